"""The host-side tile compiler, executed on the CPU and compared with the C oracle (no GPU)."""

import numpy as np
import pytest

from etha_amd import _native as nat
from oracle import c_oracle as co

from tile_interpreter import HostArena, execute

ES = {nat.F16: 2, nat.BF16: 2, nat.F32: 4, nat.F64: 8, nat.B8: 1, nat.B16: 2, nat.B32: 4, nat.B64: 8}
rs = np.random.RandomState(7)


def _mk_desc(tensor_addr, lo, hi, bucket_addr, blo, bhi, start, shape, stride, tdt, wdt):
    d = np.zeros((), dtype=nat.CHUNK_DESC)
    d["tensor_ptr"], d["tensor_lo"], d["tensor_hi"] = tensor_addr, lo, hi
    d["bucket_ptr"], d["bucket_lo"], d["bucket_hi"] = bucket_addr, blo, bhi
    nd = len(shape)
    d["ndim"] = nd
    d["start"][:nd], d["shape"][:nd], d["stride"][:nd] = start, shape, stride
    d["tensor_dtype"], d["wire_dtype"] = tdt, wdt
    return d


def _oracle_chunk(tensor_addr, start, shape, stride, tdt, wdt, off):
    return co.make_chunk(tensor_addr, start, shape, stride, tdt, wdt, bucket_off=off)


# (parent shape, permutation, slice start, chunk shape, tensor dtype, wire dtype, address skew)
GEOMETRIES = [
    ((512, 1024), None, (0, 256), (512, 256), nat.F32, nat.F32, 0),      # 1 KiB rows of a 4 KiB pitch
    ((64, 4096), None, (0, 2048), (64, 2048), nat.BF16, nat.BF16, 0),    # 4 KiB rows: run tiles per row
    ((16, 14336), None, (0, 7168), (16, 7168), nat.BF16, nat.BF16, 0),   # 14 KiB rows: ragged row tiles
    ((1024, 64), None, (0, 16), (1024, 16), nat.BF16, nat.BF16, 0),      # 32-byte rows
    ((33, 50), None, (1, 3), (31, 45), nat.BF16, nat.BF16, 0),           # odd sizes: 2-byte units
    ((33, 50), None, (1, 3), (31, 45), nat.B8, nat.B8, 3),               # byte elements at an odd address
    ((20, 30, 40), None, (2, 5, 8), (7, 11, 24), nat.F32, nat.F32, 0),   # 3-D, nothing merges
    ((20, 30, 40), (2, 0, 1), (8, 2, 5), (24, 7, 11), nat.F32, nat.F32, 0),  # permuted parent: strided elements
    ((8, 16, 64), None, (0, 0, 0), (8, 8, 64), nat.B64, nat.B64, 0),     # "slice view": half of dim 1
    ((4096,), None, (1024,), (2048,), nat.F32, nat.BF16, 0),             # fp32 -> bf16, vectorised
    ((77, 33), None, (3, 1), (70, 31), nat.F32, nat.BF16, 0),            # fp32 -> bf16, element-wise
    ((64, 256), None, (0, 0), (64, 256), nat.BF16, nat.F32, 0),          # widening wire
    ((64, 256), None, (0, 128), (64, 128), nat.F64, nat.F16, 0),
    ((64, 256), None, (0, 128), (64, 128), nat.F16, nat.BF16, 0),
    ((3,), None, (0,), (3,), nat.F32, nat.F32, 0),
    ((40000,), None, (3,), (39990,), nat.BF16, nat.BF16, 0),             # long run, the two sides skewed
    ((200000,), None, (3,), (199990,), nat.BF16, nat.BF16, 0),           # >= 256 KiB skewed run: peeled per run
    ((3, 140000), None, (0, 1), (3, 139999), nat.BF16, nat.BF16, 2),     # peeled rows of 279998 bytes
    ((64, 1024), None, (0, 5), (64, 777), nat.BF16, nat.BF16, 2),        # skewed rows of 1554 bytes
    ((9000,), None, (1,), (8990,), nat.B8, nat.B8, 1),                   # byte elements, odd everything
    ((30, 600), None, (0, 1), (30, 599), nat.F32, nat.F32, 4),           # dword-aligned skew
    ((64, 1030), None, (0, 3), (64, 1000), nat.F32, nat.BF16, 4),        # vector conversion, fp32 rows only 4-byte aligned
    ((40, 100), None, (0, 1), (40, 91), nat.BF16, nat.F16, 2),           # 8-element vectors + remainder of 3, skewed
    ((50, 77), None, (0, 0), (50, 77), nat.F64, nat.F32, 8),             # 2-element vectors + remainder of 1
    ((64, 13), None, (0, 1), (64, 12), nat.BF16, nat.BF16, 2),           # 24-byte rows at a 2-byte skew: 8-byte units
    ((64, 7), None, (0, 0), (64, 6), nat.B8, nat.B8, 1),                 # 6-byte rows at odd addresses: 2-byte units
    ((5, 0, 7), None, (0, 0, 0), (5, 0, 7), nat.F32, nat.F32, 0),        # empty chunk
]


@pytest.mark.parametrize("geom", GEOMETRIES, ids=lambda g: f"{g[0]}p{g[1]}s{g[2]}c{g[3]}t{g[4]}w{g[5]}k{g[6]}")
def test_pack_and_unpack_tiles_match_oracle(geom):
    pshape, perm, start, cshape, tdt, wdt, skew = geom
    es, ws = ES[tdt], ES[wdt]
    pn = int(np.prod(pshape))
    cn = int(np.prod(cshape))
    arena = HostArena(2 * pn * es + 4 * cn * max(es, ws) + 8192)
    t_addr = arena.alloc(pn * es, skew=skew)
    t2_addr = arena.alloc(pn * es, skew=skew)
    bucket_pad = 48  # the chunk does not start at the bucket's first byte
    b_addr = arena.alloc(cn * ws + 2 * bucket_pad)
    # element strides of the (possibly permuted) parent view
    strides = np.array([int(np.prod(pshape[i + 1:])) for i in range(len(pshape))], dtype=np.int64)
    if perm is not None:
        strides = strides[list(perm)]
    if tdt in (nat.F16, nat.BF16, nat.F32, nat.F64) and tdt != wdt:
        vals = (rs.randn(pn) * 3).astype(np.float64)
        raw = co.cast(vals.view(np.uint64), co.F64, tdt, {2: np.uint16, 4: np.uint32, 8: np.uint64}[es])
        arena.bytes_at(t_addr, pn * es)[:] = raw.view(np.uint8)
    else:
        arena.bytes_at(t_addr, pn * es)[:] = rs.randint(0, 256, pn * es)
    before_t2 = arena.bytes_at(t2_addr, pn * es).copy()
    off = bucket_pad - (bucket_pad % ws)
    desc = _mk_desc(t_addr, t_addr, t_addr + pn * es, b_addr + off, b_addr, b_addr + cn * ws + 2 * bucket_pad,
                    start, cshape, strides, tdt, wdt)
    table = nat.Table.create(desc.reshape(1), upload=False)
    assert table.info().payload_bytes == cn * ws
    # ---- pack
    src_before = arena.bytes_at(t_addr, pn * es).copy()
    bucket_before = arena.bytes_at(b_addr, cn * ws + 2 * bucket_pad).copy()
    execute(table, arena, "pack")
    want_bucket = bucket_before.copy()
    scratch = np.zeros(max(cn * es, 8), dtype=np.uint8)
    oc = _oracle_chunk(t_addr, start, cshape, strides, tdt, wdt, off)
    assert co.lib().oracle_pack_bucket(oc, 1, want_bucket.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(b_addr, cn * ws + 2 * bucket_pad), want_bucket)
    assert np.array_equal(arena.bytes_at(t_addr, pn * es), src_before), "pack wrote the source tensor"
    w = arena.writes
    assert w.max(initial=0) <= 1 and int(w.sum()) == cn * ws, "every bucket byte exactly once"
    # ---- unpack into a second tensor of the same geometry
    arena.writes[:] = 0
    desc2 = _mk_desc(t2_addr, t2_addr, t2_addr + pn * es, b_addr + off, b_addr, b_addr + cn * ws + 2 * bucket_pad,
                     start, cshape, strides, tdt, wdt)
    table2 = nat.Table.create(desc2.reshape(1), upload=False)
    execute(table2, arena, "unpack")
    want_t2 = before_t2.copy()
    oc2 = _oracle_chunk(want_t2.ctypes.data, start, cshape, strides, tdt, wdt, off)
    assert co.lib().oracle_unpack_bucket(oc2, 1, want_bucket.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(t2_addr, pn * es), want_t2), "unpack result / untouched bytes differ"
    assert arena.writes.max(initial=0) <= 1 and int(arena.writes.sum()) == cn * es


def test_skewed_chunks_use_wide_units():
    """A long chunk whose two sides are skewed must not fall back to element-sized units."""
    n, es = 1 << 20, 2
    arena = HostArena(3 * n * es + 65536)
    t = arena.alloc(n * es)
    b = arena.alloc(n * es + 64)
    d = _mk_desc(t, t, t + n * es, b + 6, b, b + n * es + 64, (0,), (n,), (1,), nat.BF16, nat.BF16)
    table = nat.Table.create(d.reshape(1), upload=False)
    run, row = table.tiles()
    body = run[(run["meta"] & (1 << 18)) != 0]
    assert len(row) == 0 and len(body) >= 1
    assert int(body["n"].sum()) * 16 >= n * es - 32  # all but head and tail move as 16-byte units
    assert len(run) - len(body) <= 2
    assert np.all(body["b"] % 16 == 0) and np.all(body["a"] % 16 == 10)


def test_odd_row_lengths_use_16_byte_bodies():
    """Rows of 150 bytes (75 bf16) at a 2-byte-aligned pitch: 9 body units + 3 remainder units per row
    instead of 75 element units."""
    rows, cols, es = 200, 75, 2
    arena = HostArena(4 * rows * 160 * es + 65536)
    t = arena.alloc(rows * 81 * es)
    arena.bytes_at(t, rows * 81 * es)[:] = rs.randint(0, 256, rows * 81 * es)
    b = arena.alloc(rows * cols * es)
    d = _mk_desc(t, t, t + rows * 81 * es, b, b, b + rows * cols * es, (0, 3), (rows, cols), (81, 1), nat.BF16, nat.BF16)
    table = nat.Table.create(d.reshape(1), upload=False)
    run, row = table.tiles()
    units = int(run["n"].sum()) + int(row["n"].sum())
    assert units == rows * (9 + 3)
    execute(table, arena, "pack")
    want = np.zeros(rows * cols * es, dtype=np.uint8)
    scratch = np.zeros(rows * cols * es, dtype=np.uint8)
    oc = co.make_chunk(t, (0, 3), (rows, cols), (81, 1), co.BF16, co.BF16, bucket_off=0)
    assert co.lib().oracle_pack_bucket(oc, 1, want.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(b, rows * cols * es), want)
    assert arena.writes.max() == 1 and int(arena.writes.sum()) == rows * cols * es


def test_bucket_ranges_and_many_chunks():
    """Chunk ranges select exactly their own tiles; un-padded prefix-sum offsets inside one bucket."""
    shapes = [(40, 24), (7, 5), (128,), (3, 9, 11), (256, 8)]
    es = 2
    total = sum(int(np.prod(s)) for s in shapes) * es
    arena = HostArena(4 * total + 65536)
    b_addr = arena.alloc(total)
    descs, ocs, off = [], [], 0
    tensors = []
    for s in shapes:
        n = int(np.prod(s))
        t = arena.alloc(n * es)
        arena.bytes_at(t, n * es)[:] = rs.randint(0, 256, n * es)
        strides = [int(np.prod(s[i + 1:])) for i in range(len(s))]
        descs.append(_mk_desc(t, t, t + n * es, b_addr + off, b_addr, b_addr + total, [0] * len(s), s, strides,
                              nat.BF16, nat.BF16))
        ocs.append((t, s, strides, off))
        tensors.append((t, n))
        off += n * es
    table = nat.Table.create(np.stack(descs), upload=False)
    run_begin, row_begin = table.ranges()
    assert len(run_begin) == len(shapes) + 1
    for first, count in ((0, 5), (1, 2), (4, 1), (2, 0)):
        arena.bytes_at(b_addr, total)[:] = 0xEE
        arena.writes[:] = 0
        execute(table, arena, "pack", first, count)
        want = np.full(total, 0xEE, dtype=np.uint8)
        scratch = np.zeros(total, dtype=np.uint8)
        for t, s, strides, o in ocs[first : first + count]:
            oc = _oracle_chunk(t, [0] * len(s), s, strides, co.BF16, co.BF16, o)
            assert co.lib().oracle_pack_bucket(oc, 1, want.ctypes.data, scratch.ctypes.data) == 0
        assert np.array_equal(arena.bytes_at(b_addr, total), want)


@pytest.mark.parametrize("op", ["sum", "avg", "max", "min", "product"])
@pytest.mark.parametrize("tdt,wdt", [(nat.BF16, nat.BF16), (nat.F32, nat.BF16), (nat.F16, nat.F16), (nat.F64, nat.F32)])
def test_reduce_tiles_match_oracle(op, tdt, wdt):
    pshape, start, cshape = (24, 96), (4, 32), (16, 64)
    es, ws = ES[tdt], ES[wdt]
    pn, cn = int(np.prod(pshape)), int(np.prod(cshape))
    n_peers = 5
    arena = HostArena(n_peers * pn * es + 2 * cn * ws + 16384)
    peers = []
    for p in range(n_peers):
        addr = arena.alloc(pn * es)
        vals = (rs.randn(pn) * (1.0 if op != "product" else 0.9) + (0.0 if op != "product" else 1.0)).astype(np.float64)
        raw = co.cast(vals.view(np.uint64), co.F64, tdt, {2: np.uint16, 4: np.uint32, 8: np.uint64}[es])
        arena.bytes_at(addr, pn * es)[:] = raw.view(np.uint8)
        peers.append(addr)
    b_addr = arena.alloc(cn * ws)
    strides = [pshape[1], 1]
    d = _mk_desc(0, 0, 0, b_addr, b_addr, b_addr + cn * ws, start, cshape, strides, tdt, wdt)
    d["n_partials"], d["partial_first"], d["reduce_op"] = n_peers, 0, nat.REDUCE_OPS[op]
    ptrs = np.asarray(peers, dtype=np.uint64)
    table = nat.Table.create(d.reshape(1), ptrs, upload=False)
    run, row = table.tiles()
    assert len(run) == 0 and len(row) > 0 and np.all(row["n_peers"] == n_peers)
    peer_bytes = [arena.bytes_at(p, pn * es).copy() for p in peers]
    execute(table, arena, "pack", peers=ptrs)
    want = np.zeros(cn * ws, dtype=np.uint8)
    scratch = np.zeros(cn * 8, dtype=np.uint8)
    oc = co.make_chunk(0, start, cshape, strides, tdt, wdt, peers=peers, op=op)
    assert co.lib().oracle_pack_bucket(oc, 1, want.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(b_addr, cn * ws), want)
    for p, before in zip(peers, peer_bytes):
        assert np.array_equal(arena.bytes_at(p, pn * es), before), "a partial was written"


def test_selfcopy_tiles():
    n = 64
    arena = HostArena(n * 4 * 4 + 8192)
    t = arena.alloc(n * 4)
    vals = np.arange(n, dtype=np.float32)
    arena.bytes_at(t, n * 4)[:] = vals.view(np.uint8)
    src = _mk_desc(t, t, t + n * 4, 0, 0, 0, (0,), (16,), (1,), nat.F32, nat.F32)
    dst = _mk_desc(t, t, t + n * 4, 0, 0, 0, (32,), (16,), (1,), nat.F32, nat.F32)
    table = nat.Table.create_selfcopy(src.reshape(1), dst.reshape(1), upload=False)
    execute(table, arena, "selfcopy")
    got = arena.bytes_at(t, n * 4).view(np.float32)
    assert np.array_equal(got[32:48], vals[:16]) and np.array_equal(got[:32], vals[:32]) and np.array_equal(got[48:], vals[48:])


def test_optimized_range_is_a_write_ordered_permutation():
    """Four column blocks of one [1024, 256] tensor arrive through four buckets; the optimized range must
    hold exactly the same tiles, ordered by the tensor address they write."""
    rows, cols, es = 1024, 256, 2
    arena = HostArena(4 * rows * cols * es + 65536)
    t = arena.alloc(rows * cols * es)
    descs, buckets = [], []
    for j in range(4):
        b = arena.alloc(rows * (cols // 4) * es)
        arena.bytes_at(b, rows * (cols // 4) * es)[:] = rs.randint(0, 256, rows * (cols // 4) * es)
        buckets.append(b)
        descs.append(_mk_desc(t, t, t + rows * cols * es, b, b, b + rows * (cols // 4) * es, (0, j * (cols // 4)),
                              (rows, cols // 4), (cols, 1), nat.BF16, nat.BF16))
    table = nat.Table.create(np.stack(descs), upload=False)
    table.optimize_range(0, 4)
    run, row = table.tiles()
    o_run, o_row = table.ordered_tiles(0, 4)
    assert len(o_run) == len(run) and len(o_row) == len(row) and len(row) > 0
    key = lambda tiles: sorted(map(bytes, tiles))
    assert key(o_row) == key(row) and key(o_run) == key(run)
    unit = 1 << (int(row[0]["meta"]) & 15)
    first_written = o_row["a"].astype(np.int64) + o_row["c0"].astype(np.int64) * unit
    assert np.all(np.diff(first_written) >= 0)
    logical = row["a"].astype(np.int64) + row["c0"].astype(np.int64) * unit
    assert not np.all(np.diff(logical) >= 0)  # bucket order is not write order here
    with pytest.raises(nat.EthaNativeError, match="not been optimized"):
        table.ordered_tiles(0, 2)


@pytest.mark.parametrize("rows,cols,blocks,tdt,wdt", [
    (1024, 64, 4, nat.BF16, nat.BF16),   # 32-byte pieces: four per 128-byte row
    (1024, 64, 8, nat.BF16, nat.BF16),   # 16-byte pieces: one unit each
    (1500, 96, 3, nat.BF16, nat.BF16),   # 64-byte pieces, three siblings, a last tile with fewer rows
    (3000, 240, 3, nat.BF16, nat.BF16),  # 160-byte pieces over several tiles per chunk: the groups continue each other
    (640, 96, 4, nat.F32, nat.BF16),     # converting: 96-byte pieces on the tensor side (48 bytes each in the bucket)
    (640, 128, 4, nat.F32, nat.BF16),    # 128-byte pieces already fill whole lines: left alone
    (300, 512, 4, nat.BF16, nat.BF16),   # 256-byte pieces likewise
    (300, 576, 4, nat.BF16, nat.BF16),   # 288-byte pieces: every piece boundary splits a line
    (40, 4032, 4, nat.BF16, nat.BF16),   # 2016-byte pieces: above the limit, left to the plain tiles
    (90, 1984, 4, nat.BF16, nat.BF16),   # 992-byte pieces: a gather tile holds four rows
    (640, 48, 6, nat.F32, nat.BF16),     # 32-byte pieces (16 bytes each in the bucket)
    (333, 40, 5, nat.B8, nat.B8),        # 8-byte pieces of byte elements
    (1000, 36, 3, nat.BF16, nat.BF16),   # 24-byte pieces: three 8-byte units, tiles hold whole rows
    (777, 48, 3, nat.BF16, nat.BF16),    # three 32-byte pieces per 96-byte row
    (515, 35, 7, nat.B8, nat.B8),        # 5-byte pieces: byte units
])
def test_short_pieces_of_one_row_are_gathered_in_an_ordered_range(rows, cols, blocks, tdt, wdt):
    """Column blocks of one tensor arrive through different buckets.  When the pieces are short, the ordered range
    holds gather tiles: each assembles whole rows from the pieces of several chunks.  Same bytes as the plain
    tiles, every destination byte written exactly once."""
    from tile_interpreter import GATHER

    es_t, es_w = ES[tdt], ES[wdt]
    piece = cols // blocks
    results = []
    for ordered in (False, True):
        arena = HostArena(rows * cols * (es_t + es_w) + 65536)
        t = arena.alloc(rows * cols * es_t)
        descs = []
        seed = np.random.RandomState(11)
        for j in range(blocks):
            nb = rows * piece * es_w
            b = arena.alloc(nb)
            if wdt == nat.BF16:  # finite values, so that a conversion has something to show
                vals = seed.randn(rows * piece).astype(np.float32)
                arena.bytes_at(b, nb)[:] = (vals.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
            else:
                arena.bytes_at(b, nb)[:] = seed.randint(0, 256, nb)
            descs.append(_mk_desc(t, t, t + rows * cols * es_t, b, b, b + nb, (0, j * piece), (rows, piece), (cols, 1), tdt, wdt))
        table = nat.Table.create(np.stack(descs), upload=False)
        if ordered:
            table.optimize_range(0, blocks)
            _, o_row = table.ordered_tiles(0, blocks)
            gathered = (o_row["meta"] & GATHER) != 0
            assert gathered.any() == (piece * es_t % 128 != 0 and piece * es_t <= 1024)
            if gathered.any():
                g = o_row[gathered]
                assert np.all(g["n_peers"] >= 2) and np.all(g["run"] == g["via"] * g["n_peers"])
                # one address per piece of every gather tile, plus the padding the kernel's fixed-size fetch needs
                assert len(table.ordered_gather(0, blocks)) == int(g["n_peers"].sum()) + 8
                # the plain tiles of the range are untouched: another range, or a pack, still uses them
                assert not np.any(table.tiles()[1]["meta"] & GATHER)
                # groups that continue each other are cut together: no short tile per group, so about as many tiles
                assert len(o_row) <= len(table.tiles()[1]) + blocks
        arena.writes = np.zeros(arena.nbytes, dtype=np.int32)
        execute(table, arena, "unpack", 0, blocks, ordered=ordered)
        counts = arena.writes[arena.offsets(np.array([t]), 1)[0]:][: rows * cols * es_t]
        assert np.all(counts == 1)
        results.append(arena.bytes_at(t, rows * cols * es_t).copy())
    assert np.array_equal(results[0], results[1])


def test_large_transposed_chunk_of_2_byte_elements_uses_wide_blocks():
    """Where 256 x 256 blocks fit, a transposing chunk of 2-byte elements is covered by them (runs of 512 bytes on
    both sides); 128 x 128 blocks and element-wise edge blocks cover the rest, every byte exactly once."""
    rows, cols, es, dt = 720, 540, 2, nat.BF16
    arena = HostArena(3 * rows * cols * es + 65536)
    t = arena.alloc(rows * cols * es)
    arena.bytes_at(t, rows * cols * es)[:] = rs.randint(0, 256, rows * cols * es)
    nj, nk = 700, 530
    b = arena.alloc(nj * nk * es)
    start, cshape, strides = (5, 3), (nj, nk), (1, rows)
    d = _mk_desc(t, t, t + rows * cols * es, b, b, b + nj * nk * es, start, cshape, strides, dt, dt)
    table = nat.Table.create(d.reshape(1), upload=False)
    tiles = table.trans_tiles()
    wide = (tiles["nj"] == 256) & (tiles["nk"] == 256)
    full = (tiles["nj"] == 128) & (tiles["nk"] == 128)
    assert int(wide.sum()) == (nj // 256) * (nk // 256) == 4
    assert int(full.sum()) == (nj // 128) * (nk // 128) - 16 == 4  # whole 128-blocks outside the 512 x 512 wide part
    assert int((~wide & ~full).sum()) == 6 * 5 - (nj // 128) * (nk // 128) == 10 and np.all(tiles["nj"][~wide] <= 128) and np.all(tiles["nk"][~wide] <= 128)
    for direction in ("pack", "unpack"):
        arena.writes[:] = 0
        if direction == "unpack":
            arena.bytes_at(t, rows * cols * es)[:] = 0
        before = arena.bytes_at(t, rows * cols * es).copy()
        execute(table, arena, direction)
        assert arena.writes.max() == 1 and int(arena.writes.sum()) == nj * nk * es
        if direction == "pack":
            want = np.zeros(nj * nk * es, dtype=np.uint8)
            scratch = np.zeros(nj * nk * es, dtype=np.uint8)
            oc = co.make_chunk(t, start, cshape, strides, dt, dt, bucket_off=0)
            assert co.lib().oracle_pack_bucket(oc, 1, want.ctypes.data, scratch.ctypes.data) == 0
            assert np.array_equal(arena.bytes_at(b, nj * nk * es), want)
            assert np.array_equal(arena.bytes_at(t, rows * cols * es), before)
        else:
            want2 = before.copy()
            oc2 = co.make_chunk(want2.ctypes.data, start, cshape, strides, dt, dt, bucket_off=0)
            assert co.lib().oracle_unpack_bucket(oc2, 1, want.ctypes.data, scratch.ctypes.data) == 0
            assert np.array_equal(arena.bytes_at(t, rows * cols * es), want2)


@pytest.mark.parametrize("wdt", [nat.BF16, nat.F16])
def test_transposed_f32_parent_converts_inside_the_lds_blocks(wdt):
    """An f32 chunk of a transposed view with a 16-bit bucket: the transposing blocks convert (pack: f32 -> wire while
    parking; unpack: wire -> f32 while emitting) instead of leaving the chunk to strided element tiles."""
    rows, cols = 310, 410
    arena = HostArena(2 * rows * cols * 4 + rows * cols * 2 + 65536)
    t = arena.alloc(rows * cols * 4)   # storage of the [cols, rows] f32 parent; the view is its transpose
    vals = (rs.randn(rows * cols) * 10.0 ** rs.uniform(-6, 6, rows * cols)).astype(np.float32)
    vals[:6] = [np.inf, -np.inf, 0.0, -0.0, 65520.0, 1e-41]
    arena.bytes_at(t, rows * cols * 4)[:] = vals.view(np.uint8)
    nj, nk = 300, 400
    b = arena.alloc(nj * nk * 2)
    start, cshape, strides = (4, 3), (nj, nk), (1, rows)
    d = _mk_desc(t, t, t + rows * cols * 4, b, b, b + nj * nk * 2, start, cshape, strides, nat.F32, wdt)
    table = nat.Table.create(d.reshape(1), upload=False)
    info, tiles = table.info(), table.trans_tiles()
    assert info.n_run_tiles == 0 and info.n_row_tiles == 0
    assert np.all(tiles["cvt"] == ((nat.F32 << 4) | wdt)) and np.all(tiles["es_log2"] == 1)
    # 128 x 256 blocks (512-byte runs on both sides) where they fit, 128 x 128 blocks and edge blocks around them
    wide = (tiles["nj"] == 128) & (tiles["nk"] == 256)
    full = (tiles["nj"] == 128) & (tiles["nk"] == 128)
    assert int(wide.sum()) == 2 and int(full.sum()) == 2 and int((~wide & ~full).sum()) == 6 and info.n_trans_tiles == 10
    before = arena.bytes_at(t, rows * cols * 4).copy()
    execute(table, arena, "pack")
    want = np.zeros(nj * nk * 2, dtype=np.uint8)
    scratch = np.zeros(nj * nk * 4, dtype=np.uint8)
    oc = co.make_chunk(t, start, cshape, strides, nat.F32, wdt, bucket_off=0)
    assert co.lib().oracle_pack_bucket(oc, 1, want.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(b, nj * nk * 2), want)
    assert np.array_equal(arena.bytes_at(t, rows * cols * 4), before)
    assert arena.writes.max() == 1 and int(arena.writes.sum()) == nj * nk * 2
    # and back: the 16-bit bucket widened into a second transposed f32 parent
    arena.writes[:] = 0
    t2 = arena.alloc(rows * cols * 4)
    before2 = arena.bytes_at(t2, rows * cols * 4).copy()
    d2 = _mk_desc(t2, t2, t2 + rows * cols * 4, b, b, b + nj * nk * 2, start, cshape, strides, nat.F32, wdt)
    table2 = nat.Table.create(d2.reshape(1), upload=False)
    assert table2.info().n_trans_tiles == 10
    execute(table2, arena, "unpack")
    want2 = before2.copy()
    oc2 = co.make_chunk(want2.ctypes.data, start, cshape, strides, nat.F32, wdt, bucket_off=0)
    assert co.lib().oracle_unpack_bucket(oc2, 1, want.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(t2, rows * cols * 4), want2)
    assert arena.writes.max() == 1 and int(arena.writes.sum()) == nj * nk * 4


@pytest.mark.parametrize("dt", [nat.B8, nat.BF16, nat.F32, nat.B64])
def test_transposed_parent_uses_lds_blocks(dt):
    """A chunk of a transposed view: the tensor side is contiguous along dim 0, the bucket along dim 1."""
    rows, cols, es = 150, 97, ES[dt]
    arena = HostArena(3 * rows * cols * es + 65536)
    t = arena.alloc(rows * cols * es)   # storage of the [cols, rows] parent; the view is its transpose
    arena.bytes_at(t, rows * cols * es)[:] = rs.randint(0, 256, rows * cols * es)
    b = arena.alloc(rows * cols * es)
    start, cshape, strides = (3, 2), (140, 90), (1, rows)  # view[i, j] = parent[j, i]
    d = _mk_desc(t, t, t + rows * cols * es, b, b, b + 140 * 90 * es, start, cshape, strides, dt, dt)
    table = nat.Table.create(d.reshape(1), upload=False)
    info = table.info()
    tiles = table.trans_tiles()
    dim = int(tiles["nj"].max())  # block side: a fixed number of bytes per row, so it depends on the element size
    assert dim >= 32 and dim * es >= 128 and int(tiles["nk"].max()) == min(dim, 90)
    assert info.n_trans_tiles == -(-140 // dim) * -(-90 // dim) and info.n_run_tiles == 0 and info.n_row_tiles == 0
    before = arena.bytes_at(t, rows * cols * es).copy()
    execute(table, arena, "pack")
    want = np.zeros(140 * 90 * es, dtype=np.uint8)
    scratch = np.zeros(140 * 90 * es, dtype=np.uint8)
    oc = co.make_chunk(t, start, cshape, strides, dt, dt, bucket_off=0)
    assert co.lib().oracle_pack_bucket(oc, 1, want.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(b, 140 * 90 * es), want)
    assert np.array_equal(arena.bytes_at(t, rows * cols * es), before)
    assert arena.writes.max() == 1 and int(arena.writes.sum()) == 140 * 90 * es
    # and back: unpack into a second transposed parent
    arena.writes[:] = 0
    t2 = arena.alloc(rows * cols * es)
    before2 = arena.bytes_at(t2, rows * cols * es).copy()
    d2 = _mk_desc(t2, t2, t2 + rows * cols * es, b, b, b + 140 * 90 * es, start, cshape, strides, dt, dt)
    execute(nat.Table.create(d2.reshape(1), upload=False), arena, "unpack")
    want2 = before2.copy()
    oc2 = co.make_chunk(want2.ctypes.data, start, cshape, strides, dt, dt, bucket_off=0)
    assert co.lib().oracle_unpack_bucket(oc2, 1, want.ctypes.data, scratch.ctypes.data) == 0
    assert np.array_equal(arena.bytes_at(t2, rows * cols * es), want2)


@pytest.mark.parametrize("tdt,wdt,ddt", [(nat.BF16, nat.BF16, nat.BF16), (nat.BF16, nat.BF16, nat.F32),
                                         (nat.F32, nat.BF16, nat.BF16), (nat.F16, nat.F16, nat.BF16),
                                         (nat.F64, nat.F32, nat.F32)])
def test_direct_reduce_tiles_round_through_the_wire_dtype(tdt, wdt, ddt):
    """A Partial source reduced straight into a (strided) target region: the result must equal reduce-pack to
    the wire dtype followed by an unpack conversion to the target dtype - two roundings, not one."""
    pshape, start, cshape = (20, 72), (2, 8), (16, 40)
    dshape, dstart = (16, 100), (0, 30)
    es, ws, ds = ES[tdt], ES[wdt], ES[ddt]
    pn, cn, dn = int(np.prod(pshape)), int(np.prod(cshape)), int(np.prod(dshape))
    n_peers = 3
    arena = HostArena(n_peers * pn * es + dn * ds + 16384)
    raw_of = {2: np.uint16, 4: np.uint32, 8: np.uint64}
    peers = []
    for p in range(n_peers):
        addr = arena.alloc(pn * es)
        vals = rs.randn(pn).astype(np.float64)
        arena.bytes_at(addr, pn * es)[:] = co.cast(vals.view(np.uint64), co.F64, tdt, raw_of[es]).view(np.uint8)
        peers.append(addr)
    d_addr = arena.alloc(dn * ds)
    arena.bytes_at(d_addr, dn * ds)[:] = 0xAB
    src = _mk_desc(0, 0, 0, 0, 0, 0, start, cshape, [pshape[1], 1], tdt, wdt)
    src["n_partials"], src["partial_first"], src["reduce_op"] = n_peers, 0, nat.REDUCE_OPS["sum"]
    dst = _mk_desc(d_addr, d_addr, d_addr + dn * ds, 0, 0, 0, dstart, cshape, [dshape[1], 1], ddt, ddt)
    ptrs = np.asarray(peers, dtype=np.uint64)
    table = nat.Table.create_selfcopy(src.reshape(1), dst.reshape(1), upload=False, partial_ptrs=ptrs)
    run, row = table.tiles()
    assert len(run) == 0 and np.all(row["n_peers"] == n_peers)
    assert np.all(row["via"] == (0 if wdt == ddt else 1 + wdt))
    execute(table, arena, "selfcopy", peers=ptrs)
    # expectation: the oracle's reduce-pack into a bucket of the wire dtype, then an element-wise cast
    bucket = np.zeros(cn * ws, dtype=np.uint8)
    scratch = np.zeros(cn * 8, dtype=np.uint8)
    oc = co.make_chunk(0, start, cshape, [pshape[1], 1], tdt, wdt, peers=peers, op="sum")
    assert co.lib().oracle_pack_bucket(oc, 1, bucket.ctypes.data, scratch.ctypes.data) == 0
    want = co.cast(bucket.view(raw_of[ws]), wdt, ddt, raw_of[ds]).reshape(cshape)
    got = arena.bytes_at(d_addr, dn * ds).view(raw_of[ds]).reshape(dshape)
    assert np.array_equal(got[dstart[0] : dstart[0] + cshape[0], dstart[1] : dstart[1] + cshape[1]], want)
    inside = np.zeros(dshape, dtype=bool)
    inside[dstart[0] : dstart[0] + cshape[0], dstart[1] : dstart[1] + cshape[1]] = True
    fill = np.frombuffer(bytes([0xAB]) * ds, dtype=raw_of[ds])[0]
    assert np.all(got[~inside] == fill), "bytes outside the destination region were written"


def test_direct_table_rejects_partial_destinations_and_selfcopy_rejects_partial_sources():
    arena = HostArena(8192)
    t = arena.alloc(1024)
    src = _mk_desc(t, t, t + 1024, 0, 0, 0, (0,), (16,), (1,), nat.F32, nat.F32)
    dst = _mk_desc(t, t, t + 1024, 0, 0, 0, (32,), (16,), (1,), nat.F32, nat.F32)
    bad_dst = dst.copy()
    bad_dst["n_partials"] = 2
    ptrs = np.asarray([t, t], dtype=np.uint64)
    with pytest.raises(nat.EthaNativeError, match="destination cannot be Partial"):
        nat.Table.create_selfcopy(src.reshape(1), bad_dst.reshape(1), upload=False, partial_ptrs=ptrs)
    bad_src = src.copy()
    bad_src["n_partials"] = 2
    with pytest.raises(nat.EthaNativeError, match="no Partial source"):
        nat.Table.create_selfcopy(bad_src.reshape(1), dst.reshape(1), upload=False)
    with pytest.raises(nat.EthaNativeError, match="outside partial_ptrs"):
        nat.Table.create_selfcopy(bad_src.reshape(1), dst.reshape(1), upload=False, partial_ptrs=ptrs[:1])


def test_expanded_source_with_zero_stride():
    """A source that is an expanded view (stride 0 along a dim) packs as that many copies; it can only be read."""
    arena = HostArena(8192)
    t = arena.alloc(64)
    row = np.arange(8, dtype=np.float32)
    arena.bytes_at(t, 32)[:] = row.view(np.uint8)
    b = arena.alloc(5 * 32 + 6 * 4 * 3)
    d = _mk_desc(t, t, t + 32, b, b, b + 5 * 32, (0, 0), (5, 8), (0, 1), nat.F32, nat.F32)
    table = nat.Table.create(d.reshape(1), upload=False)
    execute(table, arena, "pack")
    assert np.array_equal(arena.bytes_at(b, 5 * 32).view(np.float32).reshape(5, 8), np.tile(row, (5, 1)))
    # both dims expanded from one element, converting: 2 x 3 copies of one value
    d2 = _mk_desc(t + 4, t, t + 32, b, b, b + 6 * 2, (0, 0), (2, 3), (0, 0), nat.F32, nat.BF16)
    table2 = nat.Table.create(d2.reshape(1), upload=False)
    execute(table2, arena, "pack")
    want = co.cast(np.full(6, 1.0, dtype=np.float32).view(np.uint32), co.F32, co.BF16, np.uint16)
    assert np.array_equal(arena.bytes_at(b, 12).view(np.uint16), want)


@pytest.mark.parametrize("seed", range(120))
def test_random_descriptors_against_numpy(seed):
    """Random parent shapes (1-6 dims), storage permutations and padding, slices (also empty), dtype pairs,
    address skews and bucket offsets: pack must equal numpy's gather (+ the oracle's cast), unpack must write the
    region and nothing else."""
    r = np.random.RandomState(seed)
    nd = r.randint(1, 7)
    pshape = [int(r.randint(1, 7)) for _ in range(nd)]
    pshape[-1] = int(r.choice([1, 3, 8, 17, 64, 100, 257, 1024]))
    if r.rand() < 0.3 and nd > 1:
        pshape[int(r.randint(nd))] = int(r.choice([33, 70, 200]))
    floats = [nat.F16, nat.BF16, nat.F32, nat.F64]
    if r.rand() < 0.5:
        tdt, wdt = int(r.choice(floats)), int(r.choice(floats))
    else:
        tdt = wdt = int(r.choice([nat.B8, nat.B16, nat.B32, nat.B64, nat.F32, nat.BF16]))
    es, ws = ES[tdt], ES[wdt]
    raw_of = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}
    perm = list(r.permutation(nd)) if r.rand() < 0.4 else list(range(nd))
    pad = int(r.choice([0, 0, 1, 5]))  # extra elements at the end of the innermost storage dim
    stride, acc = [0] * nd, 1
    for k in range(nd - 1, -1, -1):
        stride[perm[k]] = acc
        acc *= pshape[perm[k]] + (pad if k == nd - 1 else 0)
    pn = acc
    start = [int(r.randint(0, s)) for s in pshape]
    cshape = [int(r.randint(1, s - st + 1)) for s, st in zip(pshape, start)]
    if r.rand() < 0.1:
        cshape[int(r.randint(nd))] = 0
    cn = int(np.prod(cshape))
    skew = int(r.choice([0, 0, 1, 2, 3])) * es
    arena = HostArena(2 * pn * es + cn * ws + 65536)
    t_addr, t2_addr = arena.alloc(pn * es, skew=skew), arena.alloc(pn * es, skew=skew)
    if tdt in floats:
        raw = co.cast(r.randn(pn).astype(np.float64).view(np.uint64), co.F64, tdt, raw_of[es])
    else:
        raw = r.randint(0, 256, pn * es).astype(np.uint8).view(raw_of[es])
    arena.bytes_at(t_addr, pn * es)[:] = raw.view(np.uint8)
    arena.bytes_at(t2_addr, pn * es)[:] = 0x5A
    boff = int(r.randint(0, 9)) * ws
    b_addr = arena.alloc(cn * ws + boff + 64)
    region = tuple(slice(a, a + n) for a, n in zip(start, cshape))

    def strided(flat, item):
        return np.lib.stride_tricks.as_strided(flat, shape=pshape, strides=[s * item for s in stride])

    d = _mk_desc(t_addr, t_addr, t_addr + pn * es, b_addr + boff, b_addr, b_addr + boff + cn * ws + 64, start, cshape,
                 stride, tdt, wdt)
    execute(nat.Table.create(d.reshape(1), upload=False), arena, "pack")
    want = np.ascontiguousarray(strided(raw, es)[region]).reshape(-1)
    if tdt != wdt:
        want = co.cast(want, tdt, wdt, raw_of[ws])
    assert np.array_equal(arena.bytes_at(b_addr + boff, cn * ws).view(raw_of[ws]), want), "pack"
    d2 = _mk_desc(t2_addr, t2_addr, t2_addr + pn * es, b_addr + boff, b_addr, b_addr + boff + cn * ws + 64, start, cshape,
                  stride, tdt, wdt)
    execute(nat.Table.create(d2.reshape(1), upload=False), arena, "unpack")
    back = arena.bytes_at(t2_addr, pn * es).view(raw_of[es])
    want_back = want if tdt == wdt else co.cast(want, wdt, tdt, raw_of[es])
    assert np.array_equal(strided(back, es)[region], want_back.reshape(cshape)), "unpack"
    untouched = np.ones(pn, dtype=bool)
    untouched[strided(np.arange(pn), 8)[region].reshape(-1)] = False
    fill = np.frombuffer(bytes([0x5A]) * es, dtype=raw_of[es])[0]
    assert np.all(back[untouched] == fill), "bytes outside the region were written"


def test_self_copy_buckets_that_feed_each_other_are_not_merged():
    """Two LOCAL buckets inside one tensor, the second reading what the first writes: merged launches keep
    them apart (a merged launch has no order inside), and the interpreter, run in the executor's order,
    gives the stream-ordered result."""
    import torch

    from etha_amd.comm import Chunk, LoopbackWire, Transport, chunk_to_bucket_ops
    from tile_interpreter import AbsoluteMemory

    def chunk(t, src, dst, n):
        return Chunk(chunk_shape=(n,), transport=Transport.LOCAL, is_source=True, is_target=True, src_rank=0, src_idx=(src // n,),
                     dst_ranks=(0,), dst_idx=(dst // n,), src_slice=(slice(src, src + n),), dst_slice=(slice(dst, dst + n),),
                     tensor=t, rank=0)

    t = torch.arange(64, dtype=torch.float32)
    want = t.clone()
    want[16:32] = want[0:16]
    want[32:48] = want[16:32]  # reads what the first copy wrote
    buckets = chunk_to_bucket_ops([chunk(t, 0, 16, 16), chunk(t, 16, 32, 16)], bucket_size=1)  # one chunk per bucket
    assert len(buckets) == 2
    other = torch.zeros(32)
    independent = chunk_to_bucket_ops([chunk(other, 0, 8, 8), chunk(other, 16, 24, 8)], bucket_size=1)
    for pool in ("resident", "ring"):
        wire = LoopbackWire("cpu", host_inspection=True, pool=pool)
        plan = wire.plan(buckets)
        assert [s[0] for s in plan.steps] == ["selfcopy", "selfcopy"]
        assert len(plan.merged_steps) == 2  # not fused: the second launch must run after the first
        assert len(wire.plan(independent).merged_steps) == 2  # same tensor: kept apart as well (allocation granularity)
    st = t.untyped_storage()
    mem = AbsoluteMemory(st.data_ptr(), st.data_ptr() + st.nbytes())
    for kind, first, count, _ in plan.merged_steps:
        execute(plan.local_table, mem, "selfcopy", first, count)
    assert torch.equal(t, want)
    # the ring pipeline with merged launches: both buckets become ready in one sweep, and still get a launch each,
    # the second one in stream order behind the first
    from etha_amd.comm import bucket_comm

    wire = LoopbackWire("cpu", host_inspection=True, pool="ring")
    log = wire.launch_log = []
    wire.on_launch = lambda *a: None
    bucket_comm(buckets, wire=wire, merge_launches=True, synchronize=False)
    assert [(kind, count) for kind, _, count, _ in log] == [("selfcopy", 1), ("selfcopy", 1)]
    assert log[1][3] == 0 and log[0][1] < log[1][1]
