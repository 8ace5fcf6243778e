"""A CPU interpreter of the compiled tile program (test infrastructure).

Descriptor addresses are plain integers, so a table can be compiled against *host* buffers and its
tiles executed here with numpy, doing exactly what the kernels do per work-item.  That checks the
host-side tile compiler (addresses, alignment classes, row walking, tails) with full bounds and
coverage checking and no GPU.
"""

from __future__ import annotations

import ctypes

import numpy as np

from oracle import c_oracle as co

THREADS = 256
_CODE_RAW = {0: np.uint16, 1: np.uint16, 2: np.uint32, 3: np.uint64,  # f16 bf16 f32 f64
             8: np.uint8, 9: np.uint8, 10: np.uint16, 11: np.uint32, 12: np.uint64, 13: np.uint8, 14: np.uint8, 15: np.uint8}
_CODE_SIZE = {k: np.dtype(v).itemsize for k, v in _CODE_RAW.items()}


class HostArena:
    """One host allocation holding every buffer, so that addresses map to offsets."""

    def __init__(self, nbytes: int, fill: int = 0xA5):
        self.buf = np.full(nbytes + 256, fill, dtype=np.uint8)
        base = self.buf.ctypes.data
        self.pad = (-base) % 256
        self.base = base + self.pad
        self.nbytes = nbytes
        self.cursor = 0
        self.writes = np.zeros(nbytes, dtype=np.uint16)

    def alloc(self, nbytes: int, align: int = 256, skew: int = 0) -> int:
        self.cursor = -(-self.cursor // align) * align + skew
        addr = self.base + self.cursor
        self.cursor += nbytes
        assert self.cursor <= self.nbytes
        return addr

    def bytes_at(self, addr: int, n: int) -> np.ndarray:
        off = addr - self.base
        assert 0 <= off and off + n <= self.nbytes, "address outside the arena"
        return self.buf[self.pad + off : self.pad + off + n]

    def offsets(self, addrs: np.ndarray, width: int) -> np.ndarray:
        off = addrs.astype(np.int64) - self.base
        assert off.min() >= 0 and off.max() + width <= self.nbytes, "tile touches memory outside the arena"
        return off


class AbsoluteMemory:
    """The process's own address space as the arena: tiles compiled against live host tensors.

    Only the bytes the tiles name are touched (numpy fancy indexing), so the view may span unmapped
    gaps between allocations.  No coverage counters (the span can be many gigabytes)."""

    def __init__(self, lo: int, hi: int):
        self.base, self.nbytes, self.pad = lo, hi - lo, 0
        self.buf = np.ctypeslib.as_array((ctypes.c_uint8 * (hi - lo)).from_address(lo))
        self.writes = None

    def offsets(self, addrs: np.ndarray, width: int) -> np.ndarray:
        off = addrs.astype(np.int64) - self.base
        assert off.min() >= 0 and off.max() + width <= self.nbytes, "tile touches memory outside the declared span"
        return off


GATHER = 1 << 21  # row tile that assembles each row from pieces of several chunks (ordered unpack ranges only)


def _unit_positions(run_tiles, row_tiles, gather=None):
    """Per active work-item: (a address, b address, meta, tile kind, row-tile index)."""
    out = []
    if len(run_tiles):
        n = run_tiles["n"].astype(np.int64)
        tid = np.concatenate([np.arange(k) for k in n]) if n.sum() else np.zeros(0, np.int64)
        rep = np.repeat(np.arange(len(run_tiles)), n)
        meta = run_tiles["meta"][rep]
        a = run_tiles["a"][rep].astype(np.int64) + (tid << (meta & 15))
        b = run_tiles["b"][rep].astype(np.int64) + (tid << ((meta >> 4) & 15))
        out.append((a, b, meta, np.full(len(a), -1)))
    if len(row_tiles):
        n = row_tiles["n"].astype(np.int64)
        tid = np.concatenate([np.arange(k) for k in n]) if n.sum() else np.zeros(0, np.int64)
        rep = np.repeat(np.arange(len(row_tiles)), n)
        t = row_tiles[rep]
        meta = t["meta"]
        run = t["run"].astype(np.int64)
        q = t["c0"].astype(np.int64) + tid
        assert np.all(t["c0"] < t["run"])
        big = run >= THREADS
        r = np.where(big, (q >= run).astype(np.int64), q // run)
        c = q - r * run
        assert np.all(c < run) and np.all(c >= 0)
        a = t["a"].astype(np.int64) + r * t["a_pitch"] + (c << (meta & 15))
        b = t["b"].astype(np.int64) + r * t["b_pitch"] + (c << ((meta >> 4) & 15))
        g = (meta & GATHER) != 0
        if g.any():
            assert gather is not None and np.all(t["n_peers"][g] >= 2) and np.all(t["via"][g] > 0)
            assert np.all(t["run"][g] == t["via"][g] * t["n_peers"][g])
            piece = c[g] // t["via"][g].astype(np.int64)
            base = gather[t["peer_first"][g].astype(np.int64) + piece].astype(np.int64)
            b[g] = base + r[g] * t["b_pitch"][g] + ((c[g] - piece * t["via"][g].astype(np.int64)) << ((meta[g] >> 4) & 15))
        out.append((a, b, meta, rep))
    return out


_TOUCHED: dict | None = None  # while execute(..., touched=d) runs: d["r"] / d["w"] collect byte offsets


def _note(kind: str, offsets: np.ndarray) -> None:
    if _TOUCHED is not None:
        _TOUCHED[kind].append(np.unique(offsets.reshape(-1)))


def execute(table, arena, direction: str, first: int = 0, count: int | None = None,
            peers: np.ndarray | None = None, ordered: bool = False, touched: dict | None = None) -> None:
    """Run chunks [first, first+count) of a table on the host. direction: 'pack' | 'unpack' | 'selfcopy'.
    ``ordered``: use the write-ordered copy of the range (it must have been optimized).
    ``touched``: a dict whose lists ``"r"`` and ``"w"`` receive the arena byte offsets this launch reads / writes."""
    global _TOUCHED
    _TOUCHED = touched
    if touched is not None:
        touched.setdefault("r", [])
        touched.setdefault("w", [])
    try:
        _execute(table, arena, direction, first, count, peers, ordered)
    finally:
        _TOUCHED = None


def _execute(table, arena, direction, first, count, peers, ordered) -> None:
    global THREADS
    THREADS = int(table.info().tile_threads)
    run_begin, row_begin = table.ranges()
    if count is None:
        count = len(run_begin) - 1 - first
    gather = None
    if ordered:
        run_tiles, row_tiles = table.ordered_tiles(first, count)
        gather = table.ordered_gather(first, count)
        assert direction == "unpack" or not np.any(row_tiles["meta"] & GATHER)
    else:
        run_tiles, row_tiles = table.tiles()
        run_tiles = run_tiles[run_begin[first] : run_begin[first + count]]
        row_tiles = row_tiles[row_begin[first] : row_begin[first + count]]
    trans_begin = table.trans_ranges()
    trans = table.trans_tiles()[trans_begin[first] : trans_begin[first + count]]
    if len(trans):
        _transpose_blocks(arena, trans, direction == "unpack", peers)
    assert np.all(run_tiles["n"] <= THREADS) and np.all(row_tiles["n"] <= THREADS)
    assert np.all(run_tiles["n"] > 0) and np.all(row_tiles["n"] > 0)
    rev = direction == "unpack"
    mem = arena.buf[arena.pad : arena.pad + arena.nbytes]
    for a, b, meta, row_idx in _unit_positions(run_tiles, row_tiles, gather):
        for m in np.unique(meta):
            sel = meta == m
            ua, ub = 1 << (int(m) & 15), 1 << ((int(m) >> 4) & 15)
            dta, dtb = (int(m) >> 8) & 15, (int(m) >> 12) & 15
            cvt, vec = bool(int(m) & (1 << 16)), bool(int(m) & (1 << 17))
            skew_a, skew_b = bool(int(m) & (1 << 18)), bool(int(m) & (1 << 19))
            reduce = row_idx[sel][0] >= 0 and int(row_tiles["n_peers"][row_idx[sel][0]]) > 0 and not (int(m) & GATHER)
            # (for reduce tiles the a side is an offset from each peer's base: checked against the real addresses below)
            assert reduce or skew_a or np.all(a[sel] % ua == 0), "misaligned vector access on the a side"
            assert skew_b or np.all(b[sel] % ub == 0), "misaligned vector access on the b side"
            generic = bool(int(m) & (1 << 20))  # an integer, bool or 8-bit float side: one element per unit
            if cvt and not reduce:  # typed accesses: every element must sit at a multiple of its size, skewed or not
                assert np.all(a[sel] % _CODE_SIZE[dta] == 0) and np.all(b[sel] % _CODE_SIZE[dtb] == 0), "misaligned element"
                assert generic == (dta > 3 or dtb > 3)
                if generic:
                    assert (ua, ub) == (_CODE_SIZE[dta], _CODE_SIZE[dtb]) and not vec
                else:  # the unit's element count is stated in the meta word and agrees with both unit sizes
                    n_el = 1 << ((int(m) >> 22) & 3)
                    assert ua == n_el * _CODE_SIZE[dta] and ub == n_el * _CODE_SIZE[dtb], "unit sizes and element count disagree"
            if reduce:
                _reduce_units(arena, mem, row_tiles, row_idx[sel], a[sel], b[sel], ua, ub, dta, dtb, peers, skew_a)
                continue
            src, dst, us, ud, ds_, dd = (b[sel], a[sel], ub, ua, dtb, dta) if rev else (a[sel], b[sel], ua, ub, dta, dtb)
            so = arena.offsets(src, us)[:, None] + np.arange(us)
            do = arena.offsets(dst, ud)[:, None] + np.arange(ud)
            data = mem[so]
            if cvt:
                assert not vec or (max(us, ud) in (16, 32) and min(us, ud) <= 16)
                raw_s, raw_d = _CODE_RAW[ds_], _CODE_RAW[dd]
                elems = np.ascontiguousarray(data).view(raw_s)
                data = co.cast(elems, ds_, dd, raw_d).view(np.uint8).reshape(len(so), ud)
            else:
                assert us == ud
            if arena.writes is not None:
                np.add.at(arena.writes, do.reshape(-1), 1)
            _note("r", so)
            _note("w", do)
            mem[do] = data


def _transpose_blocks(arena, trans, rev: bool, peers=None) -> None:
    mem = arena.buf[arena.pad : arena.pad + arena.nbytes]
    for t in trans:
        es = 1 << int(t["es_log2"])
        nj, nk = int(t["nj"]), int(t["nk"])
        assert 0 < nj <= 512 and 0 < nk <= 512  # block side: a fixed number of bytes per row
        cvt = int(t["cvt"])
        typed = bool(cvt & 256)
        dta, dtb = (cvt >> 4) & 15, cvt & 15
        n_peers = int(t["n_peers"])
        if typed:  # a block of the typed kernel: any pair of value types, or a Partial source reduced with one op
            dim = 64 if 8 in (_CODE_SIZE[dta], _CODE_SIZE[dtb]) else 128
            assert nj <= dim and nk <= dim and (dta != dtb or n_peers)
            assert not n_peers or (not rev and dta <= 3 and dtb <= 3 and int(t["reduce_op"]) <= 4)
        else:
            assert n_peers == 0
            if cvt:  # a converting block: f32 on the a side, f16 or bf16 in the bucket; blocks are sized by the b side
                assert dta == 2 and dtb in (0, 1) and es == 2 and nj <= 128 and nk <= 256
        esa, esb = (_CODE_SIZE[dta], _CODE_SIZE[dtb]) if cvt else (es, es)
        j, k = np.meshgrid(np.arange(nj), np.arange(nk), indexing="ij")
        a = int(t["a"]) + j * esa + k * int(t["a_pitch"])
        b = int(t["b"]) + j * int(t["b_pitch"]) + k * esb
        assert np.all(a % esa == 0) and np.all(b % esb == 0)
        src, dst, ess, esd, ds_, dd = (b, a, esb, esa, dtb, dta) if rev else (a, b, esa, esb, dta, dtb)
        do = arena.offsets(dst.reshape(-1), esd)[:, None] + np.arange(esd)
        if arena.writes is not None:
            np.add.at(arena.writes, do.reshape(-1), 1)
        _note("w", do)
        if n_peers:  # src holds offsets from each member's base
            bases = peers[int(t["peer_first"]) : int(t["peer_first"]) + n_peers].astype(np.int64)
            staged = []
            for base in bases:
                assert base % esa == 0, "misaligned member"
                so = arena.offsets(base + src.reshape(-1), ess)[:, None] + np.arange(ess)
                _note("r", so)
                staged.append(np.ascontiguousarray(mem[so]).reshape(-1).copy())
            via = int(t["via"])
            out_dt = via - 1 if via else dd
            n_el = src.size
            out = np.zeros(n_el, dtype=_CODE_RAW[out_dt])
            scratch = np.zeros(n_el, dtype=np.float64)
            op = {0: "sum", 1: "avg", 2: "max", 3: "min", 4: "product"}[int(t["reduce_op"])]
            ch = co.make_chunk(0, (0,), (n_el,), (1,), ds_, out_dt, peers=[s.ctypes.data for s in staged], op=op)
            assert co.lib().oracle_reduce(ch, out.ctypes.data, scratch.ctypes.data) == 0
            if via:
                out = co.cast(out, out_dt, dd, _CODE_RAW[dd])
            mem[do] = out.view(np.uint8).reshape(n_el, esd)
            continue
        so = arena.offsets(src.reshape(-1), ess)[:, None] + np.arange(ess)
        _note("r", so)
        data = mem[so]
        if cvt:
            elems = np.ascontiguousarray(data).view(_CODE_RAW[ds_]).reshape(-1)
            data = co.cast(elems, ds_, dd, _CODE_RAW[dd]).view(np.uint8).reshape(len(so), esd)
        mem[do] = data


def _reduce_units(arena, mem, row_tiles, row_idx, a_off, b, ua, ub, dta, dtb, peers, skew_a=False):
    es = {0: 2, 1: 2, 2: 4, 3: 8}[dta]
    n_el = ua // es
    for ti in np.unique(row_idx):
        sel = row_idx == ti
        t = row_tiles[ti]
        bases = peers[int(t["peer_first"]) : int(t["peer_first"]) + int(t["n_peers"])].astype(np.int64)
        op = {0: "sum", 1: "avg", 2: "max", 3: "min", 4: "product"}[int(t["reduce_op"]) & 7]
        offs = a_off[sel]
        n_units = len(offs)
        via = int(t["via"])  # 0, or 1 + the dtype the result is rounded to before the b-side dtype
        out_dt = via - 1 if via else dtb
        out = np.zeros(n_units * n_el, dtype=_CODE_RAW[out_dt])
        scratch = np.zeros(n_units * n_el, dtype=np.float64)
        # gather each peer's units into a contiguous staging array, then let the C oracle combine them
        staged = []
        for base in bases:
            assert skew_a or np.all((base + offs) % ua == 0), "misaligned vector access on a peer"
            assert np.all((base + offs) % es == 0), "misaligned element on a peer"
            so = arena.offsets(base + offs, ua)[:, None] + np.arange(ua)
            _note("r", so)
            staged.append(np.ascontiguousarray(mem[so]).reshape(-1).copy())
        word = int(t["reduce_op"])
        g0, g1 = (word >> 16) & 255, (word >> 24) & 255
        names = {0: "sum", 1: "avg", 2: "max", 3: "min", 4: "product"}
        if g0 == 0:  # one level over all peers, in list order
            ch = co.make_chunk(0, (0,), (n_units * n_el,), (1,), dta, out_dt, peers=[s.ctypes.data for s in staged], op=op)
            assert co.lib().oracle_reduce(ch, out.ctypes.data, scratch.ctypes.data) == 0
        else:  # nested levels: accumulators stay in fp32 (f64 for f64 inputs) between levels, one rounding at the end
            g1 = g1 or 1
            sizes = [g0, g1, len(staged) // (g0 * g1)]
            assert sizes[0] * sizes[1] * sizes[2] == len(staged)
            acc_dt = 3 if dta == 3 else 2
            values, cur_dt = staged, dta
            for level, size in enumerate(sizes):
                last = level == 2
                nxt = []
                for i in range(0, len(values), size):
                    o = out if last else np.zeros(n_units * n_el, dtype=_CODE_RAW[acc_dt])
                    ch = co.make_chunk(0, (0,), (n_units * n_el,), (1,), cur_dt, out_dt if last else acc_dt,
                                       peers=[v.ctypes.data for v in values[i:i + size]], op=names[(word >> (3 * level)) & 7])
                    assert co.lib().oracle_reduce(ch, o.ctypes.data, scratch.ctypes.data) == 0
                    nxt.append(o)
                values, cur_dt = nxt, acc_dt
            assert len(values) == 1
        if via:
            out = co.cast(out, out_dt, dtb, _CODE_RAW[dtb])
        do = arena.offsets(b[sel], ub)[:, None] + np.arange(ub)
        if arena.writes is not None:
            np.add.at(arena.writes, do.reshape(-1), 1)
        _note("w", do)
        mem[do] = out.view(np.uint8).reshape(n_units, ub)
