"""Host planner: route tables, chunk slices, bucket coalescing, uneven and same-rank cases (no GPU)."""

import numpy as np
import pytest
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from etha_amd import workloads
from etha_amd.comm import Transport, chunk_to_bucket_ops, get_m2m_map, m2m_to_chunks
from etha_amd.layout import local_shape, mesh_coord


def test_config1_grid_and_routes():
    """(2,) Shard(0) -> (4,) Shard(1): grid [2,4], source cut 4 ways along dim 1, 8 P2P routes."""
    m = get_m2m_map([0, 1], (Shard(0),), [2, 3, 4, 5], (Shard(1),))
    assert m.source_num_slicers == [1, 4] and m.target_num_slicers == [2, 1]
    assert [(r.src.rank, r.src.cell, r.dsts[0].rank, r.dsts[0].cell, r.kind) for r in m.routes] == [
        (s, (0, j), 2 + j, (s, 0), Transport.P2P) for s in (0, 1) for j in range(4)
    ]
    src = torch.empty(512, 1024, device="meta")
    chunks = m2m_to_chunks(m, 0, source_tensor=src)
    assert [c.src_slice for c in chunks] == [(slice(0, 512), slice(256 * j, 256 * (j + 1))) for j in range(4)]
    assert all(c.chunk_shape == (512, 256) and c.nbytes == 512 * 1024 for c in chunks)
    tgt = torch.empty(1024, 256, device="meta")
    rchunks = m2m_to_chunks(m, 3, target_tensor=tgt)
    assert [(c.src_rank, c.dst_slice) for c in rchunks] == [
        (0, (slice(0, 512), slice(0, 256))), (1, (slice(512, 1024), slice(0, 256)))]


def test_replicated_source_picks_replica_by_target_position():
    """Target flat position t reads the replica group of source flat position t % |source|."""
    m = get_m2m_map([[0, 1], [2, 3]], (Replicate(), Shard(0)), [4, 5, 6, 7], (Shard(0),))
    got = {(r.src.rank, r.src.cell): [(d.rank, d.cell) for d in r.dsts] for r in m.routes}
    # grid [4]; source shard j holds cells 2j, 2j+1; targets 4,5,6,7 view replicas of ranks 0,1,2,3 -> rows 0,0,1,1
    assert got == {(0, (0,)): [(4, (0,))], (0, (1,)): [(5, (0,))], (3, (0,)): [(6, (0,))], (3, (1,)): [(7, (0,))]}


def test_broadcast_routes_and_order():
    m = get_m2m_map(list(range(8)), (Shard(0),), [8, 9], (Replicate(),))
    assert all(r.kind == Transport.BROADCAST and [d.rank for d in r.dsts] == [8, 9] for r in m.routes)
    assert [r.src.rank for r in m.routes] == list(range(8))
    assert m.target_num_slicers == [8]


def test_partial_shadows_reach_the_whole_component():
    """(2,3) double Partial -> (2,) Replicate: only ranks 0,1 ship, but all 6 must take part."""
    m = get_m2m_map(np.arange(6).reshape(2, 3), (Partial(), Partial()), [6, 7], (Replicate(),))
    assert m.source_partial_reductions == [(0, "sum"), (1, "sum")]
    shipping = [(r.src.rank, [d.rank for d in r.dsts]) for r in m.routes if r.dsts]
    assert shipping == [(0, [6]), (1, [7])]
    shadows = sorted(r.src.rank for r in m.routes if r.kind == Transport.NONE)
    assert shadows == [2, 3, 4, 5]
    with pytest.raises(NotImplementedError, match="contains Partial"):
        get_m2m_map([0, 1], (Shard(0),), [2, 3], (Partial(),))


def test_bucket_rule():
    src = torch.empty(64, 64, dtype=torch.float32, device="meta")
    m = get_m2m_map([0], (Replicate(),), [1, 2], (Shard(0),))
    chunks = []
    for _ in range(5):
        chunks += m2m_to_chunks(m, 0, source_tensor=src)  # 5 tensors x 2 chunks of 8 KiB, keys (0,(1,)) and (0,(2,))
    assert [c.nbytes for c in chunks] == [8192] * 10
    one = chunk_to_bucket_ops(chunks, 1)
    assert len(one) == 10 and all(len(b.chunks) == 1 for b in one)
    b20k = chunk_to_bucket_ops(chunks, 20000)
    # per key: 3 chunks close a bucket (24576 >= 20000); the remaining 2 are flushed at the end, key order
    assert [(b.dst_ranks, len(b.chunks)) for b in b20k] == [((1,), 3), ((2,), 3), ((1,), 2), ((2,), 2)]
    assert b20k[0].offsets == [0, 8192, 16384] and b20k[0].total_bytes == 24576
    big = chunk_to_bucket_ops(chunks, 8192)  # a chunk of at least bucket_size is a bucket of its own
    assert len(big) == 10
    # every chunk lands in exactly one bucket, order inside a key preserved
    for buckets in (one, b20k, big):
        seen = [id(c) for b in buckets for c in b.chunks]
        assert sorted(seen) == sorted(id(c) for c in chunks)


def test_uneven_vocab_rows_follow_torch_chunk():
    """151936 rows over 6 ranks: 5 x 25323 + 25321; the target cuts its rows at the same places."""
    rows = 151936
    m = get_m2m_map(list(range(6)), (Shard(0),), [6, 7, 8, 9], (Shard(1),))
    sizes = [local_shape((rows, 64), (6,), (Shard(0),), mesh_coord((6,), r))[0] for r in range(6)]
    assert sizes == [25323] * 5 + [25321]
    tgt = torch.empty(rows, 16, device="meta", dtype=torch.bfloat16)
    rchunks = m2m_to_chunks(m, 6, target_tensor=tgt)
    assert [c.chunk_shape[0] for c in rchunks] == sizes
    assert rchunks[-1].dst_slice[0] == slice(5 * 25323, rows)
    for r in range(6):
        src = torch.empty(sizes[r], 64, device="meta", dtype=torch.bfloat16)
        s = m2m_to_chunks(m, r, source_tensor=src)
        assert [c.chunk_shape for c in s] == [(sizes[r], 16)] * 4
    # a dim that is cut on both sides cannot be uneven
    m2 = get_m2m_map([0, 1], (Shard(0),), [2, 3, 4, 5], (Shard(0),))
    with pytest.raises(ValueError, match="not divisible"):
        m2m_to_chunks(m2, 1, source_tensor=torch.empty(9, 4, device="meta"))


def test_same_rank_destination_becomes_local_chunk():
    m = get_m2m_map([0, 1], (Shard(0),), [0, 1], (Shard(1),))
    src = torch.empty(4, 8, device="meta")
    tgt = torch.empty(8, 4, device="meta")
    chunks = m2m_to_chunks(m, 0, source_tensor=src, target_tensor=tgt)
    kinds = [(c.transport, c.is_source, c.is_target, c.dst_ranks) for c in chunks]
    assert kinds == [
        (Transport.LOCAL, True, True, (0,)),  # cell (0,0): rank 0 -> rank 0
        (Transport.P2P, True, False, (1,)),  # cell (0,1): rank 0 -> rank 1
        (Transport.P2P, False, True, (0,)),  # from rank 1
    ]
    local = chunks[0]
    assert local.src_tensor is src and local.tensor is tgt
    assert local.src_slice == (slice(0, 4), slice(0, 4)) and local.dst_slice == (slice(0, 4), slice(0, 4))


def test_llama3_8b_share_matches_the_published_shape_of_the_workload():
    specs, targets, bucket = workloads.llama3_8b_fsdp8_to_tp2()
    assert len(specs) == 290 and targets == [8] and bucket == 64 << 20
    params = sum(int(np.prod(s.shape)) for s in specs)
    assert params == 8_030_257_152
    cache = {}
    recv, send = [], {r: [] for r in range(8)}
    for s in specs:
        key = (s.target_placements,)
        if key not in cache:
            cache[key] = get_m2m_map(s.source_mesh, s.source_placements, s.target_mesh, s.target_placements)
        m = cache[key]
        t_shape = local_shape(s.shape, (2,), s.target_placements, (0,))
        recv += m2m_to_chunks(m, 8, target_tensor=torch.empty(t_shape, dtype=s.source_dtype, device="meta"))
        for r in range(8):
            s_shape = local_shape(s.shape, (8,), s.source_placements, (r,))
            cs = m2m_to_chunks(m, r, source_tensor=torch.empty(s_shape, dtype=s.source_dtype, device="meta"))
            send[r] += [c for c in cs if 8 in c.dst_ranks]
    assert len(recv) == 1672
    assert sum(c.nbytes for c in recv) == 8_030_519_296
    assert sum(len(v) for v in send.values()) == 1672
    kinds = {"col": 0, "row": 0, "norm": 0}
    for c in recv:
        kinds["norm" if len(c.chunk_shape) == 1 else ("row" if c.dst_slice[1] == slice(0, c.tensor.shape[1]) and c.tensor.shape[1] in (2048, 7168) else "col")] += 1
    assert kinds == {"col": 648, "row": 512, "norm": 512}
    buckets = chunk_to_bucket_ops(recv, bucket)
    assert sum(b.total_bytes for b in buckets) == 8_030_519_296
    assert all(b.total_bytes < 2 * bucket or len(b.chunks) == 1 for b in buckets)


def test_partial_and_plain_tensors_bucket_alike_on_both_ends():
    """A batch with a Partial-source tensor and a plain tensor between the same ranks: the sender keeps
    them in different buckets (different reduce signature), so the receiver must too."""
    from etha_amd.world import create_partial_groups

    plain = get_m2m_map([0, 1], (Shard(0),), [2], (Replicate(),))
    part = get_m2m_map([0, 1], (Partial(),), [2], (Replicate(),))
    src_plain = {r: torch.empty(4, 8, device="meta") for r in (0, 1)}
    src_part = {r: torch.empty(8, 8, device="meta") for r in (0, 1)}
    tgt = torch.empty(8, 8, device="meta")
    groups = create_partial_groups([0, 1], part.source_partial_reductions, 0, src_part)
    send = m2m_to_chunks(plain, 0, source_tensor=src_plain[0]) + m2m_to_chunks(part, 0, source_tensor=src_part[0],
                                                                             source_partial_groups=groups)
    recv = m2m_to_chunks(plain, 2, target_tensor=tgt) + m2m_to_chunks(part, 2, target_tensor=tgt)
    send_b = [b for b in chunk_to_bucket_ops(send, 1 << 30) if b.dst_ranks]
    recv_b = [b for b in chunk_to_bucket_ops(recv, 1 << 30) if b.src_rank == 0]
    assert [[c.nbytes for c in b.chunks] for b in send_b] == [[c.nbytes for c in b.chunks] for b in recv_b]
    assert len(send_b) == 2 and recv_b[1].chunks[0].source_partial_signature == (((0, 1), "sum", ()),)
    # the receive chunks name the group exactly as the send chunks do
    assert recv_b[1].chunks[0].partial_signature == send_b[1].chunks[0].partial_signature


def test_partial_reductions_that_nest_differently_bucket_alike_on_both_ends():
    """Two Partial tensors over the same six ranks with the same two ops, but sum over 2 then avg over 3 in one and sum
    over 3 then avg over 2 in the other: different groups, so the sender keeps their chunks in separate buckets, and
    the receiver has to split the channel the same way (found by a sweep of random batches on the GPU)."""
    from etha_amd.world import create_partial_groups

    mesh_a, mesh_b = np.arange(6).reshape(2, 3), np.arange(6).reshape(3, 2)
    pl = (Partial("sum"), Partial("avg"))
    maps = [get_m2m_map(mesh_a, pl, [6], (Replicate(),)), get_m2m_map(mesh_b, pl, [6], (Replicate(),))]
    src = [{r: torch.empty(4, 8, device="meta") for r in range(6)} for _ in maps]
    tgt = torch.empty(4, 8, device="meta")
    send_keys, recv_keys = [], []
    for r in range(6):
        send = []
        for m, mesh, tensors in zip(maps, (mesh_a, mesh_b), src):
            groups = create_partial_groups(mesh, m.source_partial_reductions, r, tensors)
            send += m2m_to_chunks(m, r, source_tensor=tensors[r], source_partial_groups=groups)
        send_b = [b for b in chunk_to_bucket_ops(send, 1 << 30) if b.dst_ranks]
        recv = [c for m in maps for c in m2m_to_chunks(m, 6, target_tensor=tgt)]
        recv_b = [b for b in chunk_to_bucket_ops(recv, 1 << 30) if b.src_rank == r]
        assert [[c.nbytes for c in b.chunks] for b in send_b] == [[c.nbytes for c in b.chunks] for b in recv_b], r
        for sb, rb in zip(send_b, recv_b):
            assert sb.chunks[0].partial_signature == rb.chunks[0].partial_signature
        send_keys += [b.chunks[0].partial_signature for b in send_b]
        recv_keys += [b.chunks[0].partial_signature for b in recv_b]
    assert len(set(send_keys)) == 2 and send_keys == recv_keys  # the rank that ships the reduced chunks has one bucket per group


def test_strided_shard_grids():
    """A strided shard in its usual pairing (split factor = size of the later Shard mesh dim on the same tensor
    dim) keeps the reference's lcm-of-shard-counts grid; any other split factor scatters a rank's pieces more
    finely and the dim is gridded by the finest cut."""
    from torch.distributed.tensor.placement_types import _StridedShard

    # the reference's own table: target (R, _StridedShard(1, 2), R, Shard(1)) on mesh (1,2,1,2) - paired
    src = np.arange(4).reshape(2, 2, 1, 1)
    tgt = np.arange(4, 8).reshape(1, 2, 1, 2)
    m = get_m2m_map(src, (Replicate(), Replicate(), Shard(0), Shard(1)), tgt,
                    (Replicate(), _StridedShard(1, split_factor=2), Replicate(), Shard(1)))
    assert m.source_num_slicers == [1, 4] and m.target_num_slicers == [1, 1]
    # unpaired: mesh (2,) _StridedShard(0, 3) -> rank r holds pieces {r, 2 + r, 4 + r} of six
    m = get_m2m_map([0, 1], (_StridedShard(0, split_factor=3),), [2, 3], (Shard(0),))
    assert m.source_num_slicers == [3] and m.target_num_slicers == [3]
    got = {(r.src.rank, r.src.cell[0]): (r.dsts[0].rank, r.dsts[0].cell[0]) for r in m.routes}
    # global cell of source rank r, local piece i is 2 * i + r; target rank 2 + g // 3 holds it at local g % 3
    assert got == {(r, i): (2 + (2 * i + r) // 3, (2 * i + r) % 3) for r in (0, 1) for i in range(3)}
