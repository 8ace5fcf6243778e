"""Randomised end-to-end check of the host side, on the CPU.

Random meshes, placements, shapes, dtypes, bucket sizes and parent strides go through the product's
planner and descriptor builder; the native library compiles the tile programs against the live host
tensors (no upload), and the CPU tile interpreter executes them step by step in the executor's order.
The result must equal the oracle's restatement of the reference path and the closed-form DTensor slice.
Everything except the device kernel itself is exercised, with bounds checks, and without a GPU.
"""

import math

import numpy as np
import pytest
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard, _StridedShard

from etha_amd.comm import LoopbackWire
from etha_amd.world import ReshardJob, TensorSpec

from helpers import assert_bit_equal, cpu_fill, expected_target, mesh_of, run_oracle
from tile_interpreter import AbsoluteMemory, execute

FLOATS = [torch.float32, torch.bfloat16, torch.float16, torch.float64]


def _random_layout(rng, ndim, allow_partial):
    mesh_shape = [int(rng.choice([1, 2, 3, 4])) for _ in range(int(rng.integers(1, 4)))]
    while math.prod(mesh_shape) > 8:
        mesh_shape[int(rng.integers(len(mesh_shape)))] = 1
    placements, partial = [], False
    for _ in mesh_shape:
        kind = rng.choice(["shard", "rep", "partial"] if allow_partial else ["shard", "rep"], p=None)
        if kind == "shard" and rng.random() < 0.15:  # a strided shard, also with split factors no later Shard pairs with
            placements.append(_StridedShard(int(rng.integers(ndim)), split_factor=int(rng.choice([2, 3]))))
        elif kind == "shard":
            placements.append(Shard(int(rng.integers(ndim))))
        elif kind == "partial":  # mostly sums; sometimes another op, so that two Partial dims may differ in op
            placements.append(Partial(str(rng.choice(["sum", "sum", "sum", "max", "avg"]))))
            partial = True
        else:
            placements.append(Replicate())
    return mesh_shape, tuple(placements), partial


def _random_spec(rng, idx, wire_size):
    ndim = int(rng.integers(1, 4))
    # Partial sources need a floating dtype of at most 32 bits: only in batches whose wire items are 2 or 4 bytes
    src_mesh, src_pl, partial = _random_layout(rng, ndim, allow_partial=wire_size in (2, 4) and rng.random() < 0.25)
    tgt_mesh, tgt_pl, _ = _random_layout(rng, ndim, allow_partial=False)
    shards = []
    def cuts(mesh, placements, d):  # how finely a layout cuts dim d
        out = 1
        for m, p in zip(mesh, placements):
            if isinstance(p, _StridedShard) and p.dim == d:
                out *= m * p.split_factor
            elif isinstance(p, Shard) and p.dim == d:
                out *= m
        return out

    for d in range(ndim):
        shards.append(math.lcm(cuts(src_mesh, src_pl, d), cuts(tgt_mesh, tgt_pl, d)))
    shape = tuple(int(l * rng.integers(1, 7)) for l in shards)
    shape = shape[:-1] + (shape[-1] * int(rng.choice([1, 1, 8, 19])),)
    # one wire item size per batch: the reference cannot mix item sizes in a bucket unless every offset
    # happens to be a multiple of the larger one (its view(dtype) of the bucket slice raises, ir.py:252)
    pairs = {
        1: [(torch.int8, torch.int8), (torch.uint8, torch.uint8), (torch.float32, torch.int8), (torch.int8, torch.float16),
            (torch.bfloat16, torch.float8_e4m3fn), (torch.float8_e5m2, torch.float32), (torch.bool, torch.int32),
            (torch.float64, torch.uint8)],
        2: [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16), (torch.bfloat16, torch.float32),
            (torch.float32, torch.bfloat16), (torch.float16, torch.float64), (torch.float64, torch.bfloat16),
            (torch.float16, torch.bfloat16), (torch.float32, torch.float16), (torch.int16, torch.float32),
            (torch.float64, torch.int16)],
        4: [(torch.float32, torch.float32), (torch.int32, torch.int32), (torch.float32, torch.float64),
            (torch.float64, torch.float32), (torch.int32, torch.float64), (torch.float32, torch.int32)],
        8: [(torch.float64, torch.float64), (torch.int64, torch.int64), (torch.int64, torch.float64)],
    }[wire_size]
    if partial:  # a Partial reduction accumulates in fp32 and needs f16/bf16/f32/f64 on both sides
        pairs = [p for p in pairs if p[0] in FLOATS[:3] and p[1] in FLOATS]
    sdt, tdt = pairs[int(rng.integers(len(pairs)))]
    n_src = math.prod(src_mesh)
    # overlapping rank sets create LOCAL chunks; their wire dtype is the target dtype (as in the reference), so
    # they stay within the batch's wire item size only when the two dtypes agree
    overlap = sdt == tdt and rng.random() < 0.4  # with a Partial source: the primary delivers to its own rank too
    tgt_start = 0 if overlap else n_src
    return TensorSpec(f"t{idx}", shape, mesh_of(0, src_mesh), src_pl, mesh_of(tgt_start, tgt_mesh), tgt_pl, sdt, tdt,
                      seed=1000 + idx, std=1.0, dist="normal" if sdt in FLOATS else "bits")


def _run_step(mem, p, kind, first, count, ordered=False, touched=None):
    if kind in ("pack", "reduce_pack"):
        execute(p.send_table, mem, "pack", first, count, peers=_peers_of(p), touched=touched)
    elif kind == "unpack":
        execute(p.recv_table, mem, "unpack", first, count, ordered=ordered, touched=touched)
    elif kind in ("selfcopy", "direct"):
        execute(p.local_table, mem, "selfcopy", first, count, ordered=ordered, touched=touched)
    elif kind in ("direct_reduce", "selfcopy_reduce"):
        execute(p.local_table, mem, "selfcopy", first, count, peers=_direct_peers_of(p), touched=touched)
    else:
        assert kind == "lend"  # nothing runs for a lent bucket


class _HazardCheck:
    """Byte-level check of the wire's launch ordering, independent of how the wire decides it: launches
    issued without ordering since the last ordered one may run at the same time on the GPU, so none of them
    may read a byte another one writes, and no two may write the same byte."""

    def __init__(self):
        self.reads = np.zeros(0, np.int64)
        self.writes = np.zeros(0, np.int64)
        self.unordered = 0

    def launch(self, touched: dict, flags: int) -> None:
        r = np.unique(np.concatenate(touched["r"])) if touched.get("r") else np.zeros(0, np.int64)
        w = np.unique(np.concatenate(touched["w"])) if touched.get("w") else np.zeros(0, np.int64)
        if flags & 1:
            self.unordered += 1
            assert not len(np.intersect1d(r, self.writes)), "unordered launch reads bytes written since the last ordered launch"
            assert not len(np.intersect1d(w, self.reads)), "unordered launch writes bytes read since the last ordered launch"
            assert not len(np.intersect1d(w, self.writes)), "two unordered launches write the same bytes"
            self.reads = np.union1d(self.reads, r)
            self.writes = np.union1d(self.writes, w)
        else:
            self.reads, self.writes = r, w


def _interpret(job, merged: bool, by_sets: bool = False):
    """What ReshardJob.run would enqueue, executed on the host by the tile interpreter.  With a ring pool the
    wire's own bucket pipelines decide the order (slots are reused, so list order would be wrong); the wire
    hands every launch to the interpreter instead of the GPU."""
    plans = [job.wire.plan(b) for b in job.send_buckets.values()] + [job.wire.plan(b) for b in job.recv_buckets.values()]
    # the span of everything that may legitimately be touched: every shard's storage and the bucket pool
    ranges = []
    for d in job.source_locals + job.target_locals:
        for t in d.values():
            st = t.untyped_storage()
            if st.nbytes():
                ranges.append((st.data_ptr(), st.data_ptr() + st.nbytes()))
    if job.wire.pool is not None:
        for seg in job.wire.pool.segments:
            ranges.append((seg.data_ptr(), seg.data_ptr() + seg.numel()))
    if not ranges:
        return
    lo, hi = min(r[0] for r in ranges), max(r[1] for r in ranges)
    mem = AbsoluteMemory(lo, hi)
    if job.wire.pool_mode == "ring":
        check = _HazardCheck()

        def on_launch(p, kind, first, count, flags):
            touched = {}
            # a recurring multi-bucket scatter runs from its written-address-ordered copy, as on the GPU
            _run_step(mem, p, kind, first, count, ordered=(kind, first, count) in p._ordered_ranges, touched=touched)
            check.launch(touched, flags)

        def on_set(members, flags):
            # the members of a set run at the same time on the GPU: here in reverse, which must not matter
            if not flags & 1:
                check.launch({}, 0)  # an ordered set: everything before it has finished
            for p, kind, first, count in reversed(members):
                touched = {}
                _run_step(mem, p, kind, first, count, ordered=(kind, first, count) in p._ordered_ranges, touched=touched)
                check.launch(touched, 1)
            check.sets += 1
            check.largest = max(check.largest, len(members))

        check.sets = check.largest = 0
        if by_sets:
            job.wire.on_set = on_set
        else:
            job.wire.on_launch = on_launch
        try:
            job.run(merge_launches=merged)
        finally:
            job.wire.on_launch = job.wire.on_set = None
        return check
    for p in plans:
        steps = p.merged_steps if merged else [(k, f, c, (s,)) for k, f, c, s in p.steps]
        for kind, first, count, slots in steps:
            _run_step(mem, p, kind, first, count, ordered=merged and len(slots) > 1)


def _direct_peers_of(plan):
    """Peer pointers of a plan's direct-reduce chunks, in the order the plan registered them."""
    ptrs = []
    for (kind, _, _, slot), info in zip(plan.steps, plan.info):
        if kind == "direct_reduce":
            for _, _, _, peers in slot.sources:
                ptrs.extend(t.data_ptr() for t in peers[0])
        elif kind == "selfcopy_reduce":  # a Partial source delivered to its own rank
            for c in info.bucket.chunks:
                ptrs.extend(t.data_ptr() for t in c.partial_peers()[0])
    return np.asarray(ptrs, dtype=np.uint64) if ptrs else None


def _peers_of(plan):
    ptrs = []
    for b in plan.buckets:
        if b.chunks and b.is_source and b.chunks[0].source_partial_groups and b.transport.value in ("p2p", "broadcast"):
            for c in b.chunks:
                ptrs.extend(t.data_ptr() for t in c.partial_peers()[0])
    return np.asarray(ptrs, dtype=np.uint64) if ptrs else None


def _uneven_spec(rng, idx, wire_size):
    """Uneven shard sizes (torch.chunk rule, empty shards included) on tensors of rank 1-5: every sharded dim is
    cut by a single Shard on one side only, the layout pairs for which an uneven split is defined."""
    del wire_size
    ndim = int(rng.integers(1, 6))

    def side(free_dims, partial_ok):
        mesh = [int(rng.choice([1, 2, 3, 4, 6])) for _ in range(int(rng.integers(1, 3)))]
        while math.prod(mesh) > 8:
            mesh[int(rng.integers(len(mesh)))] = 1
        placements, used, op = [], set(), str(rng.choice(["sum", "avg", "max"]))
        for _ in mesh:
            free = [d for d in free_dims if d not in used]
            if free and rng.random() < 0.7:
                d = int(rng.choice(free))
                used.add(d)
                placements.append(Shard(d))
            elif partial_ok and rng.random() < 0.3:
                placements.append(Partial(op))
            else:
                placements.append(Replicate())
        return mesh, tuple(placements)

    dims = list(range(ndim))
    rng.shuffle(dims)
    half = int(rng.integers(0, ndim + 1))
    src_mesh, src_pl = side(dims[:half], True)
    tgt_mesh, tgt_pl = side(dims[half:], False)
    shape = tuple(int(rng.integers(1, 14)) for _ in range(ndim))
    partial = any(isinstance(p, Partial) for p in src_pl)
    tgt_start = 0 if (not partial and rng.random() < 0.3) else math.prod(src_mesh)
    return TensorSpec(f"t{idx}", shape, mesh_of(0, src_mesh), src_pl, mesh_of(tgt_start, tgt_mesh), tgt_pl,
                      torch.float32, seed=2000 + idx, std=1.0)


@pytest.mark.parametrize("seed", range(60))
def test_random_uneven_batches(seed):
    test_random_batches(100_000 + seed, spec_fn=_uneven_spec)


@pytest.mark.parametrize("seed", range(150))
def test_random_batches(seed, spec_fn=None):
    spec_fn = spec_fn or _random_spec
    rng = np.random.default_rng(seed)
    wire_size = int(rng.choice([1, 2, 2, 4, 4, 8]))
    specs = [spec_fn(rng, i, wire_size) for i in range(int(rng.integers(1, 5)))]
    # all tensors of a batch share rank numbering: re-home each spec's meshes on disjoint or overlapping ranks as drawn
    bucket_size = [None, 64, 4096, 1 << 20][int(rng.integers(4))]
    view = None
    if rng.random() < 0.35:
        def view(kind, t):  # non-contiguous parents: every local shard is a slice of a wider tensor
            if t.dim() == 0 or t.numel() == 0:
                return t
            shape = list(t.shape)
            shape[-1] = shape[-1] * 2 + 3
            wide = torch.zeros(shape, dtype=t.dtype)
            return wide[..., 1 : 1 + t.shape[-1]]
    merged = bool(rng.integers(2))
    # wire options must not change results: plain buckets, lent single-chunk buckets, or no buckets at all
    mode = ["buckets", "buckets", "zero_copy", "direct"][int(rng.integers(4))]
    # the pool: a ring of 1-3 slots per channel (the default form), or a slot per bucket
    pool = ["ring", "ring", "resident"][int(rng.integers(3))]
    depth = int(rng.integers(1, 4))
    job = ReshardJob(specs, device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill, local_view=view,
                     wire=LoopbackWire("cpu", segment_bytes=1 << 22, host_inspection=True, pool=pool, max_in_flight=depth),
                     direct=mode == "direct", zero_copy=mode == "zero_copy", max_in_flight=depth)
    ref = ReshardJob(specs, device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill, local_view=view)
    for a, b in zip(job.source_locals, ref.source_locals):  # Partial sources are drawn per job: make them equal
        for r in a:
            b[r].copy_(a[r])
    src_before = [{r: t.clone() for r, t in d.items()} for d in job.source_locals]
    # the launches one by one in issue order, or set by set with the members of every set in reverse
    _interpret(job, merged, by_sets=bool(rng.integers(2)))
    run_oracle(ref)
    for i, spec in enumerate(specs):
        for r, t in job.target_locals[i].items():
            assert_bit_equal(t, ref.target_locals[i][r], f"seed {seed} {spec.name} rank {r} vs oracle")
            if job.globals_[i] is not None:
                assert_bit_equal(t, expected_target(spec, job.globals_[i], r), f"seed {seed} {spec.name} rank {r} vs closed form")
        for r, t in job.source_locals[i].items():
            if not any(t is x for x in job.target_locals[i].values()):
                assert_bit_equal(t, src_before[i][r], f"seed {seed} {spec.name} source rank {r} mutated")
    with pytest.raises(RuntimeError, match="no CPU path"):
        job.run()


def _mutate_sources(job, ref, k):
    """New source values on both jobs (so that a replay that moved stale bytes would show), targets poisoned."""
    for a, b in zip(job.source_locals, ref.source_locals):
        for r, t in a.items():
            if any(t is x for d in job.target_locals for x in d.values()):
                continue
            if t.dtype.is_floating_point and t.dtype not in (torch.float8_e4m3fn, torch.float8_e5m2):
                t.copy_((t.double() * -0.5 + k).to(t.dtype))
            elif t.dtype == torch.bool:
                t.copy_(~t)
            elif t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
                t.copy_(t.float().roll(1, -1 if t.dim() else 0).to(t.dtype) if t.dim() else t)
            else:
                t.copy_(t.roll(1, -1) if t.dim() else t)
            b[r].copy_(t)


@pytest.mark.parametrize("staged", [False, True], ids=["one_drive", "send_then_recv"])
@pytest.mark.parametrize("seed", range(40))
def test_recorded_transfers_replay_what_the_pipelines_issue(seed, staged):
    """A transfer that repeats is served from the sets its first run recorded, not by stepping the pipelines again.
    The replayed sets go through the same byte-level hazard check and must give the oracle's result on new source
    values; a transfer whose calls arrive in another order falls back to the pipelines and is recorded as well."""
    rng = np.random.default_rng(7000 + seed)
    wire_size = int(rng.choice([2, 2, 4, 8]))
    specs = [_random_spec(rng, i, wire_size) for i in range(int(rng.integers(1, 5)))]
    bucket_size = [64, 4096, 1 << 20][int(rng.integers(3))]
    depth = int(rng.integers(1, 4))
    merged = bool(rng.integers(2))
    mode = ["buckets", "buckets", "zero_copy", "direct"][int(rng.integers(4))]
    wire = LoopbackWire("cpu", segment_bytes=1 << 22, host_inspection=True, pool="ring", max_in_flight=depth)
    job = ReshardJob(specs, device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill, wire=wire,
                     direct=mode == "direct", zero_copy=mode == "zero_copy", max_in_flight=depth)
    ref = ReshardJob(specs, device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill)
    for a, b in zip(job.source_locals, ref.source_locals):
        for r in a:
            b[r].copy_(a[r])
    ranges = []
    for d in job.source_locals + job.target_locals:
        for t in d.values():
            st = t.untyped_storage()
            if st.nbytes():
                ranges.append((st.data_ptr(), st.data_ptr() + st.nbytes()))
    for p in [wire.plan(b) for b in list(job.send_buckets.values()) + list(job.recv_buckets.values())]:
        del p  # planning allocates the pool
    if wire.pool is not None:
        ranges += [(s.data_ptr(), s.data_ptr() + s.numel()) for s in wire.pool.segments]
    if not ranges:
        return
    mem = AbsoluteMemory(min(r[0] for r in ranges), max(r[1] for r in ranges))
    check = _HazardCheck()
    issued: list = []

    def on_set(members, flags):
        issued.append((tuple((id(p), k, f, c) for p, k, f, c in members), flags))
        if not flags & 1:
            check.launch({}, 0)
        for p, kind, first, count in reversed(members):
            touched = {}
            _run_step(mem, p, kind, first, count, ordered=(kind, first, count) in p._ordered_ranges, touched=touched)
            check.launch(touched, 1)

    def transfer(order=1):
        issued.clear()
        if staged:  # the senders' calls come first and fill their rings; the receivers' calls bring the rest
            job.run_send(merged, drive=True)
            recv = list(job.recv_buckets.values())[::order]
            from etha_amd.comm import bucket_comm
            for b in recv:
                bucket_comm(b, depth, wire=wire, merge_launches=merged, synchronize=False)
        else:
            job.run(merge_launches=merged)
        assert wire.idle()
        return list(issued)

    def verify(what):
        run_oracle(ref)
        for i, spec in enumerate(specs):
            for r, t in job.target_locals[i].items():
                assert_bit_equal(t, ref.target_locals[i][r], f"seed {seed} {what}: {spec.name} rank {r} vs oracle")

    wire.on_set = on_set
    try:
        first = transfer()
        verify("recording")
        for k in (1, 2):
            _mutate_sources(job, ref, k)
            before = wire.replays
            again = transfer()
            if first:
                assert wire.replays > before, "the repeated transfer was not served from the recording"
            assert again == first, "a replay issues exactly the recorded sets"
            verify(f"replay {k}")
        if staged and len(job.recv_buckets) > 1:
            _mutate_sources(job, ref, 3)
            transfer(order=-1)  # another arrival order: not a recorded sequence from some point on
            verify("other order")
            _mutate_sources(job, ref, 4)
            before = wire.replays
            transfer(order=-1)
            assert wire.replays > before
            verify("other order, replayed")
        # switched off: the pipelines run again and give the same launches
        wire.replay_schedules = False
        _mutate_sources(job, ref, 5)
        before = wire.replays
        assert transfer() == first and wire.replays == before
        verify("pipelines")
    finally:
        wire.on_set = None
