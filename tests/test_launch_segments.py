"""etha_launch_segments: a set of independent bucket launches issued as one unit, against the same launches made
one by one through etha_pack_bucket / etha_unpack_bucket / etha_reduce_pack_bucket / etha_selfcopy_bucket."""

import numpy as np
import pytest
import torch

from etha_amd import _native as nat
from etha_amd.comm.device_plan import fill_region


def _pair_rows(pairs):
    src = np.zeros(len(pairs), dtype=nat.CHUNK_DESC)
    dst = np.zeros(len(pairs), dtype=nat.CHUNK_DESC)
    for i, (s, ss, d, ds) in enumerate(pairs):
        shape = tuple(s[ss].shape)
        assert shape == tuple(d[ds].shape)
        a, b = np.zeros((), dtype=nat.CHUNK_DESC), np.zeros((), dtype=nat.CHUNK_DESC)
        fill_region(a, s, ss, shape)
        fill_region(b, d, ds, shape)
        a["wire_dtype"], b["wire_dtype"] = a["tensor_dtype"], b["tensor_dtype"]
        src[i], dst[i] = a, b
    return src, dst


def _bucket_rows(tensors, slices, buffer, wire_code):
    """Descriptors of chunks ``tensors[i][slices[i]]`` laid back to back in ``buffer``."""
    rows = np.zeros(len(tensors), dtype=nat.CHUNK_DESC)
    off = 0
    for i, (t, sl) in enumerate(zip(tensors, slices)):
        shape = tuple(t[sl].shape)
        row = np.zeros((), dtype=nat.CHUNK_DESC)
        fill_region(row, t, sl, shape)
        row["wire_dtype"] = wire_code
        row["bucket_ptr"] = buffer.data_ptr() + off
        row["bucket_lo"], row["bucket_hi"] = buffer.data_ptr(), buffer.data_ptr() + buffer.numel() * buffer.element_size()
        rows[i] = row
        off += int(np.prod(shape)) * {nat.BF16: 2, nat.F32: 4}[wire_code]
    return rows, off


def test_bad_segments_are_rejected_before_any_launch():
    import ctypes

    d = np.zeros(1, dtype=nat.CHUNK_DESC)
    d["tensor_ptr"], d["bucket_ptr"], d["ndim"] = 0x10000, 0x900000, 1
    d["shape"][0][0], d["stride"][0][0] = 64, 1
    d["tensor_dtype"] = d["wire_dtype"] = nat.F32
    table = nat.Table.create(d, upload=False)
    nat.launch_segments([])  # nothing to do
    with pytest.raises(nat.EthaNativeError, match="unknown kind"):
        nat.launch_segments([(table, 9, 0, 1)])
    with pytest.raises(nat.EthaNativeError, match="wrong table kind"):
        nat.launch_segments([(table, nat.SEG_SELFCOPY, 0, 1)])
    with pytest.raises(nat.EthaNativeError, match="exceeds table"):
        nat.launch_segments([(table, nat.SEG_PACK, 0, 2)])
    with pytest.raises(nat.EthaNativeError, match="without upload"):
        nat.launch_segments([(table, nat.SEG_PACK, 0, 1)])
    with pytest.raises(nat.EthaNativeError, match="unknown launch flags"):
        nat.launch_segments([(table, nat.SEG_PACK, 0, 1)], flags=8)
    assert nat.lib().etha_launch_segments(None, 3, None, 0) == nat.ERR_INVALID
    assert ctypes.sizeof(nat.Segment) == 24


def _bits(t):
    return t.contiguous().view(torch.uint8).cpu()


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [0, nat.LAUNCH_UNORDERED])
def test_a_set_of_segments_equals_the_launches_one_by_one(gpu_device, flags):
    dev = gpu_device
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def build(keep):
        """Tables and the tensors they write: 20 same-rank copy tables of the same size (more than one launch's worth
        of segments; some convert, some also hold a transposing chunk), 2 larger ones, a pack, three unpacks (one of them a
        gathered range) and a Partial reduce-pack table."""
        segs, outs = [], []
        for k in range(22):
            r, c = (300, 520) if k < 20 else (900 + 300 * (k - 20), 1024)
            src = torch.randn(r + 4, c + 6, generator=torch.Generator(device=dev).manual_seed(100 + k), device=dev)
            dst = torch.full((r + 9, c + 11), -2.0, device=dev, dtype=torch.bfloat16 if k % 3 == 0 else torch.float32)
            pairs = [(src, (slice(2, 2 + r), slice(3, 3 + c)), dst, (slice(5, 5 + r), slice(1, 1 + c)))]
            if k % 4 == 1:  # a transposing chunk of its own
                tsrc = torch.randn(c + 8, 200, generator=torch.Generator(device=dev).manual_seed(300 + k), device=dev).t()
                tdst = torch.zeros(200, c + 8, device=dev)
                pairs.append((tsrc, (slice(0, 200), slice(0, c + 8)), tdst, (slice(0, 200), slice(0, c + 8))))
                outs.append(tdst)
                keep.append(tsrc)
            a, b = _pair_rows(pairs)
            table = nat.Table.create_selfcopy(a, b)
            segs.append((table, nat.SEG_SELFCOPY, 0, len(pairs)))
            outs.append(dst)
            keep += [src, table]
        # pack: three chunks of two tensors into a bf16 bucket (the fp32 one converts)
        x = torch.randn(300, 257, generator=torch.Generator(device=dev).manual_seed(7), device=dev).to(torch.bfloat16)
        y = torch.randn(129, 64, generator=torch.Generator(device=dev).manual_seed(8), device=dev)
        bucket = torch.zeros(1 << 20, dtype=torch.uint8, device=dev)
        rows, _ = _bucket_rows([x, y, x], [(slice(0, 150), slice(1, 257)), (slice(0, 129), slice(0, 64)),
                                           (slice(150, 300), slice(0, 200))], bucket, nat.BF16)
        pack = nat.Table.create(rows)
        segs.append((pack, nat.SEG_PACK, 0, 3))
        outs.append(bucket)
        # unpack: a filled bucket scattered into two tensors, the second range launched as its own segment
        filled = torch.randn(1 << 18, generator=torch.Generator(device=dev).manual_seed(9), device=dev).to(torch.bfloat16)
        u1 = torch.full((200, 300), 9.0, device=dev, dtype=torch.bfloat16)
        u2 = torch.full((77, 50), 9.0, device=dev, dtype=torch.float32)
        urows, _ = _bucket_rows([u1, u2], [(slice(10, 190), slice(0, 300)), (slice(0, 77), slice(3, 47))],
                                filled.view(torch.uint8), nat.BF16)
        unpack = nat.Table.create(urows)
        segs += [(unpack, nat.SEG_UNPACK, 0, 1), (unpack, nat.SEG_UNPACK, 1, 1)]
        outs += [u1, u2]
        # unpack of a write-ordered range whose short pieces are gathered row by row: four column blocks of one tensor
        wide = torch.full((700, 96), 5.0, device=dev, dtype=torch.bfloat16)
        blocks = torch.randn(4, 700 * 24, generator=torch.Generator(device=dev).manual_seed(11), device=dev).to(torch.bfloat16)
        grows = np.zeros(4, dtype=nat.CHUNK_DESC)
        for j in range(4):
            r, _ = _bucket_rows([wide], [(slice(0, 700), slice(24 * j, 24 * j + 24))], blocks[j].view(torch.uint8), nat.BF16)
            grows[j] = r[0]
        gathered = nat.Table.create(grows)
        gathered.optimize_range(0, 4)
        assert len(gathered.ordered_gather(0, 4)) > 0
        segs.append((gathered, nat.SEG_UNPACK, 0, 4))
        outs.append(wide)
        keep += [blocks, gathered]
        # Partial: three members summed into a bf16 bucket
        members = [torch.randn(64, 515, generator=torch.Generator(device=dev).manual_seed(20 + i), device=dev) for i in range(3)]
        rbucket = torch.zeros(64 * 515 * 2 + 64, dtype=torch.uint8, device=dev)
        rrows, _ = _bucket_rows([members[0]], [(slice(0, 64), slice(0, 515))], rbucket, nat.BF16)
        rrows["n_partials"], rrows["partial_first"], rrows["reduce_op"] = 3, 0, 0
        ptrs = np.array([m.data_ptr() for m in members], dtype=np.uint64)
        reduce = nat.Table.create(rrows, ptrs)
        segs.append((reduce, nat.SEG_REDUCE_PACK, 0, 1))
        outs.append(rbucket)
        keep += [x, y, filled, members, pack, unpack, reduce]
        return segs, outs

    keep = []
    segs_a, outs_a = build(keep)
    with pytest.raises(nat.EthaNativeError, match="not Partial chunks"):
        nat.launch_segments([segs_a[0], (segs_a[-5][0], nat.SEG_REDUCE_PACK, 0, 1)], stream)
    with pytest.raises(nat.EthaNativeError, match="holds Partial chunks"):
        nat.launch_segments([segs_a[0], (segs_a[-1][0], nat.SEG_PACK, 0, 1)], stream)
    segs_b, outs_b = build(keep)
    before = nat.kernel_launches()
    nat.launch_segments(segs_a, stream, flags)
    as_a_set = nat.kernel_launches() - before
    one = {nat.SEG_PACK: "pack", nat.SEG_UNPACK: "unpack", nat.SEG_REDUCE_PACK: "reduce_pack", nat.SEG_SELFCOPY: "selfcopy"}
    before = nat.kernel_launches()
    for table, kind, first, count in segs_b:
        getattr(table, one[kind])(first, count, stream)
    one_by_one = nat.kernel_launches() - before
    torch.cuda.synchronize()
    for k, (a, b) in enumerate(zip(outs_a, outs_b)):
        assert torch.equal(_bits(a), _bits(b)), f"output {k} differs"
    assert not torch.equal(_bits(outs_a[-1]), torch.zeros_like(_bits(outs_a[-1])))  # the reduce really ran
    # one by one: a plain-tile kernel per segment (25) plus a transposing kernel for the 6 tables that hold such a
    # chunk and the reduce.  As a set the 23 forward segments need far fewer launches (equal ones share a launch, 16
    # at most), the two unpack segments share one
    assert one_by_one == 26 + 6 + 1
    assert as_a_set <= 6 + 2 + 6 + 1


@pytest.mark.gpu
def test_pipelines_issue_sets_and_results_do_not_depend_on_it(gpu_device):
    """The wire hands what a sweep prepares and finalizes to the library as one set: fewer kernel launches than
    bucket steps, same bytes as with one launch per step."""
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from etha_amd.world import ReshardJob, TensorSpec
    from helpers import cpu_fill

    specs = [TensorSpec(f"w{i}", (512, 384), list(range(4)), (Shard(0),), [4, 5], (Shard(1),), torch.bfloat16, seed=i, std=1.0)
             for i in range(6)]
    specs.append(TensorSpec("n", (384,), list(range(4)), (Replicate(),), [4, 5], (Replicate(),), torch.float32, torch.bfloat16,
                            seed=9, std=1.0))
    results = []
    for sets in (True, False):
        job = ReshardJob(specs, device=gpu_device, bucket_size=64 * 1024, fill=cpu_fill)
        job.wire.group_launches = sets
        log = job.wire.launch_log = []
        before = nat.kernel_launches()
        job.run(merge_launches=False)
        kernels = nat.kernel_launches() - before
        results.append(([_bits(t) for d in job.target_locals for t in d.values()], kernels, len(log)))
    (with_sets, k_sets, steps), (without, k_single, steps2) = results
    assert steps == steps2 and k_single == steps
    assert k_sets < steps // 2
    assert all(torch.equal(a, b) for a, b in zip(with_sets, without))


def test_bad_schedules_are_rejected_when_they_are_created():
    import ctypes

    d = np.zeros(1, dtype=nat.CHUNK_DESC)
    d["tensor_ptr"], d["bucket_ptr"], d["ndim"] = 0x10000, 0x900000, 1
    d["shape"][0][0], d["stride"][0][0] = 64, 1
    d["tensor_dtype"] = d["wire_dtype"] = nat.F32
    table = nat.Table.create(d, upload=False)
    empty = nat.Schedule([])
    assert (empty.info().n_calls, empty.info().n_kernel_launches) == (0, 0)
    with pytest.raises(nat.EthaNativeError, match="without upload"):
        nat.Schedule([([(table, nat.SEG_PACK, 0, 1)], 0, False)])
    with pytest.raises(nat.EthaNativeError, match="unknown kind"):
        nat.Schedule([([(table, 7, 0, 1)], 0, True)])
    with pytest.raises(nat.EthaNativeError, match="unknown launch flags"):
        nat.Schedule([([(table, nat.SEG_PACK, 0, 1)], 4, False)])
    with pytest.raises(nat.EthaNativeError, match="exactly one segment"):
        nat.Schedule([([(table, nat.SEG_PACK, 0, 1), (table, nat.SEG_PACK, 0, 1)], 0, True)])
    out = ctypes.c_void_p()
    call = nat.ScheduleCall(first_segment=0, n_segments=2, flags=0, single=0)
    seg = nat.Segment(table=table._h, kind=nat.SEG_PACK, first=0, count=1)
    assert nat.lib().etha_schedule_create(ctypes.byref(seg), 1, ctypes.byref(call), 1, ctypes.byref(out)) == nat.ERR_INVALID
    assert b"outside the segment array" in nat.lib().etha_last_error()
    assert nat.lib().etha_schedule_create(None, 1, ctypes.byref(call), 1, ctypes.byref(out)) == nat.ERR_INVALID
    assert nat.lib().etha_schedule_launch(None, None) == nat.ERR_INVALID
    assert nat.lib().etha_schedule_destroy(None) == 0
    assert ctypes.sizeof(nat.ScheduleCall) == 16


@pytest.mark.gpu
def test_a_schedule_reissues_the_calls_it_was_made_from(gpu_device):
    """etha_schedule_launch against the same calls made one by one: same bytes, same number of kernels; a schedule
    whose table changed or went away refuses to launch."""
    dev = gpu_device
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def build(keep, seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        srcs = [torch.randn(400, 300, generator=g, device=dev) for _ in range(6)]
        bucket = torch.zeros(6 * 400 * 300 * 2, dtype=torch.uint8, device=dev)
        rows = np.zeros(6, dtype=nat.CHUNK_DESC)
        off = 0
        for i, s in enumerate(srcs):
            r, n = _bucket_rows([s], [(slice(0, 400), slice(0, 300))], bucket[off:], nat.BF16)
            r["bucket_lo"], r["bucket_hi"] = bucket.data_ptr(), bucket.data_ptr() + bucket.numel()
            rows[i] = r[0]
            off += n
        pack = nat.Table.create(rows)
        wide = torch.full((400, 6 * 300 + 5), 3.0, device=dev, dtype=torch.bfloat16)
        urows = np.zeros(6, dtype=nat.CHUNK_DESC)
        off = 0
        for i in range(6):
            r, n = _bucket_rows([wide], [(slice(0, 400), slice(300 * i, 300 * i + 300))], bucket[off:], nat.BF16)
            r["bucket_lo"], r["bucket_hi"] = bucket.data_ptr(), bucket.data_ptr() + bucket.numel()
            urows[i] = r[0]
            off += n
        unpack = nat.Table.create(urows)
        tsrc = torch.randn(520, 260, generator=g, device=dev).t()
        tdst = torch.zeros(260, 520, device=dev, dtype=torch.bfloat16)
        a, b = _pair_rows([(tsrc, (slice(0, 260), slice(0, 520)), tdst, (slice(0, 260), slice(0, 520)))])
        local = nat.Table.create_selfcopy(a, b)
        keep += [srcs, bucket, pack, unpack, local, tsrc]
        calls = [
            ([(pack, nat.SEG_PACK, 0, 2), (pack, nat.SEG_PACK, 2, 4), (local, nat.SEG_SELFCOPY, 0, 1)], 0, False),
            ([(unpack, nat.SEG_UNPACK, 0, 2)], 0, True),
            ([(unpack, nat.SEG_UNPACK, 2, 4)], nat.LAUNCH_UNORDERED, True),
        ]
        return calls, [wide, tdst, bucket], srcs + [tsrc], unpack

    keep = []
    calls_a, outs_a, ins_a, unpack_a = build(keep, 5)
    calls_b, outs_b, ins_b, _ = build(keep, 5)
    sched = nat.Schedule(calls_a)
    info = sched.info()
    assert info.n_calls == 3 and info.n_tables == 3 and info.n_kernel_launches >= 4
    one = {nat.SEG_PACK: "pack", nat.SEG_UNPACK: "unpack", nat.SEG_SELFCOPY: "selfcopy"}
    for round_ in range(3):
        for x, y in zip(ins_a, ins_b):  # new values every round: a replay must move what is there now
            x.mul_(-1.5).add_(round_)
            y.copy_(x)
        before = nat.kernel_launches()
        sched.launch(stream)
        by_schedule = nat.kernel_launches() - before
        before = nat.kernel_launches()
        for segs, flags, single in calls_b:
            if single:
                table, kind, first, count = segs[0]
                getattr(table, one[kind])(first, count, stream, flags)
            else:
                nat.launch_segments(segs, stream, flags)
        by_calls = nat.kernel_launches() - before
        torch.cuda.synchronize()
        assert by_schedule == by_calls == info.n_kernel_launches
        for k, (a, b) in enumerate(zip(outs_a, outs_b)):
            assert torch.equal(_bits(a), _bits(b)), f"round {round_}: output {k} differs"
        assert torch.equal(_bits(outs_a[0][:, :300]), _bits(ins_a[0].to(torch.bfloat16)))
    # a range of one of its tables gains a write-ordered copy: what the schedule would launch is no longer what a
    # call launches, so it refuses; a schedule made afterwards works
    unpack_a.optimize_range(2, 4)
    before = nat.kernel_launches()
    with pytest.raises(nat.EthaNativeError, match="stale schedule"):
        sched.launch(stream)
    assert nat.kernel_launches() == before  # nothing was launched
    again = nat.Schedule(calls_a)
    again.launch(stream)
    torch.cuda.synchronize()
    for k, (a, b) in enumerate(zip(outs_a, outs_b)):
        assert torch.equal(_bits(a), _bits(b)), f"after optimize_range: output {k} differs"
    calls_a[0][0][2][0].close()  # the same-rank table is destroyed
    with pytest.raises(nat.EthaNativeError, match="stale schedule"):
        again.launch(stream)
    torch.cuda.synchronize()


@pytest.mark.gpu
@pytest.mark.parametrize("workload", ["mixed", "partial"])
def test_a_repeated_transfer_is_served_from_its_recording(gpu_device, workload):
    """The wire records what the pipelines issue for a transfer and re-issues it when the transfer repeats
    (LoopbackWire.replay_schedules): same bytes as with the pipelines, on new source values every time."""
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    from etha_amd.world import ReshardJob, TensorSpec
    from helpers import cpu_fill

    if workload == "mixed":
        specs = [TensorSpec(f"w{i}", (512, 384 + 64 * i), list(range(4)), (Shard(0),), [4, 5], (Shard(1),), torch.bfloat16,
                            seed=i, std=1.0) for i in range(6)]
        specs.append(TensorSpec("n", (384,), list(range(4)), (Replicate(),), [4, 5], (Replicate(),), torch.float32,
                                torch.bfloat16, seed=9, std=1.0))
        specs.append(TensorSpec("t", (256, 512), list(range(4)), (Shard(0),), [4, 5], (Shard(0),), torch.float32, torch.bfloat16,
                                seed=11, std=1.0, source_layout="transposed"))
    else:
        specs = [TensorSpec(f"p{i}", (256, 320), list(range(4)), (Partial("sum"),), [2, 3], (Shard(0),), torch.bfloat16,
                            seed=10 * i, std=1.0) for i in range(5)]
    jobs = [ReshardJob(specs, device=gpu_device, bucket_size=64 * 1024, fill=cpu_fill) for _ in range(2)]
    jobs[1].wire.replay_schedules = False
    for a, b in zip(jobs[0].source_locals, jobs[1].source_locals):
        for r in a:
            b[r].copy_(a[r])
    for round_ in range(4):
        for a, b in zip(jobs[0].source_locals, jobs[1].source_locals):
            for r, t in a.items():
                if not any(t is x for d in jobs[0].target_locals for x in d.values()):
                    t.mul_(-0.75).add_(0.125 * round_)
                    b[r].copy_(t)
        launched = []
        for job in jobs:
            before = nat.kernel_launches()
            job.run(merge_launches=True)
            launched.append(nat.kernel_launches() - before)
        assert launched[0] == launched[1] > 0
        for i in range(len(specs)):
            for r, t in jobs[0].target_locals[i].items():
                assert torch.equal(_bits(t), _bits(jobs[1].target_locals[i][r])), f"round {round_}: {specs[i].name} rank {r}"
    assert jobs[0].wire.replays >= 2 and jobs[1].wire.replays == 0
    # a HIP graph captured from the wire replays the same transfer, recorded or not
    graph = jobs[0].capture(merge_launches=True)
    for t in (x for d in jobs[0].target_locals for x in d.values()):
        t.zero_()
    graph.replay()
    torch.cuda.synchronize()
    for i in range(len(specs)):
        for r, t in jobs[0].target_locals[i].items():
            assert torch.equal(_bits(t), _bits(jobs[1].target_locals[i][r]))
