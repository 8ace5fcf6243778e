"""Partial mesh dims with different reduce ops, and a Partial source delivered to its own rank.

The reference all-reduces once per Partial mesh dim, each with its own op, in mesh-dim order
(``src/etha/tensor_bus/agent.py:46-70``, ``src/etha/comm/ir.py:123-124``).  Here that is one nested
reduction with fp32 accumulators and a single rounding; the closed form below is written out with numpy,
independently of the oracle and of the product.
"""

import numpy as np
import pytest
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from etha_amd.comm import LoopbackWire
from etha_amd.world import ReshardJob, TensorSpec
from oracle import reference_path

from helpers import assert_bit_equal, cpu_fill, mesh_of, run_oracle
from test_random_layouts_cpu import _interpret

_NP = {"sum": np.add.reduce, "max": np.fmax.reduce, "min": np.fmin.reduce, "product": np.multiply.reduce}


def _level(values: np.ndarray, op: str, axis: int) -> np.ndarray:
    """Combine along ``axis`` in index order with fp32 arithmetic (np reduce on float32 adds pairwise for long
    axes; these axes have at most 4 members, where it is strictly sequential)."""
    acc = np.take(values, 0, axis=axis).astype(np.float32)
    for i in range(1, values.shape[axis]):
        v = np.take(values, i, axis=axis).astype(np.float32)
        if op in ("sum", "avg"):
            acc = (acc + v).astype(np.float32)
        elif op == "product":
            acc = (acc * v).astype(np.float32)
        elif op == "max":
            acc = np.fmax(acc, v)
        else:
            acc = np.fmin(acc, v)
    if op == "avg":
        acc = (acc / np.float32(values.shape[axis])).astype(np.float32)
    return acc


def _closed_form(members: np.ndarray, ops) -> np.ndarray:
    """``members`` has one leading axis per Partial mesh dim (mesh-dim order); reduce dim by dim, first dim first."""
    out = members.astype(np.float32)
    for op in ops:
        out = _level(out, op, 0)  # reducing axis 0 exposes the next mesh dim as the new axis 0
    return out


def test_oracle_levels_follow_mesh_dim_order():
    """Order matters: max over sums differs from sum over maxes; the oracle applies the first mesh dim first."""
    x = np.array([[1.0, 5.0], [4.0, -3.0]], dtype=np.float32)  # x[i][j]: mesh dim 0 index i, mesh dim 1 index j
    slices = [torch.tensor([x[i][j]]) for j in range(2) for i in range(2)]  # first dim fastest
    assert reference_path.reduce_levels(slices, (("sum", 2), ("max", 2))).item() == max(1 + 4, 5 - 3) == 5.0
    assert reference_path.reduce_levels(slices, (("max", 2), ("sum", 2))).item() == max(1, 4) + max(5, -3) == 9.0
    assert _closed_form(x.reshape(2, 2, 1), ("sum", "max")).item() == 5.0
    assert _closed_form(x.reshape(2, 2, 1), ("max", "sum")).item() == 9.0
    # accumulators are not rounded between levels: 256 + 1 + 1 in bf16 members, summed then averaged
    m = [torch.tensor([v], dtype=torch.bfloat16) for v in (256.0, 1.0, 1.0, 0.0)]
    assert reference_path.reduce_levels(m, (("sum", 2), ("avg", 2))).item() == (257.0 + 1.0) / 2


def _run_cpu(specs, bucket, targets=None, depth=2):
    wire = LoopbackWire("cpu", host_inspection=True, max_in_flight=depth)
    job = ReshardJob(specs, device="cpu", bucket_size=bucket, target_ranks=targets, fill=cpu_fill, wire=wire, max_in_flight=depth)
    ref = ReshardJob(specs, device="cpu", bucket_size=bucket, target_ranks=targets, fill=cpu_fill)
    for a, b in zip(job.source_locals, ref.source_locals):
        for r in a:
            b[r].copy_(a[r])
    _interpret(job, False)
    run_oracle(ref)
    return job, ref


def _expect(job, spec_index, spec, ops, dtype):
    """The numpy closed form of a fully Partial source, cast like the wire does (one rounding)."""
    mesh = np.asarray(spec.source_mesh)
    members = np.stack([job.source_locals[spec_index][int(r)].float().numpy() for r in mesh.reshape(-1)])
    members = members.reshape(*mesh.shape, *members.shape[1:])
    return torch.from_numpy(_closed_form(members, ops)).to(dtype)


@pytest.mark.parametrize("ops,mesh", [(("sum", "max"), [2, 2]), (("max", "sum"), [2, 2]), (("avg", "min"), [2, 3]),
                                      (("sum", "max", "avg"), [2, 2, 2]), (("product", "sum"), [3, 2])])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_mixed_ops_per_mesh_dim_on_the_cpu(ops, mesh, dtype):
    n = int(np.prod(mesh))
    spec = TensorSpec("p", (24, 20), mesh_of(0, mesh), tuple(Partial(o) for o in ops), mesh_of(n, [2]), (Shard(0),), dtype,
                      seed=3, std=1.0)
    job, ref = _run_cpu([spec], 256)
    want = _expect(job, 0, spec, ops, dtype)
    for j, r in enumerate((n, n + 1)):
        got = job.target_locals[0][r]
        assert_bit_equal(got, ref.target_locals[0][r], f"{ops} rank {r} vs oracle")
        assert_bit_equal(got, want[12 * j: 12 * j + 12], f"{ops} rank {r} vs the numpy closed form")


def test_partial_with_shard_and_mixed_ops():
    """(Partial(sum), Shard(1), Partial(max)) on a (2, 2, 2) mesh: two Partial dims around a sharded one."""
    spec = TensorSpec("q", (16, 24), mesh_of(0, [2, 2, 2]), (Partial("sum"), Shard(1), Partial("max")), mesh_of(8, [2]),
                      (Replicate(),), torch.float32, seed=11, std=1.0)
    job, ref = _run_cpu([spec], 512)
    mesh = np.asarray(spec.source_mesh)
    for r in (8, 9):
        assert_bit_equal(job.target_locals[0][r], ref.target_locals[0][r], f"rank {r} vs oracle")
    for col in range(2):  # the column half held by mesh coordinate (., col, .)
        members = np.stack([[job.source_locals[0][int(mesh[i, col, k])].numpy() for k in range(2)] for i in range(2)])
        want = _closed_form(members, ("sum", "max"))  # members[i][k]: first Partial dim first
        assert np.array_equal(job.target_locals[0][8][:, 12 * col: 12 * col + 12].numpy(), want)


@pytest.mark.parametrize("ops", [("sum",), ("max", "sum")])
def test_partial_source_delivered_to_its_own_rank(ops):
    """Target ranks overlap the source ranks: the primary of a cell is also one of its destinations, so the
    members are combined straight into its own target shard (a LOCAL chunk with a Partial source)."""
    mesh = [2, 2] if len(ops) == 2 else [4]
    spec = TensorSpec("p", (32, 12), mesh_of(0, mesh), tuple(Partial(o) for o in ops), mesh_of(0, [2]), (Shard(0),),
                      torch.bfloat16, seed=5, std=1.0)
    other = TensorSpec("w", (16, 8), mesh_of(0, [4]), (Shard(0),), mesh_of(0, [2]), (Shard(1),), torch.float32, seed=6)
    job, ref = _run_cpu([spec, other], 128)
    kinds = {s[0] for b in job.send_buckets.values() for s in job.wire.plan(b).steps}
    assert "selfcopy_reduce" in kinds and "selfcopy" in kinds
    want = _expect(job, 0, spec, ops, torch.bfloat16)
    for j, r in enumerate((0, 1)):
        assert_bit_equal(job.target_locals[0][r], ref.target_locals[0][r], f"rank {r} vs oracle")
        assert_bit_equal(job.target_locals[0][r], want[16 * j: 16 * j + 16], f"rank {r} vs the numpy closed form")
        assert_bit_equal(job.target_locals[1][r], ref.target_locals[1][r], f"plain tensor rank {r}")


@pytest.mark.gpu
@pytest.mark.parametrize("ops,mesh", [(("sum", "max"), [2, 2]), (("avg", "min"), [2, 3]), (("sum", "max", "avg"), [2, 2, 2])])
def test_mixed_ops_per_mesh_dim_on_the_gpu(gpu_device, ops, mesh):
    from helpers import gpu_vs_oracle

    n = int(np.prod(mesh))
    specs = [TensorSpec(f"p{i}", (96, 72 + 8 * i), mesh_of(0, mesh), tuple(Partial(o) for o in ops), mesh_of(n, [2]), (Shard(0),),
                        dt, seed=3 + i, std=1.0) for i, dt in enumerate((torch.bfloat16, torch.float32, torch.float64, torch.float16))]
    job, _ = gpu_vs_oracle(specs, gpu_device, 4096, check_closed_form=False)
    cpu = type("J", (), {"source_locals": [{r: t.cpu() for r, t in d.items()} for d in job.source_locals]})
    want = _expect(cpu, 0, specs[0], ops, torch.bfloat16)
    assert_bit_equal(job.target_locals[0][n].cpu(), want[:48], "vs the numpy closed form")


@pytest.mark.gpu
@pytest.mark.parametrize("ops", [("sum",), ("max", "sum")])
def test_partial_source_delivered_to_its_own_rank_on_the_gpu(gpu_device, ops):
    from helpers import gpu_vs_oracle

    mesh = [2, 2] if len(ops) == 2 else [4]
    specs = [TensorSpec("p", (128, 96), mesh_of(0, mesh), tuple(Partial(o) for o in ops), mesh_of(0, [2]), (Shard(0),),
                        torch.bfloat16, seed=5, std=1.0),
             TensorSpec("w", (64, 32), mesh_of(0, [4]), (Shard(0),), mesh_of(0, [2]), (Shard(1),), torch.float32, seed=6)]
    for merge in (False, True):
        job, _ = gpu_vs_oracle(specs, gpu_device, 2048, check_closed_form=False, merge_launches=merge)
    kinds = {s[0] for b in job.send_buckets.values() for s in job.wire.plan(b).steps}
    assert "selfcopy_reduce" in kinds
    gpu_vs_oracle(specs, gpu_device, 2048, check_closed_form=False, merge_launches=True, pool="resident")


def test_rounding_between_levels_is_the_only_difference_from_the_reference():
    """The reference all-reduces a buffer of the tensor's dtype once per Partial mesh dim (ir.py:123-124): 16-bit
    members are rounded after every level.  The kernels keep fp32 across levels and round once.  For f32 members the
    two forms are the same function; for bf16 members they agree wherever no intermediate rounding happens (small
    integers, max/min levels) and otherwise stay within one rounding step of the inner level's result."""
    from oracle.reference_path import reduce_levels, reduce_levels_in_tensor_dtype

    g = torch.Generator().manual_seed(4)
    levels = (("sum", 2), ("max", 3))
    f32 = [torch.randn(257, generator=g) for _ in range(6)]
    assert torch.equal(reduce_levels(f32, levels), reduce_levels_in_tensor_dtype(f32, levels))
    small = [torch.randint(-8, 9, (257,), generator=g).to(torch.bfloat16) for _ in range(6)]
    assert torch.equal(reduce_levels(small, levels).to(torch.bfloat16), reduce_levels_in_tensor_dtype(small, levels))
    only_order = (("max", 2), ("min", 3))  # no arithmetic: nothing to round
    bf = [torch.randn(257, generator=g).to(torch.bfloat16) for _ in range(6)]
    assert torch.equal(reduce_levels(bf, only_order).to(torch.bfloat16), reduce_levels_in_tensor_dtype(bf, only_order))
    # sums of random bf16 values, then a second sum: the inner sums are rounded (reference) or not (kernels)
    two_sums = (("sum", 2), ("avg", 3))
    once = reduce_levels(bf, two_sums).to(torch.bfloat16).float()
    each = reduce_levels_in_tensor_dtype(bf, two_sums).float()
    inner = torch.stack([b.double() for b in bf]).reshape(3, 2, -1).sum(1)
    exact = inner.mean(0)
    eps = torch.finfo(torch.bfloat16).eps
    # each inner sum is off by at most half a step of its own magnitude, the results by one step of theirs
    bound = eps * (inner.abs().max(0).values + exact.abs()).float()
    assert bool(((once - each).abs() <= bound).all())  # they differ, by roundings only ...
    assert not torch.equal(once, each)
    assert float((once.double() - exact).abs().mean()) <= float((each.double() - exact).abs().mean())  # ... and once is no worse
