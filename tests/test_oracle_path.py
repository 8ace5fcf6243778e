"""The oracle's restatement of the reference path, run on the reference's own test tables (CPU).

Plans come from the product planner; bytes are moved by ``oracle.reference_path``; the result is
checked against closed forms that do not involve either: the DTensor slice of the global tensor
(what the reference's tests assert through ``full_tensor()``), and an independent numpy fp32
rank-order reduction for Partial sources.
"""

import numpy as np
import pytest
import torch
from torch.distributed.tensor.placement_types import Partial

from etha_amd.comm import Chunk, Transport, chunk_to_bucket_ops
from etha_amd.world import ReshardJob, TensorSpec
from oracle import dtensor_layout, reference_path

from helpers import (DTYPES, assert_bit_equal, cpu_fill, expected_target, load_cases, mesh_of, parse_placements,
                     run_oracle)

CASES = load_cases()


def _run_case(spec, bucket_size):
    job = ReshardJob([spec], device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill)
    src_before = {r: t.clone() for r, t in job.source_locals[0].items()}
    run_oracle(job)
    for r, t in job.source_locals[0].items():
        assert torch.equal(t, src_before[r]), f"source rank {r} mutated"
    return job


def _numpy_partial_truth(job, spec):
    """fp32 sequential combination over each Partial connected component, independent of the oracle."""
    src_mesh = np.asarray(spec.source_mesh)
    partial_dims = [i for i, p in enumerate(spec.source_placements) if isinstance(p, Partial)]
    op = spec.source_placements[partial_dims[0]].reduce_op
    locals_ = job.source_locals[0]
    # ranks that differ only in Partial coordinates hold contributions to the same shard
    out = {}
    for pos, r in enumerate(src_mesh.reshape(-1)):
        coord = list(np.unravel_index(pos, src_mesh.shape))
        key = tuple(c for i, c in enumerate(coord) if i not in partial_dims)
        out.setdefault(key, []).append(int(r))
    logical_by_rank = {}
    for members in out.values():
        members = sorted(members)
        acc = locals_[members[0]].float().numpy().astype(np.float32).copy()
        for m in members[1:]:
            v = locals_[m].float().numpy().astype(np.float32)
            acc = {"sum": np.add, "avg": np.add, "max": np.fmax, "min": np.fmin, "product": np.multiply}[op](acc, v)
        if op == "avg":
            acc = (acc / np.float32(len(members))).astype(np.float32)
        for m in members:
            logical_by_rank[m] = torch.from_numpy(acc)
    # reassemble the logical global tensor from the (non-Partial) sharding of the source
    eff = tuple(p for p in spec.source_placements)
    glob = torch.zeros(spec.shape, dtype=torch.float32)
    for pos, r in enumerate(src_mesh.reshape(-1)):
        coord = dtensor_layout.mesh_coord(src_mesh.shape, pos)
        idx = torch.arange(int(np.prod(spec.shape))).reshape(spec.shape)
        where = dtensor_layout.local_shard(idx, src_mesh.shape, eff, coord)
        glob.view(-1)[where.reshape(-1)] = logical_by_rank[int(r)].reshape(-1)
    return glob


@pytest.mark.parametrize("pair", CASES["communication_cpu"]["mesh_pairs"], ids=lambda p: f"{p[0]}->{p[1]}")
def test_reference_mesh_pairs_with_strided_target(pair):
    cc = CASES["communication_cpu"]
    src_mesh, tgt_mesh = pair
    n_src = int(np.prod(src_mesh))
    spec = TensorSpec("w", tuple(cc["tensor_shape"]), mesh_of(0, src_mesh), parse_placements(cc["source_placements"]),
                      mesh_of(n_src, tgt_mesh), parse_placements(cc["target_placements"]), torch.float32,
                      seed=cc["seed"], std=1.0)
    for bucket_size in cc["bucket_sizes"]:
        job = _run_case(spec, bucket_size)
        for r, t in job.target_locals[0].items():
            assert_bit_equal(t, expected_target(spec, job.globals_[0], r), f"rank {r}")


def test_symmetric_mesh_both_directions():
    sm = CASES["symmetric_mesh"]
    pl = parse_placements(sm["placements"])
    a, b = mesh_of(0, sm["mesh"]), mesh_of(4, sm["mesh"])
    for src, tgt in ((a, b), (b, a)):
        spec = TensorSpec("w", tuple(sm["tensor_shape"]), src, pl, tgt, pl, torch.float32, seed=0, std=1.0)
        job = _run_case(spec, 1)
        for r, t in job.target_locals[0].items():
            assert_bit_equal(t, expected_target(spec, job.globals_[0], r), f"rank {r}")


def test_single_element_chunks_of_transposed_shards():
    """A chunk of one element cut from a ``.t()`` view keeps a stride other than 1 through ``.contiguous()`` and
    ``reshape(-1)``, which the byte view refuses; the oracle flattens such a chunk itself (found by the GPU sweeps)."""
    from torch.distributed.tensor.placement_types import Shard

    def transposed(kind, t):
        return torch.zeros(t.shape[1], t.shape[0], dtype=t.dtype).t() if t.dim() == 2 else torch.zeros_like(t)

    spec = TensorSpec("w", (4, 1), mesh_of(0, [1]), (Shard(1),), mesh_of(1, [4]), (Shard(0),), torch.float32, seed=5, std=1.0)
    job = ReshardJob([spec], device="cpu", bucket_size=None, keep_globals=True, fill=cpu_fill, local_view=transposed)
    run_oracle(job)
    for r, t in job.target_locals[0].items():
        assert_bit_equal(t, expected_target(spec, job.globals_[0], r), f"rank {r}")


@pytest.mark.parametrize("case", [c for c in CASES["reshard"] if not c["slice_view"]],
                         ids=lambda c: f"{c['src_mesh']}{c['src']}->{c['tgt_mesh']}{c['tgt']}")
@pytest.mark.parametrize("bucket_size", CASES["reshard_bucket_sizes"])
def test_reference_reshard_cases(case, bucket_size):
    n_src = int(np.prod(case["src_mesh"]))
    spec = TensorSpec("w", tuple(case["shape"]), mesh_of(0, case["src_mesh"]), parse_placements(case["src"]),
                      mesh_of(n_src, case["tgt_mesh"]), parse_placements(case["tgt"]), torch.float32, seed=0, std=1.0)
    job = _run_case(spec, bucket_size)
    partial = any(c.startswith("P") for c in case["src"])
    glob = _numpy_partial_truth(job, spec) if partial else job.globals_[0]
    for r, t in job.target_locals[0].items():
        assert_bit_equal(t, expected_target(spec, glob, r), f"rank {r}")


def test_partial_fp32_to_bf16_reduces_before_the_cast():
    pm = CASES["partial_mixed_dtype"]
    n_src = int(np.prod(pm["src_mesh"]))
    spec = TensorSpec("w", tuple(pm["shape"]), mesh_of(0, pm["src_mesh"]), (Partial("sum"),),
                      mesh_of(n_src, pm["tgt_mesh"]), parse_placements(["R"]), torch.float32, torch.bfloat16,
                      seed=pm["seed_base"], std=pm["scale"])
    job = _run_case(spec, 1)
    glob = _numpy_partial_truth(job, spec)
    cast_first = sum(t.to(torch.bfloat16) for t in job.source_locals[0].values())
    for r, t in job.target_locals[0].items():
        want = glob.to(torch.bfloat16)
        assert t.dtype == torch.bfloat16
        assert_bit_equal(t, want, f"rank {r}")
    assert not torch.equal(cast_first, glob.to(torch.bfloat16))  # the wrong order is distinguishable here


def _self_copy_chunk(t, src, dst):
    return Chunk(chunk_shape=(4,), transport=Transport.LOCAL, is_source=True, is_target=True, src_rank=0,
                 src_idx=(src // 4,), dst_ranks=(0,), dst_idx=(dst // 4,), src_slice=(slice(src, src + 4),),
                 dst_slice=(slice(dst, dst + 4),), tensor=t)


@pytest.mark.parametrize("case", CASES["self_copy"], ids=lambda c: c["name"])
def test_self_copy_known_answers(case):
    t = torch.tensor(case["tensor"], dtype=torch.float32)
    chunks = [_self_copy_chunk(t, s, d) for s, d in case["copies"]]
    buckets = chunk_to_bucket_ops(chunks, bucket_size=case["bucket_size"])
    if "expect_buckets" in case:
        assert len(buckets) == case["expect_buckets"] and len(buckets[0].chunks) == case["expect_chunks_in_bucket"]
    reference_path.run_rank(buckets, reference_path.Mailbox(), rank=0)
    assert t[case["tail_from"]:].tolist() == [float(x) for x in case["expect_tail"]]


@pytest.mark.parametrize("case", CASES["partial_chunk_reduce"], ids=lambda c: f"{c[0]}{c[1]}{c[2]}{c[3]}{'nc' if c[4] else ''}")
def test_partial_reduce_cases_within_reference_tolerance(case):
    """Collapse Partial -> Replicate on the same mesh size; compare with an fp64 reduction within the
    reference's tolerances, and bit-exactly with the fp32 rank-order closed form."""
    mesh_shape, codes, shape, dtype_name, non_contiguous = case
    dtype = DTYPES[dtype_name]
    n = int(np.prod(mesh_shape))
    tgt_codes = ["R" if c.startswith("P") else c for c in codes]
    spec = TensorSpec("w", tuple(shape), mesh_of(0, mesh_shape), parse_placements(codes), mesh_of(n, mesh_shape),
                      parse_placements(tgt_codes), dtype, seed=1000, std=1.0)
    job = ReshardJob([spec], device="cpu", bucket_size=1, fill=cpu_fill)
    if non_contiguous:  # rebuild the sources as every-other-column views of wider tensors
        for r, t in list(job.source_locals[0].items()):
            wide = torch.zeros(*t.shape[:-1], t.shape[-1] * 2, dtype=t.dtype)
            view = wide[..., ::2]
            view.copy_(t)
            assert not view.is_contiguous()
            job.source_locals[0][r] = view
        job = _rebuild_with_sources(spec, job.source_locals[0])
    run_oracle(job)
    glob32 = _numpy_partial_truth(job, spec)
    rtol, atol = CASES["partial_tolerances"][{"float32": "fp32"}.get(dtype_name, dtype_name)]
    for r, t in job.target_locals[0].items():
        want = expected_target(spec, glob32, r)
        assert_bit_equal(t, want.to(dtype), f"rank {r} vs fp32 rank-order closed form")
        assert torch.allclose(t.double(), expected_target(spec, glob32.double(), r).double(), rtol=rtol, atol=atol)


def _rebuild_with_sources(spec, sources):
    """A job whose source locals are the given (possibly non-contiguous) tensors."""
    from etha_amd.comm import chunk_to_bucket_ops, get_m2m_map, m2m_to_chunks
    from etha_amd.world import create_partial_groups

    job = ReshardJob([spec], device="cpu", bucket_size=1, fill=cpu_fill)
    job.source_locals[0] = sources
    m2m = get_m2m_map(spec.source_mesh, spec.source_placements, spec.target_mesh, spec.target_placements)
    send, recv = {}, {}
    for r, t in sources.items():
        groups = create_partial_groups(np.asarray(spec.source_mesh), m2m.source_partial_reductions, r, sources)
        send[r] = chunk_to_bucket_ops(m2m_to_chunks(m2m, r, source_tensor=t, source_partial_groups=groups or None), 1)
    for r, t in job.target_locals[0].items():
        recv[r] = chunk_to_bucket_ops(m2m_to_chunks(m2m, r, target_tensor=t), 1)
    job.send_buckets, job.recv_buckets = send, recv
    return job
