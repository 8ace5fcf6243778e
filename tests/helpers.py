"""Shared test plumbing: identical inputs for the HIP path (GPU) and the oracle (CPU)."""

from __future__ import annotations

import copy

import numpy as np
import torch

from etha_amd.world import ReshardJob, TensorSpec
from oracle import dtensor_layout, reference_path


def cpu_fill(spec: TensorSpec) -> torch.Tensor:
    """Seeded values generated on the CPU so that GPU and CPU jobs see the same bits."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(spec.seed)
    if spec.dist == "uniform":
        g = torch.rand(spec.shape, generator=gen, dtype=torch.float32) * 2 - 1
    elif spec.dist == "bits":  # every bit pattern class, for byte-move tests
        n = int(np.prod(spec.shape))
        raw = torch.randint(0, 256, (n * spec.source_dtype.itemsize,), generator=gen, dtype=torch.uint8)
        return raw.view(spec.source_dtype).reshape(spec.shape)
    else:
        g = torch.randn(spec.shape, generator=gen, dtype=torch.float32) * spec.std
    if not spec.source_dtype.is_floating_point:  # integers and bool: spread the values over a few hundred units
        g = g * (200.0 / max(spec.std, 1e-6))
    return g.to(spec.source_dtype)


def mirror_partials(gpu_job: ReshardJob, cpu_job: ReshardJob) -> None:
    """Partial sources are generated per device; make the CPU job's partials equal the GPU job's."""
    for g_src, c_src in zip(gpu_job.source_locals, cpu_job.source_locals):
        for r, t in c_src.items():
            t.copy_(g_src[r].cpu())


def make_cpu_job(specs, bucket_size, target_ranks=None) -> ReshardJob:
    """A CPU-resident job with seeded CPU data; module-level so that spawned rank processes can call it."""
    return ReshardJob(clone_specs(specs), device="cpu", bucket_size=bucket_size, target_ranks=target_ranks,
                      keep_globals=True, fill=cpu_fill)


def run_oracle(cpu_job: ReshardJob) -> None:
    """Execute a CPU-resident job with the oracle's restatement of the reference path."""
    box = reference_path.Mailbox()
    for r, buckets in cpu_job.send_buckets.items():
        reference_path.run_rank(buckets, box, rank=r)
    for r, buckets in cpu_job.recv_buckets.items():
        reference_path.run_rank(buckets, box, rank=r)


def expected_target(spec: TensorSpec, glob: torch.Tensor, rank: int) -> torch.Tensor:
    """Closed form: the DTensor slice of the global tensor, through the wire dtype, in target dtype."""
    from etha_amd.world import transfer_dtype_rule

    mesh = np.asarray(spec.target_mesh)
    pos = [int(x) for x in mesh.reshape(-1)].index(rank)
    shard = dtensor_layout.local_shard(glob, mesh.shape, spec.target_placements, dtensor_layout.mesh_coord(mesh.shape, pos))
    tgt = spec.target_dtype or spec.source_dtype
    return shard.to(transfer_dtype_rule(spec.source_dtype, tgt)).to(tgt)


def bits(t: torch.Tensor) -> torch.Tensor:
    """Raw bytes of a tensor, for bit-exact comparison (NaNs and -0 included)."""
    flat = t.detach().cpu().contiguous().reshape(-1)  # flat first: a size-1 last dim may carry any stride ...
    if flat.numel() == 1 and flat.stride(0) != 1:  # ... and so may a single element cut from a .t() view
        flat = flat.as_strided((1,), (1,))
    return flat.view(torch.uint8)


def assert_bit_equal(a: torch.Tensor, b: torch.Tensor, what: str = "") -> None:
    assert a.shape == b.shape and a.dtype == b.dtype, f"{what}: {a.shape}/{a.dtype} vs {b.shape}/{b.dtype}"
    ba, bb = bits(a), bits(b)
    if not torch.equal(ba, bb):
        bad = (ba != bb).nonzero().reshape(-1)
        raise AssertionError(f"{what}: {bad.numel()} differing bytes, first at byte {int(bad[0])}")


def clone_specs(specs):
    return [copy.copy(s) for s in specs]


def next_values(gpu_job: ReshardJob, cpu_job: ReshardJob, k: int) -> None:
    """New source values on both jobs (a transfer that moved stale bytes would show); targets are poisoned."""
    targets = [x for d in gpu_job.target_locals for x in d.values()]
    for g_src, c_src in zip(gpu_job.source_locals, cpu_job.source_locals):
        for r, t in g_src.items():
            if any(t is x for x in targets) or t.numel() == 0:
                continue
            if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
                t.copy_((t.float() * -0.5).to(t.dtype))
            elif t.dtype.is_floating_point:
                t.copy_((t.double() * -0.75 + 0.125 * k).to(t.dtype))
            elif t.dtype == torch.bool:
                t.copy_(~t)
            else:
                t.copy_(t.flip(-1) if t.dim() else t)
            c_src[r].copy_(t.cpu())
    sources = [x for d in gpu_job.source_locals for x in d.values()]
    for job in (gpu_job, cpu_job):
        srcs = [x for d in job.source_locals for x in d.values()]
        for d in job.target_locals:
            for t in d.values():
                if not any(t is x for x in srcs) and t.numel():
                    t.copy_(torch.ones_like(t))
    del sources


def gpu_vs_oracle(specs, device, bucket_size, target_ranks=None, merge_launches=False, check_closed_form=True,
                  pool="ring", max_in_flight=2, repeat=0, replay=True):
    """Run the same job on the GPU (HIP path) and on the CPU (oracle); compare every target shard.  ``repeat`` more
    transfers follow on new source values (with ``replay`` they are served from the wire's recording of the first)."""
    gpu_job = ReshardJob(clone_specs(specs), device=device, bucket_size=bucket_size, target_ranks=target_ranks,
                         keep_globals=True, fill=cpu_fill, pool=pool, max_in_flight=max_in_flight)
    gpu_job.wire.replay_schedules = replay
    cpu_job = ReshardJob(clone_specs(specs), device="cpu", bucket_size=bucket_size, target_ranks=target_ranks,
                         keep_globals=True, fill=cpu_fill)
    mirror_partials(gpu_job, cpu_job)
    src_before = [{r: t.clone() for r, t in d.items()} for d in gpu_job.source_locals]
    gpu_job.run(merge_launches=merge_launches)
    run_oracle(cpu_job)
    for i, spec in enumerate(specs):
        for r, t in gpu_job.target_locals[i].items():
            assert_bit_equal(t, cpu_job.target_locals[i][r], f"{spec.name} target rank {r} vs oracle")
            if check_closed_form and gpu_job.globals_[i] is not None:
                assert_bit_equal(t, expected_target(spec, cpu_job.globals_[i], r), f"{spec.name} rank {r} vs closed form")
        for r, t in gpu_job.source_locals[i].items():
            same_obj = any(t is x for x in gpu_job.target_locals[i].values())
            if not same_obj:
                assert_bit_equal(t, src_before[i][r], f"{spec.name} source rank {r} mutated")
    for k in range(repeat):
        next_values(gpu_job, cpu_job, k + 1)
        before = gpu_job.wire.replays
        gpu_job.run(merge_launches=merge_launches)
        run_oracle(cpu_job)
        for i, spec in enumerate(specs):
            for r, t in gpu_job.target_locals[i].items():
                assert_bit_equal(t, cpu_job.target_locals[i][r], f"transfer {k + 2}: {spec.name} target rank {r} vs oracle")
        if pool == "ring":
            assert (gpu_job.wire.replays > before) == bool(replay), "served from the recording exactly when that is switched on"
    return gpu_job, cpu_job


# ---- fixtures ------------------------------------------------------------------------------------
def load_cases() -> dict:
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_cases.json")) as f:
        return json.load(f)


def parse_placement(code: str):
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard, _StridedShard

    if code == "R":
        return Replicate()
    if code.startswith("SS"):
        dim, sf = code[2:].split("/")
        return _StridedShard(int(dim), split_factor=int(sf))
    if code.startswith("S"):
        return Shard(int(code[1:]))
    if code.startswith("P"):
        return Partial(code[1:])
    raise ValueError(code)


def parse_placements(codes) -> tuple:
    return tuple(parse_placement(c) for c in codes)


def mesh_of(start: int, shape) -> list:
    n = int(np.prod(shape))
    return np.arange(start, start + n).reshape(tuple(shape)).tolist()


DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16, "float32": torch.float32,
          "bfloat16": torch.bfloat16}
