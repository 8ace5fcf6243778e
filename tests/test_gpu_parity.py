"""GPU parity: the HIP path (through the C ABI) against the CPU oracle, bit for bit.

Bar: bit-exact for every byte move and every cast of a non-NaN value; NaNs stay NaNs (payload not
pinned, see oracle/reshard_oracle.c).  The Partial reduce is compared bit-exactly with the oracle's
fp32 rank-order sum, which is well inside the stated tolerance of 1 bf16 ulp.
"""

import numpy as np
import pytest
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from etha_amd import _native, workloads
from etha_amd.comm import Chunk, LoopbackWire, Transport, bucket_comm, chunk_to_bucket_ops
from etha_amd.world import ReshardJob, TensorSpec

from helpers import (DTYPES, assert_bit_equal, bits, clone_specs, cpu_fill, expected_target, gpu_vs_oracle, load_cases, mesh_of,
                     mirror_partials, next_values, parse_placements, run_oracle)

pytestmark = pytest.mark.gpu
CASES = load_cases()


# ---- the single-fp32-tensor config and the reference's own case tables ----------------------------

def test_config1_fp32_shard0_to_shard1(gpu_device):
    """fp32 [1024,1024] uniform(-1,1) seed 0; (2,) Shard(0) -> (4,) Shard(1); full reassembly."""
    specs, targets, _ = workloads.single_fp32_shard0_to_shard1()
    for bucket_size in (None, 256 * 1024, 64 << 20):
        gpu_vs_oracle(specs, gpu_device, bucket_size, target_ranks=targets)


@pytest.mark.parametrize("pair", CASES["communication_cpu"]["mesh_pairs"], ids=lambda p: f"{p[0]}->{p[1]}")
def test_reference_mesh_pairs_with_strided_target(gpu_device, pair):
    cc = CASES["communication_cpu"]
    src_mesh, tgt_mesh = pair
    n_src = int(np.prod(src_mesh))
    spec = TensorSpec("w", tuple(cc["tensor_shape"]), mesh_of(0, src_mesh), parse_placements(cc["source_placements"]),
                      mesh_of(n_src, tgt_mesh), parse_placements(cc["target_placements"]), torch.float32,
                      seed=cc["seed"], std=1.0)
    for bucket_size in cc["bucket_sizes"]:
        gpu_vs_oracle([spec], gpu_device, bucket_size)


def test_symmetric_mesh_both_directions(gpu_device):
    sm = CASES["symmetric_mesh"]
    pl = parse_placements(sm["placements"])
    a, b = mesh_of(0, sm["mesh"]), mesh_of(4, sm["mesh"])
    for src, tgt in ((a, b), (b, a)):
        spec = TensorSpec("w", tuple(sm["tensor_shape"]), src, pl, tgt, pl, torch.float32, seed=0, std=1.0)
        gpu_vs_oracle([spec], gpu_device, 1)


class _HalfOfWider:
    """Re-home a local shard as the first half (along dim 1) of a tensor twice as wide, as the
    reference's slice-view cases do; the other half must never be touched."""

    def __init__(self):
        self.parents = []

    def __call__(self, kind, t):
        shape = list(t.shape)
        shape[1] *= 2
        wide = torch.full(shape, 7.0, dtype=t.dtype, device=t.device)
        self.parents.append((wide, t.shape[1]))
        return wide[:, : t.shape[1]]

    def check_untouched(self):
        for wide, half in self.parents:
            assert bool((wide[:, half:] == 7.0).all()), "bytes outside the chunk slices were written"


@pytest.mark.parametrize("case", CASES["reshard"], ids=lambda c: f"{c['src_mesh']}{c['src']}->{c['tgt_mesh']}{c['tgt']}{'view' if c['slice_view'] else ''}")
@pytest.mark.parametrize("bucket_size", CASES["reshard_bucket_sizes"])
def test_reference_reshard_cases(gpu_device, case, bucket_size):
    n_src = int(np.prod(case["src_mesh"]))
    spec = TensorSpec("w", tuple(case["shape"]), mesh_of(0, case["src_mesh"]), parse_placements(case["src"]),
                      mesh_of(n_src, case["tgt_mesh"]), parse_placements(case["tgt"]), torch.float32, seed=0, std=1.0)
    if not case["slice_view"]:
        gpu_vs_oracle([spec], gpu_device, bucket_size)
        return
    g_view, c_view = _HalfOfWider(), _HalfOfWider()
    gpu_job = ReshardJob([spec], device=gpu_device, bucket_size=bucket_size, keep_globals=True, fill=cpu_fill, local_view=g_view)
    cpu_job = ReshardJob([spec], device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill, local_view=c_view)
    assert not next(iter(gpu_job.source_locals[0].values())).is_contiguous()
    gpu_job.run()
    run_oracle(cpu_job)
    for r, t in gpu_job.target_locals[0].items():
        assert_bit_equal(t, cpu_job.target_locals[0][r], f"rank {r} vs oracle")
        assert_bit_equal(t, expected_target(spec, cpu_job.globals_[0], r), f"rank {r} vs closed form")
    g_view.check_untouched()
    c_view.check_untouched()


def test_partial_fp32_to_bf16_reduces_before_the_cast(gpu_device):
    pm = CASES["partial_mixed_dtype"]
    n_src = int(np.prod(pm["src_mesh"]))
    spec = TensorSpec("w", tuple(pm["shape"]), mesh_of(0, pm["src_mesh"]), (Partial("sum"),),
                      mesh_of(n_src, pm["tgt_mesh"]), (Replicate(),), torch.float32, torch.bfloat16,
                      seed=pm["seed_base"], std=pm["scale"])
    for bucket_size in (1, 256 << 20):
        gpu_vs_oracle([spec], gpu_device, bucket_size)


@pytest.mark.parametrize("case", CASES["partial_chunk_reduce"], ids=lambda c: f"{c[0]}{c[1]}{c[2]}{c[3]}{'nc' if c[4] else ''}")
def test_partial_reduce_cases(gpu_device, case):
    mesh_shape, codes, shape, dtype_name, non_contiguous = case
    n = int(np.prod(mesh_shape))
    tgt_codes = ["R" if c.startswith("P") else c for c in codes]
    spec = TensorSpec("w", tuple(shape), mesh_of(0, mesh_shape), parse_placements(codes), mesh_of(n, mesh_shape),
                      parse_placements(tgt_codes), DTYPES[dtype_name], seed=1000, std=1.0)
    if not non_contiguous:
        gpu_vs_oracle([spec], gpu_device, 1)
        return

    def every_other(kind, t):  # source partials become every-other-column views (element stride 2)
        if kind != "source":
            return t
        wide = torch.zeros(*t.shape[:-1], t.shape[-1] * 2, dtype=t.dtype, device=t.device)
        return wide[..., ::2]

    gpu_job = ReshardJob([spec], device=gpu_device, bucket_size=1, local_view=every_other)
    cpu_job = ReshardJob([spec], device="cpu", bucket_size=1, local_view=every_other)
    mirror_partials(gpu_job, cpu_job)
    gpu_job.run()
    run_oracle(cpu_job)
    for r, t in gpu_job.target_locals[0].items():
        assert_bit_equal(t, cpu_job.target_locals[0][r], f"rank {r}")


# ---- dtypes ---------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.uint8, torch.int8, torch.bool, torch.int16, torch.int32, torch.int64,
                                   torch.float16, torch.bfloat16, torch.float32, torch.float64, torch.complex64,
                                   torch.float8_e4m3fn])
def test_same_dtype_is_a_byte_move(gpu_device, dtype):
    """Every bit pattern survives (NaN payloads, -0, denormals): random bytes reinterpreted as dtype."""
    spec = TensorSpec("w", (96, 80), mesh_of(0, [2, 2]), (Shard(0), Shard(1)), mesh_of(4, [4]), (Shard(1),), dtype,
                      seed=11, dist="bits")
    if dtype == torch.bool:
        spec.dist = "normal"
        gpu_vs_oracle([spec], gpu_device, 4096, check_closed_form=False)
        return
    gpu_vs_oracle([spec], gpu_device, 4096)


def _special_values(dtype):
    f = torch.tensor([0.0, -0.0, 1.0, -1.0, float("inf"), float("-inf"), 65504.0, 65520.0, 1e-8, -1e-8, 3.4e38,
                      1.17549435e-38, 1e-40, -1e-45, 2.0**-24, 2.0**-25, 1.0 + 2.0**-8, 1.0 + 3 * 2.0**-9, 0.1, 1e5],
                     dtype=torch.float64)
    return f.to(dtype)


@pytest.mark.parametrize("src_dt", ["fp16", "bf16", "fp32", "fp64"])
@pytest.mark.parametrize("dst_dt", ["fp16", "bf16", "fp32", "fp64"])
def test_float_conversions(gpu_device, src_dt, dst_dt):
    names = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32, "fp64": torch.float64}
    s, d = names[src_dt], names[dst_dt]
    if s == d:
        pytest.skip("same dtype is covered by the byte-move test")

    def fill(spec):
        g = torch.Generator().manual_seed(5)
        x = torch.randn(spec.shape, generator=g, dtype=torch.float64)
        x = x * torch.logspace(-10, 10, spec.shape[1], dtype=torch.float64)
        sp = _special_values(torch.float64)
        x.view(-1)[: sp.numel()] = sp
        with torch.no_grad():
            return x.to(spec.source_dtype)

    for shape in ((64, 256), (37, 51)):  # vector path and element-wise path
        spec = TensorSpec("w", shape, mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),), s, d, seed=5)
        gpu_job = ReshardJob([spec], device=gpu_device, bucket_size=1 << 20, keep_globals=True, fill=fill)
        cpu_job = ReshardJob([spec], device="cpu", bucket_size=1 << 20, keep_globals=True, fill=fill)
        gpu_job.run()
        run_oracle(cpu_job)
        assert_bit_equal(gpu_job.target_locals[0][1], cpu_job.target_locals[0][1], f"{src_dt}->{dst_dt} {shape}")


_VALUE_TYPES = [torch.float16, torch.bfloat16, torch.float32, torch.float64, torch.int8, torch.uint8, torch.int16, torch.int32,
                torch.int64, torch.bool, torch.float8_e4m3fn, torch.float8_e5m2]


@pytest.mark.parametrize("src", _VALUE_TYPES, ids=lambda d: str(d).replace("torch.", ""))
def test_value_type_conversions(gpu_device, src):
    """``Tensor.to`` between every pair of value types that involves an integer, bool or 8-bit float, on random bit
    patterns, magnitudes around the integer limits (out of range included) and the committed special values:
    the kernel's element-wise converter against the oracle's restatement of the reference path (torch's CPU casts)."""
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cast_kats.json")) as f:
        kats = json.load(f)
    name = {torch.float16: "f16", torch.bfloat16: "bf16", torch.float32: "f32", torch.float64: "f64",
            torch.float8_e4m3fn: "e4m3", torch.float8_e5m2: "e5m2"}.get(src)

    def fill(spec):
        g = torch.Generator().manual_seed(11)
        n = spec.shape[0] * spec.shape[1]
        raw = torch.randint(0, 256, (n * src.itemsize,), generator=g, dtype=torch.uint8)
        x = ((raw % 2).view(src) if src == torch.bool else raw.view(src)).clone()
        if src.is_floating_point:
            k = n // 3
            x[:k] = (torch.randn(k, generator=g, dtype=torch.float64) * 300).to(src)
            x[k:2 * k] = (torch.randn(k, generator=g, dtype=torch.float64) * 3e9).to(src)
            special = np.array([int(v, 16) for v in kats["float_to_int"][f"{name}->i32"]["in"]], dtype=np.uint64)
            raw_np = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[src.itemsize]
            x[2 * k:2 * k + len(special)] = torch.from_numpy(special.astype(raw_np).view(np.uint8).copy()).view(src)
        return x.reshape(spec.shape)

    for dst in _VALUE_TYPES:
        if dst == src or (src in _VALUE_TYPES[:4] and dst in _VALUE_TYPES[:4]):
            continue  # the four IEEE-style floats among themselves: test_float_conversions
        spec = TensorSpec("w", (33, 50), mesh_of(0, [2]), (Shard(1),), mesh_of(2, [3]), (Shard(0),), src, dst, seed=5)
        gpu_job = ReshardJob([spec], device=gpu_device, bucket_size=512, keep_globals=True, fill=fill)
        cpu_job = ReshardJob([spec], device="cpu", bucket_size=512, keep_globals=True, fill=fill)
        gpu_job.run()
        run_oracle(cpu_job)
        for r, got in gpu_job.target_locals[0].items():
            want = cpu_job.target_locals[0][r]
            a, b = bits(got).view(got.shape + (-1,)), bits(want).view(want.shape + (-1,))
            same = (a == b).all(-1)
            if dst.is_floating_point:  # NaN payloads are not pinned
                same |= torch.isnan(got.cpu().to(torch.float64)) & torch.isnan(want.to(torch.float64))
            assert bool(same.all()), f"{src} -> {dst} rank {r}: {int((~same).sum())} elements differ"


def test_opaque_types_can_only_be_moved(gpu_device):
    spec = TensorSpec("c", (8, 8), mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),), torch.complex64, torch.float32)
    job = ReshardJob([spec], device=gpu_device, bucket_size=1 << 20, fill=lambda s: torch.zeros(s.shape, dtype=torch.complex64))
    with pytest.raises(NotImplementedError, match="only floats, integers, bool and 8-bit floats are converted"):
        job.run()


def test_nan_stays_nan(gpu_device):
    def fill(spec):
        x = torch.zeros(spec.shape, dtype=torch.float32)
        x.view(torch.int32).view(-1)[:4] = torch.tensor([0x7FC00000, 0x7F800001, -4194304, 0x7FFFFFFF], dtype=torch.int32)
        return x

    for d in (torch.bfloat16, torch.float16, torch.float64):
        spec = TensorSpec("w", (8, 8), mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),), torch.float32, d)
        job = ReshardJob([spec], device=gpu_device, bucket_size=1 << 20, fill=fill)
        job.run()
        out = job.target_locals[0][1].cpu().reshape(-1)
        assert bool(out[:4].isnan().all()) and not bool(out[4:].isnan().any())


# ---- geometry ---------------------------------------------------------------------------------------

@pytest.mark.parametrize("shape,dtype", [((33, 50), torch.bfloat16), ((7, 3), torch.int8), ((129, 1023), torch.float32),
                                         ((4, 6, 10), torch.bfloat16), ((1, 1), torch.float64), ((2048, 16), torch.bfloat16)])
def test_odd_shapes_and_unaligned_bucket_offsets(gpu_device, shape, dtype):
    """Un-padded prefix-sum offsets put later chunks at addresses that are only element-aligned;
    the narrow vector classes must cope.  (Offsets that are not a multiple of the item size cannot
    occur in the reference: its ``view(dtype)`` of the bucket slice raises for them, ir.py:252.)"""
    specs = [
        TensorSpec("odd", (3, 5), mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),), dtype, seed=1, dist="bits"),
        TensorSpec("w", shape, mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),), dtype, seed=2, dist="bits"),
        TensorSpec("w2", shape, mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),), dtype, seed=3, dist="bits"),
    ]
    gpu_vs_oracle(specs, gpu_device, 1 << 30)


def test_permuted_parent_uses_strided_elements(gpu_device):
    def permuted(kind, t):
        if t.dim() != 3:
            return t
        base = torch.zeros(t.shape[2], t.shape[0], t.shape[1], dtype=t.dtype, device=t.device)
        return base.permute(1, 2, 0)

    spec = TensorSpec("w", (12, 20, 24), mesh_of(0, [2, 2]), (Shard(0), Shard(2)), mesh_of(4, [2]), (Shard(1),),
                      torch.bfloat16, seed=9, dist="bits")
    gpu_job = ReshardJob([spec], device=gpu_device, bucket_size=4096, keep_globals=True, fill=cpu_fill, local_view=permuted)
    cpu_job = ReshardJob([spec], device="cpu", bucket_size=4096, keep_globals=True, fill=cpu_fill, local_view=permuted)
    assert not next(iter(gpu_job.target_locals[0].values())).is_contiguous()
    gpu_job.run()
    run_oracle(cpu_job)
    for r, t in gpu_job.target_locals[0].items():
        assert_bit_equal(t, cpu_job.target_locals[0][r], f"rank {r}")
        assert_bit_equal(t, expected_target(spec, cpu_job.globals_[0], r), f"rank {r} closed form")


def test_empty_shards_and_empty_bucket_list(gpu_device):
    spec = TensorSpec("w", (3, 8), mesh_of(0, [4]), (Shard(0),), mesh_of(4, [2]), (Replicate(),), torch.float32, seed=1)
    gpu_vs_oracle([spec], gpu_device, 1)  # rank 3 holds an empty shard
    bucket_comm([])


# ---- self-copy ----------------------------------------------------------------------------------------

def _self_copy_chunk(t, src, dst, n=4):
    return Chunk(chunk_shape=(n,), transport=Transport.LOCAL, is_source=True, is_target=True, src_rank=0,
                 src_idx=(src // n,), dst_ranks=(0,), dst_idx=(dst // n,), src_slice=(slice(src, src + n),),
                 dst_slice=(slice(dst, dst + n),), tensor=t)


@pytest.mark.parametrize("case", CASES["self_copy"], ids=lambda c: c["name"])
def test_self_copy_known_answers(gpu_device, case):
    t = torch.tensor(case["tensor"], dtype=torch.float32, device=gpu_device)
    chunks = [_self_copy_chunk(t, s, d) for s, d in case["copies"]]
    buckets = chunk_to_bucket_ops(chunks, bucket_size=case["bucket_size"])
    if "expect_buckets" in case:
        assert len(buckets) == case["expect_buckets"] and len(buckets[0].chunks) == case["expect_chunks_in_bucket"]
    wire = LoopbackWire(gpu_device)
    bucket_comm(buckets, wire=wire)
    assert t[case["tail_from"]:].tolist() == [float(x) for x in case["expect_tail"]]
    assert t[: case["tail_from"]].tolist() == [float(x) for x in case["tensor"][: case["tail_from"]]]
    plan = wire.plan(buckets)
    assert [s[0] for s in plan.steps] == ["selfcopy"]  # no overlap: direct copy, no staging


def test_bundled_self_copy_with_overlap_is_staged(gpu_device):
    """A swap: chunk 0 copies a->b, chunk 1 copies b->a.  Reads must all precede writes (the reference
    stages a bundled bucket through its buffer), so the executor must not copy in place."""
    t = torch.arange(16, dtype=torch.float32, device=gpu_device)
    chunks = [_self_copy_chunk(t, 0, 8, 8), _self_copy_chunk(t, 8, 0, 8)]
    buckets = chunk_to_bucket_ops(chunks, bucket_size=1 << 20)
    wire = LoopbackWire(gpu_device)
    bucket_comm(buckets, wire=wire)
    assert t.tolist() == [float(x) for x in list(range(8, 16)) + list(range(8))]
    assert [s[0] for s in wire.plan(buckets).steps] == ["pack", "unpack"]
    t_cpu = torch.arange(16, dtype=torch.float32)
    from oracle import reference_path
    cpu_chunks = [_self_copy_chunk(t_cpu, 0, 8, 8), _self_copy_chunk(t_cpu, 8, 0, 8)]
    reference_path.run_rank(chunk_to_bucket_ops(cpu_chunks, 1 << 20), reference_path.Mailbox(), 0)
    assert t.cpu().tolist() == t_cpu.tolist()


def test_recv_before_send_is_an_error(gpu_device):
    spec = TensorSpec("w", (8, 8), [0, 1], (Shard(0),), [2, 3], (Shard(1),), torch.float32)
    job = ReshardJob([spec], device=gpu_device, bucket_size=None)
    with pytest.raises(RuntimeError, match="no matching send bucket"):
        job.run_recv()


# ---- scaled-down versions of the headline configs, against the oracle ---------------------------------

@pytest.mark.parametrize("replay", [True, False], ids=["recorded", "pipelines"])
@pytest.mark.parametrize("workload", ["llama", "short_rows", "partial", "moe_self_copy", "transposed", "fp32_to_bf16"])
def test_repeated_transfers_with_and_without_the_recording(gpu_device, workload, replay):
    """Three transfers of one registration on new values each time, scaled-down forms of the configurations: with the
    wire's recording of the first transfer switched on (the second and third are re-issued by etha_schedule_launch)
    and off (the pipelines are stepped every time), against the oracle every time."""
    if workload == "llama":
        specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=2, hidden=256, inter=896, kv=64, vocab=2056)
    elif workload == "fp32_to_bf16":
        specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=2, hidden=256, inter=896, kv=64, vocab=2056,
                                                             dtype=torch.float32, target_dtype=torch.bfloat16)
    elif workload == "short_rows":
        specs, targets, _ = workloads.many_small_2d_to_replicate(n_tensors=12, rows=64)
    elif workload == "partial":
        specs, targets, _ = workloads.partial4_to_shard2(n_tensors=3, n=256)
    elif workload == "moe_self_copy":
        specs, targets, _ = workloads.moe_experts_and_uneven_vocab(n_experts=8, hidden=64, inter=224, vocab=1030)
    else:
        specs, targets, _ = workloads.transposed_parents(n_tensors=3, n=520)
    for s in specs:
        s.std = 1.0
    gpu_vs_oracle(specs, gpu_device, 64 * 1024, target_ranks=targets, merge_launches=True, repeat=2, replay=replay)


@pytest.mark.parametrize("pool", ["ring", "resident"])
@pytest.mark.parametrize("merge", [False, True])
def test_llama_like_fsdp_to_tp_small(gpu_device, merge, pool):
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=2, hidden=256, inter=896, kv=64, vocab=2056)
    gpu_vs_oracle(specs, gpu_device, 64 * 1024, target_ranks=targets, merge_launches=merge, pool=pool)
    gpu_vs_oracle(specs, gpu_device, 64 * 1024, target_ranks=None, merge_launches=merge, pool=pool)


@pytest.mark.parametrize("depth", [1, 2, 4])
def test_ring_depths_and_unordered_launches(gpu_device, depth):
    """Many buckets per channel through rings of 1, 2 and 4 slots: same bytes as the oracle, the pool stays
    within channels x depth x bucket, most launches are issued without ordering, and switching that off
    changes nothing but the flags."""
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=6, hidden=256, inter=896, kv=64, vocab=520)
    job, _ = gpu_vs_oracle(specs, gpu_device, 32 * 1024, target_ranks=targets, max_in_flight=depth)
    channels = sum(len({(b.src_rank, b.dst_ranks, b.transport) for b in bs}) for bs in job.send_buckets.values())
    largest = max(b.total_bytes for bs in job.send_buckets.values() for b in bs)
    assert job.wire.pool.reserved_bytes <= channels * depth * (largest + 256)
    assert job.wire.pool.reserved_bytes < job.payload_bytes() // 2
    log = job.wire.launch_log = []
    for d in job.target_locals:
        for t in d.values():
            t.zero_()
    job.run()
    assert sum(1 for _, _, _, flags in log if flags & 1) > len(log) // 2
    want = [{r: t.clone() for r, t in d.items()} for d in job.target_locals]
    job.wire.unordered_launches = False
    log.clear()
    for d in job.target_locals:
        for t in d.values():
            t.zero_()
    job.run()
    assert not any(flags & 1 for _, _, _, flags in log)
    for d, w in zip(job.target_locals, want):
        for r, t in d.items():
            assert torch.equal(t.view(torch.uint8), w[r].view(torch.uint8))


def test_many_small_2d_to_replicate_small(gpu_device):
    specs, targets, _ = workloads.many_small_2d_to_replicate(n_tensors=24, rows=64)
    job, _ = gpu_vs_oracle(specs, gpu_device, 256 * 1024, target_ranks=targets, merge_launches=True)
    assert job.counts()["recv_buckets"] >= 8  # 8 source ranks -> 8 channels


@pytest.mark.parametrize("op", ["sum", "avg", "max", "min", "product"])
def test_partial4_to_shard2_small(gpu_device, op):
    specs, targets, _ = workloads.partial4_to_shard2(n_tensors=3, n=256)
    for s in specs:
        s.source_placements = (Partial(op),)
        s.std = 1.0 if op == "product" else 0.02
    gpu_job, cpu_job = gpu_vs_oracle(specs, gpu_device, 128 * 1024, target_ranks=targets)
    if op == "sum":  # stated tolerance: 1 bf16 ulp of the fp32 rank-order sum (here it is met exactly)
        for i in range(len(specs)):
            parts = [gpu_job.source_locals[i][r].float().cpu() for r in range(4)]
            acc = parts[0]
            for p in parts[1:]:
                acc = acc + p
            want = acc[: acc.shape[0] // 2].to(torch.bfloat16)
            got = gpu_job.target_locals[i][4].cpu()
            ulp = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs().max().item()
            assert ulp <= 1 and ulp == 0


def test_moe_experts_and_uneven_vocab_small(gpu_device):
    specs, _, _ = workloads.moe_experts_and_uneven_vocab(n_experts=8, hidden=64, inter=224, vocab=1000)
    job, _ = gpu_vs_oracle(specs, gpu_device, 32 * 1024, target_ranks=[0, 1, 2, 3])
    kinds = {s[0] for plan in [job.wire.plan(b) for b in job.send_buckets.values()] for s in plan.steps}
    assert "selfcopy" in kinds and "pack" in kinds  # same-rank chunks took the direct path
    sizes = [t.shape[0] for t in job.source_locals[3].values()]
    assert sizes == [167] * 5 + [165]  # uneven tail shard


# ---- full size: size-independent properties ------------------------------------------------------------

@pytest.mark.parametrize("bucket_size", [64 << 20, None, 1 << 20, 1 << 30], ids=["64MiB", "unbucketed", "1MiB", "1GiB"])
def test_llama3_8b_full_size_properties(gpu_device, bucket_size):
    """Config 2 at its real size: every target shard equals its slice of the global tensor, sources
    are untouched, and the step is idempotent - for the configured 64 MiB buckets and for other bucket sizes."""
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket_size, target_ranks=targets, keep_globals=True)
    assert job.payload_bytes() == 8_030_519_296 and job.counts()["recv_chunks"] == 1672
    if bucket_size is None:
        assert job.counts()["recv_buckets"] == 1672
    src_sums = [{r: t.view(torch.int16).sum(dtype=torch.int64).item() for r, t in d.items()} for d in job.source_locals]
    job.run(merge_launches=True)
    if bucket_size == 64 << 20:
        # the pool is a ring: 2 slots per channel, each as large as the channel's largest bucket (here the
        # 125.25 MiB single-chunk embedding buckets), instead of the 8.03 GB a slot per bucket would take
        embed = 128256 // 8 * 4096 * 2
        assert job.wire.pool.reserved_bytes <= 8 * 2 * embed + 8 * 2 * 65536
    from oracle.dtensor_layout import local_shard  # the pinned convention, not the product's planner

    def check():
        for i, spec in enumerate(specs):
            want = local_shard(job.globals_[i], (2,), spec.target_placements, (0,))
            assert torch.equal(job.target_locals[i][8].view(torch.int16), want.contiguous().view(torch.int16)), spec.name

    check()
    for i, d in enumerate(job.source_locals):
        for r, t in d.items():
            assert t.view(torch.int16).sum(dtype=torch.int64).item() == src_sums[i][r], "source mutated"
    for d in job.target_locals:
        d[8].zero_()
    job.run(merge_launches=False)  # second transfer, one launch per bucket this time
    check()


def _check_targets_against_global(job, specs, cast=None):
    import numpy as np

    from oracle.dtensor_layout import local_shard, mesh_coord  # the pinned convention, not the product's planner

    for i, spec in enumerate(specs):
        mesh = np.asarray(spec.target_mesh)
        flat = [int(x) for x in mesh.reshape(-1)]
        for r, got in job.target_locals[i].items():
            want = local_shard(job.globals_[i], mesh.shape, spec.target_placements, mesh_coord(mesh.shape, flat.index(r)))
            if cast is not None:
                want = want.to(cast)
            assert got.shape == want.shape and got.dtype == want.dtype, spec.name
            assert torch.equal(got.contiguous().view(torch.uint8), want.contiguous().view(torch.uint8)), (spec.name, r)


def test_llama3_8b_fp32_to_bf16_full_size_properties(gpu_device):
    """Config 2 with fp32 source shards and bf16 targets at full size: every target shard is the RNE
    bf16 cast of its slice of the fp32 global tensor (torch's device cast is the independent check)."""
    specs, targets, bucket = workloads.llama3_8b_fsdp8_to_tp2_fp32_to_bf16()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets, keep_globals=True)
    assert job.payload_bytes() == 8_030_519_296
    job.run(merge_launches=True)
    _check_targets_against_global(job, specs, cast=torch.bfloat16)


def test_many_small_2d_to_replicate_full_size_properties(gpu_device):
    """Config 3 at full size: the replicated target equals the global tensor; both launch granularities."""
    specs, targets, bucket = workloads.many_small_2d_to_replicate()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets, keep_globals=True)
    assert len(job.send_buckets) == 8  # one channel per source rank
    for merge in (True, False):
        for d in job.target_locals:
            for t in d.values():
                t.zero_()
        job.run(merge_launches=merge)
        _check_targets_against_global(job, specs)


def test_partial4_to_shard2_full_size_properties(gpu_device):
    """Config 4 at full size: the target shard is the fp32 rank-order sum of the four partials, cast once
    to bf16 - recomputed here with torch device ops (IEEE fp32 adds, RNE cast), so 0 ulp is required
    where 1 bf16 ulp is allowed; the partials are not modified."""
    specs, targets, bucket = workloads.partial4_to_shard2()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets)
    sums = [{r: t.view(torch.int16).sum(dtype=torch.int64).item() for r, t in d.items()} for d in job.source_locals]
    job.run(merge_launches=True)
    for i, spec in enumerate(specs):
        acc = job.source_locals[i][0][:4096].float()
        for r in (1, 2, 3):
            acc = acc + job.source_locals[i][r][:4096].float()
        want = acc.to(torch.bfloat16)
        got = job.target_locals[i][4]
        ulp = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs().max().item()
        assert ulp == 0, (spec.name, ulp)
        for r, t in job.source_locals[i].items():
            assert t.view(torch.int16).sum(dtype=torch.int64).item() == sums[i][r], "partial mutated"


def test_moe_experts_and_uneven_vocab_full_size_properties(gpu_device):
    """Config 5 at full size, all four target ranks: every shard (through buckets or the direct
    same-rank path) equals its slice of the global tensor, uneven 151936-row embedding included."""
    specs, _, bucket = workloads.moe_experts_and_uneven_vocab()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=[0, 1, 2, 3], keep_globals=True)
    assert [t.shape[0] for t in job.source_locals[3].values()] == [25323] * 5 + [25321]
    job.run(merge_launches=True)
    _check_targets_against_global(job, specs)


@pytest.mark.parametrize("target_transposed", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.int8, torch.float64])
def test_transposed_parents_small(gpu_device, dtype, target_transposed):
    """Shards that are ``.t()`` views on one or both sides: full 16-byte-vector blocks and element-wise edge
    blocks of the transposing kernel, against the oracle."""
    specs, targets, _ = workloads.transposed_parents(n_tensors=2, n=776, dtype=dtype, target_transposed=target_transposed)
    for s in specs:
        s.dist = "bits"
    job, _ = gpu_vs_oracle(specs, gpu_device, 256 * 1024, target_ranks=targets)
    assert not job.source_locals[0][0].is_contiguous()
    assert all(job.wire.plan(b).send_table.info().n_trans_tiles > 0 for b in job.send_buckets.values())
    recv = job.wire.plan(job.recv_buckets[4]).recv_table.info()
    assert (recv.n_trans_tiles > 0) == target_transposed


@pytest.mark.parametrize("target_transposed", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.int16, torch.int8])
def test_transposed_parents_wide_blocks(gpu_device, dtype, target_transposed):
    """Shards of 1- and 2-byte elements large enough for 256 x 256 blocks (each loaded whole, then staged through
    LDS in one or two panels), with 128 x 128 blocks and edge blocks around them, against the oracle."""
    specs, targets, _ = workloads.transposed_parents(n_tensors=2, n=1576, dtype=dtype, target_transposed=target_transposed)
    for s in specs:
        s.dist = "bits"
    job, _ = gpu_vs_oracle(specs, gpu_device, 4 * 1024 * 1024, target_ranks=targets)
    assert not job.source_locals[0][0].is_contiguous()
    for b in job.send_buckets.values():
        tiles = job.wire.plan(b).send_table.trans_tiles()
        wide = (tiles["nj"] == 256) & (tiles["nk"] == 256)
        full = (tiles["nj"] == 128) & (tiles["nk"] == 128)
        assert wide.any() and full.any() and (~wide & ~full).any()


@pytest.mark.parametrize("narrow", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("direction", ["f32 .t() source -> 16-bit target", "16-bit source -> f32 .t() target"])
def test_transposed_f32_parents_convert_in_the_transposing_kernel(gpu_device, narrow, direction):
    """fp32 shards that are ``.t()`` views with a 16-bit wire dtype (master weights stored [in, out] -> serving
    weights, and back): the transposing blocks convert on the way, full blocks and edge blocks, against the oracle."""
    src, tgt = mesh_of(0, [4]), mesh_of(4, [2])
    pack_side = direction.startswith("f32")
    specs = [TensorSpec(f"w{i}", (904, 904), src, (Shard(0),), tgt, (Shard(0),), torch.float32 if pack_side else narrow,
                        narrow if pack_side else torch.float32, seed=i,
                        source_layout="transposed" if pack_side else "contiguous",
                        target_layout="contiguous" if pack_side else "transposed") for i in range(2)]
    job, _ = gpu_vs_oracle(specs, gpu_device, 256 * 1024, target_ranks=[4])
    if pack_side:
        infos = [job.wire.plan(b).send_table.info() for b in job.send_buckets.values()]
        tiles = job.wire.plan(job.send_buckets[0]).send_table.trans_tiles()
    else:
        infos = [job.wire.plan(job.recv_buckets[4]).recv_table.info()]
        tiles = job.wire.plan(job.recv_buckets[4]).recv_table.trans_tiles()
    assert all(i.n_trans_tiles > 0 and i.n_row_tiles == 0 for i in infos)
    wide = (tiles["nj"] == 128) & (tiles["nk"] == 256)
    full = (tiles["nj"] == 128) & (tiles["nk"] == 128)
    assert np.all(tiles["cvt"] != 0) and wide.any() and full.any() and (~wide & ~full).any()


_TYPED_PAIRS = [
    # (source dtype, target dtype, which side is the .t() view)
    (torch.float64, torch.float32, "source"), (torch.float64, torch.bfloat16, "source"), (torch.float32, torch.int8, "source"),
    (torch.int32, torch.int16, "source"), (torch.float32, torch.float8_e4m3fn, "source"), (torch.int64, torch.float32, "source"),
    (torch.float16, torch.bfloat16, "target"), (torch.bfloat16, torch.float64, "target"), (torch.int8, torch.int32, "target"),
    (torch.float32, torch.float64, "target"), (torch.bool, torch.float16, "target"), (torch.uint8, torch.int64, "target"),
]


@pytest.mark.parametrize("src_dt,tgt_dt,side", _TYPED_PAIRS,
                         ids=lambda v: str(v).replace("torch.", "") if not isinstance(v, str) else v)
def test_transposed_parents_of_any_value_type_convert_in_lds_blocks(gpu_device, src_dt, tgt_dt, side):
    """``.t()`` shards whose element type differs from the wire's, beyond f32 <-> 16-bit: the typed transposing kernel
    converts every element while the block is parked in LDS (full blocks of 128 x 128, or 64 x 64 with an 8-byte
    side, and edge blocks), against the oracle's restatement of the reference path."""
    src, tgt = mesh_of(0, [4]), mesh_of(4, [2])
    specs = [TensorSpec(f"w{i}", (904, 652), src, (Shard(0),), tgt, (Shard(0),), src_dt, tgt_dt, seed=i, std=1.0,
                        source_layout="transposed" if side == "source" else "contiguous",
                        target_layout="transposed" if side == "target" else "contiguous") for i in range(2)]
    job, _ = gpu_vs_oracle(specs, gpu_device, 256 * 1024, target_ranks=[4], check_closed_form=False)
    if side == "source":
        tables = [job.wire.plan(b).send_table for b in job.send_buckets.values()]
    else:
        tables = [job.wire.plan(job.recv_buckets[4]).recv_table]
    dim = 64 if 8 in (src_dt.itemsize, tgt_dt.itemsize) else 128
    for table in tables:
        info, tiles = table.info(), table.trans_tiles()
        assert info.n_trans_tiles > 0 and info.n_row_tiles == 0 and info.n_run_tiles == 0
        assert np.all(tiles["cvt"] & _native.TRANS_TYPED) and np.all(tiles["n_peers"] == 0)
        full = (tiles["nj"] == dim) & (tiles["nk"] == dim)
        assert full.any() and (~full).any() and tiles["nj"].max() <= dim and tiles["nk"].max() <= dim


def test_direct_wire_converts_transposed_sources_in_lds_blocks(gpu_device):
    """The direct wire writes the target straight from a ``.t()`` source of another type (bf16 -> f32: the narrow side
    is the tensor, which no bucket table ever sees): typed blocks in the region-to-region table."""
    src, tgt = mesh_of(0, [4]), mesh_of(4, [2])
    specs = [TensorSpec("w", (776, 520), src, (Shard(0),), tgt, (Shard(0),), torch.bfloat16, torch.float32, seed=3, std=1.0,
                        source_layout="transposed")]
    jobs = []
    for direct in (True, False):
        job = ReshardJob(clone_specs(specs), device=gpu_device, bucket_size=256 * 1024, target_ranks=[4], fill=cpu_fill, direct=direct)
        job.run()
        jobs.append(job)
    assert_bit_equal(jobs[0].target_locals[0][4], jobs[1].target_locals[0][4], "direct wire vs buckets")
    tiles = jobs[0].wire.plan(jobs[0].recv_buckets[4]).local_table.trans_tiles()
    assert len(tiles) and np.all(tiles["cvt"] & _native.TRANS_TYPED)


@pytest.mark.parametrize("dtype,wire", [(torch.bfloat16, None), (torch.float32, torch.bfloat16), (torch.float16, None),
                                        (torch.float64, torch.float32)],
                         ids=["bf16", "f32_to_bf16", "f16", "f64_to_f32"])
@pytest.mark.parametrize("op", ["sum", "avg", "max"])
def test_partial_members_stored_transposed_are_reduced_in_lds_blocks(gpu_device, dtype, wire, op):
    """A Partial source whose members are ``.t()`` views: the typed transposing kernel combines the members' blocks in
    registers (fp32, list order; f64 for f64 members), rounds once and writes the bucket through LDS - full and
    edge blocks, against the oracle (bit for bit: the oracle's reduce is the same rank-order sum)."""
    src, tgt = mesh_of(0, [4]), mesh_of(4, [2])
    specs = [TensorSpec(f"p{i}", (1320, 776), src, (Partial(op),), tgt, (Shard(0),), dtype, wire, seed=10 * i, std=1.0,
                        source_layout="transposed") for i in range(2)]
    job, _ = gpu_vs_oracle(specs, gpu_device, 256 * 1024, target_ranks=[4])
    seen = 0
    for b in job.send_buckets.values():
        table = job.wire.plan(b).send_table
        if table is None or not table.info().n_chunks:
            continue
        tiles = table.trans_tiles()
        if len(tiles):
            assert table.info().n_row_tiles == 0
            assert np.all(tiles["n_peers"] == 4) and np.all(tiles["cvt"] & _native.TRANS_TYPED)
            dim = 64 if dtype == torch.float64 else 128
            full = (tiles["nj"] == dim) & (tiles["nk"] == dim)
            assert full.any() and (~full).any() and tiles["nj"].max() <= dim and tiles["nk"].max() <= dim
            seen += 1
    assert seen > 0


def test_partial_transposed_full_size_properties(gpu_device):
    """16 bf16 [8192, 8192] Partial tensors whose four members are ``.t()`` views: the target shard equals the fp32
    rank-order sum of the members, recomputed with torch device ops, rounded once (0 ulp); members unchanged."""
    specs, targets, bucket = workloads.partial4_transposed_to_shard2()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets)
    sums = [{r: t.view(torch.int16).sum(dtype=torch.int64).item() for r, t in d.items()} for d in job.source_locals[:2]]
    job.run(merge_launches=True)
    for i in range(len(specs)):
        acc = job.source_locals[i][0].float()
        for r in (1, 2, 3):
            acc = acc + job.source_locals[i][r].float()
        want = acc.to(torch.bfloat16)[:4096]
        assert torch.equal(job.target_locals[i][4].view(torch.int16), want.contiguous().view(torch.int16)), f"tensor {i}"
    for i, d in enumerate(job.source_locals[:2]):
        for r, t in d.items():
            assert not t.is_contiguous() and t.view(torch.int16).sum(dtype=torch.int64).item() == sums[i][r], "member mutated"
    info = job.wire.plan(job.send_buckets[0]).send_table.info()
    assert info.n_trans_tiles > 0 and info.n_row_tiles == 0


@pytest.mark.parametrize("src_dt,tgt_dt", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32),
                                           (torch.float16, torch.float64), (torch.float64, torch.float16),
                                           (torch.float16, torch.bfloat16)],
                         ids=lambda d: str(d).replace("torch.", ""))
def test_short_and_ragged_converting_rows_use_narrow_vectors(gpu_device, src_dt, tgt_dt):
    """Converting rows that are not whole vectors: the remainder of a row (and rows shorter than one vector) move in
    vectors of 4 and 2 elements before single elements are used.  Every row length from 1 to 23 elements, rows at
    element-aligned pitches, against torch's cast of the same slice."""
    from etha_amd.comm.device_plan import fill_region

    dev = gpu_device
    g = torch.Generator(device=dev).manual_seed(3)
    pairs, keep = [], []
    for run in range(1, 24):
        s = (torch.randn(301, run + 3, generator=g, device=dev, dtype=torch.float32) * 50).to(src_dt)
        d = torch.full((301, run + 5), 7.0, device=dev, dtype=tgt_dt)
        pairs.append((s, (slice(0, 301), slice(1, 1 + run)), d, (slice(0, 301), slice(2, 2 + run))))
    src = np.zeros(len(pairs), dtype=_native.CHUNK_DESC)
    dst = np.zeros(len(pairs), dtype=_native.CHUNK_DESC)
    for i, (s, ss, d, ds) in enumerate(pairs):
        a, b = np.zeros((), dtype=_native.CHUNK_DESC), np.zeros((), dtype=_native.CHUNK_DESC)
        fill_region(a, s, ss, tuple(s[ss].shape))
        fill_region(b, d, ds, tuple(s[ss].shape))
        a["wire_dtype"], b["wire_dtype"] = a["tensor_dtype"], b["tensor_dtype"]
        src[i], dst[i] = a, b
    table = _native.Table.create_selfcopy(src, dst)
    _, rows = table.tiles()
    elems = (rows["meta"] >> 22) & 3
    full = 16 // max(src_dt.itemsize, tgt_dt.itemsize) if min(src_dt.itemsize, tgt_dt.itemsize) * 2 < max(src_dt.itemsize, tgt_dt.itemsize) else None
    assert set(np.unique(elems)) >= {0, 1}  # single elements and pairs at least; wider ones where the pair allows
    table.selfcopy(0, len(pairs), torch.cuda.current_stream(dev).cuda_stream)
    torch.cuda.synchronize()
    for s, ss, d, ds in pairs:
        assert torch.equal(bits(d[ds]), bits(s[ss].to(tgt_dt))), f"row length {s[ss].shape[1]}"
        outside = torch.ones_like(d, dtype=torch.bool)
        outside[ds] = False
        assert bool((d[outside] == 7.0).all())


def test_transposed_parents_full_size_properties(gpu_device):
    """16 bf16 [8192, 8192] weights handed over as ``.t()`` views: every target shard equals its slice of the
    global tensor, the (non-contiguous) sources are unchanged."""
    specs, targets, bucket = workloads.transposed_parents()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets, keep_globals=True)
    assert job.payload_bytes() == 16 * 8192 * 4096 * 2
    sums = [{r: t.view(torch.int16).sum(dtype=torch.int64).item() for r, t in d.items()} for d in job.source_locals]
    job.run(merge_launches=True)
    _check_targets_against_global(job, specs)
    for i, d in enumerate(job.source_locals):
        for r, t in d.items():
            assert t.view(torch.int16).sum(dtype=torch.int64).item() == sums[i][r], "source mutated"


def test_transposed_parents_fp32_to_bf16_full_size_properties(gpu_device):
    """16 fp32 [8192, 8192] weights handed over as ``.t()`` views, bf16 targets: every target shard is the RNE bf16 cast
    of its slice of the fp32 global tensor (torch's device cast is the independent check); all chunks go through the
    converting transposing blocks."""
    specs, targets, bucket = workloads.transposed_parents_fp32_to_bf16()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets, keep_globals=True)
    assert job.payload_bytes() == 16 * 8192 * 4096 * 2
    for b in job.send_buckets.values():
        info = job.wire.plan(b).send_table.info()
        assert info.n_trans_tiles > 0 and info.n_row_tiles == 0 and info.n_run_tiles == 0
    job.run(merge_launches=True)
    _check_targets_against_global(job, specs, cast=torch.bfloat16)


@pytest.mark.parametrize("piece_bytes", [32, 96, 1024])
def test_scatter_of_short_pieces_workload(gpu_device, piece_bytes):
    """The short-piece scatter workload scaled down (four column blocks from four ranks into one replicated target),
    merged launches so that the write-ordered range with its gather tiles runs, against the oracle."""
    specs, targets, _ = workloads.scatter_32_byte_pieces(piece_bytes=piece_bytes, total_bytes=3 << 20)
    for s in specs:
        s.dist = "bits"
    for _ in range(2):  # the second transfer runs the write-ordered copy made during the first
        gpu_vs_oracle(specs, gpu_device, 256 * 1024, target_ranks=targets, merge_launches=True)


def test_moe_row_parallel_w2(gpu_device):
    """The expert layout's second reading - w2 [E, H, I] row-parallel, Shard(0)@8 -> Shard(2)@4 (rows of I/4
    elements at a pitch of I) - scaled down against the oracle, then at full size through the closed form."""
    specs, _, _ = workloads.moe_experts_row_parallel_w2(n_experts=8, hidden=64, inter=224)
    gpu_vs_oracle(specs, gpu_device, 32 * 1024, target_ranks=[0, 1, 2, 3])
    specs, _, bucket = workloads.moe_experts_row_parallel_w2()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=[0, 1, 2, 3], keep_globals=True)
    job.run(merge_launches=True)
    _check_targets_against_global(job, specs)
    w2 = [c for b in job.recv_buckets[1] for c in b.chunks if c.tensor is job.target_locals[2][1]]
    assert w2 and all(c.chunk_shape == (1, 4096, 3584) for c in w2)  # 7168-byte rows


def test_per_bucket_launches_on_side_streams(gpu_device):
    """Fan-out over side streams (fork/join with events) gives the same bytes as one stream."""
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=3, hidden=256, inter=896, kv=64, vocab=2056)
    gpu_job = ReshardJob(specs, device=gpu_device, bucket_size=32 * 1024, target_ranks=targets, keep_globals=True, fill=cpu_fill,
                         pool="resident")  # side streams run a list in list order: every bucket needs its own slot
    cpu_job = ReshardJob(specs, device="cpu", bucket_size=32 * 1024, target_ranks=targets, keep_globals=True, fill=cpu_fill)
    run_oracle(cpu_job)
    with pytest.raises(ValueError, match="resident pool"):
        ReshardJob(specs, device=gpu_device, bucket_size=32 * 1024, target_ranks=targets).run(fanout=2)
    for fanout in (3, 1, 4):
        for d in gpu_job.target_locals:
            for t in d.values():
                t.zero_()
        gpu_job.run(merge_launches=False, fanout=fanout)
        for i, spec in enumerate(specs):
            for r, t in gpu_job.target_locals[i].items():
                assert_bit_equal(t, cpu_job.target_locals[i][r], f"{spec.name} rank {r} fanout {fanout}")


def test_skewed_buckets_large(gpu_device):
    """An odd-sized first chunk skews every later chunk of its bucket; long runs then move as 16-byte
    units with an unaligned tensor-side access.  Both directions, contiguous and strided rows."""
    one = (mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),))
    specs = [
        TensorSpec("odd", (7,), *one, torch.bfloat16, seed=1, dist="bits"),            # 14 bytes
        TensorSpec("big", (1 << 20,), *one, torch.bfloat16, seed=2, dist="bits"),       # skew 14
        TensorSpec("rows", (300, 1000), mesh_of(0, [1]), (Replicate(),), mesh_of(1, [2]), (Shard(1),), torch.bfloat16,
                   seed=3, dist="bits"),                                               # 1000-byte strided rows
    ]
    job, _ = gpu_vs_oracle(specs, gpu_device, 1 << 30)
    specs32 = [
        TensorSpec("odd", (3,), *one, torch.float32, seed=5, dist="bits"),             # 12 bytes: dword-aligned skew
        TensorSpec("f32", (257, 513), *one, torch.float32, seed=4, dist="bits"),
    ]
    gpu_vs_oracle(specs32, gpu_device, 1 << 30)
    plan = job.wire.plan(job.send_buckets[0])
    run, _ = plan.send_table.tiles()
    assert ((run["meta"] & (1 << 18)) != 0).sum() > 0  # the skew path was really taken


@pytest.mark.parametrize("src_dt,tgt_dt,cols", [
    (torch.float32, torch.bfloat16, 1000),   # full vectors at a 4-byte-aligned fp32 pitch
    (torch.float32, torch.bfloat16, 1003),   # vector body + 3-element remainder
    (torch.bfloat16, torch.float16, 91),     # 8-element vectors + remainder, odd pitch
    (torch.float64, torch.float32, 77),
    (torch.bfloat16, torch.bfloat16, 12),    # 24-byte rows: 8-byte units at 2-byte-aligned addresses
    (torch.int8, torch.int8, 6),             # 6-byte rows at odd addresses
    (torch.bfloat16, torch.bfloat16, 257),   # 514-byte rows: unaligned body + 2-byte remainder
])
def test_rows_at_element_aligned_pitch(gpu_device, src_dt, tgt_dt, cols):
    """Source and target shards live inside parents whose row pitch is one element longer than the row,
    so row starts are only element-aligned: vector units must still be used and still be exact."""
    def padded(kind, t):
        if t.dim() != 2:
            return t
        parent = torch.zeros(t.shape[0], t.shape[1] + 1, dtype=t.dtype, device=t.device)
        return parent[:, : t.shape[1]]

    one = (mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),))
    specs = [TensorSpec("lead", (5,), *one, src_dt, tgt_dt, seed=1, std=1.0),
             TensorSpec("rows", (300, cols), *one, src_dt, tgt_dt, seed=2, std=1.0)]
    gpu_job = ReshardJob(clone_specs(specs), device=gpu_device, bucket_size=1 << 30, keep_globals=True, fill=cpu_fill,
                         local_view=padded)
    cpu_job = ReshardJob(clone_specs(specs), device="cpu", bucket_size=1 << 30, keep_globals=True, fill=cpu_fill,
                         local_view=padded)
    gpu_job.run()
    run_oracle(cpu_job)
    for i, spec in enumerate(specs):
        assert_bit_equal(gpu_job.target_locals[i][1], cpu_job.target_locals[i][1], spec.name)
        assert_bit_equal(gpu_job.target_locals[i][1], expected_target(spec, cpu_job.globals_[i], 1), spec.name + " closed form")
    # element-sized units only where the arithmetic forces them (remainders), never for whole rows
    plan = gpu_job.wire.plan(gpu_job.send_buckets[0])
    run, row = plan.send_table.tiles()
    units = sum(int(t["n"].sum()) for t in (run, row))
    assert units <= 5 + 300 * (cols // 2 + 8)


def test_bucket_protocol_methods(gpu_device):
    """prepare / launch / is_complete / finalize on single buckets, as the reference's bucket_comm drives them."""
    from etha_amd.comm import get_m2m_map, m2m_to_chunks

    wire = LoopbackWire(gpu_device)
    g = torch.arange(64 * 32, dtype=torch.float32).reshape(64, 32)
    src = {r: g[32 * r : 32 * (r + 1)].clone().to(gpu_device) for r in range(2)}
    tgt = {2 + j: torch.zeros(64, 16, device=gpu_device) for j in range(2)}
    m = get_m2m_map([0, 1], (Shard(0),), [2, 3], (Shard(1),))
    send = {r: chunk_to_bucket_ops(m2m_to_chunks(m, r, source_tensor=src[r]), 1 << 20) for r in src}
    recv = {r: chunk_to_bucket_ops(m2m_to_chunks(m, r, target_tensor=tgt[r]), 1 << 20) for r in tgt}
    for buckets in send.values():
        for b in buckets:
            b.prepare(wire)
            assert b.launch()
            assert not b.is_complete(wire)  # packed into its ring slot, not yet unpacked by its destination
    for buckets in recv.values():
        for b in buckets:
            b.prepare(wire)
            assert b.launch() and b.is_complete(wire)
            b.finalize(wire)
            assert not b.is_complete(wire)  # consumed: the next transfer's bytes have not arrived
            with pytest.raises(RuntimeError, match="before its send bucket was packed"):
                b.finalize(wire)
    for buckets in send.values():
        for b in buckets:
            assert b.is_complete(wire)
            b.finalize(wire)  # nothing to write on the source side
    torch.cuda.synchronize()
    for j in range(2):
        assert torch.equal(tgt[2 + j].cpu(), g[:, 16 * j : 16 * (j + 1)])


@pytest.mark.parametrize("pool", ["ring", "resident"])
def test_hip_graph_replay_matches_eager(gpu_device, pool):
    """A captured transfer replays correctly, several times, with new source values each time.  (Under capture
    the wire issues every launch in order: a captured stream is a chain anyway.)"""
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=2, hidden=256, inter=896, kv=64, vocab=2056)
    job = ReshardJob(specs, device=gpu_device, bucket_size=64 * 1024, target_ranks=targets, pool=pool)
    job.run(merge_launches=True)  # plans, uploads
    graph = job.capture(merge_launches=True)
    for round_ in range(3):
        for i, d in enumerate(job.source_locals):
            for r, t in d.items():
                t.copy_(torch.full_like(t, float(round_ + 1)) + i)  # eager work between replays
        for d in job.target_locals:
            for t in d.values():
                t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, d in enumerate(job.target_locals):
            for r, t in d.items():
                assert bool((t == float(round_ + 1) + i).all()), f"replay {round_}, tensor {i}"


def test_single_chunk_beyond_4gib(gpu_device):
    """64-bit addressing: one 5 GiB chunk; compare a strided sample and the tails with the source."""
    n = 5 * (1 << 30) + 48
    spec = TensorSpec("huge", (n,), mesh_of(0, [1]), (Replicate(),), mesh_of(1, [1]), (Replicate(),), torch.uint8, seed=1)

    def fill(spec):
        x = torch.empty(n, dtype=torch.uint8, device=gpu_device)
        x.view(torch.int64)[: n // 8] = torch.arange(n // 8, device=gpu_device, dtype=torch.int64) * 2654435761
        x[-48:] = 7
        return x

    job = ReshardJob([spec], device=gpu_device, bucket_size=1 << 20, fill=fill)
    job.run()
    src, dst = job.source_locals[0][0], job.target_locals[0][1]
    for lo in (0, (1 << 32) - 4096, (1 << 32), n - 8192):
        assert torch.equal(src[lo : lo + 8192], dst[lo : lo + 8192]), f"window at {lo}"
    assert torch.equal(src[:: 4099], dst[:: 4099])
    assert int(dst.view(torch.int64)[: n // 8].sum()) == int(src.view(torch.int64)[: n // 8].sum())


def test_equal_width_dtypes_convert_instead_of_reinterpreting(gpu_device):
    """fp16 source, bf16 target: the wire carries the source's dtype and the unpack converts."""
    spec = TensorSpec("w", (64, 96), mesh_of(0, [2]), (Shard(0),), mesh_of(2, [3]), (Shard(1),), torch.float16, torch.bfloat16,
                      seed=4, std=1.0)
    job, cpu_job = gpu_vs_oracle([spec], gpu_device, 4096)
    assert job.recv_buckets[2][0].chunks[0].transfer_dtype == torch.float16
    want = cpu_job.globals_[0][:, :32].to(torch.bfloat16)
    assert torch.equal(job.target_locals[0][2].cpu(), want)


@pytest.mark.parametrize("seed", range(60))
def test_random_batches_gpu(gpu_device, seed):
    """Random meshes / placements / shapes / dtypes / strides / bucket sizes on the GPU, against the oracle."""
    from test_random_layouts_cpu import _random_spec, _uneven_spec

    rng = np.random.default_rng(10_000 + seed)
    wire_size = int(rng.choice([1, 2, 2, 4, 4, 8]))
    spec_fn = _uneven_spec if seed % 4 == 3 else _random_spec  # every fourth batch: uneven shards, rank up to 5
    specs = [spec_fn(rng, i, wire_size) for i in range(int(rng.integers(1, 5)))]
    bucket_size = [None, 64, 4096, 1 << 20][int(rng.integers(4))]
    view = None
    if rng.random() < 0.35:
        def view(kind, t):
            if t.dim() == 0 or t.numel() == 0:
                return t
            shape = list(t.shape)
            shape[-1] = shape[-1] * 2 + 3
            wide = torch.zeros(shape, dtype=t.dtype, device=t.device)
            return wide[..., 1 : 1 + t.shape[-1]]
    merge = bool(rng.integers(2))
    mode = ["buckets", "buckets", "zero_copy", "direct"][int(rng.integers(4))]  # wire options must not change results
    fanout = 3 if seed % 5 == 4 else 1  # every fifth batch: launches spread over side streams (needs a slot per bucket)
    pool = "resident" if fanout > 1 or seed % 5 == 3 else "ring"
    depth = int(rng.integers(1, 4))
    gpu_job = ReshardJob(specs, device=gpu_device, bucket_size=bucket_size, keep_globals=True, fill=cpu_fill, local_view=view,
                         zero_copy=mode == "zero_copy", direct=mode == "direct", pool=pool, max_in_flight=depth)
    cpu_job = ReshardJob(specs, device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill, local_view=view)
    mirror_partials(gpu_job, cpu_job)
    for transfer in range(2):  # the second transfer, on new values, is served from the wire's recording of the first (ring pool)
        if transfer:
            next_values(gpu_job, cpu_job, transfer)
        gpu_job.run(merge_launches=merge, fanout=fanout)
        run_oracle(cpu_job)
        for i, spec in enumerate(specs):
            for r, t in gpu_job.target_locals[i].items():
                assert_bit_equal(t, cpu_job.target_locals[i][r],
                                 f"seed {seed} ({mode}, {pool} pool, fanout {fanout}) transfer {transfer} {spec.name} rank {r}")


@pytest.mark.parametrize("dtype", [torch.int8, torch.bfloat16, torch.float32, torch.float64])
def test_transposed_parents_go_through_lds(gpu_device, dtype):
    """Source and target shards that are transposes of their storage ([R, C] views of [C, R] tensors)."""
    def transposed(kind, t):
        if t.dim() != 2:
            return t
        return torch.zeros(t.shape[1], t.shape[0], dtype=t.dtype, device=t.device).t()

    spec = TensorSpec("w", (260, 330), mesh_of(0, [2]), (Shard(0),), mesh_of(2, [3]), (Shard(1),), dtype, seed=21, dist="bits")
    gpu_job = ReshardJob([spec], device=gpu_device, bucket_size=1 << 20, keep_globals=True, fill=cpu_fill, local_view=transposed)
    cpu_job = ReshardJob([spec], device="cpu", bucket_size=1 << 20, keep_globals=True, fill=cpu_fill, local_view=transposed)
    assert not gpu_job.source_locals[0][0].is_contiguous()
    gpu_job.run()
    run_oracle(cpu_job)
    for r, t in gpu_job.target_locals[0].items():
        assert_bit_equal(t, cpu_job.target_locals[0][r], f"rank {r}")
        assert_bit_equal(t, expected_target(spec, cpu_job.globals_[0], r), f"rank {r} closed form")
    assert gpu_job.wire.plan(gpu_job.send_buckets[0]).send_table.info().n_trans_tiles > 0
    assert gpu_job.wire.plan(gpu_job.recv_buckets[2]).recv_table.info().n_trans_tiles > 0


def test_zero_copy_single_chunk_buckets(gpu_device):
    """With the wire's zero-copy option, contiguous single-chunk buckets are lent: no pack launch, the
    consumer unpacks straight from the source shard; everything else is packed as usual."""
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=2, hidden=256, inter=896, kv=64, vocab=2056)
    gpu_job = ReshardJob(specs, device=gpu_device, bucket_size=64 * 1024, target_ranks=targets, keep_globals=True,
                         fill=cpu_fill, zero_copy=True)
    cpu_job = ReshardJob(specs, device="cpu", bucket_size=64 * 1024, target_ranks=targets, keep_globals=True, fill=cpu_fill)
    gpu_job.run(merge_launches=True)
    run_oracle(cpu_job)
    plans = [gpu_job.wire.plan(b) for b in gpu_job.send_buckets.values()]
    lent = sum(len(p.lent) for p in plans)
    packed = sum(1 for p in plans for s in p.steps if s[0] == "pack")
    assert lent > 0 and packed > 0  # the big embedding / projection chunks are lent, bundled ones are packed
    for i, spec in enumerate(specs):
        for r, t in gpu_job.target_locals[i].items():
            assert_bit_equal(t, cpu_job.target_locals[i][r], f"{spec.name} rank {r}")
    # a second transfer with new values: lent buckets must deliver the new bytes too
    for d in gpu_job.source_locals:
        for t in d.values():
            t.mul_(-1.0)
    gpu_job.run(merge_launches=False)
    for i, spec in enumerate(specs):
        for r, t in gpu_job.target_locals[i].items():
            assert_bit_equal(t, -cpu_job.target_locals[i][r], f"{spec.name} rank {r}, second transfer")
    for p in plans:
        gpu_job.wire.release(p.buckets)  # lent slots are not pool memory and must not enter its free list
    assert all(not s.borrowed for free in gpu_job.wire.pool._free.values() for s in free)


def test_direct_same_device_wire(gpu_device):
    """With the direct wire no plain bucket is packed: the target bucket's launch copies from the producer's
    regions in one pass - for a Partial source it reduces every member's region.  Same results as the bucket
    path for P2P, BROADCAST, LOCAL, converting, strided and Partial layouts; no pool memory."""
    src = mesh_of(0, (2, 2))
    specs = [
        TensorSpec("a", (64, 48), src, (Shard(0), Shard(1)), mesh_of(4, (2,)), (Replicate(),), torch.float32, seed=1),
        TensorSpec("b", (32, 40), src, (Shard(1), Shard(0)), mesh_of(1, (4,)), (Shard(0),), torch.float32, seed=2),
        TensorSpec("c", (24, 16), src, (Replicate(), Shard(0)), mesh_of(4, (2,)), (Replicate(),), torch.float32,
                   torch.bfloat16, seed=3),
        TensorSpec("d", (8, 128), src, (Shard(0), Shard(1)), mesh_of(4, (2, 2)), (Shard(1), Replicate()),
                   torch.bfloat16, torch.float32, seed=4),
        TensorSpec("p", (64, 32), mesh_of(0, (4,)), (Partial(),), mesh_of(4, (2,)), (Shard(0),), torch.bfloat16, seed=5),
        # bf16 partials into an fp32 target: the sum is still rounded to the bf16 wire dtype before widening
        TensorSpec("pw", (48, 20), mesh_of(0, (4,)), (Partial("avg"),), mesh_of(4, (2,)), (Shard(1),), torch.bfloat16,
                   torch.float32, seed=6),
        TensorSpec("pn", (16, 24), mesh_of(0, (2, 2)), (Partial(), Shard(0)), mesh_of(4, (2,)), (Replicate(),), torch.float32,
                   torch.bfloat16, seed=7),
    ]
    for bucket_size in (1, 4096, 1 << 20):
        for merge in (False, True):
            gpu_job = ReshardJob(clone_specs(specs), device=gpu_device, bucket_size=bucket_size, keep_globals=True,
                                 fill=cpu_fill, direct=True)
            cpu_job = ReshardJob(clone_specs(specs), device="cpu", bucket_size=bucket_size, keep_globals=True, fill=cpu_fill)
            mirror_partials(gpu_job, cpu_job)
            before = [{r: t.clone() for r, t in d.items()} for d in gpu_job.source_locals]
            gpu_job.run(merge_launches=merge)
            gpu_job.run(merge_launches=merge)  # plan once, transfer twice
            run_oracle(cpu_job)
            for i, spec in enumerate(specs):
                for r, t in gpu_job.target_locals[i].items():
                    assert_bit_equal(t, cpu_job.target_locals[i][r], f"{spec.name} rank {r} bucket {bucket_size} merge {merge}")
                for r, t in gpu_job.source_locals[i].items():
                    if not any(t is x for x in gpu_job.target_locals[i].values()):
                        assert_bit_equal(t, before[i][r], f"{spec.name} source {r} mutated")
            kinds = {s[0] for bs in list(gpu_job.send_buckets.values()) + list(gpu_job.recv_buckets.values())
                     for s in gpu_job.wire.plan(bs).steps}
            assert {"direct", "direct_reduce", "lend"} <= kinds
            assert not kinds & {"pack", "reduce_pack", "unpack"}  # (staged self-copies would pack; this layout has none)
            assert gpu_job.wire.pool is None or gpu_job.wire.pool.reserved_bytes == 0
    with pytest.raises(NotImplementedError):
        gpu_job.wire.export_manifest()


def test_direct_wire_full_size_llama(gpu_device):
    specs, targets, bucket = workloads.llama3_8b_fsdp8_to_tp2()
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets, keep_globals=True, direct=True)
    job.run(merge_launches=True)
    _check_targets_against_global(job, specs)
    assert job.wire.pool is None or job.wire.pool.reserved_bytes == 0


def test_direct_table_launch_refuses_mixed_ranges(gpu_device):
    """A launched range of a direct table is all plain or all Partial chunks (they run in different kernels)."""
    from etha_amd._native import EthaNativeError

    one = (mesh_of(0, (2,)), mesh_of(2, (1,)))
    specs = [TensorSpec("a", (8, 16), one[0], (Shard(0),), one[1], (Replicate(),), torch.float32, seed=1),
             TensorSpec("p", (8, 16), one[0], (Partial(),), one[1], (Replicate(),), torch.float32, seed=2)]
    job = ReshardJob(specs, device=gpu_device, bucket_size=1, direct=True)
    job.run()
    plan = job.wire.plan(job.recv_buckets[2])
    kinds = [s[0] for s in plan.steps]
    assert "direct" in kinds and "direct_reduce" in kinds
    total = sum(s[2] for s in plan.steps)
    with pytest.raises(EthaNativeError, match="mixes Partial and plain"):
        plan.local_table.selfcopy(0, total)


def test_large_resident_set_70b_shapes(gpu_device):
    """Llama-3-70B shapes, 40 layers: 70 GB of source shards resident, a 36 GB share through 37 pool segments.
    Every checked target shard equals its slice of the reassembled source (sizes well past 32-bit offsets)."""
    free, _ = torch.cuda.mem_get_info(gpu_device)
    if free < 180 << 30:
        pytest.skip("needs about 150 GB of free device memory")
    specs, targets, bucket = workloads.llama3_8b_fsdp8_to_tp2(n_layers=40, hidden=8192, inter=28672, kv=1024, vocab=128256)
    job = ReshardJob(specs, device=gpu_device, bucket_size=bucket, target_ranks=targets)
    assert job.payload_bytes() == 36_328_177_664
    job.run(merge_launches=True)
    from oracle.dtensor_layout import local_shard

    for i, spec in enumerate(specs):
        if i % 9 not in (0, 5) and i != len(specs) - 1:  # embeddings, o_proj / down_proj of every layer, lm_head
            continue
        glob = torch.cat([job.source_locals[i][r] for r in range(8)], dim=0)
        want = local_shard(glob, (2,), spec.target_placements, (0,))
        assert torch.equal(job.target_locals[i][8].view(torch.int16), want.contiguous().view(torch.int16)), spec.name
        del glob, want
    del job
    torch.cuda.empty_cache()  # hand the 150 GB back before the multi-process tests start


@pytest.mark.gpu
@pytest.mark.parametrize("pool", ["ring", "resident"])
@pytest.mark.parametrize("cols,src_dtype,tgt_dtype", [(64, torch.bfloat16, None), (32, torch.bfloat16, None),
                                                      (48, torch.float32, torch.bfloat16), (32, torch.bfloat16, torch.float32),
                                                      (320, torch.bfloat16, None), (192, torch.bfloat16, None)])
def test_short_pieces_from_several_ranks_are_gathered_per_row(gpu_device, pool, cols, src_dtype, tgt_dtype):
    """Every target row is four short pieces from four source ranks' buckets.  Merged unpack launches run from the
    write-ordered copy of their range, where such pieces are assembled row by row by gather tiles."""
    from etha_amd.comm.comm_methods import _UNPACK

    specs = [TensorSpec(f"t{i}", (2048 + 512 * i, cols), [[0, 1, 2, 3]], (Replicate(), Shard(1)), [4], (Replicate(),),
                        src_dtype, tgt_dtype, seed=40 + i, std=1.0) for i in range(3)]
    job, _ = gpu_vs_oracle(specs, gpu_device, 256 * 1024, merge_launches=True, pool=pool)
    job.run(merge_launches=True)  # the schedule repeats: by now every recurring merged range has its ordered copy
    plan = job.wire.plan(job.recv_buckets[4])
    ranges = plan._ordered_ranges if pool == "ring" else {(k, f, c) for k, f, c, s in plan.merged_steps if len(s) > 1}
    gathered = sum(len(plan.recv_table.ordered_gather(f, c)) for k, f, c in ranges if k == _UNPACK)
    assert gathered > 0
    for i, spec in enumerate(specs):
        want = expected_target(spec, job.globals_[i].cpu(), 4)
        assert_bit_equal(job.target_locals[i][4], want, spec.name)
