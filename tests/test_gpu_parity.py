"""GPU parity: the HIP path (through the C ABI) against the CPU oracle, bit for bit."""

import pytest
import torch
from torch.distributed.tensor.placement_types import Replicate, Shard

from etha_amd.world import TensorSpec

from helpers import gpu_vs_oracle

pytestmark = pytest.mark.gpu


def test_config1_fp32_shard0_to_shard1(gpu_device):
    """fp32 [1024,1024] uniform(-1,1) seed 0; (2,) Shard(0) -> (4,) Shard(1); full reassembly."""
    spec = TensorSpec("w", (1024, 1024), [0, 1], (Shard(0),), [2, 3, 4, 5], (Shard(1),), torch.float32,
                      seed=0, dist="uniform")
    for bucket_size in (None, 256 * 1024, 64 << 20):
        gpu_vs_oracle([spec], gpu_device, bucket_size)


@pytest.mark.parametrize("merge", [False, True])
def test_small_llama_like_fsdp_to_tp(gpu_device, merge):
    """Column-parallel, row-parallel and replicated norm tensors, FSDP@8 -> TP@2, one TP rank's share."""
    src = list(range(8))
    tgt = [8, 9]
    specs = []
    for layer in range(2):
        s = layer * 10
        specs += [
            TensorSpec(f"l{layer}.q", (256, 128), src, (Shard(0),), tgt, (Shard(0),), seed=s + 1),
            TensorSpec(f"l{layer}.o", (128, 256), src, (Shard(0),), tgt, (Shard(1),), seed=s + 2),
            TensorSpec(f"l{layer}.down", (128, 448), src, (Shard(0),), tgt, (Shard(1),), seed=s + 3),
            TensorSpec(f"l{layer}.norm", (128,), src, (Shard(0),), tgt, (Replicate(),), seed=s + 4),
        ]
    gpu_vs_oracle(specs, gpu_device, 16 * 1024, target_ranks=[8], merge_launches=merge)
    gpu_vs_oracle(specs, gpu_device, 16 * 1024, target_ranks=None, merge_launches=merge)
