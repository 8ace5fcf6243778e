"""Synthetic workloads: the layouts and shapes the headline numbers are quoted on.

Each builder returns ``(specs, target_ranks, bucket_size)`` for :class:`etha_amd.world.ReshardJob`.
Source ranks are numbered from 0; target ranks follow the source ranks unless a workload says
otherwise (overlapping rank sets are what creates same-rank LOCAL chunks).
"""

from __future__ import annotations

import numpy as np
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from .world import TensorSpec

MIB = 1 << 20


def _mesh(start: int, shape) -> list:
    n = int(np.prod(shape))
    return np.arange(start, start + n).reshape(shape).tolist()


def single_fp32_shard0_to_shard1():
    """fp32 [1024,1024] uniform(-1,1) seed 0; mesh (2,) Shard(0) -> mesh (4,) Shard(1)."""
    spec = TensorSpec("w", (1024, 1024), _mesh(0, (2,)), (Shard(0),), _mesh(2, (4,)), (Shard(1),),
                      torch.float32, seed=0, dist="uniform")
    return [spec], None, None


def llama3_8b_fsdp8_to_tp2(n_layers: int = 32, with_embeddings: bool = True, dtype=torch.bfloat16,
                           hidden: int = 4096, inter: int = 14336, kv: int = 1024, vocab: int = 128256,
                           target_dtype=None):
    """Llama-3-8B weight set, FSDP Shard(0) over 8 ranks -> TP=2; one TP rank's share.

    Column-parallel (q/k/v/gate/up/embed/lm_head): Shard(0) -> Shard(0).  Row-parallel (o/down):
    Shard(0) -> Shard(1).  RMSNorm weights: Shard(0) -> Replicate.  Values normal(0, 0.02), seed =
    tensor index.  290 tensors at the full size.
    """
    src, tgt = _mesh(0, (8,)), _mesh(8, (2,))
    col, row, rep = (Shard(0),), (Shard(1),), (Replicate(),)
    specs: list[TensorSpec] = []

    def add(name, shape, tgt_pl):
        specs.append(TensorSpec(name, shape, src, (Shard(0),), tgt, tgt_pl, dtype, target_dtype, seed=len(specs)))

    if with_embeddings:
        add("embed_tokens", (vocab, hidden), col)
    for i in range(n_layers):
        add(f"layers.{i}.input_layernorm", (hidden,), rep)
        add(f"layers.{i}.q_proj", (hidden, hidden), col)
        add(f"layers.{i}.k_proj", (kv, hidden), col)
        add(f"layers.{i}.v_proj", (kv, hidden), col)
        add(f"layers.{i}.o_proj", (hidden, hidden), row)
        add(f"layers.{i}.post_attention_layernorm", (hidden,), rep)
        add(f"layers.{i}.gate_proj", (inter, hidden), col)
        add(f"layers.{i}.up_proj", (inter, hidden), col)
        add(f"layers.{i}.down_proj", (hidden, inter), row)
    if with_embeddings:
        add("lm_head", (vocab, hidden), col)
    return specs, [8], 64 * MIB


def many_small_2d_to_replicate(n_tensors: int = 256, rows: int = 2048, k_seed: int = 1234, dtype=torch.bfloat16):
    """256 bf16 [2048, k], k uniform over {64, 128, ..., 4096} (numpy RandomState(1234));
    mesh (2,4) (Shard(0), Shard(1)) -> mesh (4,) Replicate; one target rank; 64 MiB buckets."""
    ks = np.random.RandomState(k_seed).randint(1, 65, size=n_tensors) * 64
    src, tgt = _mesh(0, (2, 4)), _mesh(8, (4,))
    specs = [
        TensorSpec(f"t{i}", (rows, int(k)), src, (Shard(0), Shard(1)), tgt, (Replicate(),), dtype, seed=i)
        for i, k in enumerate(ks)
    ]
    return specs, [8], 64 * MIB


def scatter_32_byte_pieces(piece_bytes: int = 32, total_bytes: int = 1 << 29, dtype=torch.bfloat16):
    """One [rows, 4 * piece] tensor whose four column blocks sit on four source ranks (mesh (1,4), Shard(1)) and
    are scattered into one replicated target: every target row is four pieces of ``piece_bytes`` from four
    buckets, 0.5 GiB in all - the shortest rows of ``many_small_2d_to_replicate`` on their own."""
    es = torch.empty((), dtype=dtype).element_size()
    cols = piece_bytes // es * 4
    rows = total_bytes // (piece_bytes * 4)
    src, tgt = _mesh(0, (1, 4)), _mesh(4, (1,))
    return [TensorSpec("t", (rows, cols), src, (Replicate(), Shard(1)), tgt, (Replicate(),), dtype, seed=1)], [4], 64 * MIB


def scatter_96_byte_pieces():
    return scatter_32_byte_pieces(piece_bytes=96)


def scatter_480_byte_pieces():
    return scatter_32_byte_pieces(piece_bytes=480)


def scatter_2048_byte_pieces():
    """Whole 128-byte lines per piece: the same scatter without partial lines, for comparison."""
    return scatter_32_byte_pieces(piece_bytes=2048)


def partial4_to_shard2(n_tensors: int = 16, n: int = 8192, dtype=torch.bfloat16):
    """16 bf16 [8192,8192], mesh (4,) Partial(sum) -> mesh (2,) Shard(0); one target rank.
    Partial of source rank r of tensor i: normal(0, 0.02) with seed 4*i + r."""
    src, tgt = _mesh(0, (4,)), _mesh(4, (2,))
    specs = [
        TensorSpec(f"p{i}", (n, n), src, (Partial("sum"),), tgt, (Shard(0),), dtype, seed=4 * i)
        for i in range(n_tensors)
    ]
    return specs, [4], 64 * MIB


def partial4_transposed_to_shard2(n_tensors: int = 16, n: int = 8192, dtype=torch.bfloat16):
    """``partial4_to_shard2`` with every member's partial stored as a ``.t()`` view (kept [in, out], handed over as
    [out, in]): the Partial collapse runs in the typed transposing kernel, which combines the four members' blocks
    in registers before they are parked in LDS."""
    specs, targets, bucket = partial4_to_shard2(n_tensors, n, dtype)
    for s in specs:
        s.source_layout = "transposed"
    return specs, targets, bucket


def moe_experts_and_uneven_vocab(n_experts: int = 8, hidden: int = 4096, inter: int = 14336, vocab: int = 151936,
                                 dtype=torch.bfloat16):
    """Mixtral-style grouped experts Shard(0)@8 -> Shard(1)@4 and a 151936-row embedding
    Shard(0)@6 (uneven tail shard) -> Shard(1)@4.  Target ranks 0..3 overlap the source ranks, so
    chunks whose source and destination rank coincide take the LOCAL (self-copy) path."""
    specs = [
        TensorSpec("experts.w1", (n_experts, inter, hidden), _mesh(0, (8,)), (Shard(0),), _mesh(0, (4,)), (Shard(1),), dtype, seed=0),
        TensorSpec("experts.w3", (n_experts, inter, hidden), _mesh(0, (8,)), (Shard(0),), _mesh(0, (4,)), (Shard(1),), dtype, seed=1),
        TensorSpec("experts.w2", (n_experts, hidden, inter), _mesh(0, (8,)), (Shard(0),), _mesh(0, (4,)), (Shard(1),), dtype, seed=2),
        TensorSpec("embed_tokens", (vocab, hidden), _mesh(0, (6,)), (Shard(0),), _mesh(0, (4,)), (Shard(1),), dtype, seed=3),
    ]
    return specs, [0], 64 * MIB


def moe_experts_row_parallel_w2(n_experts: int = 8, hidden: int = 4096, inter: int = 14336, dtype=torch.bfloat16):
    """The second reading of the expert layout: ``w2`` [E, H, I] as a true row-parallel weight, expert
    Shard(0)@8 -> TP=4 Shard(2): every target rank takes I/4 = 3584 columns, i.e. rows of 7168 bytes at a
    28672-byte pitch inside each source expert (w1/w3 stay column-parallel, Shard(1))."""
    src, tgt = _mesh(0, (8,)), _mesh(0, (4,))
    specs = [
        TensorSpec("experts.w1", (n_experts, inter, hidden), src, (Shard(0),), tgt, (Shard(1),), dtype, seed=0),
        TensorSpec("experts.w3", (n_experts, inter, hidden), src, (Shard(0),), tgt, (Shard(1),), dtype, seed=1),
        TensorSpec("experts.w2", (n_experts, hidden, inter), src, (Shard(0),), tgt, (Shard(2),), dtype, seed=2),
    ]
    return specs, [0], 64 * MIB


def transposed_parents(n_tensors: int = 16, n: int = 8192, dtype=torch.bfloat16, target_transposed: bool = False,
                       target_dtype=None):
    """16 bf16 [8192, 8192] weights whose source shards are ``.t()`` views (stored [in, out], handed over as
    [out, in]): mesh (4,) Shard(0) -> mesh (2,) Shard(0), one target rank.  The contiguous dim differs between
    shard and bucket, so every chunk goes through the LDS-staged transposing kernel."""
    src, tgt = _mesh(0, (4,)), _mesh(4, (2,))
    specs = [
        TensorSpec(f"w{i}", (n, n), src, (Shard(0),), tgt, (Shard(0),), dtype, target_dtype, seed=i, source_layout="transposed",
                   target_layout="transposed" if target_transposed else "contiguous")
        for i in range(n_tensors)
    ]
    return specs, [4], 64 * MIB


def transposed_parents_4096():
    """The same layout with 4096 x 4096 weights (64 tensors, same bytes): bucket rows at an 8 KiB pitch."""
    return transposed_parents(n_tensors=64, n=4096)


def transposed_parents_fp32_to_bf16():
    """The same with fp32 ``.t()`` sources and bf16 targets (master weights kept [in, out] -> serving weights): the
    transposing pack converts."""
    return transposed_parents(dtype=torch.float32, target_dtype=torch.bfloat16)


def llama3_8b_fsdp8_to_tp2_fp32_to_bf16():
    """Same layouts with fp32 source shards and bf16 target shards (trainer master weights -> serving
    weights): the wire dtype is bf16, so the pack kernel converts."""
    return llama3_8b_fsdp8_to_tp2(dtype=torch.float32, target_dtype=torch.bfloat16)


WORKLOADS = {
    "single_fp32_shard0_to_shard1": single_fp32_shard0_to_shard1,
    "llama3_8b_fsdp8_to_tp2": llama3_8b_fsdp8_to_tp2,
    "llama3_8b_fsdp8_to_tp2_fp32_to_bf16": llama3_8b_fsdp8_to_tp2_fp32_to_bf16,
    "many_small_2d_to_replicate": many_small_2d_to_replicate,
    "partial4_to_shard2": partial4_to_shard2,
    "partial4_transposed_to_shard2": partial4_transposed_to_shard2,
    "scatter_32_byte_pieces": scatter_32_byte_pieces,
    "scatter_96_byte_pieces": scatter_96_byte_pieces,
    "scatter_480_byte_pieces": scatter_480_byte_pieces,
    "scatter_2048_byte_pieces": scatter_2048_byte_pieces,
    "moe_experts_and_uneven_vocab": moe_experts_and_uneven_vocab,
    "moe_experts_row_parallel_w2": moe_experts_row_parallel_w2,
    "transposed_parents": transposed_parents,
    "transposed_parents_4096": transposed_parents_4096,
    "transposed_parents_fp32_to_bf16": transposed_parents_fp32_to_bf16,
}
