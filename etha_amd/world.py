"""All ranks of a redistribute job resident on one GPU.

The reference runs one agent process per rank and moves buckets between them with NCCL.  This
build shows the part one GPU can show: every source rank's shards and every (selected) target
rank's shards are tensors on the same device, each rank's chunk/bucket plan is built exactly as
the per-rank agents would build it (``src/etha/tensor_bus/agent.py:543-687``), and the wire is the
same-GPU loopback.  :class:`ReshardJob` is the harness the tests, the benchmark and the smoke check
share.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate

from .comm import LoopbackWire, PartialGroup, bucket_comm, chunk_to_bucket_ops, get_m2m_map, m2m_to_chunks
from .layout import local_shape, local_shard, mesh_coord


@dataclass
class TensorSpec:
    """One logical tensor and its two layouts."""

    name: str
    shape: tuple[int, ...]
    source_mesh: list  # nested list of global ranks
    source_placements: tuple
    target_mesh: list
    target_placements: tuple
    source_dtype: torch.dtype = torch.bfloat16
    target_dtype: torch.dtype | None = None  # None = source dtype
    seed: int = 0
    std: float = 0.02
    dist: str = "normal"  # "normal" | "uniform" (uniform(-1, 1))
    # storage of the local shards: "contiguous", or "transposed" - a 2-D shard is the ``.t()`` view of a
    # contiguous [cols, rows] tensor (a trainer that keeps a weight in [in, out] order hands over such views;
    # non-contiguous parents are legal, tests/test_communication_replicate_shard.py:99-113)
    source_layout: str = "contiguous"
    target_layout: str = "contiguous"


def transfer_dtype_rule(source: torch.dtype, target: torch.dtype) -> torch.dtype:
    """Wire dtype: the side with the smaller item size; on a tie the source's dtype.

    The reference lets each side pick its own dtype on a tie (``agent.py:635-640``), which makes
    two equally wide but different dtypes (fp16 vs bf16) reinterpret each other's bits; choosing the
    source's dtype on both sides turns that case into a real conversion at unpack time.
    """
    return source if source.itemsize <= target.itemsize else target


def create_partial_groups(mesh, partial_reductions, this_rank: int, tensors_by_rank: dict[int, torch.Tensor]):
    """The Partial reduction ``this_rank`` takes part in, as a one-element list of (PartialGroup, op).

    The reference builds one process group per Partial mesh dim and line of ranks
    (``_create_partial_groups``, ``agent.py:46-70``) and all-reduces over them one after the other
    (``ir.py:123-124``); the net effect is one reduction over every rank that differs from this one
    only in Partial mesh coordinates.  That whole set is returned as a single group, so that the
    reduce kernel can combine all members in one pass, in rank order.  Partial mesh dims with different ops
    become the levels of one nested reduction.
    """
    if not partial_reductions:
        return []
    mesh = np.asarray(mesh)
    where = np.argwhere(mesh == this_rank)
    if len(where) != 1:
        raise ValueError(f"rank {this_rank} is not a unique member of the source mesh")
    index: list = [int(c) for c in where[0]]
    for mesh_dim, _ in partial_reductions:
        index[mesh_dim] = slice(None)
    members = np.asarray(mesh[tuple(index)])  # one axis per Partial mesh dim, in mesh-dim order
    ops = [op for _, op in sorted(partial_reductions)]
    if len(set(ops)) == 1:
        ranks = sorted(int(r) for r in members.reshape(-1))
        return [(PartialGroup(ranks=ranks, tensors=[tensors_by_rank[r] for r in ranks]), ops[0])]
    # different ops: the reference all-reduces mesh dim by mesh dim, each with its own op (agent.py:46-70,
    # ir.py:123-124).  The members are listed with the first Partial mesh dim varying fastest and reduced level
    # by level in that order.
    ranks = [int(r) for r in members.transpose().reshape(-1)]
    levels = tuple((op, int(n)) for op, n in zip(ops, members.shape))
    group = PartialGroup(ranks=ranks, tensors=[tensors_by_rank[r] for r in ranks], levels=levels)
    return [(group, "+".join(ops))]


def _flat_ranks(mesh) -> list[int]:
    return [int(r) for r in np.asarray(mesh).reshape(-1)]


def _as_transposed(t: torch.Tensor) -> torch.Tensor:
    """The same values as a ``.t()`` view of a contiguous [cols, rows] tensor (2-D tensors only)."""
    if t.dim() != 2:
        return t
    out = torch.empty(t.shape[1], t.shape[0], dtype=t.dtype, device=t.device).t()
    out.copy_(t)
    return out


def make_global(spec: TensorSpec, device, seed: int | None = None, shape=None) -> torch.Tensor:
    """Synthetic values of a tensor: seeded normal(0, std) or uniform(-1, 1), generated in fp32."""
    gen = torch.Generator(device=device)
    gen.manual_seed(spec.seed if seed is None else seed)
    shape = tuple(spec.shape if shape is None else shape)
    if spec.dist == "uniform":
        g = torch.rand(shape, generator=gen, device=device, dtype=torch.float32) * 2 - 1
    else:
        g = torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * spec.std
    return g.to(spec.source_dtype)


@dataclass
class ReshardJob:
    """Shards, plans and execution of a batch of tensors on one GPU.

    ``target_ranks`` limits the job to those target ranks' share (None = all); source buckets that
    serve none of them are dropped, like a run where only those target agents exist.
    ``fill`` controls source data: "random" (seeded per spec) or a callable ``spec -> global tensor``.
    """

    specs: list[TensorSpec]
    device: torch.device | str = "cuda:0"
    bucket_size: int | None = 64 << 20
    target_ranks: list[int] | None = None
    keep_globals: bool = False
    fill: object = "random"
    wire: LoopbackWire | None = None
    local_view: object = None  # optional ``(kind, tensor) -> view``: re-home a local shard inside another parent
    zero_copy: bool = False  # lend contiguous single-chunk buckets instead of packing them (see LoopbackWire)
    direct: bool = False  # no bucket buffers for plain buckets: targets copy straight from the sources (see LoopbackWire)
    pool: str = "ring"  # "ring": max_in_flight slots per channel; "resident": one slot per bucket (see LoopbackWire)
    max_in_flight: int = 2
    source_locals: list[dict[int, torch.Tensor]] = field(default_factory=list, init=False)
    target_locals: list[dict[int, torch.Tensor]] = field(default_factory=list, init=False)
    globals_: list[torch.Tensor | None] = field(default_factory=list, init=False)
    send_buckets: dict[int, list] = field(default_factory=dict, init=False)
    recv_buckets: dict[int, list] = field(default_factory=dict, init=False)

    def __post_init__(self) -> None:
        self.device = torch.device(self.device)
        if self.wire is None:
            self.wire = LoopbackWire(self.device, pool=self.pool, max_in_flight=self.max_in_flight)
        self.pool = self.wire.pool_mode
        if self.zero_copy:
            self.wire.zero_copy_single_chunk = True
        if self.direct:
            self.wire.direct_same_device = True
        send_chunks: dict[int, list] = {}
        recv_chunks: dict[int, list] = {}
        m2m_cache: dict[tuple, object] = {}
        wanted = set(self.target_ranks) if self.target_ranks is not None else None
        if wanted is not None:  # target ranks that are not staged never unpack: the wire must not wait for them
            named = {r for spec in self.specs for r in _flat_ranks(spec.target_mesh)}
            self.wire.absent_ranks |= named - wanted
        for spec in self.specs:
            src_mesh, tgt_mesh = np.asarray(spec.source_mesh), np.asarray(spec.target_mesh)
            src_ranks, tgt_ranks = _flat_ranks(src_mesh), _flat_ranks(tgt_mesh)
            tgt_dtype = spec.target_dtype or spec.source_dtype
            partial = any(isinstance(p, Partial) for p in spec.source_placements)
            # ---- stage the shards
            src_local: dict[int, torch.Tensor] = {}
            glob = None
            if partial:
                # every member holds its own contribution: seed + flat position, where replicated mesh
                # dims do not count (replicas of a Partial layout hold identical contributions)
                for pos, r in enumerate(src_ranks):
                    coord = list(mesh_coord(src_mesh.shape, pos))
                    shape = local_shape(spec.shape, src_mesh.shape, spec.source_placements, coord)
                    for i, p in enumerate(spec.source_placements):
                        if isinstance(p, Replicate):
                            coord[i] = 0
                    canon = int(np.ravel_multi_index(coord, src_mesh.shape))
                    src_local[r] = make_global(spec, self.device, seed=spec.seed + canon, shape=shape)
            else:
                glob = self.fill(spec).to(self.device) if callable(self.fill) else make_global(spec, self.device)
                for pos, r in enumerate(src_ranks):
                    view = local_shard(glob, src_mesh.shape, spec.source_placements, mesh_coord(src_mesh.shape, pos))
                    src_local[r] = view.clone(memory_format=torch.contiguous_format)
            if spec.source_layout == "transposed":
                src_local = {r: _as_transposed(t) for r, t in src_local.items()}
            if self.local_view is not None:
                src_local = {r: self._rehome("source", t) for r, t in src_local.items()}
            tgt_local: dict[int, torch.Tensor] = {}
            for pos, r in enumerate(tgt_ranks):
                if wanted is not None and r not in wanted:
                    continue
                shape = local_shape(spec.shape, tgt_mesh.shape, spec.target_placements, mesh_coord(tgt_mesh.shape, pos))
                tgt_local[r] = torch.zeros(shape, dtype=tgt_dtype, device=self.device)
                if spec.target_layout == "transposed":
                    tgt_local[r] = _as_transposed(tgt_local[r])
                if self.local_view is not None:
                    tgt_local[r] = self._rehome("target", tgt_local[r])
            self.source_locals.append(src_local)
            self.target_locals.append(tgt_local)
            self.globals_.append(glob if self.keep_globals else None)
            # ---- plan, rank by rank
            key = (str(spec.source_mesh), spec.source_placements, str(spec.target_mesh), spec.target_placements)
            if key not in m2m_cache:
                m2m_cache[key] = get_m2m_map(src_mesh, spec.source_placements, tgt_mesh, spec.target_placements)
            m2m = m2m_cache[key]
            wire_dtype = transfer_dtype_rule(spec.source_dtype, tgt_dtype)
            for r in sorted(set(src_ranks) | set(tgt_local)):
                s_t = src_local.get(r)
                t_t = tgt_local.get(r)
                groups = None
                if partial and s_t is not None:
                    groups = create_partial_groups(src_mesh, m2m.source_partial_reductions, r, src_local) or None
                for c in m2m_to_chunks(m2m, r, source_tensor=s_t, target_tensor=t_t, transfer_dtype=wire_dtype,
                                       source_partial_groups=groups):
                    if c.is_source:  # wire source, reduce-only, or LOCAL
                        if wanted is not None and c.dst_ranks and not (set(c.dst_ranks) & wanted):
                            continue
                        if wanted is not None and not c.dst_ranks and not self._cell_wanted(m2m, c, wanted):
                            continue
                        send_chunks.setdefault(r, []).append(c)
                    else:
                        recv_chunks.setdefault(r, []).append(c)
        size = self.bucket_size or 1
        self.send_buckets = {r: chunk_to_bucket_ops(cs, size) for r, cs in sorted(send_chunks.items())}
        self.recv_buckets = {r: chunk_to_bucket_ops(cs, size) for r, cs in sorted(recv_chunks.items())}

    def _rehome(self, kind: str, t: torch.Tensor) -> torch.Tensor:
        view = self.local_view(kind, t)
        if tuple(view.shape) != tuple(t.shape) or view.dtype != t.dtype:
            raise ValueError("local_view must keep shape and dtype")
        view.copy_(t)
        return view

    @staticmethod
    def _cell_wanted(m2m, chunk, wanted) -> bool:
        """A reduce-only chunk matters if the primary of its cell ships to a wanted rank."""
        for route in m2m.routes:
            if route.src.cell == tuple(chunk.src_idx) and any(d.rank in wanted for d in route.dsts):
                return True
        return False

    # ------------------------------------------------------------------------------------------
    def run_send(self, merge_launches: bool = False, fanout: int = 1, drive: bool = True) -> None:
        for buckets in self.send_buckets.values():
            bucket_comm(buckets, self.max_in_flight, wire=self.wire, merge_launches=merge_launches, synchronize=False,
                        fanout=fanout, drive=drive)

    def run_recv(self, merge_launches: bool = False, fanout: int = 1, drive: bool = True) -> None:
        for buckets in self.recv_buckets.values():
            bucket_comm(buckets, self.max_in_flight, wire=self.wire, merge_launches=merge_launches, synchronize=False,
                        fanout=fanout, drive=drive)

    def run(self, merge_launches: bool = False, synchronize: bool = True, fanout: int = 1) -> None:
        """One transfer: every source rank calls ``bucket_comm`` on its send list, then every target rank on its
        receive list.  With a ring pool the senders fill their slots and wait on the wire; the receivers' calls
        then move both sides along until every bucket has been unpacked."""
        if self.wire.pool_mode == "ring":  # this process plays every rank: queue all pipelines, step them together
            self.run_send(merge_launches, fanout, drive=False)
            self.run_recv(merge_launches, fanout, drive=False)
            self.wire.drive()
        else:
            self.run_send(merge_launches, fanout)
            self.run_recv(merge_launches, fanout)
        if not self.wire.idle():
            raise RuntimeError(f"transfer did not complete; still waiting for a peer: {self.wire.pending()}")
        if synchronize and self.device.type == "cuda":
            torch.cuda.current_stream(self.device).synchronize()

    def capture(self, merge_launches: bool = True):
        """Record one transfer into a HIP graph and return it; ``graph.replay()`` then re-issues every
        launch of the transfer with one call.  The plans must exist (run once eagerly first): planning
        allocates and uploads, which cannot be captured.  Useful when a transfer is launch-bound."""
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.run(merge_launches=merge_launches, synchronize=False)
        return graph

    def payload_bytes(self) -> int:
        """Bytes the measured target ranks end up holding, in wire dtype (the reference's
        effective-throughput numerator, ``bench/transfer_benchmark.py:339-360``)."""
        total = 0
        for buckets in self.recv_buckets.values():
            total += sum(b.total_bytes for b in buckets)
        for buckets in self.send_buckets.values():
            total += sum(b.total_bytes for b in buckets if b.transport.value == "local")
        return total

    def counts(self) -> dict[str, int]:
        return {
            "send_buckets": sum(len(b) for b in self.send_buckets.values()),
            "recv_buckets": sum(len(b) for b in self.recv_buckets.values()),
            "send_chunks": sum(len(b.chunks) for bs in self.send_buckets.values() for b in bs),
            "recv_chunks": sum(len(b.chunks) for bs in self.recv_buckets.values() for b in bs),
        }
