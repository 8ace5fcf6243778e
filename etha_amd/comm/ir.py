"""Plan objects of the redistribute path: routes, chunks, buckets.

Same names, fields and meaning as the reference's IR (``src/etha/comm/ir.py``): ``Endpoint``,
``Route`` and ``M2MMap`` (``ir.py:16-48``) describe the shape-free mesh-to-mesh topology,
``Chunk`` (``ir.py:60-169``) one strided tensor region and its role, ``Bucket``
(``ir.py:172-310``) a group of chunks that travel as one contiguous buffer.

Differences, all additive:

* the byte work of ``Chunk.prepare/finalize`` and ``Bucket.prepare/finalize`` is not done here
  with per-chunk tensor ops; buckets are compiled into a device tile program
  (:mod:`etha_amd.comm.device_plan`) and run as batched HIP launches;
* a Partial source is described by :class:`PartialGroup` objects (the peers' tensors, all resident
  on this GPU) instead of ``ProcessGroup`` handles;
* ``Chunk.rank`` records the rank the chunk was built for, and ``Chunk.src_tensor`` lets a LOCAL
  chunk read a source tensor that is a different object than its target tensor.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any

import torch

from .transfer import Transport

REDUCE_OPS = ("sum", "avg", "max", "min", "product")  # ir.py:51-57


@dataclass(frozen=True)
class Endpoint:
    """Where a chunk lives: the owning rank and the multi-index of its cell in the lcm grid of the transfer."""

    rank: int
    cell: tuple[int, ...]


@dataclass(frozen=True)
class Route:
    """Delivery plan of one source cell: ``src`` to every endpoint in ``dsts``.

    ``kind`` is NONE for a reduce-only entry (no dsts), P2P for one dst, BROADCAST for several.
    """

    src: Endpoint
    dsts: tuple[Endpoint, ...]
    kind: Transport


@dataclass
class M2MMap:
    """Mesh-to-mesh topology; independent of tensor shapes and reusable across batches.

    The first four fields are the reference's (``ir.py:36-48``).  The remaining ones record the
    two layouts so that chunk building can treat unevenly sharded dims.
    """

    routes: list[Route] | None = None
    source_num_slicers: list[int] | None = None
    target_num_slicers: list[int] | None = None
    source_partial_reductions: list[tuple[int, str]] = field(default_factory=list)
    source_mesh: Any = None  # nested list of ranks
    source_placements: tuple = ()
    target_mesh: Any = None
    target_placements: tuple = ()


@dataclass(eq=False)
class PartialGroup:
    """The members of one Partial reduction as seen from one GPU.

    ``ranks`` are in ascending order; ``tensors[i]`` is rank ``ranks[i]``'s local partial
    tensor.  Stands in for the ``ProcessGroup`` of ``Chunk.source_partial_groups`` (``ir.py:84``):
    the reduce kernel reads the peers directly instead of running a collective.

    ``levels`` describes Partial mesh dims with *different* reduce ops: ``((op, size), ...)`` from the
    first-applied mesh dim to the last, ``ranks``/``tensors`` then listed with the first-applied dim
    varying fastest (not ascending).  The reference all-reduces once per such dim, each with its own op,
    in mesh-dim order (``tensor_bus/agent.py:46-70``, ``ir.py:123-124``).
    """

    ranks: tuple[int, ...]
    tensors: tuple[torch.Tensor, ...]
    levels: tuple = ()

    def __post_init__(self) -> None:
        self.ranks = tuple(self.ranks)
        self.tensors = tuple(self.tensors)
        self.levels = tuple((str(op), int(n)) for op, n in self.levels)
        if len(self.ranks) != len(self.tensors):
            raise ValueError("PartialGroup needs one tensor per rank")
        if self.levels:
            if not 2 <= len(self.levels) <= 3:
                raise NotImplementedError("between two and three Partial mesh dims with different ops are supported")
            if math.prod(n for _, n in self.levels) != len(self.ranks):
                raise ValueError("PartialGroup levels do not multiply up to the number of members")
            if any(op not in REDUCE_OPS for op, _ in self.levels) or any(not 1 <= n <= 255 for _, n in self.levels):
                raise ValueError(f"bad PartialGroup levels {self.levels}")
        elif list(self.ranks) != sorted(self.ranks):
            raise ValueError("PartialGroup ranks must be ascending (reduction order is rank order)")


@dataclass(kw_only=True, eq=False)
class Chunk:
    """Descriptor of one region of one tensor and of what this rank does with it (send, receive, both, or reduce only)."""

    transport: Transport
    is_source: bool
    is_target: bool
    src_rank: int
    dst_ranks: tuple[int, ...]
    chunk_shape: tuple[int, ...]
    tensor: torch.Tensor | None = None
    src_slice: tuple[slice, ...] = ()  # read here when is_source
    dst_slice: tuple[slice, ...] = ()  # written here when is_target
    transfer_dtype: torch.dtype | None = None  # wire dtype; None = tensor.dtype
    src_idx: tuple = ()
    dst_idx: tuple | None = None
    source_partial_groups: list[tuple[PartialGroup, str]] | None = None
    buffer: torch.Tensor | None = None
    # additions
    rank: int | None = None  # rank this chunk was materialised for
    src_tensor: torch.Tensor | None = None  # LOCAL chunks: tensor that src_slice indexes (default: tensor)
    # consume-only chunks: the Partial signature of the producing side, so that both ends of a wire split
    # their buckets the same way (the reference's receive chunks carry no Partial information, which makes
    # sender and receiver bundle differently when a batch mixes Partial and plain tensors)
    source_partial_signature: tuple = ()

    def __post_init__(self) -> None:
        if self.transfer_dtype is None and self.tensor is not None:
            self.transfer_dtype = self.tensor.dtype
        self.chunk_shape = tuple(int(n) for n in self.chunk_shape)
        self.dst_ranks = tuple(self.dst_ranks)

    def __repr__(self) -> str:
        role = ("S" if self.is_source else "") + ("T" if self.is_target else "") or "-"
        return f"Chunk({self.transport.name[:3]}/{role}, src={self.src_rank}->{self.dst_ranks}, shape={self.chunk_shape})"

    @property
    def partial_signature(self) -> tuple:
        if not self.source_partial_groups:
            return tuple(self.source_partial_signature)
        return tuple((g.ranks, op, g.levels) for g, op in self.source_partial_groups)

    @property
    def bucket_key(self) -> tuple:
        """Grouping key, as ``ir.py:143-164``.

        ``(src_rank, dst_ranks, partial signature, cell key, transport)``; the cell key is only
        set for reduce-only chunks so that they never bundle across cells.  The partial signature
        is built from the group's ranks and op (the reference uses ``id(group)``; equal for
        equal groups either way).
        """
        cell_key: tuple = ()
        signature = self.partial_signature
        if signature and not self.dst_ranks:
            cell_key = tuple(self.src_idx)
        return (self.src_rank, self.dst_ranks, signature, cell_key, self.transport)

    @property
    def nbytes(self) -> int:
        """Byte size on the wire (``ir.py:166-169``)."""
        return math.prod(self.chunk_shape) * self.transfer_dtype.itemsize

    # -- reduction description used by the device plan ------------------------------------
    def partial_peers(self) -> tuple[tuple[torch.Tensor, ...], str] | None:
        """Peers (rank order) and op of this chunk's Partial collapse, or None.

        The reference runs one in-place all-reduce per sub-group in sequence (``ir.py:123-124``),
        which reduces over the whole connected component of the Partial mesh dims.  Here that
        component must be given as ONE group (``etha_amd.world.create_partial_groups`` builds it):
        the union of a rank's own per-dim sub-groups would miss members that share no line with it.
        """
        if not self.source_partial_groups:
            return None
        if len(self.source_partial_groups) != 1:
            raise NotImplementedError(
                "pass one PartialGroup covering the whole Partial connected component (with levels when the mesh dims "
                "reduce with different ops), not one group per mesh dim"
            )
        group, op = self.source_partial_groups[0]
        if group.levels:
            return group.tensors, group.levels  # one op per Partial mesh dim, innermost (first applied) first
        if op not in REDUCE_OPS:
            raise ValueError(f"unknown reduce op {op!r}")
        return group.tensors, op


@dataclass(kw_only=True, eq=False)
class Bucket:
    """A transfer unit: one contiguous buffer holding its chunks back to back.

    Identity (transport, role, ranks, key) is uniform over the chunks and read from the first
    one; ``offsets`` is the un-padded prefix sum of ``chunk.nbytes`` (``ir.py:189-194``).
    """

    chunks: list[Chunk]
    device: torch.device | None = None
    buffer: torch.Tensor | None = None
    offsets: list[int] = field(init=False)

    def __post_init__(self) -> None:
        cursor, offsets = 0, []
        for chunk in self.chunks:
            offsets.append(cursor)
            cursor += chunk.nbytes
        self.offsets = offsets
        self._total = cursor

    @property
    def transport(self) -> Transport:
        return self.chunks[0].transport

    @property
    def is_source(self) -> bool:
        return self.chunks[0].is_source

    @property
    def is_target(self) -> bool:
        return self.chunks[0].is_target

    @property
    def src_rank(self) -> int:
        return self.chunks[0].src_rank

    @property
    def dst_ranks(self) -> tuple[int, ...]:
        return self.chunks[0].dst_ranks

    @property
    def key(self) -> tuple:
        return self.chunks[0].bucket_key

    @property
    def rank(self) -> int | None:
        return self.chunks[0].rank

    @property
    def total_bytes(self) -> int:
        return self._total

    def __repr__(self) -> str:
        role = ("S" if self.is_source else "") + ("T" if self.is_target else "") or "-"
        return (
            f"Bucket({self.transport.name[:3]}/{role}, n={len(self.chunks)}, bytes={self.total_bytes}, "
            f"src={self.src_rank}->{self.dst_ranks})"
        )

    # -- the reference's per-bucket protocol (ir.py:229-310), on top of the compiled plan -----------
    # ``bucket_comm`` is the normal entry; these exist for code that drives single buckets itself.
    def _plan(self, wire=None):
        if wire is None:
            from .loopback import default_wire

            wire = default_wire()
        return wire.plan([self])

    def prepare(self, wire=None) -> None:
        """Source bucket: enqueue its pack (or reduce-pack / self-copy) launch.  Target bucket: nothing
        to do, its bytes arrive in the producer's pool slot (``Bucket.prepare``, ``ir.py:229-264``)."""
        self._plan(wire).run_kinds(("pack", "reduce_pack", "selfcopy", "selfcopy_reduce", "lend"))

    def launch(self) -> bool:
        """The wire step.  Always ready: the loopback hands the pool slot over in place
        (``Bucket.launch``, ``ir.py:266-284``)."""
        return True

    def is_complete(self, wire=None) -> bool:
        """Source bucket on a ring pool: every destination has unpacked it (its slot is free again).  Target
        bucket on a ring pool: its send bucket has been packed.  Otherwise always True
        (``Bucket.is_complete``, ``ir.py:286-298``)."""
        from .comm_methods import recv_may_start

        plan = self._plan(wire)
        if plan.wire.pool_mode != "ring":
            return True
        for i in plan.steps_of.get(id(self), ()):
            entry, kind = plan.info[i].entry, plan.steps[i][0]
            if entry is None:
                continue
            if kind in ("unpack", "direct", "direct_reduce"):
                if not recv_may_start(entry, self.rank):
                    return False
            elif entry.left:
                return False
        return True

    def finalize(self, wire=None) -> None:
        """Target bucket (and staged self-copy): enqueue its unpack launch (``Bucket.finalize``,
        ``ir.py:300-310``)."""
        self._plan(wire).run_kinds(("unpack", "direct", "direct_reduce"))
