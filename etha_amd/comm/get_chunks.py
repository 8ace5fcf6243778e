"""Stage-2 planner, part 1: routes x tensor shape -> chunks.

Counterpart of ``src/etha/comm/get_chunks.py``.  Same call signature and the same chunk order
(route order; per route the source chunk first, then one chunk per destination on this rank).

Deliberate differences:

* **Uneven dims.**  The reference cuts a local dim by floor division
  (``get_chunks.py:12-19``, ``utils.py:51-57``) and silently drops a non-divisible tail.  Here a
  non-divisible local dim is cut by the ``torch.chunk`` convention - which is how DTensor lays out
  an uneven ``Shard`` - provided the *other* side shards that dim with exactly one plain
  ``Shard`` mesh dim and this side does not shard it at all; then each piece has exactly the
  extent of the peer's (uneven) local shard.  Any other non-divisible case raises ``ValueError``.
  ``chunk_shape`` is therefore taken per chunk from its slice.
* **Same-rank destinations.**  For a destination on the source rank the reference emits a LOCAL
  chunk *and* still lists that rank in the wire chunk's ``dst_ranks`` (``get_chunks.py:62-111``),
  which would post a send to itself.  Here the LOCAL chunk serves that destination, the wire
  chunk keeps only the remote destinations and disappears when none is left.  The LOCAL chunk
  reads ``source_tensor`` (``Chunk.src_tensor``) and writes ``target_tensor``.
* broadcast sub-groups need no pre-creation (``get_chunks.py:48-55``): there is no process group.
* Receive chunks of a Partial source carry the producer's Partial signature
  (``Chunk.source_partial_signature``), so that sender and receiver split a wire key's chunks into the same
  buckets when a batch mixes Partial and plain tensors.
* A role whose tensor is not given produces no chunks: without ``source_tensor`` the rank does not act
  as a source, without ``target_tensor`` not as a destination (the reference would build chunks around
  ``None`` and fail in ``Chunk.__post_init__``, ``ir.py:87-89``).
"""

from __future__ import annotations

import torch

from .get_m2m_map import _is_shard, _is_strided
from .ir import Chunk, M2MMap, PartialGroup
from .transfer import Transport
from .utils import get_slice_from_multi_index, get_slicer_tuples

__all__ = ["m2m_to_chunks", "calculate_chunk_shape"]


def calculate_chunk_shape(num_slicers: list[int], tensor_shape) -> tuple[int, ...]:
    """Nominal (even-split) chunk shape; kept for API compatibility (``get_chunks.py:12-19``)."""
    if tensor_shape is None:
        return ()
    return tuple(int(tensor_shape[d]) // int(num_slicers[d]) for d in range(len(tensor_shape)))


def _uneven_ok(dim: int, this_mesh, this_placements, other_mesh, other_placements) -> bool:
    """May a non-divisible local dim ``dim`` on this side be cut by the torch.chunk rule?"""
    if this_mesh is None or other_mesh is None:
        return False
    if any(_is_shard(p) and p.dim == dim for p in this_placements):
        return False
    on_dim = [p for p in other_placements if _is_shard(p) and p.dim == dim]
    return len(on_dim) == 1 and not _is_strided(on_dim[0])


def _side_slicers(tensor, num_slicers, this_mesh, this_pl, other_mesh, other_pl, side: str):
    shape = tuple(tensor.shape)
    ext = (list(num_slicers) + [1] * len(shape))[: len(shape)]
    for d, (n, k) in enumerate(zip(shape, ext)):
        if k > 1 and n % k != 0 and not _uneven_ok(d, this_mesh, this_pl, other_mesh, other_pl):
            raise ValueError(
                f"{side} tensor dim {d} of size {n} is not divisible into {k} cells and the layout pair "
                "does not define an uneven split for it (the reference would silently drop the tail)"
            )
    return ext, get_slicer_tuples(shape, ext)


def _partial_signature(m2m: M2MMap, src_rank: int) -> tuple:
    """``((member ranks), op, levels)`` of the Partial reduction ``src_rank`` takes part in, as one group over the
    whole connected component - what ``Chunk.partial_signature`` gives for the group that
    ``etha_amd.world.create_partial_groups`` builds on the sending side.  Two reductions over the same ranks with the
    same ops are still different groups when their mesh dims nest differently (sum over 2 then avg over 3, against
    sum over 3 then avg over 2): the sender keeps their chunks in separate buckets, so the receiver must too."""
    if not m2m.source_partial_reductions or m2m.source_mesh is None:
        return ()
    import numpy as np

    mesh = np.asarray(m2m.source_mesh)
    where = np.argwhere(mesh == src_rank)
    if len(where) != 1:
        return ()
    index: list = [int(c) for c in where[0]]
    for mesh_dim, _ in m2m.source_partial_reductions:
        index[mesh_dim] = slice(None)
    members = np.asarray(mesh[tuple(index)])  # one axis per Partial mesh dim, in mesh-dim order
    ops = [op for _, op in sorted(m2m.source_partial_reductions)]
    if len(set(ops)) == 1:
        return ((tuple(sorted(int(r) for r in members.reshape(-1))), ops[0], ()),)
    # one op per Partial mesh dim: members in level order (first Partial mesh dim fastest), and the levels themselves
    ranks = tuple(int(r) for r in members.transpose().reshape(-1))
    levels = tuple((str(op), int(n)) for op, n in zip(ops, members.shape))
    return ((ranks, "+".join(ops), levels),)


def _shape_of(slices: tuple[slice, ...]) -> tuple[int, ...]:
    return tuple(s.stop - s.start for s in slices)


def m2m_to_chunks(
    m2m: M2MMap,
    rank: int,
    source_tensor: torch.Tensor | None = None,
    target_tensor: torch.Tensor | None = None,
    transfer_dtype: torch.dtype | None = None,
    source_partial_groups: list[tuple[PartialGroup, str]] | None = None,
) -> list[Chunk]:
    """Materialise an ``M2MMap`` onto this rank's local tensors."""
    routes = m2m.routes
    if not routes:
        return []
    src_ext = src_tuples = tgt_ext = tgt_tuples = None
    if source_tensor is not None:
        src_ext, src_tuples = _side_slicers(
            source_tensor, m2m.source_num_slicers, m2m.source_mesh, m2m.source_placements,
            m2m.target_mesh, m2m.target_placements, "source",
        )
    if target_tensor is not None:
        tgt_ext, tgt_tuples = _side_slicers(
            target_tensor, m2m.target_num_slicers, m2m.target_mesh, m2m.target_placements,
            m2m.source_mesh, m2m.source_placements, "target",
        )

    chunks: list[Chunk] = []
    for route in routes:
        src_rank, src_idx = route.src.rank, route.src.cell
        all_dsts = tuple(sorted({d.rank for d in route.dsts}))
        src_slices: tuple[slice, ...] = ()
        if src_rank == rank and source_tensor is not None:
            src_slices = get_slice_from_multi_index(src_idx, src_ext, src_tuples)
            remote = tuple(r for r in all_dsts if r != rank)
            if remote or route.kind == Transport.NONE:
                kind = route.kind
                if kind != Transport.NONE:
                    kind = Transport.BROADCAST if len(remote) > 1 else Transport.P2P
                chunks.append(
                    Chunk(
                        chunk_shape=_shape_of(src_slices),
                        transport=kind,
                        is_source=True,
                        is_target=False,
                        src_rank=rank,
                        src_idx=src_idx,
                        dst_ranks=remote,
                        src_slice=src_slices,
                        tensor=source_tensor,
                        transfer_dtype=transfer_dtype,
                        source_partial_groups=source_partial_groups,
                        rank=rank,
                    )
                )
        for dst in route.dsts:
            if dst.rank != rank or target_tensor is None:
                continue
            dst_slices = get_slice_from_multi_index(dst.cell, tgt_ext, tgt_tuples)
            if src_rank == rank:
                if source_tensor is None:
                    raise ValueError(
                        f"rank {rank} is both source and destination of cell {src_idx}: pass source_tensor too"
                    )
                chunks.append(
                    Chunk(
                        chunk_shape=_shape_of(dst_slices),
                        transport=Transport.LOCAL,
                        is_source=True,
                        is_target=True,
                        src_rank=src_rank,
                        src_idx=src_idx,
                        dst_ranks=(rank,),
                        dst_idx=dst.cell,
                        src_slice=src_slices,
                        dst_slice=dst_slices,
                        tensor=target_tensor,
                        src_tensor=source_tensor,
                        # a Partial source delivered to its own rank: the members are combined into the target region
                        source_partial_groups=source_partial_groups,
                        rank=rank,
                    )
                )
            else:
                remote = tuple(r for r in all_dsts if r != src_rank)
                chunks.append(
                    Chunk(
                        chunk_shape=_shape_of(dst_slices),
                        transport=Transport.BROADCAST if len(remote) > 1 else Transport.P2P,
                        is_source=False,
                        is_target=True,
                        src_rank=src_rank,
                        src_idx=src_idx,
                        dst_ranks=remote,
                        dst_idx=dst.cell,
                        dst_slice=dst_slices,
                        tensor=target_tensor,
                        transfer_dtype=transfer_dtype,
                        rank=rank,
                        source_partial_signature=_partial_signature(m2m, src_rank),
                    )
                )
    return chunks
