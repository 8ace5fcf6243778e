"""TEST INFRASTRUCTURE.  DTensor's sharding convention, restated.

This is the closed form every end-to-end test of the reference asserts: after a transfer,
``full_tensor()`` of the target DTensor equals the source's global tensor
(``tests/test_communication_cpu.py:110-114``, ``tests/test_communication_replicate_shard.py:193-197``),
i.e. every target rank's local shard is *the slice of the global tensor that DTensor assigns to
that rank*.  ``local_shard`` computes that slice.

Convention (torch.distributed.tensor, torch 2.10): placements are applied left to right over the
mesh dims; ``Shard(d)`` keeps the ``coord``-th ``torch.chunk`` piece of dim ``d`` (uneven and
empty pieces allowed); ``_StridedShard(d, split_factor=sf)`` cuts dim ``d`` into ``sf`` pieces,
each of them into ``mesh size`` pieces, and concatenates the ``coord``-th piece of every one;
``Replicate`` keeps everything; a ``Partial`` mesh dim does not slice (every member holds a
full-shape contribution).

Pinned by ``tests/test_oracle_layout.py`` against torch's own ``distribute_tensor`` run under
a single-process fake process group, for every mesh/placement pair of the reference's test tables.
"""

from __future__ import annotations

import numpy as np
import torch
from torch.distributed.tensor.placement_types import Shard, _StridedShard


def _pieces(t: torch.Tensor, parts: int, dim: int) -> list[torch.Tensor]:
    out = list(torch.chunk(t, parts, dim=dim))
    while len(out) < parts:  # torch.chunk returns fewer pieces when it runs out of elements
        out.append(t.narrow(dim, 0, 0))
    return out


def local_shard(global_tensor: torch.Tensor, mesh_shape, placements, coord) -> torch.Tensor:
    """The local shard DTensor gives the rank at mesh coordinate ``coord``."""
    t = global_tensor
    for size, p, c in zip(mesh_shape, placements, coord):
        size, c = int(size), int(c)
        if isinstance(p, _StridedShard):
            firsts = _pieces(t, int(p.split_factor), p.dim)
            t = torch.cat([_pieces(f, size, p.dim)[c] for f in firsts], dim=p.dim)
        elif isinstance(p, Shard):
            t = _pieces(t, size, p.dim)[c]
    return t


def mesh_coord(mesh_shape, position: int) -> tuple[int, ...]:
    return tuple(int(x) for x in np.unravel_index(position, tuple(mesh_shape)))


def all_local_shards(global_tensor: torch.Tensor, mesh, placements) -> dict[int, torch.Tensor]:
    """``{rank: local shard}`` for a mesh given as a nested list / array of ranks."""
    mesh = np.asarray(mesh)
    out = {}
    for pos, rank in enumerate(mesh.reshape(-1)):
        out[int(rank)] = local_shard(global_tensor, mesh.shape, placements, mesh_coord(mesh.shape, pos))
    return out
