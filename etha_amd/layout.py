"""DTensor layout arithmetic used to stage every rank's shards on one GPU.

``local_shard`` returns the part of a global tensor that a rank holds under
``(mesh shape, placements)``, following the same left-to-right convention the planner uses
(:func:`etha_amd.comm.get_m2m_map.local_shard_indices`).
"""

from __future__ import annotations

import numpy as np
import torch

from .comm.get_m2m_map import local_shard_indices


def mesh_coord(mesh_shape, position: int) -> tuple[int, ...]:
    return tuple(int(x) for x in np.unravel_index(position, tuple(mesh_shape)))


def local_shard(global_tensor: torch.Tensor, mesh_shape, placements, coord) -> torch.Tensor:
    """View (or gathered copy, for strided shards) of the rank's part of ``global_tensor``."""
    idx = local_shard_indices(global_tensor.shape, mesh_shape, placements, coord)
    out = global_tensor
    for d, v in enumerate(idx):
        if len(v) == out.shape[d]:
            continue
        if len(v) == 0:
            out = out.narrow(d, 0, 0)
        elif int(v[-1]) - int(v[0]) + 1 == len(v):
            out = out.narrow(d, int(v[0]), len(v))
        else:
            out = out.index_select(d, torch.as_tensor(v, device=out.device))
    return out


def local_shape(global_shape, mesh_shape, placements, coord) -> tuple[int, ...]:
    return tuple(len(v) for v in local_shard_indices(global_shape, mesh_shape, placements, coord))
