"""Index helpers of the planner (pure host code).

Counterparts of ``src/etha/comm/utils.py``: ``enumerate_partial_subgroup_ranks`` (``:17-38``),
``get_slicer_tuples`` (``:41-57``) and ``get_slice_from_multi_index`` (``:60-78``).
"""

from __future__ import annotations

import itertools

import numpy as np

__all__ = [
    "enumerate_partial_subgroup_ranks",
    "get_slicer_tuples",
    "get_slice_from_multi_index",
    "split_points",
]


def _as_rank_array(mesh) -> np.ndarray:
    if hasattr(mesh, "mesh"):  # DeviceMesh
        mesh = mesh.mesh
    if hasattr(mesh, "detach"):  # torch.Tensor
        mesh = mesh.detach().cpu().numpy()
    return np.asarray(mesh, dtype=np.int64)


def enumerate_partial_subgroup_ranks(mesh_tensor, mesh_dim_idx: int) -> list[list[int]]:
    """Rank lists of the sub-groups along ``mesh_dim_idx``: one per setting of the other coords."""
    mesh = _as_rank_array(mesh_tensor)
    if not 0 <= mesh_dim_idx < mesh.ndim:
        raise ValueError(f"mesh_dim_idx must be in [0, {mesh.ndim}), got {mesh_dim_idx}")
    moved = np.moveaxis(mesh, mesh_dim_idx, -1)  # other dims keep their order
    return [list(map(int, row)) for row in moved.reshape(-1, mesh.shape[mesh_dim_idx])]


def split_points(length: int, parts: int) -> list[int]:
    """Boundaries of ``length`` cut into ``parts`` pieces.

    Even split when divisible (the reference's ``dim_size // num_slices``); otherwise the
    ``torch.chunk`` convention DTensor uses for uneven shards: pieces of ``ceil(length/parts)``,
    the last non-empty one shorter, trailing ones empty.
    """
    step = -(-length // parts) if parts else 0
    return [min(i * step, length) for i in range(parts + 1)]


def get_slicer_tuples(tensor_shape, num_slicers: list[int]) -> list[tuple[slice, ...]]:
    """All slice tuples of a tensor cut ``num_slicers[d]`` ways along each dim, row-major."""
    per_dim = []
    for dim, parts in enumerate(num_slicers):
        pts = split_points(int(tensor_shape[dim]), int(parts))
        per_dim.append([slice(pts[i], pts[i + 1]) for i in range(parts)])
    return list(itertools.product(*per_dim))


def get_slice_from_multi_index(idx: tuple, num_slicers: list[int], slicer_tuples: list[tuple[slice, ...]]):
    """Slice tuple of the cell with multi-index ``idx`` (row-major linearisation)."""
    linear = 0
    for i, n in zip(idx, num_slicers[: len(idx)]):
        linear = linear * n + i
    return slicer_tuples[linear]
