"""Stage-1 planner: the mesh-to-mesh map, in closed form.

The reference finds the map by *tracing*: it distributes a small "cell grid" tensor with
DTensor on the source mesh, writes ``(rank, local index)`` codes into the local shards, gathers
the full grid, ships it to the target ranks, distributes it there and decodes what every target
cell received (``src/etha/comm/get_m2m_map.py:117-265``).  That needs a process group per rank.

Here the same map is computed directly from DTensor's sharding convention, with no collectives:

* the grid has ``lcm(source shards, target shards)`` cells per tensor dim (``:155-172``);
* a rank's local shard is obtained by applying the placements left to right over the mesh dims:
  ``Shard(d)`` keeps the ``coord``-th ``torch.chunk`` piece of dim ``d``; ``_StridedShard(d, sf)``
  cuts dim ``d`` into ``sf`` pieces, each of those into ``mesh size`` pieces, and keeps the
  ``coord``-th piece of every one; ``Replicate`` (and ``Partial``, traced as ``Replicate``,
  ``:147-149``) keeps everything;
* the target rank at flat mesh position ``t`` reads the grid as seen by the source rank at flat
  position ``t % |source|`` (``:194-203``); that view takes replicated mesh dims from that rank's
  own coordinates and sharded mesh dims from whichever rank owns the cell.

Routes are ordered by ``(src_rank, cell)`` (``_dict_to_routes``, ``:19-37``) and Partial sources
get reduce-only entries for every member of the Partial connected component
(``_expand_partial_shadows``, ``:63-114``).
"""

from __future__ import annotations

import itertools
import math
from collections import defaultdict

import numpy as np
from torch.distributed.tensor.placement_types import Partial, Placement, Replicate, Shard, _StridedShard

from .ir import Endpoint, M2MMap, Route
from .transfer import Transport
from .utils import _as_rank_array, enumerate_partial_subgroup_ranks

__all__ = ["get_m2m_map", "get_shard_shape", "local_shard_indices"]


def _is_strided(p) -> bool:
    return isinstance(p, _StridedShard)


def _is_shard(p) -> bool:
    # in some torch versions _StridedShard derives from Shard, in others it does not
    return isinstance(p, Shard) or _is_strided(p)


def _get_tensor_ndim(placements) -> int:
    return max((p.dim for p in placements if _is_shard(p)), default=0) + 1


def get_shard_shape(mesh_shape, placements, tensor_ndim: int) -> list[int]:
    """Number of shards per tensor dim (``get_m2m_map.py:54-60``)."""
    shards = [1] * tensor_ndim
    for size, p in zip(mesh_shape, placements):
        if _is_shard(p):
            shards[p.dim] *= int(size)
    return shards


def _fine_shape(mesh_shape, placements, tensor_ndim: int) -> list[int]:
    """Finest granularity a layout cuts each tensor dim into: a strided shard cuts ``split_factor`` times finer."""
    fine = [1] * tensor_ndim
    for size, p in zip(mesh_shape, placements):
        if _is_strided(p):
            fine[p.dim] *= int(size) * int(p.split_factor)
        elif _is_shard(p):
            fine[p.dim] *= int(size)
    return fine


def _whole_cells(idx: np.ndarray, ratio: int) -> bool:
    """Is a rank's list of fine cells a sequence of whole coarse cells (``ratio`` fine cells each)?"""
    if ratio == 1:
        return True
    if len(idx) % ratio:
        return False
    rows = idx.reshape(-1, ratio)
    return bool(np.all(rows[:, 0] % ratio == 0) and np.all(rows == rows[:, :1] + np.arange(ratio)))


def _cell_grid(src_shape, src_pl, src_shards, tgt_shape, tgt_pl, tgt_shards, ndim: int) -> list[int]:
    """Cells per tensor dim: the coarsest grid on which every rank of both sides holds whole cells.

    The reference uses ``lcm(source shards, target shards)`` (``get_m2m_map.py:155-172``), which is enough
    when strided shards appear in their usual pairing (split factor = size of a later ``Shard`` mesh dim on
    the same tensor dim).  A strided shard with any other split factor scatters a rank's pieces more finely;
    then the dim is gridded by the lcm of both sides' finest cuts.
    """
    coarse = [math.lcm(s, t) for s, t in zip(src_shards, tgt_shards)]
    fine = [math.lcm(math.lcm(a, b), c) for a, b, c in
            zip(_fine_shape(src_shape, src_pl, ndim), _fine_shape(tgt_shape, tgt_pl, ndim), coarse)]
    if fine == coarse:
        return coarse
    ok = [True] * ndim
    for shape, pl in ((src_shape, src_pl), (tgt_shape, tgt_pl)):
        for pos in range(int(np.prod(shape))):
            idx = local_shard_indices(fine, shape, pl, np.unravel_index(pos, tuple(shape)))
            for d in range(ndim):
                ok[d] = ok[d] and _whole_cells(idx[d], fine[d] // coarse[d])
    return [c if good else f for c, f, good in zip(coarse, fine, ok)]


def _chunk(arr: np.ndarray, parts: int) -> list[np.ndarray]:
    """``torch.chunk`` on an index vector, padded with empty pieces up to ``parts``."""
    step = -(-len(arr) // parts) if len(arr) else 0
    if step == 0:
        return [arr[:0] for _ in range(parts)]
    return [arr[i * step : (i + 1) * step] for i in range(parts)]


def local_shard_indices(dim_sizes, mesh_shape, placements, coord) -> list[np.ndarray]:
    """Global indices, per tensor dim and in local order, held by the rank at mesh ``coord``."""
    idx = [np.arange(n) for n in dim_sizes]
    for size, p, c in zip(mesh_shape, placements, coord):
        size = int(size)
        if _is_strided(p):
            pieces = [_chunk(part, size)[c] for part in _chunk(idx[p.dim], int(p.split_factor))]
            idx[p.dim] = np.concatenate(pieces) if pieces else idx[p.dim][:0]
        elif _is_shard(p):
            idx[p.dim] = _chunk(idx[p.dim], size)[c]
    return idx


def _expand_partial_shadows(m2m: dict, source_mesh: np.ndarray, source_placements) -> dict:
    """Give every member of a Partial connected component an entry for every shipped cell."""
    groups: list[list[int]] = []
    for mesh_dim, p in enumerate(source_placements):
        if isinstance(p, Partial):
            groups.extend(enumerate_partial_subgroup_ranks(source_mesh, mesh_dim))
    out = {src: dict(cells) for src, cells in m2m.items()}
    if not groups:
        return out
    # union-find over ranks that share a sub-group
    parent = {r: r for g in groups for r in g}

    def root(x: int) -> int:
        while parent[x] != x:
            parent[x] = parent[parent[x]]
            x = parent[x]
        return x

    for g in groups:
        for r in g[1:]:
            a, b = root(g[0]), root(r)
            if a != b:
                parent[a] = b
    members: dict[int, set[int]] = defaultdict(set)
    for r in parent:
        members[root(r)].add(r)
    for src, cells in m2m.items():
        if src not in parent:
            continue
        for peer in members[root(src)]:
            if peer == src:
                continue
            for cell in cells:
                out.setdefault(peer, {}).setdefault(cell, [])
    return out


def _dict_to_routes(m2m: dict) -> list[Route]:
    routes = []
    for src in sorted(m2m):
        for cell in sorted(m2m[src]):
            dsts = tuple(Endpoint(rank=r, cell=c) for r, c in m2m[src][cell])
            kind = Transport.NONE if not dsts else (Transport.BROADCAST if len(dsts) > 1 else Transport.P2P)
            routes.append(Route(src=Endpoint(rank=src, cell=cell), dsts=dsts, kind=kind))
    return routes


def get_m2m_map(
    source_mesh,
    source_placements: tuple[Placement, ...],
    target_mesh,
    target_placements: tuple[Placement, ...],
    group=None,
    device: str = "cpu",
) -> M2MMap:
    """Mesh-to-mesh redistribution map of a source/target layout pair.

    ``source_mesh``/``target_mesh`` are ``DeviceMesh`` objects or plain (nested lists / arrays /
    tensors of) global ranks.  ``group`` and ``device`` exist for signature compatibility with the
    reference and are unused: nothing is communicated.  A ``Partial`` target raises
    ``NotImplementedError`` as in the reference (``get_m2m_map.py:137-142``).
    """
    del group, device
    source_placements = tuple(source_placements)
    target_placements = tuple(target_placements)
    if any(isinstance(p, Partial) for p in target_placements):
        raise NotImplementedError(
            f"target_placements={target_placements} contains Partial: how a tensor would be split into partial "
            "contributions across two process groups has no single answer, so Partial can only appear on the source side."
        )
    src_mesh = _as_rank_array(source_mesh)
    tgt_mesh = _as_rank_array(target_mesh)
    if src_mesh.ndim != len(source_placements) or tgt_mesh.ndim != len(target_placements):
        raise ValueError("one placement per mesh dim is required")

    partial_reductions = [(i, p.reduce_op) for i, p in enumerate(source_placements) if isinstance(p, Partial)]
    eff_source = tuple(Replicate() if isinstance(p, Partial) else p for p in source_placements)

    ndim = max(_get_tensor_ndim(eff_source), _get_tensor_ndim(target_placements))
    src_shards = get_shard_shape(src_mesh.shape, eff_source, ndim)
    tgt_shards = get_shard_shape(tgt_mesh.shape, target_placements, ndim)
    grid = _cell_grid(src_mesh.shape, eff_source, src_shards, tgt_mesh.shape, target_placements, tgt_shards, ndim)
    source_num_slicers = [g // s for g, s in zip(grid, src_shards)]
    target_num_slicers = [g // t for g, t in zip(grid, tgt_shards)]

    src_ranks = [int(r) for r in src_mesh.reshape(-1)]
    tgt_ranks = [int(r) for r in tgt_mesh.reshape(-1)]

    # who owns which grid cell on the source side, per replica
    replicated_dims = [i for i, p in enumerate(eff_source) if not _is_shard(p)]
    owner: dict[tuple, tuple[int, tuple[int, ...]]] = {}
    for pos, rank in enumerate(src_ranks):
        coord = np.unravel_index(pos, src_mesh.shape)
        idx = local_shard_indices(grid, src_mesh.shape, eff_source, coord)
        replica = tuple(int(coord[i]) for i in replicated_dims)
        for local in itertools.product(*[range(len(v)) for v in idx]):
            cell = tuple(int(idx[d][local[d]]) for d in range(ndim))
            owner[(replica, cell)] = (rank, tuple(local))

    m2m: dict[int, dict[tuple, list]] = defaultdict(lambda: defaultdict(list))
    # targets contribute in ascending rank order, each in its local iteration order
    for pos in sorted(range(len(tgt_ranks)), key=lambda i: tgt_ranks[i]):
        t_rank = tgt_ranks[pos]
        view_coord = np.unravel_index(pos % len(src_ranks), src_mesh.shape)
        replica = tuple(int(view_coord[i]) for i in replicated_dims)
        coord = np.unravel_index(pos, tgt_mesh.shape)
        idx = local_shard_indices(grid, tgt_mesh.shape, target_placements, coord)
        for local in itertools.product(*[range(len(v)) for v in idx]):
            cell = tuple(int(idx[d][local[d]]) for d in range(ndim))
            s_rank, s_local = owner[(replica, cell)]
            m2m[s_rank][s_local].append((t_rank, tuple(local)))

    plain = {src: dict(cells) for src, cells in m2m.items()}
    plain = _expand_partial_shadows(plain, src_mesh, source_placements)
    return M2MMap(
        routes=_dict_to_routes(plain),
        source_num_slicers=source_num_slicers,
        target_num_slicers=target_num_slicers,
        source_partial_reductions=partial_reductions,
        source_mesh=src_mesh.tolist(),
        source_placements=source_placements,
        target_mesh=tgt_mesh.tolist(),
        target_placements=target_placements,
    )
