"""Pins the layout convention: oracle vs torch's own DTensor, and the product's helper vs the oracle."""

import numpy as np
import pytest
import torch
import torch.distributed as dist

from etha_amd import layout as product_layout
from oracle import dtensor_layout

from helpers import load_cases, parse_placements

CASES = load_cases()


def _layouts():
    seen, out = set(), []

    def add(mesh_shape, codes, shape):
        codes = [c for c in codes]
        if any(c.startswith("P") for c in codes):  # Partial cannot enter distribute_tensor; it does not slice
            codes = ["R" if c.startswith("P") else c for c in codes]
        key = (tuple(mesh_shape), tuple(codes), tuple(shape))
        if key not in seen:
            seen.add(key)
            out.append(key)

    cc = CASES["communication_cpu"]
    for src_mesh, tgt_mesh in cc["mesh_pairs"]:
        add(src_mesh, cc["source_placements"], cc["tensor_shape"])
        add(tgt_mesh, cc["target_placements"], cc["tensor_shape"])
    for c in CASES["reshard"]:
        add(c["src_mesh"], c["src"], c["shape"])
        add(c["tgt_mesh"], c["tgt"], c["shape"])
    # uneven shards and strided shards beyond the reference's tables
    add([6], ["S0"], [31, 4])
    add([2, 2], ["SS0/2", "S0"], [8, 8])
    add([2, 3], ["S1", "S0"], [7, 10])
    add([4], ["S0"], [3, 5])  # more ranks than rows: empty shards
    # random layouts with strided shards of arbitrary split factors (also unpaired ones), even sizes
    rng = np.random.RandomState(7)
    for _ in range(40):
        ndim = int(rng.randint(1, 4))
        mesh = [int(rng.choice([1, 2, 3, 4])) for _ in range(int(rng.randint(1, 4)))]
        while int(np.prod(mesh)) > 8:
            mesh[int(rng.randint(len(mesh)))] = 1
        codes, mult = [], [1] * ndim
        for n in mesh:
            kind, d = rng.choice(["S", "SS", "R"]), int(rng.randint(ndim))
            if kind == "S":
                codes.append(f"S{d}")
                mult[d] *= n
            elif kind == "SS":
                sf = int(rng.choice([2, 3]))
                codes.append(f"SS{d}/{sf}")
                mult[d] *= n * sf
            else:
                codes.append("R")
        add(mesh, codes, [m * int(rng.randint(1, 4)) for m in mult])
    return out


@pytest.fixture(scope="module")
def torch_truth():
    """Local shards computed by torch's distribute_tensor under a single-process fake group."""
    from torch.distributed.tensor import DeviceMesh, distribute_tensor
    from torch.testing._internal.distributed.fake_pg import FakeStore

    cache = {}

    def get(mesh_shape, codes, shape):
        key = (mesh_shape, codes, shape)
        if key in cache:
            return cache[key]
        world = int(np.prod(mesh_shape))
        g = torch.arange(int(np.prod(shape)), dtype=torch.float32).reshape(shape)
        res = []
        for r in range(world):
            dist.init_process_group("fake", rank=r, world_size=world, store=FakeStore())
            try:
                mesh = DeviceMesh("cpu", torch.arange(world).view(mesh_shape))
                dt = distribute_tensor(g, mesh, list(parse_placements(codes)), src_data_rank=None)
                res.append(dt.to_local().clone())
            finally:
                dist.destroy_process_group()
        cache[key] = (g, res)
        return cache[key]

    return get


@pytest.mark.parametrize("mesh_shape,codes,shape", _layouts())
def test_layout_matches_torch_distribute_tensor(torch_truth, mesh_shape, codes, shape):
    g, truth = torch_truth(mesh_shape, codes, shape)
    pl = parse_placements(codes)
    for pos, want in enumerate(truth):
        coord = dtensor_layout.mesh_coord(mesh_shape, pos)
        got = dtensor_layout.local_shard(g, mesh_shape, pl, coord)
        assert got.shape == want.shape and torch.equal(got, want), f"oracle, rank {pos}"
        got_p = product_layout.local_shard(g, mesh_shape, pl, coord)
        assert got_p.shape == want.shape and torch.equal(got_p, want), f"product, rank {pos}"
        assert product_layout.local_shape(shape, mesh_shape, pl, coord) == tuple(want.shape)
