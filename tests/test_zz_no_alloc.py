"""etha_copy_regions_noalloc: the region copy that allocates no device memory, against the table-based entry
points it is a variant of (etha_selfcopy_table_create + etha_selfcopy_bucket), bit for bit, through the C ABI."""

import numpy as np
import pytest
import torch

from etha_amd import _native as nat
from etha_amd.comm.device_plan import fill_region

pytestmark = pytest.mark.gpu


def _rows(pairs):
    """Descriptor arrays for ``[(src tensor, src slices, dst tensor, dst slices), ...]``."""
    src = np.zeros(len(pairs), dtype=nat.CHUNK_DESC)
    dst = np.zeros(len(pairs), dtype=nat.CHUNK_DESC)
    for i, (s, ss, d, ds) in enumerate(pairs):
        shape = tuple(s[ss].shape)
        assert shape == tuple(d[ds].shape)
        a, b = np.zeros((), dtype=nat.CHUNK_DESC), np.zeros((), dtype=nat.CHUNK_DESC)
        fill_region(a, s, ss, shape)
        fill_region(b, d, ds, shape)
        a["wire_dtype"], b["wire_dtype"] = a["tensor_dtype"], b["tensor_dtype"]
        src[i], dst[i] = a, b
    return src, dst


def _bits(t):
    return t.contiguous().view(torch.uint8).cpu()


def _case(dev, seed, scale):
    """A few region pairs of mixed kinds; ``scale`` sizes them.  Returns (pairs into dst set 1, same into dst set 2)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    r, c = 37 * scale, 51 * scale
    f32 = torch.randn(r + 9, c + 13, generator=g, device=dev)
    i8 = torch.randint(-128, 128, (r * 3 + 5,), generator=g, device=dev, dtype=torch.int8)
    tr = torch.randn(c + 8, r + 8, generator=g, device=dev).to(torch.bfloat16).t()  # contiguous along dim 0
    f64 = torch.randn(r, 7, generator=g, device=dev, dtype=torch.float64)

    def targets():
        return (torch.full((r + 20, c + 40), -1.0, device=dev, dtype=torch.bfloat16),
                torch.full((r * 3 + 64,), 7, device=dev, dtype=torch.int8),
                torch.full((r + 8, c + 24), 3.0, device=dev, dtype=torch.bfloat16),
                torch.full((r, 16), 2.0, device=dev, dtype=torch.float16))

    def pairs(t):
        return [
            (f32, (slice(5, 5 + r), slice(7, 7 + c)), t[0], (slice(11, 11 + r), slice(3, 3 + c))),  # converting, strided rows
            (i8, (slice(3, 3 + r * 3),), t[1], (slice(17, 17 + r * 3),)),  # skewed byte move
            (tr, (slice(0, r + 8), slice(2, 2 + c)), t[2], (slice(0, r + 8), slice(5, 5 + c))),  # transposing
            (f64, (slice(0, r), slice(0, 7)), t[3], (slice(0, r), slice(4, 11))),  # short converting rows
        ]

    t1, t2 = targets(), targets()
    return pairs(t1), pairs(t2), t1, t2


def test_noalloc_region_copy_matches_the_table_path(gpu_device):
    torch.cuda.set_device(gpu_device)
    nat.noalloc_setup()
    nat.noalloc_setup()  # idempotent
    stream = torch.cuda.current_stream(gpu_device).cuda_stream
    kept = []
    # two calls in a row on one stream, the second with a smaller input; neither waits for the other
    for seed, scale in ((1, 40), (2, 3)):
        p1, p2, t1, t2 = _case(gpu_device, seed, scale)
        src1, dst1 = _rows(p1)
        nat.copy_regions_noalloc(src1, dst1, stream)
        kept.append((p2, t1, t2, seed))
    torch.cuda.synchronize()
    for p2, t1, t2, seed in kept:
        src2, dst2 = _rows(p2)
        table = nat.Table.create_selfcopy(src2, dst2)
        info = table.info()
        assert info.n_trans_tiles > 0 and info.n_row_tiles > 0 and info.n_run_tiles > 0
        table.selfcopy(0, len(src2), stream)
        torch.cuda.synchronize()
        for k, (a, b) in enumerate(zip(t1, t2)):
            assert torch.equal(_bits(a), _bits(b)), f"call with seed {seed}: target {k} differs from the table path"
    # and what either path means, for every pair of every call: the slice, converted by torch, landed; bytes outside
    # the destination slice kept their fill value
    for p2, t1, t2, seed in kept:
        fills = (-1.0, 7, 3.0, 2.0)
        for k, ((s, ss, d, ds), first, fill) in enumerate(zip(p2, t1, fills)):
            want = s[ss].to(d.dtype)
            assert torch.equal(_bits(first[ds]), _bits(want)), f"call with seed {seed}: pair {k} is not torch's slice.to()"
            outside = torch.ones_like(first, dtype=torch.bool)
            outside[ds] = False
            assert bool((first[outside] == fill).all()), f"call with seed {seed}: pair {k} wrote outside its region"


def test_noalloc_refuses_what_does_not_fit_and_what_it_cannot_do(gpu_device):
    torch.cuda.set_device(gpu_device)
    nat.noalloc_setup()
    rows, row_bytes, pitch = 640_000, 2000, 2016  # 125 units per row: row tiles, 64 bytes per 16 KiB of payload
    src = torch.zeros(rows, pitch, dtype=torch.uint8, device=gpu_device)
    dst = torch.ones(rows, pitch, dtype=torch.uint8, device=gpu_device)
    a, b = _rows([(src, (slice(0, rows), slice(0, row_bytes)), dst, (slice(0, rows), slice(0, row_bytes)))])
    with pytest.raises(nat.EthaNativeError, match="holds at most") as e:
        nat.copy_regions_noalloc(a, b)
    assert e.value.code == nat.ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert int(dst[0, 0]) == 1 and int(dst[-1, row_bytes - 1]) == 1  # nothing was launched
    # half of it fits
    h = rows // 2
    a, b = _rows([(src, (slice(0, h), slice(0, row_bytes)), dst, (slice(0, h), slice(0, row_bytes)))])
    nat.copy_regions_noalloc(a, b)
    torch.cuda.synchronize()
    assert int(dst[:h, :row_bytes].max()) == 0 and int(dst[:h, row_bytes:].min()) == 1 and int(dst[h:].min()) == 1
    a["n_partials"] = 2
    with pytest.raises(nat.EthaNativeError, match="Partial"):
        nat.copy_regions_noalloc(a, b)


def test_noalloc_refuses_a_capturing_stream(gpu_device):
    """Recorded into a graph, the upload of the tile program would be replayed from a staging buffer that later
    calls overwrite: the entry point refuses a stream under capture and launches nothing."""
    torch.cuda.set_device(gpu_device)
    nat.noalloc_setup()
    src = torch.arange(4096, device=gpu_device, dtype=torch.float32)
    dst = torch.zeros(4096, device=gpu_device, dtype=torch.float32)
    a, b = _rows([(src, (slice(0, 4096),), dst, (slice(0, 4096),))])
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device=gpu_device)
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            before = nat.kernel_launches()
            with pytest.raises(nat.EthaNativeError, match="capturing") as e:
                nat.copy_regions_noalloc(a, b, torch.cuda.current_stream(gpu_device).cuda_stream)
            assert e.value.code == nat.ERR_UNSUPPORTED and nat.kernel_launches() == before
            dst.add_(0)  # the capture itself stays valid: it records this and ends normally
    torch.cuda.synchronize()
    assert float(dst.abs().sum()) == 0.0
    nat.copy_regions_noalloc(a, b, torch.cuda.current_stream(gpu_device).cuda_stream)  # eagerly it still works
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
