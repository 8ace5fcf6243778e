"""The C-ABI library: loads, exports what the header declares, validates descriptors (no GPU)."""

import os
import re

import numpy as np
import pytest

from etha_amd import _native as nat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_functions():
    text = open(os.path.join(ROOT, "include", "etha_reshard.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(etha_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    declared = _header_functions()
    assert len(declared) >= 15
    lib = nat.lib()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(nat.exported_symbols()) == declared
    assert lib.etha_abi_version() == nat.ABI_VERSION


def test_struct_layouts_match_header():
    assert nat.CHUNK_DESC.itemsize == 6 * 8 + 3 * 8 * nat.ETHA_MAX_NDIM + 6 * 4
    assert nat.CHUNK_DESC.fields["start"][1] == 48
    assert nat.CHUNK_DESC.fields["ndim"][1] == 48 + 3 * 64
    info = nat.TableInfo()
    assert info.n_chunks == 0


def _desc(**kw):
    d = np.zeros(1, dtype=nat.CHUNK_DESC)
    d["tensor_ptr"], d["bucket_ptr"] = 0x10000, 0x900000
    d["ndim"] = 2
    d["shape"][0][:2] = [8, 16]
    d["stride"][0][:2] = [16, 1]
    d["tensor_dtype"] = d["wire_dtype"] = nat.F32
    for k, v in kw.items():
        if isinstance(v, (list, tuple)):
            d[k][0][: len(v)] = v
        else:
            d[k] = v
    return d


def test_host_only_table_and_tile_counts():
    t = nat.Table.create(_desc(), upload=False)
    info = t.info()
    assert (info.n_chunks, info.payload_bytes) == (1, 8 * 16 * 4)
    assert info.tile_threads % 64 == 0  # a tile is executed by tile_threads / 64 one-wavefront workgroups
    run, row = t.tiles()
    assert len(run) == 1 and len(row) == 0  # fully contiguous: one run of 32 16-byte units
    assert int(run[0]["n"]) == 32 and int(run[0]["a"]) == 0x10000 and int(run[0]["b"]) == 0x900000
    with pytest.raises(nat.EthaNativeError, match="without upload"):
        t.pack(0, 1)


def test_validation_rejects_bad_descriptors():
    with pytest.raises(nat.EthaNativeError, match="leaves the allowed range"):
        nat.Table.create(_desc(tensor_lo=0x10000, tensor_hi=0x10000 + 8 * 16 * 4 - 1), upload=False)
    with pytest.raises(nat.EthaNativeError, match="leave the bucket buffer"):
        nat.Table.create(_desc(bucket_lo=0x900000, bucket_hi=0x900000 + 100), upload=False)
    with pytest.raises(nat.EthaNativeError, match="ndim"):
        nat.Table.create(_desc(ndim=9), upload=False)
    with pytest.raises(nat.EthaNativeError, match="can only be moved, not converted"):
        nat.Table.create(_desc(tensor_dtype=nat.B32, wire_dtype=nat.F32), upload=False)
    generic = nat.Table.create(_desc(tensor_dtype=nat.I32, wire_dtype=nat.F32), upload=False)  # a value type: converted
    assert all(int(m) & (1 << 20) for tiles in generic.tiles() for m in tiles["meta"])
    with pytest.raises(nat.EthaNativeError, match="unknown"):
        nat.Table.create(_desc(wire_dtype=99), upload=False)
    with pytest.raises(nat.EthaNativeError, match="null tensor"):
        nat.Table.create(_desc(tensor_ptr=0), upload=False)
    with pytest.raises(nat.EthaNativeError, match="partial pointer range"):
        nat.Table.create(_desc(n_partials=2, partial_first=0), upload=False)
    with pytest.raises(nat.EthaNativeError, match="not aligned"):
        nat.Table.create(_desc(tensor_ptr=0x10002, wire_dtype=nat.BF16), upload=False)
    ok = nat.Table.create(_desc(tensor_lo=0x10000, tensor_hi=0x10000 + 8 * 16 * 4), upload=False)
    with pytest.raises(nat.EthaNativeError, match="exceeds table"):
        ok.pack(0, 2)


def test_empty_and_zero_sized():
    t = nat.Table.create(np.zeros(0, dtype=nat.CHUNK_DESC), upload=False)
    assert t.info().n_chunks == 0
    t = nat.Table.create(_desc(shape=[0, 16]), upload=False)
    assert t.info().n_run_tiles + t.info().n_row_tiles == 0


def test_executor_refuses_cpu_tensors():
    import torch
    from torch.distributed.tensor.placement_types import Shard

    from etha_amd.world import ReshardJob, TensorSpec

    job = ReshardJob([TensorSpec("w", (8, 8), [0, 1], (Shard(0),), [2, 3], (Shard(1),), torch.float32)],
                     device="cpu", bucket_size=None)
    with pytest.raises(RuntimeError, match="no CPU path"):
        job.run()


def test_ipc_entry_points_reject_bad_arguments_without_a_gpu():
    import ctypes

    h = nat.IpcHandle()
    h.size = 2 << 30  # allocations of 2 GiB and more are refused before any HIP call
    out = ctypes.c_void_p()
    assert nat.lib().etha_ipc_open(ctypes.byref(h), ctypes.byref(out)) == nat.ERR_UNSUPPORTED
    assert b"under 2 GiB" in nat.lib().etha_last_error()
    assert nat.lib().etha_ipc_open(None, ctypes.byref(out)) == nat.ERR_INVALID
    with pytest.raises(nat.EthaNativeError, match="not returned by etha_ipc_open"):
        nat.ipc_close(0x1234)
    nat.ipc_close(0)  # null is a no-op
    assert nat.lib().etha_arena_create(0, ctypes.byref(out)) == nat.ERR_INVALID


def test_missing_library_fails_loudly(tmp_path):
    """No fallback: with the library absent, the first use of the product raises and names the build step."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import torch\n"
        "from torch.distributed.tensor.placement_types import Shard\n"
        "from etha_amd.world import ReshardJob, TensorSpec\n"
        "from etha_amd.comm import LoopbackWire\n"
        "spec = TensorSpec('w', (8, 8), [0, 1], (Shard(0),), [2], (Shard(1),), torch.float32)\n"
        "job = ReshardJob([spec], device='cpu', wire=LoopbackWire('cpu', host_inspection=True))\n"
        "job.wire.plan(job.send_buckets[0])\n"
    )
    env = dict(os.environ, ETHA_AMD_LIB=str(tmp_path / "absent.so"), PYTHONPATH=root)
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=120)
    assert proc.returncode != 0
    assert "is missing: the HIP extension is not built" in proc.stderr and "no CPU fallback" in proc.stderr


def test_library_reports_the_sources_it_was_built_from():
    """The harnesses rebuild a library that is older than the tree: the library carries a digest of its sources."""
    from etha_amd import build

    assert build.library_hash(build.LIB_PATH) == build.source_hash()
    assert nat.lib().etha_source_hash().decode() == build.source_hash()
    assert build.library_hash(os.path.join(ROOT, "README.md")) is None  # a file without the marker counts as stale


def test_exceptions_stay_inside_the_library(tmp_path):
    """The ABI is plain C: a C++ exception raised while a tile program is being compiled (a host allocation that
    fails) comes back as ETHA_ERR_NOMEM with a message, never as an exception.  A test build of the library
    raises std::bad_alloc once a program passes 40 tiles."""
    import subprocess
    import sys

    from etha_amd import build

    lib_path = str(tmp_path / "libetha_throwing.so")
    build.build_library(defines=("ETHA_TEST_THROW_AT_TILE=40",), out_path=lib_path)
    code = (
        "import numpy as np\n"
        "from etha_amd import _native as nat\n"
        "def desc(rows):\n"
        "    d = np.zeros(1, dtype=nat.CHUNK_DESC)\n"
        "    d['tensor_ptr'], d['bucket_ptr'], d['ndim'] = 0x10000, 0x9000000, 2\n"
        "    d['shape'][0][:2] = [rows, 4096]\n"
        "    d['stride'][0][:2] = [4096, 1]\n"
        "    d['tensor_dtype'] = d['wire_dtype'] = nat.F32\n"
        "    return d\n"
        "small = nat.Table.create(desc(8), upload=False)\n"  # 8 tiles: below the limit
        "assert small.info().n_run_tiles == 8\n"
        "for make in (lambda: nat.Table.create(desc(64), upload=False),\n"
        "             lambda: nat.Table.create_selfcopy(desc(64), desc(64), upload=False)):\n"
        "    try:\n"
        "        make()\n"
        "    except nat.EthaNativeError as e:\n"
        "        assert e.code == nat.ERR_NOMEM and 'out of host memory' in str(e), str(e)\n"
        "    else:\n"
        "        raise SystemExit('the oversized program was accepted')\n"
        "assert nat.Table.create(desc(8), upload=False).info().n_run_tiles == 8\n"  # the library still works
        "print('contained')\n"
    )
    env = dict(os.environ, ETHA_AMD_LIB=lib_path, PYTHONPATH=ROOT)
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=180)
    assert proc.returncode == 0 and "contained" in proc.stdout, proc.stderr[-2000:]
