"""Build recipe for the HIP library (gfx950 only).

``python -m etha_amd.build`` compiles ``csrc/etha_reshard.hip`` into
``etha_amd/libetha_reshard.so`` next to this file.  hipcc cross-compiles, so no GPU is needed.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
SOURCE = os.path.join(PKG_DIR, "csrc", "etha_reshard.hip")
INCLUDE_DIR = os.path.join(REPO_DIR, "include")
# ETHA_AMD_LIB selects another build of the same library (kernel tuning experiments)
LIB_PATH = os.environ.get("ETHA_AMD_LIB") or os.path.join(PKG_DIR, "libetha_reshard.so")

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # kernel arguments arrive in scalar registers with the wave instead of through a load at its start: every
    # workgroup here lives only a few microseconds, and that load is on its critical path (measured +0.3 %)
    "-mllvm", "-amdgpu-kernarg-preload-count=8",
    "-fPIC",
    "-shared",
    "-std=c++17",
]


def hipcc_path() -> str:
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        raise RuntimeError("hipcc not found; the ROCm toolchain is required to build etha_amd")
    return path


HEADER = os.path.join(INCLUDE_DIR, "etha_reshard.h")


def source_hash() -> str:
    """Digest of the sources and compiler flags the library is built from; the library carries the one it was
    built with."""
    h = hashlib.sha256(" ".join(HIPCC_FLAGS).encode())
    for path in (SOURCE, HEADER):
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:32]


def library_hash(path: str) -> str | None:
    """The source digest a built library carries, read from the file (the library is not loaded: it must only
    ever be loaded after torch, so that both use one HIP runtime).  None for a library without one."""
    marker = b"etha-source-digest:"
    try:
        with open(path, "rb") as f:
            blob = f.read()
    except OSError:
        return None
    at = blob.find(marker)
    if at < 0:
        return None
    end = blob.find(b"\0", at)
    return blob[at + len(marker):end].decode(errors="replace")


def build_library(verbose: bool = False, defines: tuple[str, ...] = (), out_path: str | None = None) -> str:
    """Compile the shared library (always recompiles) and return its path."""
    out_path = out_path or LIB_PATH
    defines = (*defines, f'ETHA_SOURCE_HASH="{source_hash()}"')
    cmd = [hipcc_path(), *HIPCC_FLAGS, *[f"-D{d}" for d in defines], f"-I{INCLUDE_DIR}", "-o", out_path + ".tmp", SOURCE]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    if verbose and proc.stderr:
        sys.stderr.write(proc.stderr)
    os.replace(out_path + ".tmp", out_path)
    return out_path


def ensure_built() -> str:
    """Build the library only if none is there, or if the one there was built from other sources than the
    ones in the tree (test / benchmark harnesses; the product itself never builds: ``etha_amd._native.lib()``
    raises when the library is missing)."""
    if not os.path.exists(LIB_PATH):
        return build_library()
    if os.environ.get("ETHA_AMD_LIB"):
        return LIB_PATH  # an explicitly selected build (kernel tuning experiments) is taken as it is
    built_from = library_hash(LIB_PATH)
    if built_from != source_hash():
        sys.stderr.write(f"[etha_amd.build] {LIB_PATH} was built from other sources ({built_from}); rebuilding\n")
        return build_library()
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
