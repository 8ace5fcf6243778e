"""TEST INFRASTRUCTURE.  ctypes binding of ``reshard_oracle.c`` (built by ``oracle/Makefile``)."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

ORACLE_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(ORACLE_DIR, "liboracle.so")
MAX_NDIM = 8
F16, BF16, F32, F64, B8, B16, B32, B64, I8, U8, I16, I32, I64, BOOL, F8E4M3, F8E5M2 = range(16)
OPS = {"sum": 0, "avg": 1, "max": 2, "min": 3, "product": 4}


class OracleChunk(ctypes.Structure):
    _fields_ = [
        ("tensor", ctypes.c_void_p),
        ("start", ctypes.c_int64 * MAX_NDIM),
        ("shape", ctypes.c_int64 * MAX_NDIM),
        ("stride", ctypes.c_int64 * MAX_NDIM),
        ("ndim", ctypes.c_int32),
        ("tensor_dtype", ctypes.c_int32),
        ("wire_dtype", ctypes.c_int32),
        ("n_partials", ctypes.c_int32),
        ("peers", ctypes.POINTER(ctypes.c_void_p)),
        ("reduce_op", ctypes.c_int32),
        ("pad", ctypes.c_int32),
        ("bucket_off", ctypes.c_int64),
    ]


def build() -> str:
    subprocess.run(["make", "-C", ORACLE_DIR, "-B", "liboracle.so"], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        source = os.path.join(ORACLE_DIR, "reshard_oracle.c")
        if not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(source):
            build()  # missing, or older than its source
        h = ctypes.CDLL(LIB_PATH)
        h.oracle_f32_to_bf16.restype = ctypes.c_uint16
        h.oracle_f32_to_bf16.argtypes = [ctypes.c_uint32]
        h.oracle_f32_to_f16.restype = ctypes.c_uint16
        h.oracle_f32_to_f16.argtypes = [ctypes.c_uint32]
        h.oracle_bf16_to_f32.restype = ctypes.c_uint32
        h.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        h.oracle_f16_to_f32.restype = ctypes.c_uint32
        h.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        h.oracle_cast.restype = ctypes.c_int
        h.oracle_cast.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64]
        h.oracle_gather.restype = None
        h.oracle_gather.argtypes = [ctypes.POINTER(OracleChunk), ctypes.c_void_p]
        h.oracle_scatter.restype = None
        h.oracle_scatter.argtypes = [ctypes.POINTER(OracleChunk), ctypes.c_void_p]
        h.oracle_reduce.restype = ctypes.c_int
        h.oracle_reduce.argtypes = [ctypes.POINTER(OracleChunk), ctypes.c_void_p, ctypes.c_void_p]
        h.oracle_pack_bucket.restype = ctypes.c_int
        h.oracle_pack_bucket.argtypes = [ctypes.POINTER(OracleChunk), ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
        h.oracle_unpack_bucket.restype = ctypes.c_int
        h.oracle_unpack_bucket.argtypes = [ctypes.POINTER(OracleChunk), ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
        _lib = h
    return _lib


def cast(src: np.ndarray, src_dt: int, dst_dt: int, dst_np_dtype) -> np.ndarray:
    """Cast a contiguous array of raw element storage (e.g. uint16 for bf16) element-wise."""
    src = np.ascontiguousarray(src)
    out = np.empty(src.size, dtype=dst_np_dtype)
    rc = lib().oracle_cast(src.ctypes.data, src_dt, out.ctypes.data, dst_dt, src.size)
    if rc:
        raise ValueError("unsupported cast")
    return out.reshape(src.shape)


def make_chunk(base_ptr: int, start, shape, stride, tensor_dt: int, wire_dt: int, bucket_off: int = 0,
               peers: list[int] | None = None, op: str = "sum") -> OracleChunk:
    c = OracleChunk()
    c.tensor = base_ptr
    nd = len(shape)
    c.ndim = nd
    for i in range(nd):
        c.start[i], c.shape[i], c.stride[i] = int(start[i]), int(shape[i]), int(stride[i])
    c.tensor_dtype, c.wire_dtype = tensor_dt, wire_dt
    c.bucket_off = bucket_off
    if peers:
        arr = (ctypes.c_void_p * len(peers))(*peers)
        c.peers = ctypes.cast(arr, ctypes.POINTER(ctypes.c_void_p))
        c.n_partials = len(peers)
        c.reduce_op = OPS[op]
        c._keep = arr
    return c
