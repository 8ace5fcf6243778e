"""ctypes binding of ``libetha_reshard.so`` (the C ABI declared in ``include/etha_reshard.h``).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_int, c_uint32, c_uint64, c_void_p

import numpy as np

from .build import LIB_PATH

ETHA_MAX_NDIM = 8
ABI_VERSION = 6
LAUNCH_UNORDERED = 1  # ETHA_LAUNCH_UNORDERED
SEG_PACK, SEG_UNPACK, SEG_REDUCE_PACK, SEG_SELFCOPY = 0, 1, 2, 3  # ETHA_SEG_*
MAX_SEGMENTS = 16

# element type codes (include/etha_reshard.h)
F16, BF16, F32, F64, B8, B16, B32, B64, I8, U8, I16, I32, I64, BOOL, F8E4M3, F8E5M2 = range(16)
REDUCE_OPS = {"sum": 0, "avg": 1, "max": 2, "min": 3, "product": 4}

ERR_INVALID, ERR_UNSUPPORTED, ERR_HIP, ERR_NOMEM = -1, -2, -3, -4

# numpy mirror of ``struct EthaChunkDesc``
CHUNK_DESC = np.dtype(
    [
        ("tensor_ptr", "<u8"),
        ("tensor_lo", "<u8"),
        ("tensor_hi", "<u8"),
        ("bucket_ptr", "<u8"),
        ("bucket_lo", "<u8"),
        ("bucket_hi", "<u8"),
        ("start", "<i8", (ETHA_MAX_NDIM,)),
        ("shape", "<i8", (ETHA_MAX_NDIM,)),
        ("stride", "<i8", (ETHA_MAX_NDIM,)),
        ("ndim", "<u4"),
        ("tensor_dtype", "<u4"),
        ("wire_dtype", "<u4"),
        ("n_partials", "<u4"),
        ("partial_first", "<u4"),
        ("reduce_op", "<u4"),
    ],
    align=True,
)
assert CHUNK_DESC.itemsize == 264, CHUNK_DESC.itemsize

RUN_TILE = np.dtype([("a", "<u8"), ("b", "<u8"), ("n", "<u4"), ("meta", "<u4")])
ROW_TILE = np.dtype(
    [
        ("a", "<u8"),
        ("b", "<u8"),
        ("a_pitch", "<i8"),
        ("b_pitch", "<i8"),
        ("n", "<u4"),
        ("meta", "<u4"),
        ("run", "<u4"),
        ("c0", "<u4"),
        ("peer_first", "<u4"),
        ("n_peers", "<u4"),
        ("reduce_op", "<u4"),
        ("via", "<u4"),
    ]
)
TRANS_TILE = np.dtype([("a", "<u8"), ("b", "<u8"), ("a_pitch", "<i8"), ("b_pitch", "<i8"), ("nj", "<u4"), ("nk", "<u4"),
                       ("es_log2", "<u4"), ("cvt", "<u4"), ("peer_first", "<u4"), ("n_peers", "<u4"), ("reduce_op", "<u4"),
                       ("via", "<u4")])
TRANS_TYPED = 1 << 8  # TransTile.cvt: a block of the typed transposing kernel
assert RUN_TILE.itemsize == 24 and ROW_TILE.itemsize == 64 and TRANS_TILE.itemsize == 64


class Segment(ctypes.Structure):
    """EthaSegment: one chunk range of one table, run as the entry point named by ``kind`` would."""

    _fields_ = [("table", c_void_p), ("kind", c_uint32), ("first", c_uint32), ("count", c_uint32), ("reserved", c_uint32)]


class ScheduleCall(ctypes.Structure):
    """EthaScheduleCall: one recorded launch call (a set of segments, or one range run by itself)."""

    _fields_ = [("first_segment", c_uint32), ("n_segments", c_uint32), ("flags", c_uint32), ("single", c_uint32)]


class ScheduleInfo(ctypes.Structure):
    _fields_ = [("n_calls", c_uint32), ("n_kernel_launches", c_uint32), ("n_tables", c_uint32), ("reserved", c_uint32)]


class TableInfo(ctypes.Structure):
    _fields_ = [
        ("n_chunks", c_uint32),
        ("n_run_tiles", c_uint32),
        ("n_row_tiles", c_uint32),
        ("tile_threads", c_uint32),
        ("device_bytes", c_uint64),
        ("payload_bytes", c_uint64),
        ("n_trans_tiles", c_uint32),
        ("reserved", c_uint32),
    ]


class IpcHandle(ctypes.Structure):
    _fields_ = [("handle", ctypes.c_uint8 * 64), ("offset", c_uint64), ("size", c_uint64)]


class EthaNativeError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, func: str, code: int, message: str):
        super().__init__(f"{func} failed ({code}): {message}")
        self.code = code


# name -> (restype, argtypes); every symbol the header declares
_SIGNATURES = {
    "etha_abi_version": (c_int, []),
    "etha_last_error": (c_char_p, []),
    "etha_source_hash": (c_char_p, []),
    "etha_table_create": (c_int, [c_void_p, c_uint32, c_void_p, c_uint32, c_int, POINTER(c_void_p)]),
    "etha_selfcopy_table_create": (c_int, [c_void_p, c_void_p, c_uint32, c_int, POINTER(c_void_p)]),
    "etha_direct_table_create": (c_int, [c_void_p, c_void_p, c_uint32, c_void_p, c_uint32, c_int, POINTER(c_void_p)]),
    "etha_table_destroy": (c_int, [c_void_p]),
    "etha_table_info": (c_int, [c_void_p, POINTER(TableInfo)]),
    "etha_table_read_tiles": (c_int, [c_void_p, c_int, c_void_p, c_uint64, POINTER(c_uint64)]),
    "etha_table_read_ranges": (c_int, [c_void_p, c_void_p, c_void_p]),
    "etha_table_read_trans_ranges": (c_int, [c_void_p, c_void_p]),
    "etha_table_optimize_range": (c_int, [c_void_p, c_uint32, c_uint32]),
    "etha_table_read_ordered": (c_int, [c_void_p, c_uint32, c_uint32, c_int, c_void_p, c_uint64, POINTER(c_uint64)]),
    "etha_pack_bucket": (c_int, [c_void_p, c_uint32, c_uint32, c_void_p, c_uint32]),
    "etha_unpack_bucket": (c_int, [c_void_p, c_uint32, c_uint32, c_void_p, c_uint32]),
    "etha_reduce_pack_bucket": (c_int, [c_void_p, c_uint32, c_uint32, c_void_p, c_uint32]),
    "etha_selfcopy_bucket": (c_int, [c_void_p, c_uint32, c_uint32, c_void_p, c_uint32]),
    "etha_launch_segments": (c_int, [c_void_p, c_uint32, c_void_p, c_uint32]),
    "etha_schedule_create": (c_int, [c_void_p, c_uint32, c_void_p, c_uint32, POINTER(c_void_p)]),
    "etha_schedule_launch": (c_int, [c_void_p, c_void_p]),
    "etha_schedule_info": (c_int, [c_void_p, POINTER(ScheduleInfo)]),
    "etha_schedule_destroy": (c_int, [c_void_p]),
    "etha_kernel_launches": (c_uint64, []),
    "etha_noalloc_setup": (c_int, []),
    "etha_copy_regions_noalloc": (c_int, [c_void_p, c_void_p, c_uint32, c_void_p]),
    "etha_arena_create": (c_int, [c_uint64, POINTER(c_void_p)]),
    "etha_arena_destroy": (c_int, [c_void_p]),
    "etha_ipc_export": (c_int, [c_void_p, POINTER(IpcHandle)]),
    "etha_ipc_open": (c_int, [POINTER(IpcHandle), POINTER(c_void_p)]),
    "etha_ipc_close": (c_int, [c_void_p]),
}

_lib = None


def exported_symbols() -> list[str]:
    return list(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load the HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension is not built. "
                "Run `python -m etha_amd.build` (needs hipcc); there is no CPU fallback."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the symbol is not exported
            fn.restype = restype
            fn.argtypes = argtypes
        if handle.etha_abi_version() != ABI_VERSION:
            raise RuntimeError(f"ABI mismatch: library {handle.etha_abi_version()}, binding {ABI_VERSION}")
        _lib = handle
    return _lib


def _check(func: str, rc: int) -> None:
    if rc != 0:
        raise EthaNativeError(func, rc, lib().etha_last_error().decode(errors="replace"))


class Table:
    """Owner of one compiled tile program (``EthaTable*``)."""

    def __init__(self, handle: int, keepalive: tuple = ()):
        self._h = c_void_p(handle)
        self._keepalive = keepalive

    @classmethod
    def create(cls, descs: np.ndarray, partial_ptrs: np.ndarray | None = None, upload: bool = True) -> "Table":
        descs = np.ascontiguousarray(descs, dtype=CHUNK_DESC)
        out = c_void_p()
        pp, npp = None, 0
        if partial_ptrs is not None and len(partial_ptrs):
            partial_ptrs = np.ascontiguousarray(partial_ptrs, dtype=np.uint64)
            pp, npp = partial_ptrs.ctypes.data, len(partial_ptrs)
        rc = lib().etha_table_create(descs.ctypes.data, len(descs), pp, npp, int(upload), byref(out))
        _check("etha_table_create", rc)
        return cls(out.value)

    @classmethod
    def create_selfcopy(cls, src: np.ndarray, dst: np.ndarray, upload: bool = True,
                        partial_ptrs: np.ndarray | None = None) -> "Table":
        """Region-to-region table.  With ``partial_ptrs`` some sources may be Partial (``etha_direct_table_create``)."""
        src = np.ascontiguousarray(src, dtype=CHUNK_DESC)
        dst = np.ascontiguousarray(dst, dtype=CHUNK_DESC)
        if len(src) != len(dst):
            raise ValueError("src and dst descriptor arrays differ in length")
        out = c_void_p()
        if partial_ptrs is not None and len(partial_ptrs):
            partial_ptrs = np.ascontiguousarray(partial_ptrs, dtype=np.uint64)
            rc = lib().etha_direct_table_create(src.ctypes.data, dst.ctypes.data, len(src), partial_ptrs.ctypes.data,
                                                len(partial_ptrs), int(upload), byref(out))
            _check("etha_direct_table_create", rc)
        else:
            rc = lib().etha_selfcopy_table_create(src.ctypes.data, dst.ctypes.data, len(src), int(upload), byref(out))
            _check("etha_selfcopy_table_create", rc)
        return cls(out.value)

    def info(self) -> TableInfo:
        info = TableInfo()
        _check("etha_table_info", lib().etha_table_info(self._h, byref(info)))
        return info

    def tiles(self) -> tuple[np.ndarray, np.ndarray]:
        """Host copies of the (run tiles, row tiles) arrays."""
        res = []
        for which, dt in ((0, RUN_TILE), (1, ROW_TILE)):
            need = c_uint64()
            _check("etha_table_read_tiles", lib().etha_table_read_tiles(self._h, which, None, 0, byref(need)))
            arr = np.zeros(need.value // dt.itemsize, dtype=dt)
            if need.value:
                _check(
                    "etha_table_read_tiles",
                    lib().etha_table_read_tiles(self._h, which, arr.ctypes.data, need.value, byref(need)),
                )
            res.append(arr)
        return res[0], res[1]

    def trans_tiles(self) -> np.ndarray:
        """Host copy of the transposing tiles."""
        need = c_uint64()
        _check("etha_table_read_tiles", lib().etha_table_read_tiles(self._h, 2, None, 0, byref(need)))
        arr = np.zeros(need.value // TRANS_TILE.itemsize, dtype=TRANS_TILE)
        if need.value:
            _check("etha_table_read_tiles",
                   lib().etha_table_read_tiles(self._h, 2, arr.ctypes.data, need.value, byref(need)))
        return arr

    def trans_ranges(self) -> np.ndarray:
        out = np.zeros(self.info().n_chunks + 1, dtype=np.uint32)
        _check("etha_table_read_trans_ranges", lib().etha_table_read_trans_ranges(self._h, out.ctypes.data))
        return out

    def ranges(self) -> tuple[np.ndarray, np.ndarray]:
        n = self.info().n_chunks
        run_begin = np.zeros(n + 1, dtype=np.uint32)
        row_begin = np.zeros(n + 1, dtype=np.uint32)
        _check(
            "etha_table_read_ranges",
            lib().etha_table_read_ranges(self._h, run_begin.ctypes.data, row_begin.ctypes.data),
        )
        return run_begin, row_begin

    def optimize_range(self, first: int, count: int) -> None:
        """Order the tiles of a range that is always launched as one unit by written address."""
        _check("etha_table_optimize_range", lib().etha_table_optimize_range(self._h, first, count))

    def ordered_tiles(self, first: int, count: int) -> tuple[np.ndarray, np.ndarray]:
        res = []
        for which, dt in ((0, RUN_TILE), (1, ROW_TILE)):
            need = c_uint64()
            _check("etha_table_read_ordered",
                   lib().etha_table_read_ordered(self._h, first, count, which, None, 0, byref(need)))
            arr = np.zeros(need.value // dt.itemsize, dtype=dt)
            if need.value:
                _check("etha_table_read_ordered",
                       lib().etha_table_read_ordered(self._h, first, count, which, arr.ctypes.data, need.value, byref(need)))
            res.append(arr)
        return res[0], res[1]

    def ordered_gather(self, first: int, count: int) -> np.ndarray:
        """Piece addresses of the gather tiles of an optimized range (``peer_first`` of such a tile indexes it)."""
        need = c_uint64()
        _check("etha_table_read_ordered", lib().etha_table_read_ordered(self._h, first, count, 3, None, 0, byref(need)))
        arr = np.zeros(need.value // 8, dtype=np.uint64)
        if need.value:
            _check("etha_table_read_ordered",
                   lib().etha_table_read_ordered(self._h, first, count, 3, arr.ctypes.data, need.value, byref(need)))
        return arr

    def pack(self, first: int, count: int, stream: int = 0, flags: int = 0) -> None:
        _check("etha_pack_bucket", lib().etha_pack_bucket(self._h, first, count, c_void_p(stream), flags))

    def unpack(self, first: int, count: int, stream: int = 0, flags: int = 0) -> None:
        _check("etha_unpack_bucket", lib().etha_unpack_bucket(self._h, first, count, c_void_p(stream), flags))

    def reduce_pack(self, first: int, count: int, stream: int = 0, flags: int = 0) -> None:
        _check("etha_reduce_pack_bucket", lib().etha_reduce_pack_bucket(self._h, first, count, c_void_p(stream), flags))

    def selfcopy(self, first: int, count: int, stream: int = 0, flags: int = 0) -> None:
        _check("etha_selfcopy_bucket", lib().etha_selfcopy_bucket(self._h, first, count, c_void_p(stream), flags))

    def close(self) -> None:
        if self._h:
            lib().etha_table_destroy(self._h)
            self._h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


NOALLOC_SCRATCH_BYTES = 4 << 20  # ETHA_NOALLOC_SCRATCH_BYTES


def noalloc_setup() -> None:
    """Once per device, with that device current: prepare ``copy_regions_noalloc``."""
    _check("etha_noalloc_setup", lib().etha_noalloc_setup())


def copy_regions_noalloc(src: np.ndarray, dst: np.ndarray, stream: int = 0) -> None:
    """Copy src region i into dst region i (descriptor arrays as for ``Table.create_selfcopy``) without any device
    allocation; at most ``NOALLOC_SCRATCH_BYTES`` of tile program per call."""
    src = np.ascontiguousarray(src, dtype=CHUNK_DESC)
    dst = np.ascontiguousarray(dst, dtype=CHUNK_DESC)
    if len(src) != len(dst):
        raise ValueError("src and dst descriptor arrays differ in length")
    _check("etha_copy_regions_noalloc",
           lib().etha_copy_regions_noalloc(src.ctypes.data, dst.ctypes.data, len(src), c_void_p(stream)))


def arena_create(nbytes: int) -> int:
    out = c_void_p()
    _check("etha_arena_create", lib().etha_arena_create(nbytes, byref(out)))
    return out.value


def arena_destroy(ptr: int) -> None:
    _check("etha_arena_destroy", lib().etha_arena_destroy(c_void_p(ptr)))


def ipc_export(ptr: int) -> bytes:
    h = IpcHandle()
    _check("etha_ipc_export", lib().etha_ipc_export(c_void_p(ptr), byref(h)))
    return bytes(h)


def kernel_launches() -> int:
    """Kernels launched through the library by this process so far."""
    return int(lib().etha_kernel_launches())


def launch_segments(segments, stream: int = 0, flags: int = 0) -> None:
    """Issue ``segments`` - ``(table, kind, first, count)`` with ``kind`` one of ``SEG_*`` - as one set of launches
    that do not depend on each other (``etha_launch_segments``)."""
    arr = (Segment * max(len(segments), 1))()
    for i, (table, kind, first, count) in enumerate(segments):
        arr[i].table, arr[i].kind, arr[i].first, arr[i].count = table._h, kind, first, count
    _check("etha_launch_segments", lib().etha_launch_segments(arr, len(segments), c_void_p(stream), flags))


class Schedule:
    """Owner of one recorded transfer (``EthaSchedule*``): launch calls planned once, re-issued with one call.

    ``calls`` is a list of ``(segments, flags, single)`` in issue order, ``segments`` as for :func:`launch_segments`;
    ``single`` marks a one-segment call that runs as its single-range entry point would.  The tables are kept alive.
    """

    def __init__(self, calls):
        n_seg = sum(len(c[0]) for c in calls)
        segs = (Segment * max(n_seg, 1))()
        recs = (ScheduleCall * max(len(calls), 1))()
        self._tables = []
        k = 0
        for i, (segments, flags, single) in enumerate(calls):
            recs[i].first_segment, recs[i].n_segments, recs[i].flags, recs[i].single = k, len(segments), flags, int(bool(single))
            for table, kind, first, count in segments:
                segs[k].table, segs[k].kind, segs[k].first, segs[k].count = table._h, kind, first, count
                self._tables.append(table)
                k += 1
        out = c_void_p()
        _check("etha_schedule_create", lib().etha_schedule_create(segs, n_seg, recs, len(calls), byref(out)))
        self._h = out
        self._launch = lib().etha_schedule_launch

    def launch(self, stream: int = 0) -> None:
        rc = self._launch(self._h, stream)
        if rc != 0:
            _check("etha_schedule_launch", rc)

    def info(self) -> ScheduleInfo:
        info = ScheduleInfo()
        _check("etha_schedule_info", lib().etha_schedule_info(self._h, byref(info)))
        return info

    def close(self) -> None:
        if self._h:
            lib().etha_schedule_destroy(self._h)
            self._h = c_void_p()
        self._tables = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def ipc_open(handle_bytes: bytes) -> int:
    h = IpcHandle.from_buffer_copy(handle_bytes)
    out = c_void_p()
    _check("etha_ipc_open", lib().etha_ipc_open(byref(h), byref(out)))
    return out.value


def ipc_close(ptr: int) -> None:
    _check("etha_ipc_close", lib().etha_ipc_close(c_void_p(ptr)))
