"""From planner objects to the flat chunk-descriptor table the HIP library consumes.

Everything here runs once per registered batch ("plan once, transfer N times"): chunks are
turned into ``EthaChunkDesc`` rows (``include/etha_reshard.h``), the library compiles them into a
device-resident tile program, and a transfer is then a handful of kernel launches.  This is the
replacement for the per-transfer Python loops of ``Bucket.prepare`` / ``Bucket.finalize``
(``src/etha/comm/ir.py:246-259,306-308``).
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from .. import _native as nat
from .ir import Bucket, Chunk

_FLOAT_CODES = {
    torch.float16: nat.F16,
    torch.bfloat16: nat.BF16,
    torch.float32: nat.F32,
    torch.float64: nat.F64,
}
# value types beyond the four floats: converted element by element with ``Tensor.to`` semantics
_VALUE_CODES = {
    torch.int8: nat.I8,
    torch.uint8: nat.U8,
    torch.int16: nat.I16,
    torch.int32: nat.I32,
    torch.int64: nat.I64,
    torch.bool: nat.BOOL,
    torch.float8_e4m3fn: nat.F8E4M3,
    torch.float8_e5m2: nat.F8E5M2,
}
_OPAQUE_CODES = {1: nat.B8, 2: nat.B16, 4: nat.B32, 8: nat.B64}


def dtype_code(dtype: torch.dtype) -> int:
    if dtype in _FLOAT_CODES:
        return _FLOAT_CODES[dtype]
    if dtype in _VALUE_CODES:
        return _VALUE_CODES[dtype]
    code = _OPAQUE_CODES.get(dtype.itemsize)
    if code is None:
        raise NotImplementedError(f"dtype {dtype} (itemsize {dtype.itemsize}) is not supported")
    return code


def check_cast(src: torch.dtype, dst: torch.dtype) -> None:
    """Same dtype is a byte move; otherwise both must be value types the library converts (the floats, the
    integers, bool, the 8-bit floats).  Other types (complex, unsigned 16/32/64) can only be moved."""
    known = (_FLOAT_CODES, _VALUE_CODES)
    if src != dst and not (any(src in k for k in known) and any(dst in k for k in known)):
        raise NotImplementedError(f"conversion {src} -> {dst}: only floats, integers, bool and 8-bit floats are converted")


def reduce_op_word(op) -> int:
    """``reduce_op`` of a descriptor: the op's code, or ``ETHA_REDUCE_LEVELS`` for ``((op, size), ...)`` levels."""
    if isinstance(op, str):
        return nat.REDUCE_OPS[op]
    ops = [nat.REDUCE_OPS[o] for o, _ in op]
    sizes = [n for _, n in op]
    if len(op) == 2:  # two levels: the outer one takes what the inner one leaves
        return ops[0] | (ops[1] << 3) | (ops[1] << 6) | (sizes[0] << 16) | (1 << 24)
    return ops[0] | (ops[1] << 3) | (ops[2] << 6) | (sizes[0] << 16) | (sizes[1] << 24)


def _storage_range(t) -> tuple[int, int]:
    st = t.untyped_storage()
    lo = st.data_ptr()
    return lo, lo + st.nbytes()


def fill_region(row, tensor: torch.Tensor, slices: tuple, chunk_shape: tuple) -> None:
    """Tensor-side fields of one descriptor row: pointer, strides, slice starts, chunk shape."""
    nd = tensor.dim()
    if nd > nat.ETHA_MAX_NDIM:
        raise NotImplementedError(f"tensors of more than {nat.ETHA_MAX_NDIM} dims are not supported")
    if len(slices) > nd:
        raise ValueError(f"slice of rank {len(slices)} on a tensor of rank {nd}")
    shape = tuple(tensor.shape)
    starts, extents = [], []
    for d in range(nd):
        if d < len(slices):
            s = slices[d]
            if s.step not in (None, 1):
                raise NotImplementedError("chunk slices must have unit step")
            lo, hi, _ = s.indices(shape[d])
            starts.append(lo)
            extents.append(max(hi - lo, 0))
        else:
            starts.append(0)
            extents.append(shape[d])
    cs = tuple(chunk_shape)
    if nd == 0:
        if int(np.prod(cs, dtype=np.int64)) != 1:
            raise ValueError(f"chunk_shape {cs} does not match a scalar tensor")
    elif tuple(extents) != cs:
        raise ValueError(f"chunk_shape {cs} does not match the slice extents {tuple(extents)} of tensor {shape}")
    row["tensor_ptr"] = tensor.data_ptr()
    lo, hi = _storage_range(tensor)
    row["tensor_lo"], row["tensor_hi"] = lo, hi
    row["ndim"] = nd
    row["start"][:nd] = starts
    row["shape"][:nd] = extents
    row["stride"][:nd] = tensor.stride()
    row["tensor_dtype"] = dtype_code(tensor.dtype)


@dataclass(eq=False)
class Slot:
    """A bucket buffer inside the pool.  In a ring pool one slot serves every ``depth``-th bucket of its channel."""

    ptr: int
    nbytes: int
    lo: int  # bounds of the allocation holding the slot
    hi: int
    filled: int = 0  # number of times a pack has been enqueued into this slot
    drained: int = 0  # number of unpacks enqueued from it (per consumer bookkeeping is the wire's job)
    borrowed: bool = False  # the slot is source-tensor memory (zero-copy single-chunk bucket, direct wire), not pool memory
    keepalive: object = None  # the tensor(s) a borrowed slot aliases
    # direct wire: per chunk of the send bucket ``(source tensor, src_slice, wire dtype, Partial peers or None)``;
    # the consumer copies from these regions straight into its own tensors and no bucket buffer exists (ptr is 0)
    sources: list | None = None
    # the send bucket (a wire entry) whose bytes are in the slot and have not been read by all of its
    # consumers yet; None = free.  A ring slot is packed again only when it is free.
    holder: object = None


def _rows_to_array(rows: list[np.ndarray]) -> np.ndarray:
    """One descriptor array from 0-d rows (np.stack spends most of its time promoting the struct dtype)."""
    out = np.empty(len(rows), dtype=nat.CHUNK_DESC)
    for i, r in enumerate(rows):
        out[i] = r
    return out


class DescBuilder:
    """Accumulates descriptor rows bucket by bucket and remembers each bucket's chunk range."""

    def __init__(self) -> None:
        self.rows: list[np.ndarray] = []
        self.partial_ptrs: list[int] = []
        self.keepalive: list[torch.Tensor] = []

    def __len__(self) -> int:
        return len(self.rows)

    def add_chunk(self, chunk: Chunk, tensor: torch.Tensor, slices: tuple, slot: Slot, offset: int,
                  reduce: bool) -> None:
        row = np.zeros((), dtype=nat.CHUNK_DESC)
        fill_region(row, tensor, slices, chunk.chunk_shape)
        wire = chunk.transfer_dtype or tensor.dtype
        check_cast(tensor.dtype, wire)
        row["wire_dtype"] = dtype_code(wire)
        row["bucket_ptr"] = slot.ptr + offset
        row["bucket_lo"], row["bucket_hi"] = slot.ptr, slot.ptr + slot.nbytes
        peers = chunk.partial_peers() if reduce else None
        if peers is not None:
            tensors, op = peers
            for t in tensors:
                if t.dtype != tensor.dtype or tuple(t.shape) != tuple(tensor.shape) or t.stride() != tensor.stride():
                    raise NotImplementedError("Partial peers must share dtype, shape and strides")
                if t.device != tensor.device:
                    raise NotImplementedError("Partial peers must live on the same device")
            row["n_partials"] = len(tensors)
            row["partial_first"] = len(self.partial_ptrs)
            row["reduce_op"] = reduce_op_word(op)
            self.partial_ptrs.extend(t.data_ptr() for t in tensors)
            self.keepalive.extend(tensors)
        self.keepalive.append(tensor)
        self.rows.append(row)

    def build(self, upload: bool = True) -> nat.Table | None:
        if not self.rows:
            return None
        descs = _rows_to_array(self.rows)
        ptrs = np.asarray(self.partial_ptrs, dtype=np.uint64) if self.partial_ptrs else None
        return nat.Table.create(descs, ptrs, upload=upload)


class SelfCopyBuilder:
    """Accumulates region-to-region rows: LOCAL chunks, and the chunks of a direct (bucket-less) wire."""

    def __init__(self) -> None:
        self.src: list[np.ndarray] = []
        self.dst: list[np.ndarray] = []
        self.partial_ptrs: list[int] = []
        self.keepalive: list[torch.Tensor] = []

    def __len__(self) -> int:
        return len(self.src)

    def add_chunk(self, chunk: Chunk) -> None:
        src_t = chunk.src_tensor if chunk.src_tensor is not None else chunk.tensor
        # a same-rank chunk of a Partial source: the members are combined straight into the target region
        self.add_pair(src_t, chunk.src_slice, chunk.tensor, chunk.dst_slice, chunk.chunk_shape,
                      peers=chunk.partial_peers(), wire_dtype=chunk.transfer_dtype)

    def add_pair(self, src_t, src_slice: tuple, dst_t, dst_slice: tuple, chunk_shape: tuple, peers=None,
                 wire_dtype: torch.dtype | None = None) -> None:
        """Copy ``src_t[src_slice]`` to ``dst_t[dst_slice]`` (same shape), converting between their dtypes.
        ``peers = (tensors, op)`` makes the source a Partial one: the members' slices are combined, rounded to
        ``wire_dtype`` and then converted, as the bucket path would."""
        a = np.zeros((), dtype=nat.CHUNK_DESC)
        b = np.zeros((), dtype=nat.CHUNK_DESC)
        fill_region(a, src_t, src_slice, chunk_shape)
        fill_region(b, dst_t, dst_slice, chunk_shape)
        check_cast(src_t.dtype, dst_t.dtype)
        a["wire_dtype"] = a["tensor_dtype"]
        b["wire_dtype"] = b["tensor_dtype"]
        if peers is not None:
            tensors, op = peers
            wire = wire_dtype or src_t.dtype
            check_cast(src_t.dtype, wire)
            check_cast(wire, dst_t.dtype)
            for t in tensors:
                if t.dtype != src_t.dtype or tuple(t.shape) != tuple(src_t.shape) or t.stride() != src_t.stride():
                    raise NotImplementedError("Partial peers must share dtype, shape and strides")
                if t.device != src_t.device:
                    raise NotImplementedError("Partial peers must live on the same device")
            a["wire_dtype"] = dtype_code(wire)
            a["n_partials"] = len(tensors)
            a["partial_first"] = len(self.partial_ptrs)
            a["reduce_op"] = reduce_op_word(op)
            self.partial_ptrs.extend(t.data_ptr() for t in tensors)
            self.keepalive.extend(tensors)
        self.src.append(a)
        self.dst.append(b)
        self.keepalive += [src_t, dst_t]

    def build(self, upload: bool = True) -> nat.Table | None:
        if not self.src:
            return None
        ptrs = np.asarray(self.partial_ptrs, dtype=np.uint64) if self.partial_ptrs else None
        return nat.Table.create_selfcopy(_rows_to_array(self.src), _rows_to_array(self.dst), upload=upload,
                                         partial_ptrs=ptrs)


def region_hull(tensor, slices: tuple) -> tuple[int, int]:
    """Smallest byte interval covering ``tensor[slices]`` (empty regions give lo == hi).

    Pure arithmetic on shape/stride/data_ptr, so it also works for tensors that only exist as an
    IPC-mapped pointer.
    """
    shape, stride, es = tuple(tensor.shape), tuple(tensor.stride()), tensor.element_size()
    lo_el, span_el, empty = 0, 0, False
    for d, n in enumerate(shape):
        start, stop = 0, n
        if d < len(slices):
            start, stop, _ = slices[d].indices(n)
        ext = max(stop - start, 0)
        if ext == 0:
            empty = True
        lo_el += start * stride[d]
        span_el += (ext - 1) * stride[d] if ext > 0 else 0
    lo = tensor.data_ptr() + lo_el * es
    if empty:
        return lo, lo
    return lo, lo + (span_el + 1) * es


def zero_copy_region(bucket: Bucket):
    """``(address, storage lo, storage hi, keepalive tensor)`` when the bucket's bytes already exist, in bucket
    layout, inside its source tensor - else None.

    That is the reference's single-entry path: one chunk, its slice contiguous, no Partial reduce and no
    cast, so that ``bucket.buffer = chunk.buffer.view(uint8)`` aliases the tensor (``ir.py:238-244``)."""
    if len(bucket.chunks) != 1:
        return None
    c = bucket.chunks[0]
    t = c.tensor
    if c.source_partial_groups or t is None or (c.transfer_dtype or t.dtype) != t.dtype or c.nbytes == 0:
        return None
    shape, stride = tuple(t.shape), tuple(t.stride())
    start_el, expect, contiguous = 0, 1, True
    for d in range(len(shape) - 1, -1, -1):
        lo, hi = 0, shape[d]
        if d < len(c.src_slice):
            lo, hi, _ = c.src_slice[d].indices(shape[d])
        ext = hi - lo
        start_el += lo * stride[d]
        if ext != 1 and stride[d] != expect:
            contiguous = False
        expect *= ext
    if not contiguous:
        return None
    lo_b, hi_b = _storage_range(t)
    return t.data_ptr() + start_el * t.element_size(), lo_b, hi_b, t


def local_bucket_needs_staging(bucket: Bucket) -> bool:
    """True when some chunk's source bytes may overlap some chunk's destination bytes.

    The reference stages a bundled self-copy bucket through the bucket buffer - all reads happen
    before all writes (``ir.py:246-259,306-308``).  A direct copy gives the same result exactly
    when no source region overlaps a destination region, which is the common case.
    """
    srcs, dsts = [], []
    for c in bucket.chunks:
        src_t = c.src_tensor if c.src_tensor is not None else c.tensor
        srcs.append(region_hull(src_t, c.src_slice))
        dsts.append(region_hull(c.tensor, c.dst_slice))
    if bucket.chunks[0].source_partial_groups:
        return False  # the members' partials are separate tensors from the target
    if len(bucket.chunks) == 1:
        return False  # single-entry path of the reference copies directly (ir.py:238-244)
    for s_lo, s_hi in srcs:
        for d_lo, d_hi in dsts:
            if s_lo < d_hi and d_lo < s_hi:
                return True
    return False
