"""TEST INFRASTRUCTURE.  The reference's byte work, restated op for op on torch CPU tensors.

``run_rank`` does for one rank's bucket list what the reference's ``bucket_comm`` does
(``src/etha/comm/comm_methods.py:53-119``), with the wire replaced by an in-memory mailbox:

* source bucket  - ``Bucket.prepare`` (``ir.py:229-264``): single chunk: ``tensor[src_slice]``,
  ``.contiguous()``, (reduce), ``.to(transfer_dtype)``, viewed as bytes; several chunks: a fresh
  ``torch.empty(total_bytes, uint8)`` and per chunk ``narrow -> view(dtype) -> view(shape)`` +
  ``copy_``.  Then the buffer is "sent": stored in the mailbox under the wire key.
* target bucket  - the buffer is taken from the mailbox ("received"), then ``Bucket.finalize``
  (``ir.py:300-310``): per chunk ``.to(tensor.dtype)`` and ``tensor[dst_slice].copy_`` (``ir.py:134-141``).
* LOCAL bucket   - prepare then finalize on the same rank (``ir.py:238-244,254-257``).

The Partial collapse (``ir.py:116-124``) is restated as its defining closed form - the fp32 sum
(or avg/max/min/product) of the members' slices in rank order, then one cast - not as a ring.
The objects consumed are duck-typed (attributes of the reference's ``Chunk``/``Bucket``), nothing
is imported from the product package.  Also used, timed, as the CPU baseline ("port").
"""

from __future__ import annotations

from collections import defaultdict

import torch

_LOW = (torch.float16, torch.bfloat16, torch.float32)


def reduce_rank_order(slices: list[torch.Tensor], op: str) -> torch.Tensor:
    """Combine the members' slices in list (= rank) order; fp32 accumulation for <= 32-bit floats."""
    acc_dtype = torch.float32 if slices[0].dtype in _LOW else torch.float64
    acc = slices[0].to(acc_dtype).clone()
    for s in slices[1:]:
        v = s.to(acc_dtype)
        if op in ("sum", "avg"):
            acc = acc + v
        elif op == "product":
            acc = acc * v
        elif op == "max":
            acc = torch.fmax(acc, v)
        elif op == "min":
            acc = torch.fmin(acc, v)
        else:
            raise ValueError(op)
    if op == "avg":
        acc = acc / float(len(slices))
    return acc


def reduce_levels(slices: list[torch.Tensor], levels) -> torch.Tensor:
    """Partial mesh dims with different ops (``ir.py:123-124``: one all-reduce per group, each with its own op, in
    mesh-dim order).  ``levels = ((op, size), ...)`` from the first-applied dim to the last; ``slices`` lists the
    members with the first-applied dim varying fastest.  After the first all-reduce every member of a line holds
    the line's result, so the whole sequence is a nested reduction: level by level, accumulators kept in fp32."""
    values = list(slices)
    for op, size in levels:
        assert len(values) % size == 0
        values = [reduce_rank_order(values[i:i + size], op) for i in range(0, len(values), size)]
    assert len(values) == 1
    return values[0]


def reduce_levels_in_tensor_dtype(slices: list[torch.Tensor], levels) -> torch.Tensor:
    """The same nested reduction with the reference's intermediate roundings: each of its all-reduces runs in place on a
    buffer of the *tensor's* dtype (``ir.py:123-124``), so for f16 / bf16 members the value is rounded to that dtype
    after every level.  ``reduce_levels`` above - which the kernels follow - keeps the accumulator in fp32 across levels
    and rounds once: for f32 / f64 members the two are the same function; for 16-bit members they can differ in the
    last place of a level's result.  Kept to quantify that difference (``tests/test_partial_levels.py``); what an
    all-reduce does inside one level is the backend's business and is not restated here."""
    dtype = slices[0].dtype
    values = list(slices)
    for op, size in levels:
        assert len(values) % size == 0
        values = [reduce_rank_order(values[i:i + size], op).to(dtype) for i in range(0, len(values), size)]
    assert len(values) == 1
    return values[0]


def _peers(chunk):
    groups = getattr(chunk, "source_partial_groups", None)
    if not groups:
        return None
    assert len(groups) == 1, "oracle: the Partial connected component comes as one group"
    group, op = groups[0]
    levels = getattr(group, "levels", ())
    return list(group.tensors), (tuple(levels) if levels else op)


def chunk_prepare(chunk, contiguous: bool = True) -> torch.Tensor:
    """``Chunk.prepare`` for a producing chunk (``ir.py:112-126``)."""
    src_t = getattr(chunk, "src_tensor", None)
    tensor = src_t if src_t is not None else chunk.tensor
    buf = tensor[chunk.src_slice]
    if contiguous:
        buf = buf.contiguous()
    peers = _peers(chunk)
    if peers is not None:
        tensors, op = peers
        members = [t[chunk.src_slice] for t in tensors]
        red = reduce_levels(members, op) if isinstance(op, tuple) else reduce_rank_order(members, op)
        wire = chunk.transfer_dtype or tensor.dtype
        return red.to(wire)  # single rounding from the accumulator
    if chunk.transfer_dtype and chunk.transfer_dtype != buf.dtype:
        buf = buf.to(chunk.transfer_dtype)
    return buf


def chunk_finalize(chunk, buf: torch.Tensor) -> None:
    """``Chunk.finalize`` (``ir.py:134-141``)."""
    if buf.dtype != chunk.tensor.dtype:
        buf = buf.to(chunk.tensor.dtype)
    chunk.tensor[chunk.dst_slice].copy_(buf)


def bucket_offsets(bucket) -> list[int]:
    """Un-padded prefix sum of the chunks' wire bytes (``ir.py:189-194``)."""
    out, cur = [], 0
    for c in bucket.chunks:
        out.append(cur)
        cur += c.nbytes
    return out


def bucket_prepare_source(bucket) -> torch.Tensor:
    """``Bucket.prepare`` of a producing bucket: returns the uint8 wire buffer (``ir.py:229-264``)."""
    chunks = bucket.chunks
    if len(chunks) == 1:
        # (flattened before the byte view: the reference's plain .view(torch.uint8) refuses a last dim of one
        # element that carries a stride other than 1, which torch reports for some slices - and for a single
        # element cut from a .t() view even after flattening; the bytes are the same)
        flat = chunk_prepare(chunks[0]).contiguous().reshape(-1)
        if flat.numel() == 1 and flat.stride(0) != 1:
            flat = flat.as_strided((1,), (1,))
        return flat.view(torch.uint8)
    offsets = bucket_offsets(bucket)
    total = offsets[-1] + chunks[-1].nbytes
    buffer = torch.empty(total, dtype=torch.uint8)
    for off, c in zip(offsets, chunks):
        dtype = c.transfer_dtype
        numel = c.nbytes // dtype.itemsize
        view = buffer.narrow(0, off, c.nbytes).view(dtype)[:numel].view(c.chunk_shape)
        view.copy_(chunk_prepare(c, contiguous=False))
    return buffer


def bucket_finalize_target(bucket, buffer: torch.Tensor) -> None:
    """``Bucket.finalize`` of a consuming bucket (``ir.py:300-310``)."""
    for off, c in zip(bucket_offsets(bucket), bucket.chunks):
        dtype = c.transfer_dtype
        numel = c.nbytes // dtype.itemsize
        view = buffer.narrow(0, off, c.nbytes).view(dtype)[:numel].view(c.chunk_shape)
        chunk_finalize(c, view)


class Mailbox:
    """In-memory wire: k-th buffer sent on a key is the k-th received on it."""

    def __init__(self) -> None:
        self.sent = defaultdict(list)
        self.taken = defaultdict(lambda: defaultdict(int))

    @staticmethod
    def key(bucket):
        c = bucket.chunks[0]
        return (c.src_rank, tuple(c.dst_ranks), c.transport.value)

    def send(self, bucket, buffer):
        self.sent[self.key(bucket)].append(buffer)

    def recv(self, bucket, rank):
        k = self.key(bucket)
        i = self.taken[k][rank]
        self.taken[k][rank] += 1
        return self.sent[k][i]


def run_rank(buckets, mailbox: Mailbox, rank=None) -> None:
    """One rank's ``bucket_comm``: all its source buckets, then its target buckets, in list order."""
    for b in buckets:
        kind = b.chunks[0].transport.value
        first = b.chunks[0]
        if kind == "none":
            continue
        if kind == "local":
            buffer = bucket_prepare_source(b)
            bucket_finalize_target(b, buffer)
        elif first.is_source:
            mailbox.send(b, bucket_prepare_source(b))
        elif first.is_target:
            bucket_finalize_target(b, mailbox.recv(b, rank if rank is not None else getattr(first, "rank", None)))
