"""Stage-2 planner, part 2: coalesce chunks into buckets.

Counterpart of ``src/etha/comm/get_buckets.py:12-43`` - same rule, same bucket order: a chunk of
at least ``bucket_size`` bytes is a bucket of its own (emitted at once); smaller chunks are
appended to the open bucket of their ``bucket_key``, which closes as soon as it holds at least
``bucket_size`` bytes; what is still open at the end is flushed in first-seen key order.
``bucket_size=1`` therefore means one chunk per bucket.
"""

from __future__ import annotations

from .ir import Bucket, Chunk

__all__ = ["chunk_to_bucket_ops"]


def _make_bucket(chunks: list[Chunk]) -> Bucket:
    tensor = chunks[0].tensor
    return Bucket(chunks=chunks, device=tensor.device if tensor is not None else None)


def chunk_to_bucket_ops(chunks: list[Chunk], bucket_size: int) -> list[Bucket]:
    buckets: list[Bucket] = []
    open_chunks: dict[tuple, list[Chunk]] = {}
    open_bytes: dict[tuple, int] = {}
    for chunk in chunks:
        size = chunk.nbytes
        if size >= bucket_size:
            buckets.append(_make_bucket([chunk]))
            continue
        key = chunk.bucket_key
        open_chunks.setdefault(key, []).append(chunk)
        open_bytes[key] = open_bytes.get(key, 0) + size
        if open_bytes[key] >= bucket_size:
            buckets.append(_make_bucket(open_chunks[key]))
            open_chunks[key] = []
            open_bytes[key] = 0
    for pending in open_chunks.values():
        if pending:
            buckets.append(_make_bucket(pending))
    return buckets
