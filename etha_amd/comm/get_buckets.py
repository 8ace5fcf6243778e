"""Stage-2 planner, part 2: coalesce chunks into buckets.

Counterpart of ``src/etha/comm/get_buckets.py:12-43`` with the same rule and the same bucket order:

* a chunk of at least ``bucket_size`` wire bytes is a bucket of its own and is emitted immediately;
* a smaller chunk joins the open bucket of its ``bucket_key``; that bucket is emitted as soon as it
  holds at least ``bucket_size`` bytes (so a bucket may exceed ``bucket_size`` by less than one chunk);
* buckets still open after the last chunk are emitted in the order their keys first appeared.

``bucket_size=1`` therefore means one chunk per bucket.
"""

from __future__ import annotations

from .ir import Bucket, Chunk

__all__ = ["chunk_to_bucket_ops"]


class _OpenBucket:
    """Chunks collected so far for one key."""

    __slots__ = ("members", "nbytes")

    def __init__(self) -> None:
        self.members: list[Chunk] = []
        self.nbytes = 0

    def take(self) -> list[Chunk]:
        members, self.members, self.nbytes = self.members, [], 0
        return members


def _seal(members: list[Chunk]) -> Bucket:
    first = members[0].tensor
    return Bucket(chunks=members, device=None if first is None else first.device)


def chunk_to_bucket_ops(chunks: list[Chunk], bucket_size: int) -> list[Bucket]:
    sealed: list[Bucket] = []
    pending: dict[tuple, _OpenBucket] = {}  # insertion order = first appearance of the key
    for chunk in chunks:
        wire_bytes = chunk.nbytes
        if wire_bytes >= bucket_size:
            sealed.append(_seal([chunk]))
            continue
        slot = pending.setdefault(chunk.bucket_key, _OpenBucket())
        slot.members.append(chunk)
        slot.nbytes += wire_bytes
        if slot.nbytes >= bucket_size:
            sealed.append(_seal(slot.take()))
    sealed.extend(_seal(slot.take()) for slot in pending.values() if slot.members)
    return sealed
