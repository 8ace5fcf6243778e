"""The wire step of this build: a same-GPU loopback.

In the reference a prepared bucket crosses ranks with ``dist.isend/irecv`` or a sub-group
``dist.broadcast`` (``src/etha/comm/transfer.py:20-41``).  Here every rank's shards live on one
GPU, so "sending" a bucket means handing its buffer over in HBM: the producer packs into a slot
of a persistent bucket pool, the consumer unpacks from the very same slot (zero copy).  Slots are
assigned when a bucket list is first planned and reused by every later transfer, so the
consumer's tile program can hold absolute addresses.

Matching follows the point-to-point rule of the reference's transports: the k-th bucket a rank
sends on a wire key ``(src_rank, dst_ranks, transport)`` is the k-th bucket each of its peers
receives on that key.  Because slots are assigned when bucket lists are *planned*, "k-th" counts
over everything ever planned on the key: several registered batches between the same ranks get
consecutive sequence numbers, provided both ends plan their lists in the same order.  A caller that
cannot promise that order names a ``scope`` (any hashable, e.g. a batch id) when planning: sequence
numbers are then counted per scope.
"""

from __future__ import annotations

from collections import defaultdict

import torch

from .device_plan import Slot
from .ir import Bucket

_SLOT_ALIGN = 256


class BucketPool:
    """Persistent device memory for bucket buffers, carved from < 2 GiB segments.

    Segments stay below 2 GiB so that each one can be shared with another process through
    ``hipIpcGetMemHandle`` (larger shared allocations are not reliable on this platform).
    """

    def __init__(self, device: torch.device, segment_bytes: int = 1 << 30):
        self.device = device
        self.segment_bytes = segment_bytes
        self.segments: list[torch.Tensor] = []
        self._cursor = 0  # offset inside the last segment
        self._free: dict[int, list[Slot]] = {}  # released slots, reused for requests of exactly their size

    def release(self, slot: Slot) -> None:
        slot.filled = slot.drained = 0
        self._free.setdefault(slot.nbytes, []).append(slot)

    def alloc(self, nbytes: int) -> Slot:
        free = self._free.get(nbytes)
        if free:
            return free.pop()
        need = max(nbytes, 1)
        if need > self.segment_bytes or not self.segments or self._cursor + need > self.segments[-1].numel():
            size = max(self.segment_bytes, need)
            self.segments.append(torch.empty(size, dtype=torch.uint8, device=self.device))
            self._cursor = 0
        seg = self.segments[-1]
        ptr = seg.data_ptr() + self._cursor
        self._cursor = -(-(self._cursor + need) // _SLOT_ALIGN) * _SLOT_ALIGN
        return Slot(ptr=ptr, nbytes=nbytes, lo=seg.data_ptr(), hi=seg.data_ptr() + seg.numel())

    def view(self, slot: Slot) -> torch.Tensor:
        """uint8 tensor aliasing a slot (for inspection and tests)."""
        for seg in self.segments:
            base = seg.data_ptr()
            if base <= slot.ptr and slot.ptr + slot.nbytes <= base + seg.numel():
                return seg[slot.ptr - base : slot.ptr - base + slot.nbytes]
        raise ValueError("slot does not belong to this pool")

    @property
    def reserved_bytes(self) -> int:
        return sum(s.numel() for s in self.segments)


def wire_key(bucket: Bucket) -> tuple:
    return (bucket.src_rank, tuple(bucket.dst_ranks), bucket.transport.value)


class LoopbackWire:
    """Process-wide stand-in for the process groups of the reference's executor."""

    def __init__(self, device: torch.device | str | None = None, segment_bytes: int = 1 << 30,
                 host_inspection: bool = False):
        self.device = torch.device(device) if device is not None else None
        self.segment_bytes = segment_bytes
        # True: bucket lists on host tensors may be *planned* (tile programs compiled against host
        # addresses, for checking them on the CPU); they still cannot be run
        self.host_inspection = host_inspection
        # True: a single-chunk bucket whose bytes already lie contiguously in its source tensor is not
        # packed at all - the consumer unpacks straight from the tensor, as the reference's single-entry
        # path sends straight from it (ir.py:238-244).  The producer must then leave that tensor alone
        # until the consumer has unpacked: "sent" no longer means "copied".
        self.zero_copy_single_chunk = False
        # True: no bucket buffers at all.  Producer and consumer tensors are on one device, so the consumer's
        # launch reads the producer's chunk regions (every member's, for a Partial source) and writes its own:
        # one pass (read source dtype, write target dtype) instead of pack + unpack, and no pool memory.
        # This is what a pull over a peer mapping does between GPUs, minus the link.  Like a lent bucket,
        # a "sent" tensor must be left alone until the consumer has run.  Only within one process.
        self.direct_same_device = False
        self.pool: BucketPool | None = None
        # per wire key: sequence number -> (slot, chunk sizes) of every planned send bucket still alive
        self._sent: dict[tuple, dict[int, tuple[Slot, tuple[int, ...]]]] = defaultdict(dict)
        self._send_seq: dict[tuple, int] = defaultdict(int)  # next number to hand to a send bucket, per key
        self._recv_seq: dict[tuple, int] = defaultdict(int)  # next number a receiver expects, per (key, rank)
        self._plans: dict[tuple, object] = {}
        self._side_streams: list[torch.cuda.Stream] = []

    def _pool_for(self, device: torch.device) -> BucketPool:
        if self.pool is None:
            self.device = self.device or device
            self.pool = BucketPool(self.device, self.segment_bytes)
        if device != self.pool.device:
            raise RuntimeError(f"loopback wire is bound to {self.pool.device}, got a bucket on {device}")
        return self.pool

    # -- plan-time rendezvous -------------------------------------------------------------------
    def slot_for_send(self, bucket: Bucket, device: torch.device, scope=None) -> Slot:
        """Assign the next sequence number on this bucket's wire key (within ``scope``) and a slot to go with it."""
        key = (scope, *wire_key(bucket))
        sizes = tuple(c.nbytes for c in bucket.chunks)
        slot = None
        if self.direct_same_device:
            self._pool_for(device)
            slot = Slot(ptr=0, nbytes=bucket.total_bytes, lo=0, hi=0, borrowed=True)
            slot.sources = [(c.tensor, c.src_slice, c.transfer_dtype or c.tensor.dtype, c.partial_peers())
                            for c in bucket.chunks]
            slot.keepalive = [c.tensor for c in bucket.chunks]
        if slot is None and self.zero_copy_single_chunk:
            from .device_plan import zero_copy_region

            region = zero_copy_region(bucket)
            if region is not None:
                self._pool_for(device)
                slot = Slot(ptr=region[0], nbytes=bucket.total_bytes, lo=region[1], hi=region[2], borrowed=True)
                slot.keepalive = region[3]
        if slot is None:
            slot = self._pool_for(device).alloc(bucket.total_bytes)
        seq = self._send_seq[key]
        self._send_seq[key] = seq + 1
        self._sent[key][seq] = (slot, sizes)
        return slot

    def slot_for_recv(self, bucket: Bucket, scope=None) -> Slot:
        """Slot of the send bucket this receive bucket pairs with: the next one its rank has not yet planned."""
        key = (scope, *wire_key(bucket))
        who = (key, bucket.rank)
        seq = self._recv_seq[who]
        entry = self._sent.get(key, {}).get(seq)
        if entry is None:
            raise RuntimeError(
                f"{bucket}: no matching send bucket #{seq} has been planned on this wire "
                "(plan/run the source side first; a real wire would deadlock here)"
            )
        slot, sizes = entry
        if sizes != tuple(c.nbytes for c in bucket.chunks):
            raise RuntimeError(f"{bucket}: chunk layout differs from the matching send bucket")
        self._recv_seq[who] = seq + 1
        return slot

    # -- across processes ----------------------------------------------------------------------
    def export_manifest(self) -> dict:
        """Describe every planned send slot so that another process on the same GPU can consume it.

        Pool segments are exported with ``hipIpcGetMemHandle`` (allocation base + offset); a slot is
        ``(segment, offset)``.  The producer sends this once, after planning; afterwards only
        "generation n is packed" notifications are needed per transfer.
        """
        from .. import _native as nat

        if self.pool is None:
            return {"device": None, "segments": [], "slots": {}}
        segments = []
        with torch.cuda.device(self.pool.device):
            for seg in self.pool.segments:
                segments.append({"ipc": nat.ipc_export(seg.data_ptr()), "nbytes": seg.numel()})
        slots: dict = {}
        for key, entries in self._sent.items():
            out = []
            for seq, (slot, sizes) in sorted(entries.items()):
                if slot.sources is not None:
                    raise NotImplementedError("a direct wire has no bucket buffers to export; it works inside one process")
                if slot.borrowed:  # lives in a source tensor: export that allocation, range = the slot itself
                    with torch.cuda.device(self.pool.device):
                        segments.append({"ipc": nat.ipc_export(slot.ptr), "nbytes": slot.nbytes})
                    out.append({"seq": seq, "segment": len(segments) - 1, "offset": 0, "nbytes": slot.nbytes, "sizes": sizes})
                    continue
                idx = next(i for i, seg in enumerate(self.pool.segments)
                           if seg.data_ptr() <= slot.ptr and slot.ptr + slot.nbytes <= seg.data_ptr() + seg.numel())
                out.append({"seq": seq, "segment": idx, "offset": slot.ptr - self.pool.segments[idx].data_ptr(),
                            "nbytes": slot.nbytes, "sizes": sizes})
            slots[key] = out
        return {"device": self.pool.device.index, "segments": segments, "slots": slots}

    @classmethod
    def from_manifest(cls, manifest: dict, device: torch.device | str | None = None) -> "LoopbackWire":
        """Consumer side: map the producer's pool segments and expose its slots for receive planning."""
        from .. import _native as nat

        dev = torch.device(device) if device is not None else torch.device("cuda", manifest["device"] or 0)
        wire = cls(dev)
        wire._imported = []
        bases = []
        with torch.cuda.device(dev):
            for seg in manifest["segments"]:
                ptr = nat.ipc_open(seg["ipc"])
                wire._imported.append(ptr)
                bases.append((ptr, seg["nbytes"]))
        for key, entries in manifest["slots"].items():
            for e in entries:
                base, nbytes = bases[e["segment"]]
                slot = Slot(ptr=base + e["offset"], nbytes=e["nbytes"], lo=base, hi=base + nbytes)
                wire._sent[key][e["seq"]] = (slot, tuple(e["sizes"]))
        return wire

    def mark_packed(self) -> None:
        """Consumer side: the producer reported that every exported slot has been packed (and its stream
        synchronised) once more."""
        for entries in self._sent.values():
            for slot, _ in entries.values():
                slot.filled += 1

    def close_imported(self) -> None:
        from .. import _native as nat

        for ptr in getattr(self, "_imported", []):
            nat.ipc_close(ptr)
        self._imported = []

    def private_slot(self, nbytes: int, device: torch.device) -> Slot:
        return self._pool_for(device).alloc(nbytes)

    def side_streams(self, device: torch.device, n: int) -> list:
        """``n`` extra streams of default priority, created on first use and kept."""
        while len(self._side_streams) < n:
            self._side_streams.append(torch.cuda.Stream(device=device))
        return self._side_streams[:n]

    # -- plan cache -----------------------------------------------------------------------------
    def plan(self, buckets: list[Bucket], scope=None):
        """Compiled plan of a bucket list (cached by the identity of its buckets).  ``scope`` only matters when the
        plan is first built: it namespaces the send/receive pairing."""
        from .comm_methods import TransferPlan

        key = tuple(id(b) for b in buckets)
        plan = self._plans.get(key)
        if plan is None:
            plan = TransferPlan(self, list(buckets), scope=scope)
            self._plans[key] = plan
        return plan

    def release(self, buckets: list[Bucket]) -> None:
        """Forget a bucket list: drop its compiled plan and hand its send slots back to the pool.
        The caller guarantees that no transfer of these buckets, on either end, is still in flight."""
        plan = self._plans.pop(tuple(id(b) for b in buckets), None)
        if plan is None:
            return
        for kind, _, _, slot in plan.steps:
            if slot is None or self.pool is None:
                continue
            owned = False
            for key, entries in list(self._sent.items()):
                mine = [seq for seq, (s, _) in entries.items() if s is slot]
                for seq in mine:  # sequence numbers are never reused: later plans on this key keep theirs
                    del entries[seq]
                    owned = True
            if (owned or kind == "pack") and not slot.borrowed:
                if not any(slot is s for s in self.pool._free.get(slot.nbytes, [])):
                    self.pool.release(slot)

    def reset(self) -> None:
        self._plans.clear()
        self._sent.clear()
        self._send_seq.clear()
        self._recv_seq.clear()
        self.pool = None


_default_wire: LoopbackWire | None = None


def default_wire() -> LoopbackWire:
    global _default_wire
    if _default_wire is None:
        _default_wire = LoopbackWire()
    return _default_wire


def reset_default_wire() -> None:
    global _default_wire
    if _default_wire is not None:
        _default_wire.reset()
    _default_wire = None
