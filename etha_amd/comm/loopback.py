"""The wire step of this build: a same-GPU loopback.

In the reference a prepared bucket crosses ranks with ``dist.isend/irecv`` or a sub-group
``dist.broadcast`` (``src/etha/comm/transfer.py:20-41``).  Here every rank's shards live on one
GPU, so "sending" a bucket means handing its buffer over in HBM: the producer packs into a slot
of a persistent bucket pool, the consumer unpacks from the very same slot (zero copy).  Slots are
assigned when a bucket list is first planned and reused by every later transfer, so the
consumer's tile program can hold absolute addresses.

Pool.  By default the pool is a **ring**: every wire key (channel) of a planned send list owns
``max_in_flight`` slots, each as large as the channel's largest bucket, and the channel's k-th bucket
uses slot ``k mod max_in_flight``.  That is the reference's memory bound - at most ``max_in_flight``
buckets per channel are prepared or in flight, and a bucket's buffer is dropped at ``finalize``
(``comm_methods.py:53-119``, ``ir.py:246,310``).  A slot is packed again only after every consumer of
its previous bucket has unpacked, so senders and receivers advance together: the wire keeps the bucket
pipelines (:class:`etha_amd.comm.comm_methods.Program`) of every rank that has called ``bucket_comm``
and steps them in turn, the single-process form of the ranks' concurrent ``bucket_comm`` loops.
``pool="resident"`` gives every bucket a slot of its own for the life of its plan (pool = payload);
that form allows one launch over many buckets, side streams and graph capture.  Either form can be exported to a
consumer in another process (``export_manifest`` / ``from_manifest``); a ring's slots then change hands through
"packed" / "unpacked" notifications (``exchange``).

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
from dataclasses import dataclass, field

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
        self.segment_bytes = segment_bytes  # 0: every slot is an allocation of its own, exactly as large as asked
        self.segments: list[torch.Tensor] = []
        self._cursor = 0  # offset inside the last segment
        self._free: dict[int, list[Slot]] = {}  # released slots, reused for requests of exactly their size

    def release(self, slot: Slot) -> None:
        slot.filled = slot.drained = 0
        slot.holder = None
        self._free.setdefault(slot.nbytes, []).append(slot)

    def alloc(self, nbytes: int) -> Slot:
        free = self._free.get(nbytes)
        if free:
            return free.pop()
        need = max(nbytes, 1)
        if self.segment_bytes == 0:
            seg = torch.empty(-(-need // _SLOT_ALIGN) * _SLOT_ALIGN, dtype=torch.uint8, device=self.device)
            self.segments.append(seg)
            return Slot(ptr=seg.data_ptr(), nbytes=nbytes, lo=seg.data_ptr(), hi=seg.data_ptr() + seg.numel())
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


@dataclass(eq=False)
class WireEntry:
    """One planned send bucket on a wire key: where its bytes travel and who still has to read them."""

    key: tuple
    seq: int
    slot: Slot
    sizes: tuple
    dst_ranks: tuple
    submitted: int = 0  # transfers the sender has been asked for
    packed: int = 0  # transfers packed into the slot so far
    arrived: dict = field(default_factory=dict)  # destination rank -> transfers it has asked for
    left: set = field(default_factory=set)  # consumers of the bytes now in the slot that have not unpacked yet
    remote: bool = False  # a copy, in a consumer process, of an entry that a producer process owns


class _no_context:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


# steps that are launched at once: the few, large one-pass copies of the direct wire measured 2 % slower in sets
_UNGROUPED = ("direct", "direct_reduce")

_DRIVE = ("d",)
_MAX_TRACE_NODES = 4096


class _TraceNode:
    """One point of a recorded transfer (see :attr:`LoopbackWire.replay_schedules`): reached from its parent by a
    ``submit`` or a ``drive`` event.  A node reached by a drive holds what that drive issued."""

    __slots__ = ("children", "calls", "schedule", "pending", "recorded", "outbox")

    def __init__(self):
        self.children: dict = {}
        self.calls: list = []  # [(group, flags, single)], group = [(plan, kind, first, count), ...], in issue order
        self.schedule = None  # the same as one native schedule (built on first replay on a GPU)
        self.pending: frozenset = frozenset()  # ids of the plans whose pipelines are still waiting after this drive
        self.recorded = False
        self.outbox: tuple = ()  # what this drive left for the peer process (a wire with a remote end)


def wire_key(bucket: Bucket) -> tuple:
    return (bucket.src_rank, tuple(bucket.dst_ranks), bucket.transport.value)


class LoopbackWire:
    """Process-wide stand-in for the process groups of the reference's executor."""

    def __init__(self, device: torch.device | str | None = None, segment_bytes: int = 1 << 30,
                 host_inspection: bool = False, pool: str = "ring", max_in_flight: int = 2):
        if pool not in ("ring", "resident"):
            raise ValueError(f"pool must be 'ring' or 'resident', got {pool!r}")
        self.device = torch.device(device) if device is not None else None
        self.segment_bytes = segment_bytes
        self.pool_mode = pool
        # slots per channel of a ring pool; a plan's rings are sized when it is first compiled
        self.max_in_flight = max(1, int(max_in_flight))
        # destination ranks that buckets name but that do not exist on this wire (a job that only stages some
        # target ranks): nobody will unpack for them, so a slot does not wait for them
        self.absent_ranks: set[int] = set()
        # launches that do not depend on each other are issued without ordering between them
        # (ETHA_LAUNCH_UNORDERED), which hides the gap between one bucket's kernel and the next one's
        self.unordered_launches = True
        # launches that do not depend on each other are handed to the library as one set (etha_launch_segments):
        # what a sweep over all pipelines prepares and finalizes shares kernel launches
        self.group_launches = True
        self._group: list = []  # (plan, kind, first, count) of the set being collected
        self._group_flags = 0
        # host inspection: called as ``on_launch(plan, kind, first, count, flags)`` instead of launching
        self.on_launch = None
        # host inspection of the sets: called as ``on_set([(plan, kind, first, count), ...], flags)`` instead of
        # handing the set to the library (its members may run in any order, or at the same time)
        self.on_set = None
        self.launch_log: list | None = None  # when a list: (kind, first, count, flags) of every launch
        self._programs: list = []  # bucket pipelines that still have work, in arrival order
        self._epoch_reads: set[int] = set()  # allocations read / written by launches since the last ordered one
        self._epoch_writes: set[int] = set()
        self._ordered_next = True
        self._stream = None
        self._carried = False  # pipelines were left pending by an earlier drive (their launches sit on _stream)
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
        # True: a transfer that repeats one seen before is not walked through the pipelines again.  The reference
        # plans once and transfers N times (tensor_bus/batch_state.py:38-40); the pipelines here are deterministic,
        # so from an idle wire the same sequence of submit / drive calls issues the same launches.  The wire keeps
        # what every drive of such a sequence issued and, when the sequence recurs, re-issues it with one library
        # call per drive (etha_schedule_launch) instead of stepping the Python pipelines.  A sequence that departs
        # from every recorded one falls back to the pipelines (their state is rebuilt first) and is recorded too.
        self.replay_schedules = True
        self._trace_root = _TraceNode()
        self._trace_nodes = 0
        self._trace_absent: set = set()
        self._tx_events: list = []  # events of the transfer under way since the wire was last idle
        self._tx_node: _TraceNode | None = None  # trie node of those events; None: this transfer is not traced
        self._tx_replaying = False  # the transfer under way follows a recorded one: no pipelines exist for it
        self._tx_dirty = False  # slots changed hands outside a transfer (a peer's early notification): do not trace the next one
        self._tx_pending: set = set()  # replaying: ids of plans submitted and not yet finished
        self._tx_calls: list | None = None  # recording: what the drive under way has issued so far
        self._suppress = False  # rebuilding pipeline state: steps are walked, nothing is launched
        self.replays = 0  # drives served from a recorded schedule (statistics)
        # Across processes (export_manifest / from_manifest with a ring pool): a list that collects what the peer
        # process must be told - ("packed", key, seq) once a send bucket is in its slot, ("unpacked", key, seq, rank)
        # once a destination has read it.  None: every rank of this wire lives in this process.
        self.outbox: list | None = None
        self.local_ranks: set | None = None  # consumer process: the destination ranks that live here
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
            self.pool = BucketPool(self.device, 0 if self.pool_mode == "ring" else self.segment_bytes)
        if device != self.pool.device:
            raise RuntimeError(f"loopback wire is bound to {self.pool.device}, got a bucket on {device}")
        return self.pool

    # -- plan-time rendezvous -------------------------------------------------------------------
    def open_rings(self, buckets: list[Bucket], device: torch.device, depth: int) -> dict:
        """Ring pool: the slots of one send list, ``{wire key: [slot, ...]}``.  A channel gets ``depth`` slots
        (fewer if it has fewer buckets) of its largest bucket's size."""
        need: dict[tuple, list[int]] = {}
        for b in buckets:
            if not b.chunks or not b.is_source or b.transport.value not in ("p2p", "broadcast"):
                continue
            if self.direct_same_device:
                continue
            if self.zero_copy_single_chunk:
                from .device_plan import zero_copy_region

                if zero_copy_region(b) is not None:
                    continue
            need.setdefault(wire_key(b), []).append(b.total_bytes)
        pool = self._pool_for(device) if need else None
        return {key: [pool.alloc(max(sizes)) for _ in range(min(depth, len(sizes)))] for key, sizes in need.items()}

    def entry_for_send(self, bucket: Bucket, device: torch.device, scope=None, ring: list | None = None,
                       ordinal: int = 0) -> WireEntry:
        """Assign the next sequence number on this bucket's wire key (within ``scope``) and a slot to go with it:
        slot ``ordinal mod depth`` of ``ring`` in a ring pool, else a slot of the bucket's own."""
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
        if slot is None and ring:
            slot = ring[ordinal % len(ring)]
        if slot is None:
            slot = self._pool_for(device).alloc(bucket.total_bytes)
        seq = self._send_seq[key]
        self._send_seq[key] = seq + 1
        entry = WireEntry(key=key, seq=seq, slot=slot, sizes=sizes, dst_ranks=tuple(bucket.dst_ranks))
        self._sent[key][seq] = entry
        return entry

    def entry_for_recv(self, bucket: Bucket, scope=None) -> WireEntry:
        """The send bucket this receive bucket pairs with: the next one on its key that its rank has not yet planned."""
        key = (scope, *wire_key(bucket))
        who = (key, bucket.rank)
        seq = self._recv_seq[who]
        entry = self._sent.get(key, {}).get(seq)
        if entry is None:
            raise RuntimeError(
                f"{bucket}: no matching send bucket #{seq} has been planned on this wire "
                "(plan/run the source side first; a real wire would deadlock here)"
            )
        if entry.sizes != tuple(c.nbytes for c in bucket.chunks):
            raise RuntimeError(f"{bucket}: chunk layout differs from the matching send bucket")
        self._recv_seq[who] = seq + 1
        return entry

    def consumers(self, entry: WireEntry) -> set:
        return {r for r in entry.dst_ranks if r not in self.absent_ranks}

    # -- a ring whose two ends live in different processes ----------------------------------------
    def take_outbox(self) -> list:
        """What the peer process has to be told since the last call.  The caller synchronises the stream first (the
        hand-over between processes is ordered by a host-side fence) and sends the list over its own channel."""
        out, self.outbox = self.outbox or [], []
        return out

    def apply_remote(self, messages) -> None:
        """The peer's notifications: a producer learns that destinations have unpacked (their slots become free), a
        consumer that send buckets have been packed (they may now be unpacked).  The same hand-shake
        ``mark_sent`` / ``mark_received`` keep inside one process."""
        messages = tuple((m[0], (m[1][0], m[1][1], tuple(m[1][2]), m[1][3]), *m[2:]) for m in messages)
        event = ("r", messages)
        if self._tx_replaying:
            child = self._tx_node.children.get(event)
            if child is not None:  # the peer follows the recorded transfer too: nothing to update, no pipelines exist
                self._tx_node = child
                self._tx_events.append(event)
                return
            self._rebuild_pipelines()
        self._apply_remote(messages)
        if self._programs or self._tx_events:
            self._tx_events.append(event)
            if self._tx_node is not None:
                self._tx_node = self._child(self._tx_node, event)
        else:  # between transfers: the next one does not start from the state every recording starts from
            self._tx_dirty = True

    def _apply_remote(self, messages) -> None:
        from .comm_methods import mark_received

        for msg in messages:
            what, key, seq = msg[0], tuple(msg[1]), msg[2]
            key = (key[0], key[1], tuple(key[2]), key[3])
            entry = self._sent.get(key, {}).get(seq)
            if entry is None:
                raise RuntimeError(f"the peer process names bucket #{seq} of {key}, which is not planned on this wire")
            if what == "packed":
                if entry.slot.holder is not None:
                    raise RuntimeError(f"bucket #{seq} of {key} was packed into a slot that still holds unread bytes")
                entry.packed += 1
                entry.left = {r for r in self.consumers(entry) if self.local_ranks is None or r in self.local_ranks}
                entry.slot.filled += 1
                entry.slot.holder = entry if entry.left else None
            elif what == "unpacked":
                if entry.slot.holder is not entry or msg[3] not in entry.left:
                    raise RuntimeError(f"rank {msg[3]} reports bucket #{seq} of {key} as unpacked, which it was not sent")
                mark_received(entry, msg[3])
            else:
                raise ValueError(f"unknown wire notification {what!r}")

    def exchange(self, conn, synchronize=None) -> None:
        """Run the transfers queued on this wire to completion against the peer process at the other end of ``conn``
        (a ``multiprocessing`` connection): step the pipelines, fence, send what the peer must know, wait for its
        notifications, until nothing is pending here.  Both processes call this once per transfer."""
        if self.outbox is None:
            raise RuntimeError("this wire has no peer process (see export_manifest / from_manifest)")
        sync = synchronize or (lambda: torch.cuda.current_stream(self.device).synchronize())
        while True:
            self.drive()
            out = self.take_outbox()
            if out:
                sync()  # the peer may touch the slots as soon as it hears of them
                conn.send(("wire", out))
            if self.idle():
                return
            kind, messages = conn.recv()
            if kind != "wire":
                raise RuntimeError(f"unexpected message from the peer process: {kind!r}: {messages}")
            self.apply_remote(messages)

    # -- across processes ----------------------------------------------------------------------
    def export_manifest(self) -> dict:
        """Describe every planned send slot so that another process on the same GPU can consume it.

        Pool segments are exported with ``hipIpcGetMemHandle`` (allocation base + offset); a slot is
        ``(segment, offset)``.  The producer sends this once, after planning.  Per transfer a resident pool needs
        one "packed" notification; a ring's two ends trade notifications while the transfer runs (``exchange``).
        """
        from .. import _native as nat

        if self.pool_mode == "ring":
            # slots are recycled: from now on the consumers' progress arrives as notifications (apply_remote)
            self.outbox = []
            self.forget_recorded_transfers()
        if self.pool is None:
            return {"device": None, "pool": self.pool_mode, "segments": [], "slots": {}}
        segments = []
        host = self.pool.device.type != "cuda"  # host inspection: the "other process" is this one, addresses are shared
        with torch.cuda.device(self.pool.device) if not host else _no_context():
            for seg in self.pool.segments:
                segments.append({"ptr": seg.data_ptr(), "nbytes": seg.numel()} if host else
                                {"ipc": nat.ipc_export(seg.data_ptr()), "nbytes": seg.numel()})
        slots: dict = {}
        for key, entries in self._sent.items():
            out = []
            for seq, entry in sorted(entries.items()):
                slot, sizes = entry.slot, entry.sizes
                if slot.sources is not None:
                    raise NotImplementedError("a direct wire has no bucket buffers to export; it works inside one process")
                if slot.borrowed:  # lives in a source tensor: export that allocation, range = the slot itself
                    with torch.cuda.device(self.pool.device) if not host else _no_context():
                        segments.append({"ptr": slot.ptr, "nbytes": slot.nbytes} if host else
                                        {"ipc": nat.ipc_export(slot.ptr), "nbytes": slot.nbytes})
                    out.append({"seq": seq, "segment": len(segments) - 1, "offset": 0, "nbytes": slot.nbytes, "sizes": sizes})
                    continue
                idx = next(i for i, seg in enumerate(self.pool.segments)
                           if seg.data_ptr() <= slot.ptr and slot.ptr + slot.nbytes <= seg.data_ptr() + seg.numel())
                out.append({"seq": seq, "segment": idx, "offset": slot.ptr - self.pool.segments[idx].data_ptr(),
                            "nbytes": slot.nbytes, "sizes": sizes})
            slots[key] = out
        return {"device": None if host else self.pool.device.index, "pool": self.pool_mode, "segments": segments, "slots": slots}

    @classmethod
    def from_manifest(cls, manifest: dict, device: torch.device | str | None = None) -> "LoopbackWire":
        """Consumer side: map the producer's pool segments and expose its slots for receive planning."""
        from .. import _native as nat

        dev = torch.device(device) if device is not None else torch.device("cuda", manifest["device"] or 0)
        ring = manifest.get("pool", "resident") == "ring"
        wire = cls(dev, pool="ring" if ring else "resident", host_inspection=dev.type != "cuda")
        wire._imported = []
        bases = []
        with torch.cuda.device(dev) if dev.type == "cuda" else _no_context():
            for seg in manifest["segments"]:
                if "ptr" in seg:  # exported by a host-inspection wire of this very process
                    bases.append((seg["ptr"], seg["nbytes"]))
                    continue
                ptr = nat.ipc_open(seg["ipc"])
                wire._imported.append(ptr)
                bases.append((ptr, seg["nbytes"]))
        slots: dict = {}  # buckets of one channel that share a ring slot share the Slot object here too
        for key, entries in manifest["slots"].items():
            for e in entries:
                base, nbytes = bases[e["segment"]]
                where = (e["segment"], e["offset"], e["nbytes"]) if ring else (key, e["seq"])
                slot = slots.get(where)
                if slot is None:
                    slot = slots[where] = Slot(ptr=base + e["offset"], nbytes=e["nbytes"], lo=base, hi=base + nbytes)
                wire._sent[key][e["seq"]] = WireEntry(key=key, seq=e["seq"], slot=slot, sizes=tuple(e["sizes"]),
                                                      dst_ranks=tuple(key[2]), remote=True)
        if ring:
            wire.outbox = []
        return wire

    def mark_packed(self) -> None:
        """Consumer side: the producer reported that every exported slot has been packed (and its stream
        synchronised) once more."""
        for entries in self._sent.values():
            for entry in entries.values():
                entry.slot.filled += 1

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
    def plan(self, buckets: list[Bucket], scope=None, max_in_flight: int | None = None):
        """Compiled plan of a bucket list (cached by the identity of its buckets).  ``scope`` and ``max_in_flight``
        only matter when the plan is first built: the scope namespaces the send/receive pairing, and a ring pool
        gives every channel of the list ``max_in_flight`` slots (default: the wire's)."""
        from .comm_methods import TransferPlan

        key = tuple(id(b) for b in buckets)
        plan = self._plans.get(key)
        if plan is None:
            plan = TransferPlan(self, list(buckets), scope=scope, max_in_flight=max_in_flight or self.max_in_flight)
            self._plans[key] = plan
        return plan

    def release(self, buckets: list[Bucket]) -> None:
        """Forget a bucket list: drop its compiled plan and hand its slots back to the pool.
        The caller guarantees that no transfer of these buckets, on either end, is still in flight."""
        plan = self._plans.pop(tuple(id(b) for b in buckets), None)
        if plan is None:
            return
        self.forget_recorded_transfers()  # they name this plan's tables
        self._programs = [p for p in self._programs if p.plan is not plan]
        for entry in plan.owned_entries:  # sequence numbers are never reused: later plans on this key keep theirs
            self._sent.get(entry.key, {}).pop(entry.seq, None)
        if self.pool is not None:
            for slot in plan.owned_slots:
                if not slot.borrowed and not any(slot is s for s in self.pool._free.get(slot.nbytes, [])):
                    self.pool.release(slot)

    def reset(self) -> None:
        self._plans.clear()
        self._sent.clear()
        self._send_seq.clear()
        self._recv_seq.clear()
        self._programs.clear()
        self._tx_replaying = False
        self.forget_recorded_transfers()
        self._tx_events, self._tx_pending = [], set()
        self.pool = None

    # -- the bucket pipelines of every rank on this wire ---------------------------------------
    # -- recorded transfers ----------------------------------------------------------------------
    def _tracing(self) -> bool:
        if not (self.replay_schedules and self.pool_mode == "ring" and self.on_launch is None and self.launch_log is None
                and (self.on_set is not None or (self.device is not None and self.device.type == "cuda"))):
            return False
        if self.absent_ranks != self._trace_absent:  # who unpacks decides when a slot is free again
            self.forget_recorded_transfers()
            self._trace_absent = set(self.absent_ranks)
        return True

    def forget_recorded_transfers(self) -> None:
        """Drop every recorded transfer (a plan they name is going away, or the wire was driven by hand).  A transfer
        under way that was following one goes back to the pipelines."""
        if self._tx_replaying:
            self._rebuild_pipelines()
        self._trace_root = _TraceNode()
        self._trace_nodes = 0
        self._tx_node = None

    def _child(self, node: _TraceNode, event) -> _TraceNode | None:
        child = node.children.get(event)
        if child is None:
            if self._trace_nodes >= _MAX_TRACE_NODES:
                return None
            child = node.children[event] = _TraceNode()
            self._trace_nodes += 1
        return child

    def _rebuild_pipelines(self) -> None:
        """The transfer under way was following a recorded one and now departs from it: bring the pipelines to the
        state they would be in, by walking the events so far with launching switched off."""
        from .comm_methods import Program

        events, self._tx_replaying = self._tx_events, False
        self._tx_pending = set()
        self._suppress = True
        try:
            outbox = self.outbox
            if outbox is not None:
                self.outbox = []  # what the walk leaves there has been handed out by the replayed drives already
            for ev in events:
                if ev[0] == "s":
                    self._programs.append(Program(ev[1], ev[2], ev[3]))
                elif ev[0] == "r":
                    self._apply_remote(ev[1])
                else:
                    self._drive_pipelines()
        finally:
            self._suppress = False
            self.outbox = outbox

    def _end_of_drive(self, idle: bool) -> None:
        if idle:  # the transfer is over: the next submit starts a new one
            self._tx_events, self._tx_node, self._tx_replaying = [], None, False
            self._tx_pending = set()
            self._tx_dirty = False

    # -- the bucket pipelines of every rank on this wire ---------------------------------------
    def submit(self, plan, max_in_flight: int, merge_launches: bool = False):
        """Start one transfer of a planned bucket list: its pipeline joins the ones :meth:`drive` steps."""
        from .comm_methods import Program

        event = ("s", id(plan), max_in_flight, merge_launches, self.unordered_launches, self.group_launches)
        if not self._programs and not self._tx_events:  # an idle wire: a new transfer begins
            self._tx_replaying = False
            self._tx_node = self._trace_root if self._tracing() and not self._tx_dirty else None
            if self._tx_node is not None and event in self._tx_node.children:
                self._tx_replaying = True
        if self._tx_replaying:
            child = self._tx_node.children.get(event) if id(plan) not in self._tx_pending else None
            if child is not None:
                self._tx_node = child
                self._tx_events.append(("s", plan, max_in_flight, merge_launches))
                self._tx_pending.add(id(plan))
                return None
            self._rebuild_pipelines()
        if any(p.plan is plan for p in self._programs):
            raise RuntimeError(
                "the previous transfer of these buckets has not completed: its receivers have not unpacked yet "
                "(a real wire would block here)")
        program = Program(plan, max_in_flight, merge_launches)
        self._programs.append(program)
        self._tx_events.append(("s", plan, max_in_flight, merge_launches))
        if self._tx_node is not None:
            self._tx_node = self._child(self._tx_node, event)
        return program

    def drive(self) -> None:
        """Step every pending pipeline, in arrival order, until none can move.  Launches go to the current stream
        of the wire's device.  A sender's pipeline that is waiting for its receivers stays pending and is picked
        up by the call that brings them."""
        if self._tx_replaying and self._drive_recorded():
            return
        if not self._programs:
            return
        record = self._tx_node is not None and not self._suppress
        if record and self.on_set is None and torch.cuda.is_current_stream_capturing():
            record, self._tx_node = False, None  # what a capture leaves out (uploads) must not end up in a recorded transfer
        self._tx_calls = [] if record else None
        outbox_before = len(self.outbox) if self.outbox is not None else 0
        try:
            self._drive_pipelines()
        except BaseException:
            self._tx_node, self._tx_calls = None, None
            raise
        calls, self._tx_calls = self._tx_calls, None
        self._tx_events.append(_DRIVE)
        if record:
            node = self._tx_node = self._child(self._tx_node, _DRIVE)
            if node is not None and not node.recorded:
                node.calls, node.pending, node.recorded = calls, frozenset(id(p.plan) for p in self._programs), True
                node.outbox = tuple(self.outbox[outbox_before:]) if self.outbox is not None else ()
        self._end_of_drive(not self._programs)

    def _drive_recorded(self) -> bool:
        """Serve a drive from the recorded transfer the events so far follow; False when they follow none
        (the pipelines have then been rebuilt and the caller steps them)."""
        from .. import _native as nat

        node = self._tx_node.children.get(_DRIVE)
        if node is None or not node.recorded:
            self._rebuild_pipelines()
            return False
        if self.on_set is not None:
            for group, flags, _ in node.calls:
                self.on_set(group, flags)
        elif node.calls:
            stream = torch.cuda.current_stream(self.device)
            if self._carried and self._stream is not None and self._stream != stream:
                done = torch.cuda.Event()
                done.record(self._stream)
                stream.wait_event(done)
            self._stream = stream
            try:
                if node.schedule is None:
                    node.schedule = nat.Schedule([([plan.segment(kind, first, count) for plan, kind, first, count in group],
                                                   flags, single) for group, flags, single in node.calls])
                with torch.cuda.device(self.device):
                    node.schedule.launch(stream.cuda_stream)
            except nat.EthaNativeError as e:
                if "stale schedule" not in str(e):
                    raise
                # a table gained a write-ordered range since the recording: nothing was launched; start over
                self.forget_recorded_transfers()
                return False
        self.replays += 1
        if self.outbox is not None:
            self.outbox.extend(node.outbox)
        self._tx_node = node
        self._tx_events.append(_DRIVE)
        self._tx_pending = set(node.pending)
        self._carried = bool(node.pending)
        self._end_of_drive(not node.pending)
        return True

    def _drive_pipelines(self) -> None:
        cuda = self.device is not None and self.device.type == "cuda" and self.on_launch is None and self.on_set is None
        if cuda and not self._suppress:
            stream = torch.cuda.current_stream(self.device)
            if self._carried and self._stream is not None and self._stream != stream:
                # work enqueued earlier for pipelines that are still pending sits on another stream
                done = torch.cuda.Event()
                done.record(self._stream)
                stream.wait_event(done)
            self._stream = stream
        # whatever is on the stream already (the caller's own kernels) must be finished before the first launch
        self._ordered_next = True
        self._epoch_reads, self._epoch_writes = set(), set()
        with torch.cuda.device(self.device) if cuda else _no_context():
            try:
                moved = True
                while moved:
                    moved = False
                    for program in list(self._programs):
                        if program.sweep(self):
                            moved = True
                        if program.finished:
                            self._programs.remove(program)
                    self._flush()  # what one pass over the pipelines made ready goes to the device now
            finally:
                self._flush()  # what was issued is marked as sent / received: it must reach the stream
        self._carried = bool(self._programs)

    def idle(self) -> bool:
        """True when no pipeline is waiting for a peer."""
        return not self._programs and not (self._tx_replaying and self._tx_pending)

    def in_progress(self, buckets: list[Bucket]) -> bool:
        """True while a transfer of this bucket list is still waiting for a peer (a send whose receivers have
        not all unpacked, a receive whose senders have not packed everything yet)."""
        plan = self._plans.get(tuple(id(b) for b in buckets))
        if plan is None:
            return False
        if self._tx_replaying:
            return id(plan) in self._tx_pending
        return any(p.plan is plan for p in self._programs)

    def pending(self) -> list[str]:
        if self._tx_replaying:
            return [f"pipeline of {ev[1].buckets[0]} ..." for ev in self._tx_events if ev[0] == "s" and id(ev[1]) in self._tx_pending]
        return [repr(p) for p in self._programs]

    def emit(self, plan, indices: list[int], merge: bool = False) -> None:
        """Issue steps ``indices`` of ``plan``, which became ready in the same phase of one pipeline sweep; with
        ``merge`` those that are neighbours in their table and touch no allocation that the other writes share a
        launch.  Each launch is ordered against earlier launches only where their bytes meet."""
        todo = []
        for i in indices:
            kind, first, count, _ = plan.steps[i]
            info = plan.info[i]
            if info.tiles:  # else nothing to move (empty shards): no launch, so nothing that could order later launches
                todo.append([kind, first, count, info.reads, info.writes, info.excl])
        if merge and len(todo) > 1:
            todo.sort(key=lambda t: (t[0], t[1]))
            runs = [todo[0]]
            for t in todo[1:]:
                last = runs[-1]
                # steps of one phase are independent except LOCAL buckets inside one tensor, where a later bucket
                # may read what an earlier one writes: those keep their own launches, in list order
                if t[0] == last[0] and last[1] + last[2] == t[1] and last[4].isdisjoint(t[3]) and last[3].isdisjoint(t[4]):
                    last[2] += t[2]
                    last[3], last[4], last[5] = last[3] | t[3], last[4] | t[4], last[5] | t[5]
                    last.append(True)  # covers several buckets
                else:
                    runs.append(t)
            todo = runs
            for t in todo:
                if len(t) > 6:
                    plan.order_by_written_address(t[0], t[1], t[2])
        for kind, first, count, reads, writes, excl, *_ in todo:
            self._issue(plan, kind, first, count, reads, writes, excl)

    def _issue(self, plan, kind, first, count, reads, writes, excl) -> None:
        ordered = (self._ordered_next or not self.unordered_launches or not self._epoch_writes.isdisjoint(reads)
                   or not self._epoch_reads.isdisjoint(writes) or not self._epoch_writes.isdisjoint(excl))
        if ordered:
            self._epoch_reads, self._epoch_writes = set(reads), set(writes)
        else:
            self._epoch_reads |= reads
            self._epoch_writes |= writes
        self._ordered_next = False
        from .. import _native as nat

        flags = 0 if ordered else nat.LAUNCH_UNORDERED
        if self.launch_log is not None:
            self.launch_log.append((kind, first, count, flags))
        if self._suppress:
            return
        if self.on_launch is not None:
            self.on_launch(plan, kind, first, count, flags)
            return
        if self.on_set is None and (plan.device is None or plan.device.type != "cuda"):
            raise RuntimeError("this plan was compiled for host inspection; the executor only runs on a GPU (there is no CPU path)")
        if not self.group_launches or kind in _UNGROUPED:
            self._flush()
            if self._tx_calls is not None:
                self._tx_calls.append(([(plan, kind, first, count)], flags, True))
            if self.on_set is not None:
                self.on_set([(plan, kind, first, count)], flags)
            else:
                plan.launch_step(kind, first, count, self._stream.cuda_stream, flags)
            return
        # an ordered launch closes the set before it and opens the next one; an unordered launch depends on
        # nothing since the last ordered one, members of the open set included, so it joins the set
        if ordered:
            self._flush()
            self._group_flags = 0
        elif not self._group:
            self._group_flags = nat.LAUNCH_UNORDERED
        self._group.append((plan, kind, first, count))

    def _flush(self) -> None:
        """Hand the collected set of independent launches to the library."""
        if not self._group:
            return
        from .. import _native as nat

        group, self._group = self._group, []
        if self._tx_calls is not None:
            self._tx_calls.append((group, self._group_flags, len(group) == 1))
        if self.on_set is not None:
            self.on_set(group, self._group_flags)
            return
        if len(group) == 1:
            plan, kind, first, count = group[0]
            plan.launch_step(kind, first, count, self._stream.cuda_stream, self._group_flags)
            return
        nat.launch_segments([plan.segment(kind, first, count) for plan, kind, first, count in group],
                            self._stream.cuda_stream, self._group_flags)


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
