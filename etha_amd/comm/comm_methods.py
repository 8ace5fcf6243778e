"""Executor: run planned buckets on the GPU.

Counterpart of ``bucket_comm`` (``src/etha/comm/comm_methods.py:53-119``).  The reference walks
per-key channels through prepare -> launch -> complete -> finalize with one ATen launch per chunk and
at most ``max_in_flight`` buckets per channel alive.  Here a bucket list is compiled once into tile
programs (:class:`TransferPlan`) and a transfer walks the same per-channel pipeline
(:class:`Program`), where

* ``prepare`` of a source bucket is one pack (or reduce-pack) launch into the channel's next ring slot,
  possible only once every consumer of the slot's previous bucket has unpacked;
* the wire step is nothing: the consumer reads the producer's pool slot;
* ``is_complete`` of a target bucket is "its send bucket has been packed", and its ``finalize`` is one
  unpack launch; ``is_complete`` of a source bucket is "every destination has unpacked";
* LOCAL buckets: one direct self-copy launch, or pack + unpack through a private slot when source and
  destination bytes may overlap; for a Partial source the launch combines the members straight into the
  target region;
* NONE buckets: nothing - the primary's reduce-pack already read this member's partial;
* with the wire's ``zero_copy_single_chunk`` option, a single-chunk source bucket whose bytes already lie
  contiguously in the tensor is lent, not packed: the consumer unpacks straight from the tensor;
* with the wire's ``direct_same_device`` option no bucket is packed at all: the target bucket's launch
  copies (for a Partial source: reduces) from the producer's chunk regions into its own tensors in one pass.

Every rank's pipeline lives on the wire (:meth:`LoopbackWire.drive`): a sender that has filled its ring
waits there for its receivers' ``bucket_comm`` call, as the reference's sender process waits for the
receiver's.  All work goes to one stream; launches that do not touch the same bytes are issued without
ordering between them, so that one bucket's kernel starts while the previous one drains.  With a
resident pool (``LoopbackWire(pool="resident")``) a bucket list runs in list order instead, and
consecutive buckets of one kind can share a launch (``merge_launches=True``).  The call returns after
synchronising the stream, like the reference's final ``torch.cuda.synchronize()`` (``comm_methods.py:119``).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

import torch

from .device_plan import DescBuilder, SelfCopyBuilder, _storage_range, local_bucket_needs_staging
from .ir import Bucket
from .transfer import Transport

__all__ = ["bucket_comm", "TransferPlan", "Program"]

_PACK, _REDUCE, _UNPACK, _SELF, _LEND, _DIRECT, _DIRECT_REDUCE, _SELF_REDUCE = (
    "pack", "reduce_pack", "unpack", "selfcopy", "lend", "direct", "direct_reduce", "selfcopy_reduce")


@dataclass
class StepInfo:
    """What the pipeline needs to know about one step beyond its launch arguments."""

    bucket: Bucket
    entry: object = None  # the wire entry of a wire bucket's step
    reads: frozenset = frozenset()  # allocations (tensor storages, pool slots) the launch reads
    writes: frozenset = frozenset()  # allocations it writes
    excl: frozenset = frozenset()  # written allocations that no other launch may write at the same time (pool slots)
    tiles: bool = True  # False: the step moves nothing (empty shards) and launches nothing


def _storages(tensors) -> frozenset:
    return frozenset(_storage_range(t)[0] for t in tensors if t is not None)


class TransferPlan:
    """Compiled form of one rank's bucket list."""

    def __init__(self, wire, buckets: list[Bucket], scope=None, max_in_flight: int = 2):
        self.wire = wire
        self.scope = scope
        self.buckets = buckets
        self.max_in_flight = max(1, int(max_in_flight))
        self.device: torch.device | None = None
        send, recv, local = DescBuilder(), DescBuilder(), SelfCopyBuilder()
        # steps: (kind, first_chunk, n_chunks, slot or None), in bucket-list order; info[i] belongs to steps[i]
        self.steps: list[tuple[str, int, int, object]] = []
        self.info: list[StepInfo] = []
        self.steps_of: dict[int, list[int]] = {}  # id(bucket) -> indices of its steps
        self.bucket_steps: dict[int, list] = {}  # id(bucket) -> [(index, kind, info)], filled on first use
        self.lent: set[int] = set()  # ids of source buckets that are consumed straight from their tensor
        self.direct_read_bytes = 0  # bytes the direct steps read from producers' tensors (source dtype)
        self.owned_entries: list = []  # wire entries of this list's send buckets
        self.owned_slots: list = []  # pool slots this plan allocated (ring slots, resident slots, private slots)
        self._ordered_ranges: set = set()  # merged launches whose tiles the library keeps in written-address order
        for bucket in buckets:
            if not bucket.chunks:
                continue
            first_tensor = bucket.chunks[0].tensor
            if first_tensor is None:
                raise ValueError(f"{bucket}: chunks without a tensor cannot be executed")
            device = first_tensor.device
            if device.type != "cuda" and not getattr(wire, "host_inspection", False):
                raise RuntimeError(
                    f"{bucket}: tensors live on {device}; this executor only runs on a GPU (there is no CPU path)"
                )
            if self.device is None:
                self.device = device
            elif device != self.device:
                raise RuntimeError("all buckets of one call must live on the same GPU")
        rings, ordinal = {}, {}
        if wire.pool_mode == "ring" and self.device is not None:
            rings = wire.open_rings(buckets, self.device, self.max_in_flight)
            for ring in rings.values():
                self.owned_slots.extend(ring)
        for bucket in buckets:
            if not bucket.chunks:
                continue
            device = self.device
            transport = bucket.transport
            if transport == Transport.NONE:
                continue
            if transport == Transport.LOCAL:
                srcs = [c.src_tensor if c.src_tensor is not None else c.tensor for c in bucket.chunks]
                dsts = [c.tensor for c in bucket.chunks]
                if local_bucket_needs_staging(bucket):
                    slot = wire.private_slot(bucket.total_bytes, device)
                    self.owned_slots.append(slot)
                    f_send, f_recv = len(send), len(recv)
                    for off, c, src_t in zip(bucket.offsets, bucket.chunks, srcs):
                        send.add_chunk(c, src_t, c.src_slice, slot, off, reduce=False)
                        recv.add_chunk(c, c.tensor, c.dst_slice, slot, off, reduce=False)
                    sid = frozenset((slot.ptr,))
                    self._add(_PACK, f_send, len(bucket.chunks), slot,
                              StepInfo(bucket, reads=_storages(srcs), writes=sid, excl=sid))
                    self._add(_UNPACK, f_recv, len(bucket.chunks), slot, StepInfo(bucket, reads=sid, writes=_storages(dsts)))
                else:
                    first = len(local)
                    reduce = bool(bucket.chunks[0].source_partial_groups)  # buckets never mix Partial and plain chunks
                    for c in bucket.chunks:
                        local.add_chunk(c)
                        if reduce:
                            srcs.extend(c.partial_peers()[0])
                    self._add(_SELF_REDUCE if reduce else _SELF, first, len(bucket.chunks), None,
                              StepInfo(bucket, reads=_storages(srcs), writes=_storages(dsts)))
                continue
            if bucket.is_source:
                from .loopback import wire_key

                key = wire_key(bucket)
                k = ordinal.get(key, 0)
                entry = wire.entry_for_send(bucket, device, scope, ring=rings.get(key), ordinal=k)
                ordinal[key] = k + 1
                self.owned_entries.append(entry)
                slot = entry.slot
                if slot.borrowed:  # zero-copy: the consumer reads the tensor itself; nothing to launch
                    self._add(_LEND, 0, 0, slot, StepInfo(bucket, entry=entry, tiles=False))
                    self.lent.add(id(bucket))
                    continue
                if wire.pool_mode != "ring":
                    self.owned_slots.append(slot)
                first = len(send)
                reduce = bool(bucket.chunks[0].source_partial_groups)
                read_from = []
                for off, c in zip(bucket.offsets, bucket.chunks):
                    send.add_chunk(c, c.tensor, c.src_slice, slot, off, reduce=reduce)
                    peers = c.partial_peers() if reduce else None
                    read_from.extend(peers[0] if peers else (c.tensor,))
                sid = frozenset((slot.ptr,))
                self._add(_REDUCE if reduce else _PACK, first, len(bucket.chunks), slot,
                          StepInfo(bucket, entry=entry, reads=_storages(read_from), writes=sid, excl=sid))
            elif bucket.is_target:
                entry = wire.entry_for_recv(bucket, scope)
                slot = entry.slot
                dsts = _storages(c.tensor for c in bucket.chunks)
                if slot.sources is not None:  # direct wire: copy from the producer's regions, no bucket
                    first = len(local)
                    reduce = slot.sources[0][3] is not None  # buckets never mix Partial and plain chunks
                    read_from = []
                    for c, (src_t, src_slice, wire_dtype, peers) in zip(bucket.chunks, slot.sources):
                        if peers is None and wire_dtype not in (src_t.dtype, c.tensor.dtype):
                            raise NotImplementedError(
                                f"{bucket}: wire dtype {wire_dtype} differs from both tensor dtypes; one direct "
                                "conversion cannot reproduce the two roundings")
                        local.add_pair(src_t, src_slice, c.tensor, c.dst_slice, c.chunk_shape, peers=peers,
                                       wire_dtype=wire_dtype)
                        members = len(peers[0]) if peers is not None else 1
                        self.direct_read_bytes += c.nbytes // wire_dtype.itemsize * src_t.element_size() * members
                        read_from.extend(peers[0] if peers is not None else (src_t,))
                    self._add(_DIRECT_REDUCE if reduce else _DIRECT, first, len(bucket.chunks), slot,
                              StepInfo(bucket, entry=entry, reads=_storages(read_from), writes=dsts))
                    continue
                first = len(recv)
                for off, c in zip(bucket.offsets, bucket.chunks):
                    recv.add_chunk(c, c.tensor, c.dst_slice, slot, off, reduce=False)
                read_from = frozenset((slot.ptr,)) if not slot.borrowed else _storages([slot.keepalive])
                self._add(_UNPACK, first, len(bucket.chunks), slot, StepInfo(bucket, entry=entry, reads=read_from, writes=dsts))
        self._keepalive = send.keepalive + recv.keepalive + local.keepalive
        self.merged_steps = self._merge(self.steps, self.info)
        self.send_table = self.recv_table = self.local_table = None
        if self.device is None:
            return
        if self.device.type != "cuda":  # host inspection: compile the programs, never upload or launch them
            self.send_table = send.build(upload=False)
            self.recv_table = recv.build(upload=False)
            self.local_table = local.build(upload=False)
        else:
            with torch.cuda.device(self.device):  # the tile programs are uploaded to the tensors' device
                self.send_table = send.build()
                self.recv_table = recv.build()
                self.local_table = local.build()
        self._mark_empty_steps()
        if wire.pool_mode == "resident":
            with torch.cuda.device(self.device) if self.device.type == "cuda" else _nullcontext():
                self._optimize_merged_ranges()

    def _add(self, kind: str, first: int, count: int, slot, info: StepInfo) -> None:
        self.steps_of.setdefault(id(info.bucket), []).append(len(self.steps))
        self.steps.append((kind, first, count, slot))
        self.info.append(info)

    def _table_of(self, kind: str):
        if kind in (_PACK, _REDUCE):
            return self.send_table
        if kind == _UNPACK:
            return self.recv_table
        if kind in (_SELF, _SELF_REDUCE, _DIRECT, _DIRECT_REDUCE):
            return self.local_table
        return None

    def _mark_empty_steps(self) -> None:
        """A step whose chunks are all empty launches no kernel; the pipeline must know, because a launch that
        does not happen orders nothing."""
        begins = {}
        for table in (self.send_table, self.recv_table, self.local_table):
            if table is not None:
                run, row = table.ranges()
                begins[id(table)] = (run, row, table.trans_ranges())
        for (kind, first, count, _), info in zip(self.steps, self.info):
            table = self._table_of(kind)
            if table is None:
                info.tiles = False
                continue
            info.tiles = any(int(b[first + count]) > int(b[first]) for b in begins[id(table)])

    def _optimize_merged_ranges(self) -> None:
        """Merged unpack / self-copy launches cover several buckets: let the library order their tiles by
        written address, so that rows of one tensor arriving through different buckets are written together."""
        for kind, first, count, slots in self.merged_steps:
            if len(slots) > 1 and kind == _UNPACK:
                self.recv_table.optimize_range(first, count)
            elif len(slots) > 1 and kind in (_SELF, _DIRECT):
                self.local_table.optimize_range(first, count)

    @staticmethod
    def _merge(steps, info=None):
        """Fuse consecutive steps of one kind whose chunk ranges are adjacent.  A step that reads an allocation
        an earlier step of the run writes (or the other way round) - two self-copy buckets inside one tensor -
        starts a new launch, so that it still runs after the earlier one, as it does unmerged."""
        merged: list[list] = []
        touched: list[tuple[set, set]] = []  # per merged launch: allocations read / written
        lends = [s[3] for s in steps if s[0] == _LEND]
        if lends:  # nothing is launched for them; keep them out of the way of merging their neighbours
            merged.append([_LEND, 0, 0, list(lends)])
            touched.append((set(), set()))
        for i, (kind, first, count, slot) in enumerate(steps):
            if kind == _LEND:
                continue
            reads = set(info[i].reads) if info is not None else set()
            writes = set(info[i].writes) if info is not None else set()
            if merged and merged[-1][0] == kind and merged[-1][1] + merged[-1][2] == first \
                    and not (reads & touched[-1][1]) and not (writes & touched[-1][0]):
                merged[-1][2] += count
                merged[-1][3].append(slot)
                touched[-1][0].update(reads)
                touched[-1][1].update(writes)
            else:
                merged.append([kind, first, count, [slot]])
                touched.append((reads, writes))
        return [(k, f, c, tuple(s)) for k, f, c, s in merged]

    def order_by_written_address(self, kind: str, first: int, count: int) -> None:
        """A scattering launch that covers several buckets and keeps recurring (the pipelines repeat the same
        schedule every transfer): let the library keep that range's tiles ordered by written address."""
        if kind not in (_UNPACK, _SELF, _DIRECT) or (kind, first, count) in self._ordered_ranges:
            return
        if self.device is not None and self.device.type == "cuda" and torch.cuda.is_current_stream_capturing():
            return  # uploads cannot be captured; the range keeps its list order
        self._ordered_ranges.add((kind, first, count))
        self._table_of(kind).optimize_range(first, count)

    def launch_step(self, kind: str, first: int, count: int, stream: int, flags: int = 0) -> None:
        """One launch: chunks ``[first, first + count)`` of the table that ``kind`` runs on."""
        if kind == _PACK:
            self.send_table.pack(first, count, stream, flags)
        elif kind == _REDUCE:
            self.send_table.reduce_pack(first, count, stream, flags)
        elif kind == _UNPACK:
            self.recv_table.unpack(first, count, stream, flags)
        elif kind in (_SELF, _SELF_REDUCE, _DIRECT, _DIRECT_REDUCE):
            self.local_table.selfcopy(first, count, stream, flags)

    def segment(self, kind: str, first: int, count: int) -> tuple:
        """The same launch as an entry of a set for ``_native.launch_segments``."""
        from .. import _native as nat

        if kind == _PACK:
            return (self.send_table, nat.SEG_PACK, first, count)
        if kind == _REDUCE:
            return (self.send_table, nat.SEG_REDUCE_PACK, first, count)
        if kind == _UNPACK:
            return (self.recv_table, nat.SEG_UNPACK, first, count)
        return (self.local_table, nat.SEG_SELFCOPY, first, count)

    # ---- resident pool: the bucket list in list order -------------------------------------------------
    def run(self, stream: int | None = None, merge_launches: bool = False, fanout: int = 1) -> None:
        """Enqueue this bucket list's launches in list order (resident pool only: with a ring the list's
        buckets share slots and must go through the wire's pipelines, see :func:`bucket_comm`).

        ``fanout > 1`` spreads the launches of independent buckets over that many side streams,
        forked from and joined back into the current stream with events, so that the tail of one
        bucket's kernel overlaps the head of the next (a single stream serialises kernels).  Buckets
        that share a pool slot (a staged self-copy's pack and unpack) stay on one stream, in order.
        """
        if self.device is None:
            return
        if self.device.type != "cuda":
            raise RuntimeError("this plan was compiled for host inspection; the executor only runs on a GPU (there is no CPU path)")
        if self.wire.pool_mode != "resident":
            raise RuntimeError("a plan on a ring pool runs through bucket_comm (its buckets share slots)")
        steps = self.merged_steps if merge_launches else [(k, f, c, (s,)) for k, f, c, s in self.steps]
        if fanout > 1 and stream is None and len(steps) > 1:
            self._run_fanout(steps, fanout)
            return
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            self._enqueue(steps, lambda i, slots: stream)

    def run_kinds(self, kinds: tuple[str, ...]) -> None:
        """Enqueue only the steps of the given kinds on the current stream (single-bucket protocol).  On a ring
        pool a step that would have to wait (a slot still held, a send bucket not packed yet) raises."""
        if self.device is None:
            return
        if self.device.type != "cuda":
            raise RuntimeError("this plan was compiled for host inspection; the executor only runs on a GPU (there is no CPU path)")
        stream = torch.cuda.current_stream(self.device).cuda_stream
        if self.wire.pool_mode == "resident":
            steps = [(k, f, c, (s,)) for k, f, c, s in self.steps if k in kinds]
            with torch.cuda.device(self.device):
                self._enqueue(steps, lambda i, slots: stream)
            return
        # buckets stepped by hand move slots outside the pipelines: transfers recorded on this wire no longer
        # describe what its pipelines would do
        self.wire.replay_schedules = False
        self.wire.forget_recorded_transfers()
        with torch.cuda.device(self.device):
            for (kind, first, count, _), info in zip(self.steps, self.info):
                if kind not in kinds:
                    continue
                entry = info.entry
                if kind in (_PACK, _REDUCE, _LEND) and entry is not None:
                    if not send_may_start(entry):
                        raise RuntimeError(f"{info.bucket}: its ring slot still holds a bucket that has not been unpacked "
                                           "(a real wire would block here)")
                    if info.tiles:
                        self.launch_step(kind, first, count, stream)
                    mark_sent(self.wire, entry)
                elif kind in (_UNPACK, _DIRECT, _DIRECT_REDUCE) and entry is not None:
                    if not recv_may_start(entry, info.bucket.rank):
                        raise RuntimeError(f"{info.bucket}: recv bucket runs before its send bucket was packed "
                                           "(a real wire would block here)")
                    if info.tiles:
                        self.launch_step(kind, first, count, stream)
                    mark_received(entry, info.bucket.rank, self.wire)
                elif info.tiles:
                    self.launch_step(kind, first, count, stream)

    def _run_fanout(self, steps, fanout: int) -> None:
        main = torch.cuda.current_stream(self.device)
        side = self.wire.side_streams(self.device, fanout)
        fork = torch.cuda.Event()
        fork.record(main)
        for s in side:
            s.wait_event(fork)
        lane_of_slot: dict[int, int] = {}
        lane_of_alloc: dict[int, int] = {}  # allocations written by a self-copy: later steps that touch them follow it
        local = [(f, info.reads | info.writes, info.writes)
                 for (k, f, _, _), info in zip(self.steps, self.info) if k == _SELF]

        def pick(i, slots):
            key = id(slots[0]) if slots and slots[0] is not None else None
            kind, first, count = steps[i][0], steps[i][1], steps[i][2]
            touched, written = set(), set()
            if kind == _SELF:
                for f, t, w in local:
                    if first <= f < first + count:
                        touched |= t
                        written |= w
            follow = [lane_of_alloc[a] for a in touched if a in lane_of_alloc]
            if key is not None and key in lane_of_slot:
                lane = lane_of_slot[key]
            elif follow:
                lane = follow[0]
            else:
                lane = i % len(side)
            if key is not None:
                lane_of_slot[key] = lane
            for a in written:
                lane_of_alloc[a] = lane
            return side[lane].cuda_stream

        with torch.cuda.device(self.device):
            self._enqueue(steps, pick)
        for s in side:
            done = torch.cuda.Event()
            done.record(s)
            main.wait_event(done)

    def _enqueue(self, steps, stream_of) -> None:
        for i, (kind, first, count, slots) in enumerate(steps):
            stream = stream_of(i, slots)
            if kind in (_UNPACK, _DIRECT, _DIRECT_REDUCE):
                for s in slots:
                    if s is not None and s.filled == 0:
                        raise RuntimeError(
                            "recv bucket runs before its send bucket was ever packed (a real wire would block here)"
                        )
            self.launch_step(kind, first, count, stream)
            if kind in (_PACK, _REDUCE, _LEND):
                for s in slots:
                    if s is not None:
                        s.filled += 1

    def lends_tensor_memory(self) -> bool:
        """True when some send bucket of this plan is consumed straight from its source tensor."""
        return any(kind == _LEND for kind, _, _, _ in self.steps)

    def payload_bytes(self) -> dict[str, int]:
        out = {}
        for name, table in (("send", self.send_table), ("recv", self.recv_table), ("local", self.local_table)):
            out[name] = table.info().payload_bytes if table is not None else 0
        return out


class _nullcontext:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


# ---- slot hand-over between a send bucket and its receivers ------------------------------------------
def send_may_start(entry) -> bool:
    """A send bucket may be packed once its slot is free: every consumer of the slot's previous bucket (this
    bucket's previous transfer, or the bucket ``max_in_flight`` places ahead on the channel) has unpacked."""
    return entry.slot.holder is None


def mark_sent(wire, entry) -> None:
    entry.packed += 1
    entry.left = wire.consumers(entry)
    entry.slot.filled += 1
    entry.slot.holder = entry if entry.left else None
    if wire.outbox is not None and entry.left:  # the consumers live in another process: tell them
        wire.outbox.append(("packed", entry.key, entry.seq))


def recv_may_start(entry, rank) -> bool:
    return entry.slot.holder is entry and rank in entry.left


def mark_received(entry, rank, wire=None) -> None:
    entry.left.discard(rank)
    entry.slot.drained += 1
    if not entry.left:
        entry.slot.holder = None
    if wire is not None and wire.outbox is not None and entry.remote:  # the producer lives in another process
        wire.outbox.append(("unpacked", entry.key, entry.seq, rank))


@dataclass
class _Channel:
    candidate: deque = field(default_factory=deque)
    prepared: deque = field(default_factory=deque)
    in_flight: deque = field(default_factory=deque)

    def busy(self) -> bool:
        return bool(self.candidate or self.prepared or self.in_flight)


class Program:
    """One transfer of one rank's bucket list: the reference's ``bucket_comm`` loop as a resumable object.

    Buckets queue per channel (``bucket.key``) and move candidate -> prepared -> in flight -> finalized in
    FIFO order, at most ``max_in_flight`` of a channel prepared or in flight (``comm_methods.py:63-117``).
    :meth:`sweep` is one turn of that loop and never blocks: a bucket that would have to wait for another
    rank simply stays where it is until a later sweep.
    """

    def __init__(self, plan: TransferPlan, max_in_flight: int = 2, merge_launches: bool = False):
        self.plan = plan
        self.max_in_flight = max(1, int(max_in_flight))
        self.merge = merge_launches
        self.channels: dict[tuple, _Channel] = {}
        buckets = [b for b in plan.buckets if b.chunks and b.transport != Transport.NONE]
        # a receive bucket can only ever complete if its sender has been asked for this transfer
        for b in buckets:
            for i in plan.steps_of.get(id(b), ()):
                entry, kind = plan.info[i].entry, plan.steps[i][0]
                if entry is not None and kind in (_UNPACK, _DIRECT, _DIRECT_REDUCE) and not entry.remote:
                    if entry.submitted < entry.arrived.get(b.rank, 0) + 1:
                        raise RuntimeError(
                            f"{b}: recv bucket runs before its send bucket was ever sent (a real wire would block here)")
        for b in buckets:
            for i in plan.steps_of.get(id(b), ()):
                entry, kind = plan.info[i].entry, plan.steps[i][0]
                if entry is None:
                    continue
                if kind in (_UNPACK, _DIRECT, _DIRECT_REDUCE):
                    entry.arrived[b.rank] = entry.arrived.get(b.rank, 0) + 1
                else:
                    entry.submitted += 1
            self.channels.setdefault(b.key, _Channel()).candidate.append(b)

    def __repr__(self) -> str:
        left = sum(len(c.candidate) + len(c.prepared) + len(c.in_flight) for c in self.channels.values())
        return f"Program({left} of {sum(1 for b in self.plan.buckets if b.chunks)} buckets left, first: {self.plan.buckets[0]})"

    @property
    def finished(self) -> bool:
        return not any(c.busy() for c in self.channels.values())

    def _steps(self, bucket):
        plan = self.plan
        cached = plan.bucket_steps.get(id(bucket))
        if cached is None:  # the plan's steps never change once it is compiled
            cached = plan.bucket_steps[id(bucket)] = [(i, plan.steps[i][0], plan.info[i]) for i in plan.steps_of.get(id(bucket), ())]
        return cached

    def _prepare(self, bucket, wire, todo: list) -> bool:
        steps = self._steps(bucket)
        if bucket.transport == Transport.LOCAL:
            todo.append(steps[0][0])  # the direct copy, or the pack of a staged one
            return True
        for i, kind, info in steps:
            if kind in (_PACK, _REDUCE, _LEND):
                if not send_may_start(info.entry):
                    return False
                todo.append(i)
                mark_sent(wire, info.entry)
        return True

    def _is_complete(self, bucket) -> bool:
        for _, kind, info in self._steps(bucket):
            if kind in (_PACK, _REDUCE, _LEND) and info.entry is not None and info.entry.left:
                return False  # a destination has not unpacked yet
            if kind in (_UNPACK, _DIRECT, _DIRECT_REDUCE) and info.entry is not None \
                    and not recv_may_start(info.entry, bucket.rank):
                return False  # nothing has arrived yet
        return True

    def _finalize(self, bucket, todo: list, wire=None) -> None:
        steps = self._steps(bucket)
        if bucket.transport == Transport.LOCAL:
            todo.extend(i for i, _, _ in steps[1:])  # the unpack of a staged copy
            return
        for i, kind, info in steps:
            if kind in (_UNPACK, _DIRECT, _DIRECT_REDUCE):
                todo.append(i)
                mark_received(info.entry, bucket.rank, wire)

    def sweep(self, wire) -> bool:
        """One turn of the prepare / launch / complete phases over all channels; True if anything moved.
        The launches of one phase are handed to the wire together: they are independent of each other."""
        moved = False
        todo: list[int] = []
        progress = True
        while progress:
            progress = False
            for ch in self.channels.values():
                if ch.candidate and len(ch.prepared) + len(ch.in_flight) < self.max_in_flight \
                        and self._prepare(ch.candidate[0], wire, todo):
                    ch.prepared.append(ch.candidate.popleft())
                    progress = moved = True
        if todo:
            wire.emit(self.plan, todo, self.merge)
        for ch in self.channels.values():  # the wire step is a hand-over in place: always ready
            while ch.prepared:
                ch.in_flight.append(ch.prepared.popleft())
                moved = True
        todo = []
        progress = True
        while progress:
            progress = False
            for ch in self.channels.values():
                if ch.in_flight and self._is_complete(ch.in_flight[0]):
                    self._finalize(ch.in_flight.popleft(), todo, wire)
                    progress = moved = True
        if todo:
            wire.emit(self.plan, todo, self.merge)
        return moved


def bucket_comm(
    buckets: list[Bucket],
    max_in_flight: int = 2,
    *,
    wire=None,
    merge_launches: bool = False,
    synchronize: bool = True,
    fanout: int = 1,
    scope=None,
    drive: bool = True,
) -> None:
    """Run the bucket pipeline for one rank's buckets.

    ``max_in_flight`` bounds the buckets of one channel that are prepared or in flight, and with the
    default ring pool it is also the number of pool slots the channel owns (fixed when the list is
    first planned).  The call enqueues what this rank can do now and whatever it unblocks in the
    pipelines of ranks that called earlier; a sender whose receivers have not called yet leaves the
    rest of its pipeline on the wire, where the receivers' calls pick it up.

    The keyword-only arguments are additions: ``wire`` selects the loopback wire (default: the
    process-wide one), ``merge_launches`` lets neighbouring buckets that become ready together share
    a launch (ring pool) or fuses consecutive buckets of one kind (resident pool),
    ``synchronize=False`` leaves the stream un-synchronised, ``fanout`` spreads per-bucket launches
    over that many side streams (resident pool only, see :meth:`TransferPlan.run`), ``scope``
    namespaces the pairing of send and receive buckets on the wire (see :class:`LoopbackWire`),
    ``drive=False`` (ring pool) only queues this rank's pipeline on the wire: a process that plays several
    ranks queues all of them and then calls ``wire.drive()`` once, which costs one ordered launch for the
    whole group instead of one per rank.
    """
    if wire is None:
        from .loopback import default_wire

        wire = default_wire()
    if not buckets:
        return
    plan = wire.plan(buckets, scope=scope, max_in_flight=max_in_flight)
    if wire.pool_mode == "resident":
        plan.run(merge_launches=merge_launches, fanout=fanout)
    else:
        if fanout > 1:
            raise ValueError("side streams need a resident pool: LoopbackWire(pool='resident')")
        if plan.device is not None:
            wire.submit(plan, max_in_flight, merge_launches)
            if drive:
                wire.drive()
    if synchronize and plan.device is not None and plan.device.type == "cuda":
        torch.cuda.current_stream(plan.device).synchronize()
