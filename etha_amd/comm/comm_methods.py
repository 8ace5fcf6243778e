"""Executor: run planned buckets on the GPU.

Counterpart of ``bucket_comm`` (``src/etha/comm/comm_methods.py:53-119``).  The reference walks
per-key channels through prepare -> launch -> complete -> finalize with one ATen launch per chunk.
Here a bucket list is compiled once into tile programs and a call enqueues, in bucket-list order:

* source buckets:  one pack (or reduce-pack) launch each - ``Bucket.prepare``;
* the wire step:   nothing to do, the consumer reads the producer's pool slot;
* target buckets:  one unpack launch each - ``Bucket.finalize``;
* LOCAL buckets:   one direct self-copy launch each, or pack + unpack through a private slot when
                   source and destination bytes may overlap;
* NONE buckets:    nothing - the primary's reduce-pack already read this member's partial;
* with the wire's ``zero_copy_single_chunk`` option, a single-chunk source bucket whose bytes already lie
  contiguously in the tensor is lent, not packed: the consumer unpacks straight from the tensor;
* with the wire's ``direct_same_device`` option no bucket is packed at all: the target bucket's launch
  copies (for a Partial source: reduces) from the producer's chunk regions into its own tensors in one pass.

Consecutive buckets of the same kind can be merged into one launch (``merge_launches=True``).
All work goes to one stream, so per-channel FIFO order and "pack before unpack" hold by stream
order; the call returns after synchronising that stream, like the reference's final
``torch.cuda.synchronize()`` (``comm_methods.py:119``).
"""

from __future__ import annotations

import torch

from .device_plan import DescBuilder, SelfCopyBuilder, local_bucket_needs_staging
from .ir import Bucket
from .transfer import Transport

__all__ = ["bucket_comm", "TransferPlan"]

_PACK, _REDUCE, _UNPACK, _SELF, _LEND, _DIRECT, _DIRECT_REDUCE = (
    "pack", "reduce_pack", "unpack", "selfcopy", "lend", "direct", "direct_reduce")


class TransferPlan:
    """Compiled form of one rank's bucket list."""

    def __init__(self, wire, buckets: list[Bucket], scope=None):
        self.wire = wire
        self.scope = scope
        self.buckets = buckets
        self.device: torch.device | None = None
        send, recv, local = DescBuilder(), DescBuilder(), SelfCopyBuilder()
        # steps: (kind, first_chunk, n_chunks, slot or None), in execution order
        self.steps: list[tuple[str, int, int, object]] = []
        self.lent: set[int] = set()  # ids of source buckets that are consumed straight from their tensor
        self.direct_read_bytes = 0  # bytes the direct steps read from producers' tensors (source dtype)
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
            transport = bucket.transport
            if transport == Transport.NONE:
                continue
            if transport == Transport.LOCAL:
                if local_bucket_needs_staging(bucket):
                    slot = wire.private_slot(bucket.total_bytes, device)
                    f_send, f_recv = len(send), len(recv)
                    for off, c in zip(bucket.offsets, bucket.chunks):
                        src_t = c.src_tensor if c.src_tensor is not None else c.tensor
                        send.add_chunk(c, src_t, c.src_slice, slot, off, reduce=False)
                        recv.add_chunk(c, c.tensor, c.dst_slice, slot, off, reduce=False)
                    self.steps.append((_PACK, f_send, len(bucket.chunks), slot))
                    self.steps.append((_UNPACK, f_recv, len(bucket.chunks), slot))
                else:
                    first = len(local)
                    for c in bucket.chunks:
                        local.add_chunk(c)
                    self.steps.append((_SELF, first, len(bucket.chunks), None))
                continue
            if bucket.is_source:
                slot = wire.slot_for_send(bucket, device, scope)
                if slot.borrowed:  # zero-copy: the consumer reads the tensor itself; nothing to launch
                    self.steps.append((_LEND, 0, 0, slot))
                    self.lent.add(id(bucket))
                    continue
                first = len(send)
                reduce = bool(bucket.chunks[0].source_partial_groups)
                for off, c in zip(bucket.offsets, bucket.chunks):
                    send.add_chunk(c, c.tensor, c.src_slice, slot, off, reduce=reduce)
                self.steps.append((_REDUCE if reduce else _PACK, first, len(bucket.chunks), slot))
            elif bucket.is_target:
                slot = wire.slot_for_recv(bucket, scope)
                if slot.sources is not None:  # direct wire: copy from the producer's regions, no bucket
                    first = len(local)
                    reduce = slot.sources[0][3] is not None  # buckets never mix Partial and plain chunks
                    for c, (src_t, src_slice, wire_dtype, peers) in zip(bucket.chunks, slot.sources):
                        if peers is None and wire_dtype not in (src_t.dtype, c.tensor.dtype):
                            raise NotImplementedError(
                                f"{bucket}: wire dtype {wire_dtype} differs from both tensor dtypes; one direct "
                                "conversion cannot reproduce the two roundings")
                        local.add_pair(src_t, src_slice, c.tensor, c.dst_slice, c.chunk_shape, peers=peers,
                                       wire_dtype=wire_dtype)
                        members = len(peers[0]) if peers is not None else 1
                        self.direct_read_bytes += c.nbytes // wire_dtype.itemsize * src_t.element_size() * members
                    self.steps.append((_DIRECT_REDUCE if reduce else _DIRECT, first, len(bucket.chunks), slot))
                    continue
                first = len(recv)
                for off, c in zip(bucket.offsets, bucket.chunks):
                    recv.add_chunk(c, c.tensor, c.dst_slice, slot, off, reduce=False)
                self.steps.append((_UNPACK, first, len(bucket.chunks), slot))
        self._keepalive = send.keepalive + recv.keepalive + local.keepalive
        self.merged_steps = self._merge(self.steps)
        self.send_table = self.recv_table = self.local_table = None
        if self.device is None:
            return
        if self.device.type != "cuda":  # host inspection: compile the programs, never upload or launch them
            self.send_table = send.build(upload=False)
            self.recv_table = recv.build(upload=False)
            self.local_table = local.build(upload=False)
            self._optimize_merged_ranges()
            return
        with torch.cuda.device(self.device):  # the tile programs are uploaded to the tensors' device
            self.send_table = send.build()
            self.recv_table = recv.build()
            self.local_table = local.build()
            self._optimize_merged_ranges()

    def _optimize_merged_ranges(self) -> None:
        """Merged unpack / self-copy launches cover several buckets: let the library order their tiles by
        written address, so that rows of one tensor arriving through different buckets are written together."""
        for kind, first, count, slots in self.merged_steps:
            if len(slots) > 1 and kind == _UNPACK:
                self.recv_table.optimize_range(first, count)
            elif len(slots) > 1 and kind in (_SELF, _DIRECT):
                self.local_table.optimize_range(first, count)

    @staticmethod
    def _merge(steps):
        merged: list[list] = []
        lends = [s[3] for s in steps if s[0] == _LEND]
        if lends:  # nothing is launched for them; keep them out of the way of merging their neighbours
            merged.append([_LEND, 0, 0, list(lends)])
        for kind, first, count, slot in steps:
            if kind == _LEND:
                continue
            if merged and merged[-1][0] == kind and merged[-1][1] + merged[-1][2] == first:
                merged[-1][2] += count
                merged[-1][3].append(slot)
            else:
                merged.append([kind, first, count, [slot]])
        return [(k, f, c, tuple(s)) for k, f, c, s in merged]

    def run(self, stream: int | None = None, merge_launches: bool = False, fanout: int = 1) -> None:
        """Enqueue this bucket list's launches.

        ``fanout > 1`` spreads the launches of independent buckets over that many side streams,
        forked from and joined back into the current stream with events, so that the tail of one
        bucket's kernel overlaps the head of the next (a single stream serialises kernels).  Buckets
        that share a pool slot (a staged self-copy's pack and unpack) stay on one stream, in order.
        """
        if self.device is None:
            return
        if self.device.type != "cuda":
            raise RuntimeError("this plan was compiled for host inspection; the executor only runs on a GPU (there is no CPU path)")
        steps = self.merged_steps if merge_launches else [(k, f, c, (s,)) for k, f, c, s in self.steps]
        if fanout > 1 and stream is None and len(steps) > 1:
            self._run_fanout(steps, fanout)
            return
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            self._enqueue(steps, lambda i, slots: stream)

    def run_kinds(self, kinds: tuple[str, ...]) -> None:
        """Enqueue only the steps of the given kinds on the current stream (single-bucket protocol)."""
        if self.device is None:
            return
        if self.device.type != "cuda":
            raise RuntimeError("this plan was compiled for host inspection; the executor only runs on a GPU (there is no CPU path)")
        stream = torch.cuda.current_stream(self.device).cuda_stream
        steps = [(k, f, c, (s,)) for k, f, c, s in self.steps if k in kinds]
        with torch.cuda.device(self.device):
            self._enqueue(steps, lambda i, slots: stream)

    def _run_fanout(self, steps, fanout: int) -> None:
        main = torch.cuda.current_stream(self.device)
        side = self.wire.side_streams(self.device, fanout)
        fork = torch.cuda.Event()
        fork.record(main)
        for s in side:
            s.wait_event(fork)
        lane_of_slot: dict[int, int] = {}

        def pick(i, slots):
            key = id(slots[0]) if slots and slots[0] is not None else None
            if key is not None and key in lane_of_slot:
                lane = lane_of_slot[key]
            else:
                lane = i % len(side)
                if key is not None:
                    lane_of_slot[key] = lane
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
            if kind == _PACK:
                self.send_table.pack(first, count, stream)
            elif kind == _REDUCE:
                self.send_table.reduce_pack(first, count, stream)
            elif kind == _UNPACK:
                for s in slots:
                    if s is not None and s.filled == 0:
                        raise RuntimeError(
                            "recv bucket runs before its send bucket was ever packed (a real wire would block here)"
                        )
                self.recv_table.unpack(first, count, stream)
            elif kind == _SELF:
                self.local_table.selfcopy(first, count, stream)
            elif kind in (_DIRECT, _DIRECT_REDUCE):
                for s in slots:
                    if s is not None and s.filled == 0:
                        raise RuntimeError(
                            "recv bucket runs before its send bucket was ever sent (a real wire would block here)"
                        )
                self.local_table.selfcopy(first, count, stream)
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


def bucket_comm(
    buckets: list[Bucket],
    max_in_flight: int = 2,
    *,
    wire=None,
    merge_launches: bool = False,
    synchronize: bool = True,
    fanout: int = 1,
    scope=None,
) -> None:
    """Run the bucket pipeline for one rank's buckets.

    ``max_in_flight`` is accepted for compatibility; every bucket owns a persistent pool slot, so
    there is nothing to throttle.  The keyword-only arguments are additions: ``wire`` selects the
    loopback wire (default: the process-wide one), ``merge_launches`` fuses consecutive buckets of
    one kind into a single launch, ``synchronize=False`` leaves the stream un-synchronised, ``fanout``
    spreads per-bucket launches over that many side streams (see :meth:`TransferPlan.run`), ``scope``
    namespaces the pairing of send and receive buckets on the wire (see :class:`LoopbackWire`).
    """
    del max_in_flight
    if wire is None:
        from .loopback import default_wire

        wire = default_wire()
    if not buckets:
        return
    plan = wire.plan(buckets, scope=scope)
    plan.run(merge_launches=merge_launches, fanout=fanout)
    if synchronize and plan.device is not None:
        torch.cuda.current_stream(plan.device).synchronize()
