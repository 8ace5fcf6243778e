"""TEST INFRASTRUCTURE.  The reference's CPU/gloo redistribute: one process per rank, real wire.

``reference_path`` replaces the wire by an in-memory mailbox.  This module keeps the byte work of
``reference_path`` and restates the wire step itself, so that a whole redistribute runs the way the
reference's CPU tests run it (``tests/test_communication_cpu.py:25-118``): ``world_size`` processes
in one gloo process group, every rank executing only its own buckets.

* P2P bucket       - ``dist.isend(buffer, dst)`` on the source, ``dist.irecv(buffer, src)`` on the
  target (``src/etha/comm/transfer.py:20-31``).
* BROADCAST bucket - ``dist.broadcast(buffer, src, group, async_op=True)`` over the sorted ranks of
  source and destinations (``transfer.py:34-42``); the sub-groups are created up front by every rank
  in one sorted order, as the reference does while building chunks (``get_chunks.py:48-55``).
* LOCAL bucket     - prepare then finalize, no wire (``ir.py:277-279``).
* pipeline         - per channel key at most two buckets prepared or in flight, FIFO within a channel,
  sweeps of prepare -> launch -> complete over all channels (``comm_methods.py:53-119``); on CPU
  "complete" waits for the work (``ir.py:294-297``).

Receive buffers are fresh ``torch.empty`` per bucket, as in the reference (``ir.py:246``).  The
plan (chunks, buckets) is duck-typed and comes from the caller's ``make_job``; every process
builds the same job and then touches only its own rank's buckets, so matching between a sender's
k-th bucket and a receiver's k-th bucket is left to gloo's ordering, as in the reference.

Partial sources are collapsed by ``reference_path.chunk_prepare``'s closed form (every process
holds all members' contributions), not by an all-reduce.
"""

from __future__ import annotations

import os
import socket
import time
from collections import deque

import torch

from . import reference_path


def _free_port() -> int:
    with socket.socket(socket.AF_INET, socket.SOCK_STREAM) as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def _kind(bucket) -> str:
    return bucket.chunks[0].transport.value


def _broadcast_ranks(bucket) -> tuple[int, ...]:
    c = bucket.chunks[0]
    return tuple(sorted({int(c.src_rank), *(int(d) for d in c.dst_ranks)}))


class _InFlight:
    __slots__ = ("bucket", "buffer", "work")

    def __init__(self, bucket, buffer, work):
        self.bucket, self.buffer, self.work = bucket, buffer, work


def run_rank_gloo(buckets, rank: int, groups: dict, max_in_flight: int = 2) -> None:
    """One rank's ``bucket_comm`` over the default gloo group."""
    import torch.distributed as dist

    channels: dict = {}
    for b in buckets:
        if _kind(b) == "none":
            continue
        channels.setdefault(b.key, {"todo": deque(), "ready": deque(), "flying": deque()})["todo"].append(b)

    def prepare(b):
        first = b.chunks[0]
        if _kind(b) == "local" or first.is_source:
            return reference_path.bucket_prepare_source(b)
        return torch.empty(b.total_bytes, dtype=torch.uint8)

    def launch(b, buffer):
        first, kind = b.chunks[0], _kind(b)
        if kind == "local":
            return None
        if kind == "p2p":
            if first.is_source:
                return dist.isend(buffer, dst=int(first.dst_ranks[0]))
            return dist.irecv(buffer, src=int(first.src_rank))
        return dist.broadcast(buffer, src=int(first.src_rank), group=groups[_broadcast_ranks(b)], async_op=True)

    def finish(item: _InFlight):
        if item.work is not None:
            item.work.wait()
        b = item.bucket
        if _kind(b) == "local" or b.chunks[0].is_target:
            reference_path.bucket_finalize_target(b, item.buffer)

    while any(ch["todo"] or ch["ready"] or ch["flying"] for ch in channels.values()):
        for ch in channels.values():
            while ch["todo"] and len(ch["ready"]) + len(ch["flying"]) < max_in_flight:
                b = ch["todo"].popleft()
                ch["ready"].append((b, prepare(b)))
        for ch in channels.values():
            while ch["ready"]:
                b, buffer = ch["ready"].popleft()
                ch["flying"].append(_InFlight(b, buffer, launch(b, buffer)))
        for ch in channels.values():
            while ch["flying"]:
                finish(ch["flying"].popleft())


def _rank_main(rank: int, world_size: int, port: int, make_job, make_job_args, passes: int, result_queue) -> None:
    import torch.distributed as dist

    os.dup2(2, 1)  # gloo reports its connections on stdout; keep the parent's stdout for the parent
    torch.set_num_threads(max(1, (os.cpu_count() or 1) // world_size))
    os.environ["MASTER_ADDR"] = "127.0.0.1"
    os.environ["MASTER_PORT"] = str(port)
    dist.init_process_group(backend="gloo", rank=rank, world_size=world_size)
    try:
        job = make_job(*make_job_args)
        every = [b for bs in list(job.send_buckets.values()) + list(job.recv_buckets.values()) for b in bs]
        groups = {}
        for ranks in sorted({_broadcast_ranks(b) for b in every if _kind(b) == "broadcast"}):
            groups[ranks] = dist.new_group(list(ranks), backend="gloo")
        mine = list(job.send_buckets.get(rank, [])) + list(job.recv_buckets.get(rank, []))
        times = []
        for _ in range(passes):
            dist.barrier()
            t0 = time.perf_counter()
            run_rank_gloo(mine, rank, groups)
            dist.barrier()
            times.append(time.perf_counter() - t0)
        # plain bytes, not shared-memory tensors: the parent may read them after this process has gone
        locals_ = {i: (str(d[rank].dtype), tuple(d[rank].shape),
                       d[rank].contiguous().reshape(-1).view(torch.uint8).numpy().tobytes())
                   for i, d in enumerate(job.target_locals) if rank in d}
        result_queue.put((rank, times, locals_, torch.get_num_threads()))
    finally:
        dist.destroy_process_group()


def run(make_job, make_job_args: tuple, world_size: int, passes: int = 1, timeout: float = 120.0):
    """Run a whole redistribute over ``world_size`` gloo processes on this host.

    ``make_job(*make_job_args)`` must be a picklable module-level callable returning an object with
    ``send_buckets``/``recv_buckets`` (rank -> bucket list) and ``target_locals`` (per tensor:
    rank -> CPU tensor); every process calls it and gets the same plan and the same source data.
    Returns ``(target_locals, seconds, threads)``: per tensor index the dict rank -> target local
    after the transfer, per pass the slowest rank's wall time between two barriers, and the compute
    threads each process used.
    """
    import torch.multiprocessing as mp

    ctx = mp.get_context("spawn")
    queue = ctx.Queue()
    port = _free_port()
    procs = [ctx.Process(target=_rank_main, args=(r, world_size, port, make_job, make_job_args, passes, queue),
                         daemon=True) for r in range(world_size)]
    for p in procs:
        p.start()
    results = {}
    deadline = time.monotonic() + timeout
    try:
        while len(results) < world_size:
            left = deadline - time.monotonic()
            if left <= 0:
                raise TimeoutError(f"gloo redistribute: {len(results)}/{world_size} ranks reported in {timeout} s")
            try:
                rank, times, locals_, threads = queue.get(timeout=min(left, 1.0))
            except Exception:
                dead = [p for p in procs if p.exitcode not in (None, 0)]
                if dead:
                    raise RuntimeError(f"gloo redistribute: rank process exited with {dead[0].exitcode}") from None
                continue
            results[rank] = (times, locals_, threads)
    finally:
        for p in procs:
            p.join(timeout=10.0)
        for p in procs:
            if p.is_alive():
                p.kill()
    merged: dict[int, dict[int, torch.Tensor]] = {}
    for rank, (_, locals_, _) in results.items():
        for i, (dtype, shape, raw) in locals_.items():
            t = torch.frombuffer(bytearray(raw), dtype=torch.uint8).view(getattr(torch, dtype.split(".")[1]))
            merged.setdefault(i, {})[rank] = t.reshape(shape)
    seconds = [max(results[r][0][k] for r in results) for k in range(passes)]
    return merged, seconds, results[0][2]
