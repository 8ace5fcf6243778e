"""The wire step between two processes on one GPU, timed.

    python -m etha_amd.comm.bench_wire [--workload NAME] [--steps K] [--warmup W] [--pool ring|resident] [--max-in-flight D]

A producer process holds every source rank's shards and the bucket pool; a consumer process holds the measured
target ranks' shards and maps the pool with ``hipIpcOpenMemHandle``.  The reference's counterpart is the step
between ``Bucket.prepare`` and ``Bucket.finalize`` - ``isend/irecv/broadcast`` between two jobs
(``src/etha/comm/transfer.py:20-41``) with at most ``max_in_flight`` buckets per channel alive
(``comm_methods.py:63-117``).  With a ring pool the producer owns ``max_in_flight`` slots per channel and the two
processes trade "packed" / "unpacked" notifications behind host-side fences while the transfer runs
(:meth:`LoopbackWire.exchange`); with a resident pool (a slot per bucket) one notification per transfer is enough.

One transfer is timed on the host clock from the moment the producer starts packing to the moment the consumer's
last unpack has completed on the device.  After the timed transfers the consumer's shards are compared, bit for
bit, with the same transfer done inside one process.  Prints ONE JSON line.
"""

from __future__ import annotations

import argparse
import json
import multiprocessing as mp
import sys
import time
import traceback


def _job(workload, device, pool, depth, wire=None):
    from etha_amd import workloads
    from etha_amd.world import ReshardJob

    specs, targets, bucket = workloads.WORKLOADS[workload]()
    return ReshardJob(specs, device=device, bucket_size=bucket, target_ranks=targets, pool=pool, max_in_flight=depth, wire=wire)


def _consumer(workload, device, pool, depth, rounds, conn, out_q) -> None:
    try:
        import torch

        from etha_amd.comm import LoopbackWire
        from etha_amd.tensor_bus.bootstrap import setup_ptrace

        setup_ptrace()
        kind, manifest = conn.recv()
        assert kind == "manifest", manifest
        wire = LoopbackWire.from_manifest(manifest, device)
        job = _job(workload, device, pool, depth, wire=wire)
        for buckets in job.recv_buckets.values():
            wire.plan(buckets)
        conn.send(("ready", None))
        for _ in range(rounds):
            if pool == "ring":
                job.run_recv(merge_launches=True, drive=False)
                wire.exchange(conn)
            else:
                assert conn.recv()[0] == "packed"
                wire.mark_packed()
                job.run_recv(merge_launches=True)
            torch.cuda.current_stream(job.device).synchronize()
            conn.send(("done", time.time()))
        # the same transfer inside this process: same seeds, so the same source values
        ref = _job(workload, device, "ring", 2)
        ref.run(merge_launches=True)
        bad = []
        for i, (mine, theirs) in enumerate(zip(job.target_locals, ref.target_locals)):
            for r, t in mine.items():
                if not torch.equal(t.contiguous().view(torch.uint8), theirs[r].contiguous().view(torch.uint8)):
                    bad.append((job.specs[i].name, r))
        wire.close_imported()
        out_q.put(("ok" if not bad else "mismatch", {"bad": bad[:5], "tensors": sum(len(d) for d in job.target_locals)}))
    except BaseException:
        out_q.put(("error", traceback.format_exc()))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="llama3_8b_fsdp8_to_tp2")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--pool", choices=["ring", "resident"], default="ring")
    ap.add_argument("--max-in-flight", type=int, default=2)
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args()

    import torch

    from etha_amd import _native
    from etha_amd.tensor_bus.bootstrap import setup_ptrace

    _native.lib()
    if not torch.cuda.is_available():
        print("bench_wire needs a GPU: the hot path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    setup_ptrace()
    ctx = mp.get_context("spawn")
    mine, theirs = ctx.Pipe()
    out_q = ctx.Queue()
    rounds = args.warmup + args.steps
    proc = ctx.Process(target=_consumer, args=(args.workload, args.device, args.pool, args.max_in_flight, rounds, theirs, out_q))
    proc.start()
    try:
        job = _job(args.workload, args.device, args.pool, args.max_in_flight)
        for buckets in job.send_buckets.values():
            job.wire.plan(buckets)
        mine.send(("manifest", job.wire.export_manifest()))
        if not mine.poll(300):
            raise RuntimeError("the consumer process did not come up")
        assert mine.recv()[0] == "ready"
        lat = []
        for k in range(rounds):
            t0 = time.time()
            if args.pool == "ring":
                job.run_send(merge_launches=True, drive=False)
                job.wire.exchange(mine)
            else:
                job.run_send(merge_launches=True)
                torch.cuda.current_stream(job.device).synchronize()
                mine.send(("packed", k))
            if not mine.poll(120):
                raise RuntimeError("the consumer process stopped answering")
            kind, t1 = mine.recv()
            assert kind == "done", (kind, t1)
            if k >= args.warmup:
                lat.append(t1 - t0)
        status, detail = out_q.get(timeout=300)
        if status != "ok":
            raise RuntimeError(f"consumer: {status}: {detail}")
    finally:
        proc.join(timeout=60)
        if proc.is_alive():
            proc.kill()
    lat.sort()
    med = lat[len(lat) // 2]
    payload = job.payload_bytes()
    print(json.dumps({
        "metric": "pack in a producer process, unpack in a consumer process, one GPU (bucket pool shared over hipIPC)",
        "value": payload / med / 1e9, "unit": "GB/s", "ms_per_transfer": med * 1e3, "min_ms": lat[0] * 1e3,
        "steps": args.steps, "warmup": args.warmup, "payload_bytes": payload,
        "config": {"workload": args.workload, "pool": args.pool, "max_in_flight": args.max_in_flight,
                   "pool_reserved_bytes": job.wire.pool.reserved_bytes if job.wire.pool is not None else 0},
        "target_tensors_bit_equal_to_the_in_process_transfer": detail["tensors"],
    }))


if __name__ == "__main__":
    main()
