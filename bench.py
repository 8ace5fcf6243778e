"""Headline benchmark: effective reshard GB/s (pack + unpack) on one MI355X.

One step = one pass of the hot path over the workload: every source rank packs its buckets for the
measured target rank's share, then that target rank unpacks them.  Inputs are resident in HBM
before the timed region.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--per-bucket]
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# HBM bytes per launch of the dominant kernel, from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE), each
# scaled by what the counter reads for a plain 1 GiB copy; the summary of those runs is
# profiles/etha_tile_kernel_llama3_8b_fsdp8_to_tp2.txt.  Keyed by (workload, kernel, launch granularity).
MEASURED_TRAFFIC_BYTES = {
    ("llama3_8b_fsdp8_to_tp2", "etha_tile_kernel<false>", "run of buckets"): 2043040739,
    ("llama3_8b_fsdp8_to_tp2", "etha_tile_kernel<true>", "run of buckets"): 16249517705,
    # profiles/etha_reduce_kernel_partial4_to_shard2.txt
    ("partial4_to_shard2", "etha_reduce_kernel", "run of buckets"): 5436000000,
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3_8b_fsdp8_to_tp2")
    ap.add_argument("--per-bucket", action="store_true", help="one launch per bucket instead of one per run of buckets")
    ap.add_argument("--fanout", type=int, default=1, help="side streams for per-bucket launches (with --per-bucket)")
    ap.add_argument("--zero-copy", action="store_true",
                    help="lend contiguous single-chunk buckets to the consumer instead of packing them")
    ap.add_argument("--direct", action="store_true",
                    help="no bucket buffers: the target side copies straight from the source shards (one pass; "
                         "not the pack+unpack path the headline is quoted on)")
    ap.add_argument("--graph", action="store_true", help="replay the step from a captured HIP graph (whole step timed)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-per-bucket-leg", action="store_true",
                    help="skip the extra one-launch-per-bucket measurement after the timed region (use under a "
                         "profiler, so that per-kernel statistics cover the timed configuration only)")
    ap.add_argument("--cpu-layers", type=int, default=8, help="layers of the workload the CPU baseline sample covers")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU work the baseline leg is bounded to")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="after the timed region run three plain 1 GiB torch copies (known traffic, for scaling "
                         "hardware counters collected with rocprofv3 --pmc)")
    return ap.parse_args()


def _cheap_fill(spec):  # values do not affect timing; avoid minutes of CPU randn
    import torch

    n = 1
    for s in spec.shape:
        n *= s
    return (torch.arange(n, dtype=torch.int32) % 251).to(spec.source_dtype).reshape(spec.shape)


def _cpu_job(workload: str):
    """The whole workload staged on the CPU; module-level so that spawned rank processes can build it too."""
    from etha_amd import workloads
    from etha_amd.world import ReshardJob

    specs, targets, bucket = workloads.WORKLOADS[workload]()
    return ReshardJob(specs, device="cpu", bucket_size=bucket, target_ranks=targets, fill=_cheap_fill)


def gloo_baseline(workload: str, passes: int = 20):
    """The same CPU path with one process per rank and gloo isend/irecv/broadcast as the wire: the
    reference's own CPU way of running a redistribute (its tests/test_communication_cpu.py:25-118)."""
    from oracle import gloo_redistribute

    job = _cpu_job(workload)
    ranks = {int(r) for spec in job.specs for mesh in (spec.source_mesh, spec.target_mesh)
             for r in __import__("numpy").asarray(mesh).reshape(-1)}
    world = max(ranks) + 1
    _, seconds, threads = gloo_redistribute.run(_cpu_job, (workload,), world, passes=passes + 1, timeout=300.0)
    seconds = sorted(seconds[1:])
    med = seconds[len(seconds) // 2]
    return {
        "value": job.payload_bytes() / med / 1e9,
        "unit": "GB/s",
        "processes": world,
        "threads_per_process": threads,
        "ms_per_transfer": med * 1e3,
        "sample": f"whole workload, median of {len(seconds)} transfers between barriers",
    }


def cpu_baseline(workload: str, layers: int, seconds: float):
    """The oracle's op-for-op restatement of the reference path, timed on this host's cores."""
    import torch

    from etha_amd import workloads
    from etha_amd.world import ReshardJob
    from oracle import reference_path

    if workload == "llama3_8b_fsdp8_to_tp2":
        specs, targets, bucket = workloads.llama3_8b_fsdp8_to_tp2(n_layers=layers, with_embeddings=False)
        sample = f"{layers} decoder layers of the workload (no embeddings), same layouts and 64 MiB buckets"
    else:
        specs, targets, bucket = workloads.WORKLOADS[workload]()
        sample = "whole workload"

    job = ReshardJob(specs, device="cpu", bucket_size=bucket, target_ranks=targets, fill=_cheap_fill)
    payload = job.payload_bytes()

    def one_pass():
        box = reference_path.Mailbox()
        for r, buckets in job.send_buckets.items():
            reference_path.run_rank(buckets, box, rank=r)
        for r, buckets in job.recv_buckets.items():
            reference_path.run_rank(buckets, box, rank=r)

    one_pass()
    times = []
    t_end = time.perf_counter() + seconds
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 200):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": payload / med / 1e9,
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{sample}; {payload} payload bytes per pass, median of {len(times)} passes "
                  f"({sum(times):.1f} s of CPU work)",
        "host_cpus": os.cpu_count(),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the reshard; runs with --gpus > 1 are not part of this build",
              file=sys.stderr)
        sys.exit(2)
    import torch

    from etha_amd import _native, workloads
    from etha_amd.build import ensure_built
    from etha_amd.world import ReshardJob

    ensure_built()  # loads what is built; compiles only if nothing is
    _native.lib()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the hot path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    specs, targets, bucket = workloads.WORKLOADS[args.workload]()
    t0 = time.time()
    job = ReshardJob(specs, device=dev, bucket_size=bucket, target_ranks=targets, zero_copy=args.zero_copy,
                     direct=args.direct)
    merge = not args.per_bucket
    # plan (compiles the tile programs) + warm-up
    for _ in range(max(args.warmup, 1)):
        job.run(merge_launches=merge, fanout=args.fanout)
    setup_s = time.time() - t0

    S = job.payload_bytes()
    send_plans = [job.wire.plan(b) for b in job.send_buckets.values()]
    recv_plans = [job.wire.plan(b) for b in job.recv_buckets.values()]
    steps_of = (lambda p: p.merged_steps) if merge else (lambda p: p.steps)
    n_pack = sum(1 for p in send_plans for s in steps_of(p) if s[0] in ("pack", "reduce_pack"))
    n_self = sum(1 for p in send_plans + recv_plans for s in steps_of(p) if s[0] == "selfcopy")
    n_unpack = sum(1 for p in send_plans + recv_plans for s in steps_of(p) if s[0] in ("unpack", "direct", "direct_reduce"))

    # algorithmic bytes: pack reads the source dtype and writes the wire dtype; unpack reads the wire
    # dtype and writes the target dtype; a reduce-pack reads every member's partial
    def table_bytes(plan, which):
        t = getattr(plan, which)
        return t.info().payload_bytes if t is not None else 0

    wire_bytes = sum(table_bytes(p, "send_table") for p in send_plans)
    pack_read = 0
    for p in send_plans:
        for b in p.buckets:
            if b.transport.value in ("p2p", "broadcast") and b.is_source and id(b) not in p.lent:
                for c in b.chunks:
                    peers = c.partial_peers()
                    n = 1
                    for d in c.chunk_shape:
                        n *= d
                    pack_read += n * c.tensor.element_size() * (len(peers[0]) if peers else 1)
    unpack_write = 0
    for p in recv_plans:
        for b in p.buckets:
            for c in b.chunks:
                n = 1
                for d in c.chunk_shape:
                    n *= d
                unpack_write += n * c.tensor.element_size()
    unpack_read = sum(table_bytes(p, "recv_table") for p in recv_plans)
    unpack_read += sum(p.direct_read_bytes for p in recv_plans)  # direct wire: reads the source regions themselves
    # LOCAL chunks run inside the send phase as direct copies: read the source region, write the target
    self_bytes = 0
    for p in send_plans:
        for b in p.buckets:
            if b.transport.value == "local":
                for c in b.chunks:
                    n = 1
                    for d in c.chunk_shape:
                        n *= d
                    src_t = c.src_tensor if c.src_tensor is not None else c.tensor
                    self_bytes += n * (src_t.element_size() + c.tensor.element_size())
    pack_bytes = pack_read + wire_bytes + self_bytes
    unpack_bytes = unpack_read + unpack_write

    stream = torch.cuda.current_stream(dev)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    graph = None
    if args.graph:
        graph = job.capture(merge_launches=merge)
        graph.replay()
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    for k in range(args.steps):
        ev[k][0].record(stream)
        if graph is not None:
            graph.replay()
            ev[k][1].record(stream)
        else:
            job.run_send(merge, args.fanout)
            ev[k][1].record(stream)
            job.run_recv(merge, args.fanout)
        ev[k][2].record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    pack_ms = [ev[k][0].elapsed_time(ev[k][1]) for k in range(args.steps)]
    unpack_ms = [ev[k][1].elapsed_time(ev[k][2]) for k in range(args.steps)]
    if graph is not None:  # a replayed graph is one unit: split the step time by algorithmic bytes
        whole = [p + u for p, u in zip(pack_ms, unpack_ms)]
        share = pack_bytes / max(pack_bytes + unpack_bytes, 1)
        pack_ms = [w * share for w in whole]
        unpack_ms = [w * (1 - share) for w in whole]
    step_ms = wall * 1e3 / args.steps
    pack_avg, unpack_avg = sum(pack_ms) / len(pack_ms), sum(unpack_ms) / len(unpack_ms)
    dev_ms = pack_avg + unpack_avg

    value = S / (step_ms * 1e-3) / 1e9
    pack_gbs = pack_bytes / (pack_avg * 1e-3) / 1e9 if pack_avg > 0 else 0.0
    unpack_gbs = unpack_bytes / (unpack_avg * 1e-3) / 1e9 if unpack_avg > 0 else 0.0
    dominant = "pack" if pack_avg >= unpack_avg else "unpack"
    dom_bytes, dom_ms, dom_launches = (
        (pack_bytes, pack_avg, max(n_pack, 1)) if dominant == "pack" else (unpack_bytes, unpack_avg, max(n_unpack, 1))
    )
    kernel_name = {"pack": "etha_tile_kernel<false>", "unpack": "etha_tile_kernel<true>"}[dominant]
    if dominant == "pack" and any(s[0] == "reduce_pack" for p in send_plans for s in steps_of(p)):
        kernel_name = "etha_reduce_kernel"
    if dominant == "unpack" and args.direct:
        kernel_name = "etha_tile_kernel<false>"  # the direct copy runs source region -> target region
        if any(s[0] == "direct_reduce" for p in recv_plans for s in steps_of(p)):
            kernel_name = "etha_reduce_kernel"
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    out = {
        "metric": "effective reshard GB/s (pack+unpack, 1 GPU) and % of HBM peak",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8" if pack_read == wire_bytes else "f32",
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "payload_bytes": S,
            "bucket_bytes": bucket,
            "launch_granularity": "run of buckets" if merge else "bucket",
            "fanout_streams": args.fanout,
            "hip_graph": bool(args.graph),
            "zero_copy_single_chunk": bool(args.zero_copy),
            "direct_same_device": bool(args.direct),
            **job.counts(),
        },
        "device_ms_per_step": round(dev_ms, 4),
        "pct_of_hbm_peak": round(100.0 * (pack_bytes + unpack_bytes) / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "pack": {"GB/s": round(pack_gbs, 1), "ms": round(pack_avg, 4), "bytes": pack_bytes, "launches": n_pack},
        "unpack": {"GB/s": round(unpack_gbs, 1), "ms": round(unpack_avg, 4), "bytes": unpack_bytes, "launches": n_unpack},
        "selfcopy": {"launches": n_self, "bytes": self_bytes, "note": "timed inside the pack phase"},
        "roofline": {
            "bound": "hbm",
            "kernel": kernel_name,
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            # measured for the default configuration only
            "traffic": None if (args.zero_copy or args.direct or args.graph or args.fanout > 1) else
            MEASURED_TRAFFIC_BYTES.get((args.workload, kernel_name, "run of buckets" if merge else "bucket")),
            "bytes_per_launch": dom_bytes // dom_launches,
            "avg_launch_ms": round(dom_ms / dom_launches, 5),
            "launches_per_step": dom_launches,
        },
        "setup_s": round(setup_s, 1),
    }
    if merge and graph is None and args.fanout == 1 and not args.no_per_bucket_leg:
        # the strict form of the same step, one launch per bucket, for comparison (not the headline)
        n_strict = sum(1 for p in send_plans + recv_plans for s in p.steps if s[0] != "lend")
        for _ in range(2):
            job.run(merge_launches=False)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = max(3, min(args.steps, 10))
        e0.record(stream)
        for _ in range(reps):
            job.run(merge_launches=False, synchronize=False)
        e1.record(stream)
        torch.cuda.synchronize()
        strict_ms = e0.elapsed_time(e1) / reps
        out["one_launch_per_bucket"] = {
            "device_ms_per_step": round(strict_ms, 4),
            "pct_of_hbm_peak": round(100.0 * (pack_bytes + unpack_bytes) / (strict_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
            "launches_per_step": n_strict,
            "effective_GB/s": round(S / (strict_ms * 1e-3) / 1e9, 1),
        }
    if args.calibration_copy:
        a = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        b = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        out["calibration_copy"] = {"bytes_read": 1 << 30, "bytes_written": 1 << 30, "launches": 3}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.workload, args.cpu_layers, args.cpu_seconds)
        if args.workload == "single_fp32_shard0_to_shard1":
            out["cpu_baseline"]["gloo"] = gloo_baseline(args.workload)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
