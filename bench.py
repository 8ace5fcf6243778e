"""Headline benchmark: effective reshard GB/s (pack + unpack) on one MI355X.

One step = one pass of the hot path over the workload: every source rank packs its buckets for the
measured target rank's share and that target rank unpacks them, through a bounded bucket pool (a ring
of ``--max-in-flight`` slots per channel).  Inputs are resident in HBM before the timed region.
Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--per-bucket] [--pool resident]
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
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.txt")


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama3_8b_fsdp8_to_tp2")
    ap.add_argument("--pool", choices=["ring", "resident"], default="ring",
                    help="ring: max-in-flight slots per channel (the reference's memory bound); resident: a slot per bucket")
    ap.add_argument("--max-in-flight", type=int, default=2, help="buckets of one channel prepared or in flight (= ring slots)")
    ap.add_argument("--per-bucket", action="store_true",
                    help="strictly one launch per bucket (default: buckets that become ready together and are neighbours "
                         "in their table share a launch)")
    ap.add_argument("--bucket-segments", action="store_true",
                    help="every bucket stays a launch segment of its own (no merging of neighbouring buckets), "
                         "independent segments still share launches")
    ap.add_argument("--in-order", action="store_true", help="issue every launch ordered after the previous one")
    ap.add_argument("--no-sets", action="store_true",
                    help="one kernel launch per bucket step instead of shared launches for independent steps "
                         "(implied by --per-bucket)")
    ap.add_argument("--fanout", type=int, default=1, help="side streams for per-bucket launches (resident pool only)")
    ap.add_argument("--zero-copy", action="store_true",
                    help="lend contiguous single-chunk buckets to the consumer instead of packing them")
    ap.add_argument("--direct", action="store_true",
                    help="no bucket buffers: the target side copies straight from the source shards (one pass; "
                         "not the pack+unpack path the headline is quoted on)")
    ap.add_argument("--graph", action="store_true", help="replay the step from a captured HIP graph (whole step timed)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-legs", action="store_true",
                    help="only the timed configuration (use under a profiler, so that per-kernel statistics cover one "
                         "configuration)")
    ap.add_argument("--cpu-layers", type=int, default=8,
                    help="decoder layers of the sample the CPU baseline falls back to when host memory is short")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU work the baseline leg is bounded to")
    ap.add_argument("--no-process-legs", action="store_true",
                    help="skip the legs that start worker processes (the two-process wire and the tensor bus end to end)")
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


def _host_memory_available() -> int:
    try:
        import psutil

        return int(psutil.virtual_memory().available)
    except Exception:
        return 0


def cpu_baseline(workload: str, layers: int, seconds: float):
    """The oracle's op-for-op restatement of the reference path, timed on this host's cores: the whole workload
    where host memory allows (shards + target share + one pass of bucket buffers), else a sample of it."""
    import torch

    from etha_amd import workloads
    from etha_amd.world import ReshardJob
    from oracle import reference_path

    specs, targets, bucket = workloads.WORKLOADS[workload]()
    sample = "whole workload"
    if workload.startswith("llama3_8b_fsdp8_to_tp2"):
        # the whole share: 16 GB of source shards + 8 GB of targets + 8 GB of bucket buffers alive during a pass
        need = 48 << 30
        have = _host_memory_available()
        if have < need:
            specs, targets, bucket = workloads.llama3_8b_fsdp8_to_tp2(n_layers=layers, with_embeddings=False)
            sample = (f"{layers} decoder layers of the workload (no embeddings), same layouts and 64 MiB buckets - "
                      f"host memory available {have >> 30} GiB < {need >> 30} GiB needed for the whole share")
        else:
            sample = "whole workload (embeddings included)"

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
        "sample": f"{sample}; {payload} payload bytes per pass, median of {len(times)} passes after one warm-up "
                  f"({sum(times):.1f} s of CPU work)",
        "host_cpus": os.cpu_count(),
    }


def read_traffic(workload: str, mode: str):
    """HBM bytes per step of a workload from the committed counter summary (``profiles/hbm_traffic.txt``), with the
    commit, command and library build it was measured at.
    Lines: ``workload | mode | fetch_bytes | write_bytes | launches | commit | library digest``."""
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                parts = [p.strip() for p in line.split("|")]
                if len(parts) >= 6 and parts[0] == workload and parts[1] == mode:
                    return {"fetch_bytes_per_step": int(parts[2]), "write_bytes_per_step": int(parts[3]),
                            "launches_per_step": int(parts[4]), "measured_at_commit": parts[5],
                            "library_digest": parts[6] if len(parts) > 6 else None,
                            "source": "profiles/hbm_traffic.txt"}
    except OSError:
        pass
    return None


def with_library_check(traffic):
    """The counters were read under rocprofv3 in a run of their own: say which build of the library that was, and
    whether it is the one running now."""
    if traffic is None:
        return None
    from etha_amd import _native

    running = _native.lib().etha_source_hash().decode()
    return {**traffic, "running_library_digest": running, "stale": traffic.get("library_digest") != running}


def _numel(shape):
    n = 1
    for d in shape:
        n *= d
    return n


def algorithmic_bytes(job):
    """(pack side bytes, unpack side bytes) per step: pack reads the source dtype (every member's partial for a
    reduce-pack) and writes the wire dtype; unpack reads the wire dtype and writes the target dtype; a same-rank
    chunk is one direct copy (read source region, write target region), counted with the pack side."""
    send_plans = [job.wire.plan(b) for b in job.send_buckets.values()]
    recv_plans = [job.wire.plan(b) for b in job.recv_buckets.values()]

    def table_bytes(plan, which):
        t = getattr(plan, which)
        return t.info().payload_bytes if t is not None else 0

    wire_bytes = sum(table_bytes(p, "send_table") for p in send_plans)
    pack_read = self_bytes = 0
    for p in send_plans:
        for b in p.buckets:
            if b.transport.value in ("p2p", "broadcast") and b.is_source and id(b) not in p.lent:
                for c in b.chunks:
                    peers = c.partial_peers()
                    pack_read += _numel(c.chunk_shape) * c.tensor.element_size() * (len(peers[0]) if peers else 1)
            elif b.transport.value == "local":
                for c in b.chunks:
                    src_t = c.src_tensor if c.src_tensor is not None else c.tensor
                    self_bytes += _numel(c.chunk_shape) * (src_t.element_size() + c.tensor.element_size())
    unpack_write = sum(_numel(c.chunk_shape) * c.tensor.element_size() for p in recv_plans for b in p.buckets for c in b.chunks)
    unpack_read = sum(table_bytes(p, "recv_table") for p in recv_plans)
    unpack_read += sum(p.direct_read_bytes for p in recv_plans)  # direct wire: reads the source regions themselves
    kinds = {s[0] for p in send_plans + recv_plans for s in p.steps}
    return pack_read + wire_bytes + self_bytes, unpack_read + unpack_write, self_bytes, kinds, pack_read == wire_bytes


def time_steps(job, steps, run):
    """Per-step device time (HIP events on the stream the launches go to) and wall time per step."""
    import torch

    stream = torch.cuda.current_stream(job.device)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    import gc

    # a full collection stalls the host for tens of milliseconds: none inside the timed region, and the one here
    # comes before the untimed burst, not between it and the first timed step (the GPU would sit idle meanwhile
    # and the steps after such a pause measured 5-6 % slower on a 1.2 ms step)
    gc.collect()
    gc.disable()
    try:
        # an untimed burst first: the first time steps queue up behind each other without a host synchronisation
        # the HIP runtime grows its internal pools once (a host stall of tens of milliseconds)
        for _ in range(min(steps, 5)):
            run()
        torch.cuda.synchronize()
        wall0 = time.perf_counter()
        ev[0].record(stream)
        for k in range(steps):
            run()
            ev[k + 1].record(stream)
        HOST_MS["issue"] = (time.perf_counter() - wall0) * 1e3 / steps  # the host's share: planning sweeps + launch calls
        torch.cuda.synchronize()
        wall = time.perf_counter() - wall0
    finally:
        gc.enable()
    dev = [ev[k].elapsed_time(ev[k + 1]) for k in range(steps)]
    return sum(dev) / steps, wall * 1e3 / steps


HOST_MS: dict = {}


def launches_per_step(job, run):
    """(kernel launches, bucket steps, bucket steps issued unordered) of one step."""
    import torch

    from etha_amd import _native

    log = job.wire.launch_log = []
    before = _native.kernel_launches()
    run()
    torch.cuda.synchronize()
    job.wire.launch_log = None
    return _native.kernel_launches() - before, len(log), sum(1 for entry in log if entry[3] & 1)


OTHER_WORKLOADS = ("single_fp32_shard0_to_shard1", "many_small_2d_to_replicate", "partial4_to_shard2",
                   "moe_experts_and_uneven_vocab", "llama3_8b_fsdp8_to_tp2_fp32_to_bf16", "transposed_parents",
                   "partial4_transposed_to_shard2")


def measure_workload(name: str, dev, steps: int, warmup: int):
    """One workload in the default form (ring of 2 slots per channel, independent steps share launches): device
    time per step by HIP events, algorithmic bytes, launches."""
    import torch

    from etha_amd import workloads
    from etha_amd.world import ReshardJob

    specs, targets, bucket = workloads.WORKLOADS[name]()
    job = ReshardJob(specs, device=dev, bucket_size=bucket, target_ranks=targets)
    for _ in range(max(warmup, 3)):
        job.run(merge_launches=True)
    dev_ms, wall_ms = time_steps(job, max(steps, 20), lambda: job.run(merge_launches=True, synchronize=False))
    host_ms = HOST_MS.get("issue")
    n_launch, n_steps, _ = launches_per_step(job, lambda: job.run(merge_launches=True, synchronize=False))
    pack_bytes, unpack_bytes, self_bytes, _, _ = algorithmic_bytes(job)
    total = pack_bytes + unpack_bytes
    S = job.payload_bytes()
    traffic = read_traffic(name, "ring/sets")
    out = {
        "payload_bytes": S,
        "device_ms_per_step": round(dev_ms, 4),
        "ms_per_step": round(wall_ms, 4),
        "host_issue_ms_per_step": round(host_ms, 4),
        "algorithmic_bytes_per_step": total,
        "pct_of_hbm_peak": round(100.0 * total / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "effective_GB/s": round(S / (dev_ms * 1e-3) / 1e9, 1),
        "launches_per_step": n_launch,
        "bucket_steps_per_step": n_steps,
        "steps": max(steps, 20),
        "warmup": max(warmup, 3),
        "pool_reserved_bytes": job.wire.pool.reserved_bytes if job.wire.pool is not None else 0,
        "hbm_GB/s": None if traffic is None else
        round((traffic["fetch_bytes_per_step"] + traffic["write_bytes_per_step"]) / (dev_ms * 1e-3) / 1e9, 1),
    }
    del job
    torch.cuda.empty_cache()
    return out


def copy_ceiling(dev, reps: int = 10):
    """What a plain copy reaches on this device through the library's own pack kernel: one contiguous 4 GiB tensor
    packed into one bucket (read 4 GiB, write 4 GiB), and the same tensor as fp32 packed into a bf16 bucket (read
    4 GiB, write 2 GiB).  The workloads above are bounded by this, not by the published 8 TB/s."""
    import torch
    from torch.distributed.tensor.placement_types import Replicate

    from etha_amd.world import ReshardJob, TensorSpec, transfer_dtype_rule

    out = {}
    stream = torch.cuda.current_stream(dev)
    for label, n, sdt, tdt in (("bf16_to_bf16", 1 << 31, torch.bfloat16, None), ("fp32_to_bf16", 1 << 30, torch.float32, torch.bfloat16)):
        spec = TensorSpec("c", (n,), [0], (Replicate(),), [1], (Replicate(),), sdt, tdt, seed=1)
        job = ReshardJob([spec], device=dev, bucket_size=64 << 20, pool="resident")
        for _ in range(3):
            job.run()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        ev[0].record(stream)
        for k in range(reps):
            job.run_send()
            ev[k + 1].record(stream)
        torch.cuda.synchronize()
        ms = sorted(ev[k].elapsed_time(ev[k + 1]) for k in range(reps))
        wire = transfer_dtype_rule(sdt, tdt or sdt).itemsize
        nbytes = n * sdt.itemsize + n * wire
        out[label] = {"bytes_read": n * sdt.itemsize, "bytes_written": n * wire, "median_ms": round(ms[len(ms) // 2], 4),
                      "GB/s": round(nbytes / (ms[len(ms) // 2] * 1e-3) / 1e9, 1),
                      "pct_of_hbm_peak": round(100.0 * nbytes / (ms[len(ms) // 2] * 1e-3) / 1e9 / HBM_PEAK_GBS, 2)}
        del job
        torch.cuda.empty_cache()
    return out


def process_leg(module: str, *flags, timeout: float = 180.0):
    """A leg that needs worker processes of its own: run the module as a child and take the JSON line it prints."""
    import subprocess

    proc = subprocess.run([sys.executable, "-m", module, *flags], cwd=ROOT, capture_output=True, text=True, timeout=timeout)
    lines = [l for l in proc.stdout.splitlines() if l.startswith("{")]
    if proc.returncode != 0 or not lines:
        raise RuntimeError(f"{module} exited with {proc.returncode}: {proc.stderr[-500:]}")
    return json.loads(lines[-1])


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
    merge = not (args.per_bucket or args.bucket_segments)
    if args.fanout > 1 and args.pool != "resident":
        print("--fanout needs --pool resident (side streams run a bucket list in list order)", file=sys.stderr)
        sys.exit(2)

    def make_job(pool, depth):
        return ReshardJob(specs, device=dev, bucket_size=bucket, target_ranks=targets, zero_copy=args.zero_copy,
                          direct=args.direct, pool=pool, max_in_flight=depth)

    t0 = time.time()
    job = make_job(args.pool, args.max_in_flight)
    job.wire.unordered_launches = not args.in_order
    sets = not (args.no_sets or args.per_bucket)
    job.wire.group_launches = sets
    for _ in range(max(args.warmup, 1)):  # plans (compiles the tile programs) + warm-up
        job.run(merge_launches=merge, fanout=args.fanout)
    setup_s = time.time() - t0

    S = job.payload_bytes()
    pack_bytes, unpack_bytes, self_bytes, kinds, byte_move = algorithmic_bytes(job)
    total_bytes = pack_bytes + unpack_bytes
    graph = None
    if args.graph:
        graph = job.capture(merge_launches=merge)
        graph.replay()
    step = graph.replay if graph is not None else (lambda: job.run(merge_launches=merge, fanout=args.fanout, synchronize=False))
    dev_ms, step_ms = time_steps(job, args.steps, step)
    host_ms = HOST_MS.get("issue")
    n_launch, n_steps, n_unordered = launches_per_step(
        job, lambda: job.run(merge_launches=merge, fanout=args.fanout, synchronize=False))
    if args.pool != "ring":
        plans = [job.wire.plan(b) for bs in (job.send_buckets, job.recv_buckets) for b in bs.values()]
        n_steps = sum(1 for p in plans for s in (p.merged_steps if merge else p.steps) if s[0] != "lend")

    kernels = []
    tables = [t for p in (job.wire.plan(b) for bs in (job.send_buckets, job.recv_buckets) for b in bs.values())
              for t in (p.send_table, p.recv_table, p.local_table) if t is not None]
    infos = [t.info() for t in tables]
    if any(i.n_trans_tiles for i in infos):
        kernels.append("etha_transpose_kernel")
    if any(i.n_run_tiles + i.n_row_tiles for i in infos) and kinds & {"pack", "unpack", "selfcopy", "direct"}:
        kernels.append("etha_tile_kernel")
    if kinds & {"reduce_pack", "direct_reduce"}:
        kernels.insert(0, "etha_reduce_kernel")
    granularity = ("bucket" if not merge and not sets else
                   "one segment per bucket, independent segments share launches" if not merge else
                   "run of buckets" if args.pool != "ring" else
                   "independent steps share launches" if sets else "buckets ready together")
    mode = f"{args.pool}/{'bucket' if not merge and not sets else 'bucket-sets' if not merge else 'sets' if sets and args.pool == 'ring' else 'runs'}"
    element = str(specs[0].source_dtype).replace("torch.", "")
    achieved = total_bytes / (dev_ms * 1e-3) / 1e9
    traffic = None if (args.zero_copy or args.direct or args.graph or args.fanout > 1 or args.in_order
                       or args.max_in_flight != 2) else read_traffic(args.workload, mode)
    out = {
        "metric": "effective reshard GB/s (pack+unpack, 1 GPU) and % of HBM peak",
        "value": round(S / (step_ms * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": f"{element} (byte move)" if byte_move else f"{element} -> wire dtype (f32 arithmetic)",
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "payload_bytes": S,
            "bucket_bytes": bucket,
            "pool": args.pool,
            "max_in_flight": args.max_in_flight,
            "pool_reserved_bytes": job.wire.pool.reserved_bytes if job.wire.pool is not None else 0,
            "launch_granularity": granularity,
            "unordered_launches": bool(job.wire.unordered_launches and args.pool == "ring"),
            "fanout_streams": args.fanout,
            "hip_graph": bool(args.graph),
            "zero_copy_single_chunk": bool(args.zero_copy),
            "direct_same_device": bool(args.direct),
            **job.counts(),
        },
        "device_ms_per_step": round(dev_ms, 4),
        "host_issue_ms_per_step": round(host_ms, 4),
        "pct_of_hbm_peak": round(100.0 * achieved / HBM_PEAK_GBS, 2),
        "algorithmic_bytes_per_step": {"pack": pack_bytes, "unpack": unpack_bytes, "of_which_self_copy": self_bytes},
        "launches_per_step": n_launch,
        "bucket_steps_per_step": n_steps,
        "unordered_bucket_steps_per_step": n_unordered,
        "roofline": {
            "bound": "hbm",
            "kernel": " + ".join(kernels),
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            # HBM bytes per launch from the committed rocprofv3 counter summary (null when this configuration has none)
            "traffic": None if traffic is None else
            (traffic["fetch_bytes_per_step"] + traffic["write_bytes_per_step"]) // max(traffic["launches_per_step"], 1),
            "traffic_detail": with_library_check(traffic),
            # achieved HBM rate by the counters: (FETCH_SIZE + WRITE_SIZE bytes per step) / device time per step
            "hbm_GB/s": None if traffic is None else
            round((traffic["fetch_bytes_per_step"] + traffic["write_bytes_per_step"]) / (dev_ms * 1e-3) / 1e9, 1),
            "bytes_per_launch": total_bytes // max(n_launch, 1),
            # launches overlap their neighbours: the average is the timed region over the launches in it
            "avg_launch_ms": round(dev_ms / max(n_launch, 1), 5),
            "launches_per_step": n_launch,
        },
        "setup_s": round(setup_s, 1),
        "library_digest": _native.lib().etha_source_hash().decode(),
    }

    def leg(j, reps=None, **kw):
        reps = reps or max(3, min(args.steps, 10))
        for _ in range(2):
            j.run(**kw)
        ms, _ = time_steps(j, reps, lambda: j.run(synchronize=False, **kw))
        return ms

    def describe(ms, launches=None, pool_bytes=None):
        d = {"device_ms_per_step": round(ms, 4),
             "pct_of_hbm_peak": round(100.0 * total_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
             "effective_GB/s": round(S / (ms * 1e-3) / 1e9, 1)}
        if launches is not None:
            d["launches_per_step"] = launches
        if pool_bytes is not None:
            d["pool_reserved_bytes"] = pool_bytes
        return d

    plain = not (args.no_extra_legs or args.graph or args.fanout > 1 or args.zero_copy or args.direct or args.in_order)
    if plain and args.pool == "ring":
        try:
            # the same step in its other forms, for comparison (none of them is `value`)
            pool_bytes = job.wire.pool.reserved_bytes if job.wire.pool is not None else 0
            def other_leg(merge_, sets_, unordered=True):
                job.wire.group_launches, job.wire.unordered_launches = sets_, unordered
                ms = leg(job, merge_launches=merge_)
                n = launches_per_step(job, lambda: job.run(merge_launches=merge_, synchronize=False))[0]
                job.wire.group_launches, job.wire.unordered_launches = sets, True
                return describe(ms, n, pool_bytes)

            if merge or sets:
                out["one_launch_per_bucket"] = other_leg(False, False)
            if merge or not sets:
                out["one_segment_per_bucket"] = other_leg(False, True)
            if not (merge and not sets):
                out["one_launch_per_run_of_buckets"] = other_leg(True, False)
            if not (merge and sets):
                out["independent_steps_share_launches"] = other_leg(True, True)
            out["every_launch_in_order"] = other_leg(merge, False, unordered=False)
            # the same launches recorded once into a HIP graph and replayed (a chain of kernel nodes)
            captured = job.capture(merge_launches=merge)
            captured.replay()
            torch.cuda.synchronize()
            ms, _ = time_steps(job, max(3, min(args.steps, 10)), captured.replay)
            out["hip_graph_replay"] = describe(ms, n_launch, pool_bytes)
            del captured
            del job
            torch.cuda.empty_cache()
            deeper = make_job("ring", 2 * args.max_in_flight)
            deeper.wire.group_launches = sets
            ms = leg(deeper, merge_launches=merge)
            n = launches_per_step(deeper, lambda: deeper.run(merge_launches=merge, synchronize=False))[0]
            out[f"ring_of_{2 * args.max_in_flight}_slots"] = describe(ms, n, deeper.wire.pool.reserved_bytes if deeper.wire.pool else 0)
            del deeper
            torch.cuda.empty_cache()
            # a slot per bucket: all packs, then all unpacks, each side in as few launches as the lists allow
            res = make_job("resident", args.max_in_flight)
            for _ in range(2):
                res.run(merge_launches=True)
            stream = torch.cuda.current_stream(dev)
            reps = max(3, min(args.steps, 10))
            ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(reps)]
            for k in range(reps):
                ev[k][0].record(stream)
                res.run_send(True)
                ev[k][1].record(stream)
                res.run_recv(True)
                ev[k][2].record(stream)
            torch.cuda.synchronize()
            p_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / reps
            u_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / reps
            plans = [res.wire.plan(b) for bs in (res.send_buckets, res.recv_buckets) for b in bs.values()]
            d = describe(p_ms + u_ms, sum(1 for p in plans for s in p.merged_steps if s[0] != "lend"), res.wire.pool.reserved_bytes)
            d["pack"] = {"GB/s": round(pack_bytes / (p_ms * 1e-3) / 1e9, 1), "ms": round(p_ms, 4)}
            d["unpack"] = {"GB/s": round(unpack_bytes / (u_ms * 1e-3) / 1e9, 1), "ms": round(u_ms, 4)}
            out["resident_pool_run_of_buckets"] = d
            del res
            torch.cuda.empty_cache()
            if args.workload == "llama3_8b_fsdp8_to_tp2":
                # the Partial collapse has no part in this workload: its rates on config 4, beside pack and unpack above
                p_specs, p_targets, p_bucket = workloads.WORKLOADS["partial4_to_shard2"]()
                red = ReshardJob(p_specs, device=dev, bucket_size=p_bucket, target_ranks=p_targets, pool="resident")
                for _ in range(2):
                    red.run(merge_launches=True)
                r_pack, r_unpack = algorithmic_bytes(red)[:2]
                ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(reps)]
                for k in range(reps):
                    ev[k][0].record(stream)
                    red.run_send(True)
                    ev[k][1].record(stream)
                    red.run_recv(True)
                    ev[k][2].record(stream)
                torch.cuda.synchronize()
                p_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / reps
                u_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / reps
                out["partial_reduce"] = {
                    "workload": "partial4_to_shard2",
                    "reduce_pack": {"GB/s": round(r_pack / (p_ms * 1e-3) / 1e9, 1), "ms": round(p_ms, 4),
                                    "bytes": r_pack, "pool": "resident"},
                    "unpack": {"GB/s": round(r_unpack / (u_ms * 1e-3) / 1e9, 1), "ms": round(u_ms, 4), "bytes": r_unpack,
                               "pool": "resident"},
                }
                del red
                torch.cuda.empty_cache()
        except Exception as e:  # an optional leg must not take the measured line with it
            out["extra_legs_error"] = f"{type(e).__name__}: {e}"

    if plain and args.pool == "ring" and args.workload == "llama3_8b_fsdp8_to_tp2":
        # every other configuration in its default form, and what a plain copy reaches through the same kernels
        job = None
        torch.cuda.empty_cache()
        out["workloads"] = {}
        for name in OTHER_WORKLOADS:
            try:
                out["workloads"][name] = measure_workload(name, dev, args.steps, args.warmup)
            except Exception as e:
                out["workloads"][name] = {"error": f"{type(e).__name__}: {e}"}
        try:
            out["copy_ceiling"] = copy_ceiling(dev)
        except Exception as e:
            out["copy_ceiling"] = {"error": f"{type(e).__name__}: {e}"}
        if not args.no_process_legs:
            torch.cuda.empty_cache()
            try:
                d = process_leg("etha_amd.comm.bench_wire", "--workload", args.workload, "--steps", "10", "--warmup", "3")
                out["two_process_wire"] = {"ms_per_transfer": round(d["ms_per_transfer"], 3), "min_ms": round(d["min_ms"], 3),
                                           "effective_GB/s": round(d["value"], 1), "payload_bytes": d["payload_bytes"],
                                           "steps": d["steps"], **d["config"],
                                           "clock": "host wall clock: producer starts packing -> consumer's last unpack done",
                                           "bit_equal_target_tensors": d["target_tensors_bit_equal_to_the_in_process_transfer"]}
            except Exception as e:
                out["two_process_wire"] = {"error": f"{type(e).__name__}: {e}"}
            try:
                d = process_leg("etha_amd.tensor_bus.bench_transfer", "--workload", args.workload, "--steps", "10", "--warmup", "3")
                out["bus_end_to_end"] = {"ms_per_transfer": round(d["ms_per_transfer"], 3), "min_ms": round(d["min_ms"], 3),
                                         "effective_GB/s": round(d["value"], 1), "payload_bytes": d["payload_bytes"],
                                         "steps": d["steps"], **d["config"], "agent": d["agent"],
                                         "clock": "host wall clock: first rank's transfer('send') -> last rank's blocking transfer('recv') returns",
                                         "tensors_verified_by_checksum": d["tensors_verified_by_checksum"]}
            except Exception as e:
                out["bus_end_to_end"] = {"error": f"{type(e).__name__}: {e}"}

    if args.calibration_copy:
        a = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        b = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        out["calibration_copy"] = {"bytes_read": 1 << 30, "bytes_written": 1 << 30, "launches": 3}
    if not args.no_cpu_baseline:
        try:
            out["cpu_baseline"] = cpu_baseline(args.workload, args.cpu_layers, args.cpu_seconds)
            if args.workload == "single_fp32_shard0_to_shard1":
                out["cpu_baseline"]["gloo"] = gloo_baseline(args.workload)
        except Exception as e:  # the GPU figures above are measured: report them even if the host leg could not run
            out["cpu_baseline"] = {"value": None, "unit": "GB/s", "cores": 0, "kind": "port",
                                   "sample": f"not measured: {type(e).__name__}: {e}"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
