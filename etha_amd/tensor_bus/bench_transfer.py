"""End-to-end timing of ``handler.transfer`` through the tensor bus on one GPU.

    python -m etha_amd.tensor_bus.bench_transfer [--workload NAME] [--steps K] [--warmup W] [--zero-copy | --direct] [--thread-per-rank]

This process runs the hub agent; every source rank ("trainer") and every target rank ("inference") is a worker
process of its own on the same GPU, as the reference's workers are (``--thread-per-rank``: one worker process per
side with a thread per rank instead - the rank threads then issue their commands one after the other).  Workers
register their tensors over hipIPC once (``register_tensors``) and then repeat ``transfer("send")`` /
``transfer("recv")``.
One step is timed on the host wall clock from the moment the first source rank issues its send to
the moment the last target rank's blocking recv returns, so it includes the command round trips,
the agent's launches and the device work.  After the last step every same-dtype tensor is verified by a
checksum of checksums (raw bits summed over all target ranks against all source ranks).  Prints ONE JSON line.

All target ranks of the workload take part (a pair needs its whole mesh), so the payload is every
target rank's share, not the single share ``bench.py`` measures.
"""

from __future__ import annotations

import argparse
import json
import multiprocessing as mp
import os
import sys
import tempfile
import threading
import time
import traceback

import numpy as np


def _naming(tmpdir: str):
    def fn(rank: int):
        return os.path.join(tmpdir, f"agent_rank{rank}_command"), os.path.join(tmpdir, f"agent_rank{rank}_state")

    return fn


def _pairs(specs):
    """One pair per distinct layout pair; returns (pair name per spec, {pair name: spec})."""
    names, first = [], {}
    for s in specs:
        key = (str(s.source_mesh), str(s.source_placements), str(s.target_mesh), str(s.target_placements))
        if key not in first:
            first[key] = (f"pair{len(first)}", s)
        names.append(first[key][0])
    return names, {n: s for n, s in first.values()}


def _worker(role: str, workload: str, tmpdir: str, device: str, steps: int, warmup: int, out_q, only_rank=None,
            shared_barrier=None) -> None:
    """Body of a worker process: every rank of one side, one thread per rank - or, with ``only_rank``, that rank
    alone (one process per rank, as in a deployment; ``shared_barrier`` then lines the processes of a side up)."""
    try:
        import torch

        from etha_amd import workloads
        from etha_amd.layout import local_shape, mesh_coord
        from etha_amd.tensor_bus import TensorBusClient
        from etha_amd.tensor_bus.bootstrap import setup_ptrace

        setup_ptrace()
        specs, _, bucket = workloads.WORKLOADS[workload]()
        pair_names, pair_specs = _pairs(specs)
        naming = _naming(tmpdir)
        source = role == "trainer"
        my_ranks = sorted({int(r) for s in specs for r in np.asarray(s.source_mesh if source else s.target_mesh).reshape(-1)})
        if only_rank is not None:
            my_ranks = [r for r in my_ranks if r == only_rank]
        shards: dict[int, list] = {r: [] for r in my_ranks}
        gen = torch.Generator(device=device)
        for i, s in enumerate(specs):
            mesh = np.asarray(s.source_mesh if source else s.target_mesh)
            placements = s.source_placements if source else s.target_placements
            dtype = s.source_dtype if source else (s.target_dtype or s.source_dtype)
            for pos, r in enumerate(int(x) for x in mesh.reshape(-1)):
                if r not in shards:
                    continue
                shape = local_shape(s.shape, mesh.shape, placements, mesh_coord(mesh.shape, pos))
                if source:  # values are irrelevant to timing; seeded so that runs repeat
                    gen.manual_seed(1000 * i + r)
                    t = (torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * s.std).to(dtype)
                else:
                    t = torch.zeros(shape, dtype=dtype, device=device)
                shards[r].append((t, pair_names[i]))
        torch.cuda.synchronize()
        barrier = shared_barrier if shared_barrier is not None else threading.Barrier(len(my_ranks))
        stamps = {r: [] for r in my_ranks}
        errors = []

        def rank_body(r: int) -> None:
            try:
                cmd, state = naming(r)
                client = TensorBusClient(r, cmd, state, connection_timeout=60)
                for name, s in pair_specs.items():
                    mesh = np.asarray(s.source_mesh if source else s.target_mesh)
                    if r not in mesh.reshape(-1):
                        continue
                    client.init_pair(name, role, "inference" if source else "trainer", int(mesh.size),
                                     device_mesh=torch.arange(mesh.size).reshape(mesh.shape),
                                     placements=s.source_placements if source else s.target_placements, timeout=120)
                handler = client.register_tensors("weights", shards[r], bucket_size=bucket, timeout=300)
                for _ in range(warmup + steps):
                    barrier.wait(120)
                    t0 = time.time()
                    handler.transfer("send" if source else "recv", blocking=True, timeout=120)
                    stamps[r].append((t0, time.time()))
                handler.close()
                client.close()
            except BaseException:
                errors.append(traceback.format_exc())
                barrier.abort()

        threads = [threading.Thread(target=rank_body, args=(r,)) for r in my_ranks]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        if errors:
            out_q.put((role, "error", errors[0]))
            return
        nbytes = sum(t.numel() * t.element_size() for r in my_ranks for t, _ in shards[r])
        # checksum per logical tensor over every rank of this side: the raw bits summed as integers
        raw = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}
        sums = [0] * len(specs)
        for r in my_ranks:
            for i, (t, _) in enumerate(shards[r]):
                if t.numel():
                    sums[i] += int(t.contiguous().view(raw[t.element_size()]).sum(dtype=torch.int64).item())
        out_q.put((role, "ok", {"stamps": stamps, "bytes": nbytes, "ranks": my_ranks, "checksums": sums}))
    except BaseException:
        if shared_barrier is not None:
            shared_barrier.abort()
        out_q.put((role, "error", traceback.format_exc()))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="llama3_8b_fsdp8_to_tp2")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--zero-copy", action="store_true", help="lend contiguous single-chunk buckets (agent option)")
    ap.add_argument("--direct", action="store_true", help="no bucket buffers: receivers copy from the senders' tensors")
    ap.add_argument("--thread-per-rank", action="store_true",
                    help="one worker process per side with a thread per rank, instead of a process per rank "
                         "(taken anyway when the workload has more than 12 ranks)")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args()

    import torch

    from etha_amd import _native, workloads
    from etha_amd.tensor_bus import TensorBusAgent

    _native.lib()
    if not torch.cuda.is_available():
        print("bench_transfer needs a GPU: the hot path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    specs, _, _ = workloads.WORKLOADS[args.workload]()
    src_ranks = {int(r) for s in specs for r in np.asarray(s.source_mesh).reshape(-1)}
    tgt_ranks = {int(r) for s in specs for r in np.asarray(s.target_mesh).reshape(-1)}
    if src_ranks & tgt_ranks:
        print("bench_transfer: this workload's source and target rank sets overlap; a rank is served over one "
              "connection, so it cannot live in both worker processes", file=sys.stderr)
        sys.exit(2)
    world = 1 + max(int(r) for s in specs for m in (s.source_mesh, s.target_mesh) for r in np.asarray(m).reshape(-1))
    tmpdir = tempfile.mkdtemp(prefix="etha_bus_")
    agent = TensorBusAgent(world, _naming(tmpdir), device=args.device, zero_copy_single_chunk=args.zero_copy,
                           direct_same_device=args.direct)
    agent.start_in_thread()
    ctx = mp.get_context("spawn")
    out_q = ctx.Queue()
    if not args.thread_per_rank and len(src_ranks) + len(tgt_ranks) <= 12:
        # the ranks of a side start a step together: one barrier per side, shared by its processes
        barriers = {"trainer": ctx.Barrier(len(src_ranks)), "inference": ctx.Barrier(len(tgt_ranks))}
        procs = [ctx.Process(target=_worker, args=(role, args.workload, tmpdir, args.device, args.steps, args.warmup, out_q, r,
                                                   barriers[role]))
                 for role, ranks in (("trainer", src_ranks), ("inference", tgt_ranks)) for r in sorted(ranks)]
    else:
        procs = [ctx.Process(target=_worker, args=(role, args.workload, tmpdir, args.device, args.steps, args.warmup, out_q))
                 for role in ("trainer", "inference")]
    for p in procs:
        p.start()
    results = {}
    try:
        answered = 0
        while answered < len(procs):
            try:
                role, status, payload = out_q.get(timeout=1.0)
            except Exception:
                if any(p.exitcode not in (None, 0) for p in procs):
                    raise RuntimeError("a worker process died") from None
                continue
            if status != "ok":
                raise RuntimeError(f"{role} failed:\n{payload}")
            answered += 1
            if role not in results:
                results[role] = payload
            else:  # another rank of the same side
                mine = results[role]
                mine["stamps"].update(payload["stamps"])
                mine["bytes"] += payload["bytes"]
                mine["ranks"] = sorted(mine["ranks"] + payload["ranks"])
                mine["checksums"] = [a + b for a, b in zip(mine["checksums"], payload["checksums"])]
    finally:
        for p in procs:
            p.join(timeout=30)
        for p in procs:
            if p.is_alive():
                p.kill()
        agent_stats = dict(agent.stats, drives_served_from_a_recording=agent.wire.replays,
                           host_ms_of_transfer_passes={k: round(v, 3) for k, v in agent.timing.items()})
        agent.close()
    # checksum of checksums: a same-dtype tensor's bits, summed over all target ranks, equal the sum over all
    # source ranks times the number of copies the target layout holds of each element (per copy the source holds)
    from torch.distributed.tensor.placement_types import Partial, Replicate

    def copies(mesh, placements):
        shape = np.asarray(mesh).shape
        return int(np.prod([n for n, p in zip(shape, placements) if isinstance(p, Replicate)] or [1]))

    verified = 0
    for i, s in enumerate(specs):
        if (s.target_dtype or s.source_dtype) != s.source_dtype or any(isinstance(p, Partial) for p in s.source_placements):
            continue
        want = results["trainer"]["checksums"][i] * copies(s.target_mesh, s.target_placements)
        got = results["inference"]["checksums"][i] * copies(s.source_mesh, s.source_placements)
        if want != got:
            raise RuntimeError(f"{s.name}: checksum over the target ranks differs from the source ranks' ({got} vs {want})")
        verified += 1
    send, recv = results["trainer"]["stamps"], results["inference"]["stamps"]
    lat, spread = [], []
    for k in range(args.warmup, args.warmup + args.steps):
        start = min(v[k][0] for v in send.values())
        end = max(v[k][1] for v in recv.values())
        lat.append(end - start)
        # from the first rank's command to the last rank's, either direction
        spread.append(max(v[k][0] for side in (send, recv) for v in side.values()) - start)
    lat.sort()
    spread.sort()
    med = lat[len(lat) // 2]
    payload = results["inference"]["bytes"]
    print(json.dumps({
        "metric": "end-to-end handler.transfer through the tensor bus, agent and worker processes on one GPU",
        "value": payload / med / 1e9, "unit": "GB/s", "ms_per_transfer": med * 1e3, "min_ms": lat[0] * 1e3,
        "steps": args.steps, "warmup": args.warmup, "payload_bytes": payload,
        "ms_between_first_and_last_rank_command": spread[len(spread) // 2] * 1e3,
        "config": {"workload": args.workload, "source_ranks": len(results["trainer"]["ranks"]),
                   "target_ranks": len(results["inference"]["ranks"]), "zero_copy_single_chunk": args.zero_copy,
                   "direct_same_device": args.direct, "worker_processes": len(procs)},
        "agent": agent_stats, "tensors_verified_by_checksum": verified,
    }))


if __name__ == "__main__":
    main()
