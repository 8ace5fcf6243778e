"""Worker-process bodies for the tensor-bus tests (importable by multiprocessing 'spawn')."""

from __future__ import annotations

import os
import sys
import threading
import traceback

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def path_naming(tmpdir):
    def fn(rank: int):
        return os.path.join(tmpdir, f"agent_rank{rank}_command.lmdb"), os.path.join(tmpdir, f"agent_rank{rank}_state.lmdb")

    return fn


def run_ranks(fn, ranks):
    """Run ``fn(rank)`` for every rank in its own thread (each rank blocks on the others)."""
    errors, results = [], {}

    def body(r):
        try:
            results[r] = fn(r)
        except BaseException:
            errors.append((r, traceback.format_exc()))

    threads = [threading.Thread(target=body, args=(r,)) for r in ranks]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    if errors:
        raise RuntimeError("rank %d failed:\n%s" % errors[0])
    return results


# specs of the two-process test: (name, shape, source placements code, target placements code, src dtype, tgt dtype)
BUS_TENSORS = [
    ("q", (256, 128), ["S0"], ["S0"], "bfloat16", "bfloat16"),
    ("o", (128, 256), ["S0"], ["S1"], "bfloat16", "bfloat16"),
    ("norm", (64,), ["S0"], ["R"], "float32", "bfloat16"),
]
SRC_RANKS, TGT_RANKS = [0, 1, 2, 3], [4, 5]


def _global(i, round_):
    import torch

    g = torch.Generator().manual_seed(100 * round_ + i)
    return torch.randn(BUS_TENSORS[i][1], generator=g)


def trainer_process(tmpdir, device, rounds, out_q):
    """All source ranks of the pair, in one worker process: fill shards, send, twice."""
    try:
        import torch

        from oracle.dtensor_layout import local_shard  # the pinned convention, not the product's planner
        from etha_amd.tensor_bus import TensorBusClient
        from etha_amd.tensor_bus.bootstrap import setup_ptrace
        from helpers import parse_placements

        setup_ptrace()
        naming = path_naming(tmpdir)
        names = {"float32": torch.float32, "bfloat16": torch.bfloat16}
        shards = {r: [] for r in SRC_RANKS}
        for i, (_, shape, src, _, sdt, _) in enumerate(BUS_TENSORS):
            g = _global(i, 0).to(names[sdt])
            for pos, r in enumerate(SRC_RANKS):
                shard = local_shard(g, (len(SRC_RANKS),), parse_placements(src), (pos,)).clone().to(device)
                if i == 1:  # a view at a storage offset inside a wider parent: strides and offset must travel too
                    parent = torch.zeros(shard.shape[0], shard.shape[1] + 6, dtype=shard.dtype, device=device)
                    view = parent[:, 3 : 3 + shard.shape[1]]
                    view.copy_(shard)
                    shard = view
                shards[r].append(shard)
        barrier = threading.Barrier(len(SRC_RANKS))

        def rank_body(r):
            cmd, state = naming(r)
            client = TensorBusClient(r, cmd, state, connection_timeout=20)
            for i, (name, _, src, _, _, _) in enumerate(BUS_TENSORS):
                client.init_pair(f"pair_{name}", "trainer", "inference", len(SRC_RANKS), device_mesh=torch.arange(len(SRC_RANKS)),
                                 placements=parse_placements(src), timeout=30)
            handler = client.register_tensors("weights", [(t, f"pair_{BUS_TENSORS[i][0]}") for i, t in enumerate(shards[r])],
                                              bucket_size=16 * 1024, timeout=30)
            for round_ in range(rounds):
                if round_ > 0:  # new values in the same registered tensors: plan once, transfer N times
                    for i, (_, _, src, _, sdt, _) in enumerate(BUS_TENSORS):
                        g = _global(i, round_).to(names[sdt])
                        pos = SRC_RANKS.index(r)
                        shards[r][i].copy_(local_shard(g, (len(SRC_RANKS),), parse_placements(src), (pos,)))
                    torch.cuda.synchronize()
                barrier.wait(60)
                handler.transfer("send", blocking=True, timeout=60)
            handler.close()
            client.close()
            return True

        run_ranks(rank_body, SRC_RANKS)
        out_q.put(("trainer", "ok", None))
    except BaseException:
        out_q.put(("trainer", "error", traceback.format_exc()))


def inference_process(tmpdir, device, rounds, out_q):
    """All target ranks in another worker process: receive and compare with the closed form."""
    try:
        import torch

        from oracle.dtensor_layout import local_shard  # the pinned convention, not the product's planner
        from etha_amd.tensor_bus import TensorBusClient
        from etha_amd.tensor_bus.bootstrap import setup_ptrace
        from helpers import parse_placements

        setup_ptrace()
        naming = path_naming(tmpdir)
        names = {"float32": torch.float32, "bfloat16": torch.bfloat16}
        locals_ = {r: [] for r in TGT_RANKS}
        for i, (_, shape, _, tgt, _, tdt) in enumerate(BUS_TENSORS):
            for pos, r in enumerate(TGT_RANKS):
                shp = tuple(local_shard(torch.empty(shape, device="meta"), (len(TGT_RANKS),), parse_placements(tgt), (pos,)).shape)
                locals_[r].append(torch.full(shp, -1.0, dtype=names[tdt], device=device))
        mismatches = []

        def rank_body(r):
            cmd, state = naming(r)
            client = TensorBusClient(r, cmd, state, connection_timeout=20)
            for i, (name, _, _, tgt, _, _) in enumerate(BUS_TENSORS):
                client.init_pair(f"pair_{name}", "inference", "trainer", len(TGT_RANKS), device_mesh=torch.arange(len(TGT_RANKS)),
                                 placements=parse_placements(tgt), timeout=30)
            handler = client.register_tensors("weights", [(t, f"pair_{BUS_TENSORS[i][0]}") for i, t in enumerate(locals_[r])],
                                              bucket_size=16 * 1024, timeout=30)
            for round_ in range(rounds):
                handler.transfer("recv", blocking=True, timeout=60)
                torch.cuda.synchronize()
                for i, (name, _, _, tgt, sdt, tdt) in enumerate(BUS_TENSORS):
                    g = _global(i, round_).to(names[sdt])
                    want = local_shard(g, (len(TGT_RANKS),), parse_placements(tgt), (TGT_RANKS.index(r),))
                    wire = names[sdt] if names[sdt].itemsize <= names[tdt].itemsize else names[tdt]
                    want = want.to(wire).to(names[tdt])
                    got = locals_[r][i].cpu()
                    if not torch.equal(got.view(torch.uint8), want.contiguous().view(torch.uint8)):
                        mismatches.append((round_, r, name))
            signal = handler.query_transfer_signal()
            handler.close()
            client.close()
            return signal

        signals = run_ranks(rank_body, TGT_RANKS)
        out_q.put(("inference", "ok" if not mismatches else "mismatch", {"mismatches": mismatches, "signals": signals}))
    except BaseException:
        out_q.put(("inference", "error", traceback.format_exc()))


# ---- bucket pool handed from a producer process to a consumer process ------------------------------------
def _pool_specs():
    import torch
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from etha_amd.world import TensorSpec

    src, tgt = list(range(4)), [4, 5]
    specs = [
        TensorSpec("q", (512, 256), src, (Shard(0),), tgt, (Shard(0),), torch.bfloat16, seed=11, std=1.0),
        TensorSpec("o", (256, 512), src, (Shard(0),), tgt, (Shard(1),), torch.bfloat16, seed=12, std=1.0),
        TensorSpec("norm", (256,), src, (Shard(0),), tgt, (Replicate(),), torch.float32, torch.bfloat16, seed=13, std=1.0),
    ]
    # several buckets per channel, so that a ring of one or two slots is recycled while a transfer runs
    for i in range(3):
        specs.append(TensorSpec(f"up{i}", (256, 320), src, (Shard(0),), tgt, (Shard(1),), torch.bfloat16, seed=20 + i, std=1.0))
        specs.append(TensorSpec(f"n{i}", (512,), src, (Shard(0),), tgt, (Replicate(),), torch.bfloat16, seed=30 + i, std=1.0))
    return specs


def producer_process(device, conn, rounds, zero_copy=False, pool="resident", depth=2):
    """Owns the source shards and the bucket pool: plans, exports the pool, packs each round.  With a ring pool the
    slots are recycled while the transfer runs: ``exchange`` trades "packed" / "unpacked" notifications with the
    consumer process; with a resident pool one "packed" message per round is enough."""
    try:
        import torch

        from etha_amd.tensor_bus.bootstrap import setup_ptrace
        from etha_amd.world import ReshardJob
        from helpers import cpu_fill

        setup_ptrace()
        job = ReshardJob(_pool_specs(), device=device, bucket_size=32 * 1024, fill=cpu_fill, zero_copy=zero_copy,
                         pool=pool, max_in_flight=depth)
        lent = 0
        for buckets in job.send_buckets.values():
            lent += len(job.wire.plan(buckets).lent)  # planning assigns the slots
        assert (lent > 0) == bool(zero_copy)
        conn.send(("manifest", job.wire.export_manifest()))
        payload = job.payload_bytes()
        reserved = job.wire.pool.reserved_bytes if job.wire.pool is not None else 0
        if pool == "ring":  # the reference's bound: max_in_flight buckets per channel, not the payload
            channels = {(b.src_rank, tuple(b.dst_ranks), b.transport.value) for bs in job.send_buckets.values() for b in bs
                        if b.transport.value in ("p2p", "broadcast")}
            largest = max(b.total_bytes for bs in job.send_buckets.values() for b in bs)
            assert reserved <= len(channels) * depth * (-(-largest // 256) * 256), (reserved, len(channels), depth, largest)
            per_channel = {}
            for bs in job.send_buckets.values():
                for b in bs:
                    if b.transport.value in ("p2p", "broadcast"):
                        k = (b.src_rank, tuple(b.dst_ranks), b.transport.value)
                        per_channel[k] = per_channel.get(k, 0) + 1
            assert zero_copy or max(per_channel.values()) > depth  # slots really are reused within one transfer
        for round_ in range(rounds):
            if round_ > 0:
                for d in job.source_locals:
                    for t in d.values():
                        t.mul_(-2.0)
            if pool == "ring":
                job.run_send(merge_launches=True, drive=False)
                job.wire.exchange(conn)
                assert job.wire.idle()
            else:
                job.run_send(merge_launches=True)
                torch.cuda.synchronize()  # cross-process ordering is a host-side fence
                conn.send(("packed", round_))
            assert conn.recv() == ("consumed", round_)
        conn.send(("done", None))
    except BaseException:
        conn.send(("error", traceback.format_exc()))


def consumer_process(device, conn, rounds, out_q):
    """Maps the producer's pool, plans its receive side against the mapped addresses, unpacks, checks."""
    try:
        import torch

        from etha_amd.comm import LoopbackWire
        from etha_amd.tensor_bus.bootstrap import setup_ptrace
        from etha_amd.world import ReshardJob
        from helpers import cpu_fill, expected_target

        setup_ptrace()
        kind, manifest = conn.recv()
        assert kind == "manifest", manifest
        wire = LoopbackWire.from_manifest(manifest, device)
        ring = wire.pool_mode == "ring"
        specs = _pool_specs()
        job = ReshardJob(specs, device=device, bucket_size=32 * 1024, fill=cpu_fill, keep_globals=True, wire=wire)
        bad = []
        for round_ in range(rounds):
            if ring:
                job.run_recv(merge_launches=True, drive=False)
                wire.exchange(conn)
                assert wire.idle()
            else:
                assert conn.recv() == ("packed", round_)
                wire.mark_packed()
                job.run_recv(merge_launches=True)
            torch.cuda.synchronize()
            for i, spec in enumerate(specs):
                glob = job.globals_[i].cpu().float() * ((-2.0) ** round_)
                for r, t in job.target_locals[i].items():
                    want = expected_target(spec, glob.to(spec.source_dtype), r)
                    if not torch.equal(t.cpu().view(torch.uint8), want.contiguous().view(torch.uint8)):
                        bad.append((round_, spec.name, r))
            conn.send(("consumed", round_))
        assert wire.pool is None or wire.pool.reserved_bytes == 0  # the consumer holds no bucket memory of its own
        wire.close_imported()
        out_q.put(("consumer", "ok" if not bad else "mismatch", bad))
    except BaseException:
        out_q.put(("consumer", "error", traceback.format_exc()))
