"""The bounded bucket pool and the per-rank bucket pipelines, checked on the CPU.

The wire's pipelines (the reference's ``bucket_comm`` loop, ``src/etha/comm/comm_methods.py:53-119``, one per
rank, stepped in turn) decide the order of launches; every launch is handed to the tile interpreter instead
of the GPU.  Checked: the bytes (against the oracle's restatement of the reference path), the pool bound
(``max_in_flight`` slots per channel), and - byte by byte - that launches issued without ordering between
them never touch each other's bytes.
"""

import numpy as np
import pytest
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from etha_amd import workloads
from etha_amd.comm import LoopbackWire, bucket_comm, loopback
from etha_amd.world import ReshardJob, TensorSpec

from helpers import assert_bit_equal, cpu_fill, expected_target, mesh_of, run_oracle
from test_random_layouts_cpu import _interpret


def _jobs(specs, bucket_size, depth, targets=None, pool="ring", **kw):
    wire = LoopbackWire("cpu", host_inspection=True, pool=pool, max_in_flight=depth)
    job = ReshardJob(specs, device="cpu", bucket_size=bucket_size, target_ranks=targets, keep_globals=True,
                     fill=cpu_fill, wire=wire, max_in_flight=depth, **kw)
    ref = ReshardJob(specs, device="cpu", bucket_size=bucket_size, target_ranks=targets, keep_globals=True, fill=cpu_fill)
    for a, b in zip(job.source_locals, ref.source_locals):
        for r in a:
            b[r].copy_(a[r])
    return job, ref


def _compare(job, ref, specs, what=""):
    for i, spec in enumerate(specs):
        for r, t in job.target_locals[i].items():
            assert_bit_equal(t, ref.target_locals[i][r], f"{what} {spec.name} rank {r} vs oracle")
            if job.globals_[i] is not None:
                assert_bit_equal(t, expected_target(spec, job.globals_[i], r), f"{what} {spec.name} rank {r} closed form")


def _ring_bound(job, depth):
    """channels x depth x largest bucket of the channel, summed over the job's send lists."""
    bound = 0
    for buckets in job.send_buckets.values():
        per_key = {}
        for b in buckets:
            if b.transport.value in ("p2p", "broadcast"):
                per_key.setdefault(loopback.wire_key(b), []).append(b.total_bytes)
        for sizes in per_key.values():
            bound += min(depth, len(sizes)) * (-(-max(sizes) // 256) * 256)
    return bound


@pytest.mark.parametrize("depth", [1, 2, 4])
@pytest.mark.parametrize("merged", [False, True], ids=["per_bucket", "ready_runs"])
def test_sets_of_independent_launches(depth, merged):
    """The wire hands an ordered launch and the unordered ones that follow it to the library as one set, whose
    members run at the same time: executed in reverse inside every set the result must be the same, no member may
    touch a byte another one writes, and the eight senders' packs of a sweep must really share sets."""
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=6, hidden=64, inter=224, kv=16, vocab=136)
    job, ref = _jobs(specs, 2048, depth, targets)
    log = job.wire.launch_log = []
    check = _interpret(job, merged, by_sets=True)
    run_oracle(ref)
    _compare(job, ref, specs, f"depth {depth}")
    assert check.sets < len(log) / 2 and check.largest >= 8
    job.wire.group_launches = False  # every step a set of its own
    check = _interpret(job, merged, by_sets=True)
    assert check.largest == 1
    _compare(job, ref, specs, f"depth {depth}, ungrouped")


@pytest.mark.parametrize("depth", [1, 2, 3])
@pytest.mark.parametrize("merged", [False, True], ids=["per_bucket", "ready_runs"])
def test_llama_like_through_a_ring(depth, merged):
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=6, hidden=64, inter=224, kv=16, vocab=136)
    job, ref = _jobs(specs, 2048, depth, targets)
    log = job.wire.launch_log = []
    check = _interpret(job, merged)
    run_oracle(ref)
    _compare(job, ref, specs, f"depth {depth}")
    n_send = sum(len(b) for b in job.send_buckets.values())
    per_channel = max(len([b for b in bs if b.transport.value == "p2p"]) for bs in job.send_buckets.values())
    assert per_channel > 2 * depth, "the workload must cycle every ring several times"
    assert job.wire.pool.reserved_bytes <= _ring_bound(job, depth)
    assert job.wire.pool.reserved_bytes < job.payload_bytes() / 2  # far below one slot per bucket
    assert check.unordered > len(log) // 2  # most launches overlap their predecessor
    if not merged:
        n_recv = sum(len(b) for b in job.recv_buckets.values())
        assert len(log) == n_send + n_recv  # one launch per bucket
    else:
        assert len(log) < n_send + sum(len(b) for b in job.recv_buckets.values())
    assert job.wire.idle()
    # a second transfer through the same plans and slots, with new values
    for d in job.source_locals:
        for t in d.values():
            t.mul_(-3)
    for d in ref.source_locals:
        for t in d.values():
            t.mul_(-3)
    _interpret(job, merged)
    run_oracle(ref)
    for i in range(len(specs)):
        for r, t in job.target_locals[i].items():
            assert_bit_equal(t, ref.target_locals[i][r], f"second transfer, tensor {i} rank {r}")


def test_both_target_ranks_and_broadcast_channels():
    """Both TP ranks receive: the broadcast channels (norm weights) are drained by two consumers, so the
    first receiver's call leaves its pipeline waiting on the wire until the second receiver has called."""
    specs, _, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=3, hidden=64, inter=224, kv=16, vocab=520)
    job, ref = _jobs(specs, 512, 2, None)
    _interpret(job, False)
    run_oracle(ref)
    _compare(job, ref, specs)
    assert job.wire.idle()


@pytest.mark.parametrize("op", ["sum", "max"])
def test_partial_and_self_copy_through_a_ring(op):
    specs = [
        TensorSpec("p", (48, 40), mesh_of(0, [4]), (Partial(op),), mesh_of(4, [2]), (Shard(0),), torch.bfloat16, seed=5),
        TensorSpec("q", (64, 24), mesh_of(0, [2, 2]), (Partial(op), Shard(1)), mesh_of(4, [2]), (Replicate(),), torch.float32, seed=9),
        # overlapping rank sets: same-rank chunks take the LOCAL path
        TensorSpec("e", (8, 24, 16), mesh_of(0, [4]), (Shard(0),), mesh_of(0, [2]), (Shard(1),), torch.float16, seed=2),
    ]
    job, ref = _jobs(specs, 256, 2)
    check = _interpret(job, False)
    run_oracle(ref)
    _compare(job, ref, specs)
    assert check.unordered > 0


@pytest.mark.parametrize("name,kw", [
    ("transposed_parents", dict(n_tensors=2, n=392)),
    ("transposed_parents", dict(n_tensors=2, n=392, target_transposed=True, dtype=torch.float32)),
    ("transposed_parents", dict(n_tensors=1, n=264, target_transposed=True, dtype=torch.float64)),
    ("transposed_parents", dict(n_tensors=1, n=520, dtype=torch.int8)),
    ("transposed_parents", dict(n_tensors=2, n=776, dtype=torch.float32, target_dtype=torch.bfloat16)),
    ("transposed_parents", dict(n_tensors=1, n=600, dtype=torch.float16, target_dtype=torch.float32, target_transposed=True)),
    ("moe_experts_row_parallel_w2", dict(n_experts=8, hidden=64, inter=224)),
])
def test_other_workloads_scaled_down(name, kw):
    """Transposed parents (LDS-staged blocks, full and edge, every element size) and the row-parallel expert
    layout, through the planner, the tile compiler and the interpreter."""
    specs, targets, _ = workloads.WORKLOADS[name](**kw)
    job, ref = _jobs(specs, 64 * 1024, 2, targets)
    _interpret(job, False)
    run_oracle(ref)
    _compare(job, ref, specs, name)


def test_missing_ordering_is_caught_by_the_byte_check(monkeypatch):
    """The byte-level check must fail when the wire forgets what earlier launches touched."""
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=2, hidden=64, inter=224, kv=16, vocab=520)
    job, _ = _jobs(specs, 2048, 2, targets)
    orig = LoopbackWire._issue

    def forgetful(self, *launch):
        self._epoch_reads, self._epoch_writes = set(), set()
        orig(self, *launch)

    monkeypatch.setattr(LoopbackWire, "_issue", forgetful)
    with pytest.raises(AssertionError, match="unordered launch"):
        _interpret(job, False)


def test_ordered_launches_only_when_switched_off():
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=1, hidden=64, inter=224, kv=16, vocab=520)
    job, ref = _jobs(specs, 2048, 2, targets)
    job.wire.unordered_launches = False
    check = _interpret(job, False)
    run_oracle(ref)
    _compare(job, ref, specs)
    assert check.unordered == 0


def test_recv_before_send_and_repeated_send_are_errors():
    spec = TensorSpec("w", (64, 8), [0, 1], (Shard(0),), [2, 3], (Shard(1),), torch.float32)
    job, _ = _jobs([spec], 64, 2)
    job.wire.on_launch = lambda *a: None
    for buckets in job.send_buckets.values():  # planning pairs receive buckets with send buckets: senders first
        job.wire.plan(buckets)
    with pytest.raises(RuntimeError, match="before its send bucket was ever sent"):
        job.run_recv()
    job.run_send()
    assert not job.wire.idle()  # the senders filled their rings and wait for the receivers
    assert len(job.wire.pending()) == 2
    with pytest.raises(RuntimeError, match="previous transfer of these buckets has not completed"):
        job.run_send()
    job.run_recv()
    assert job.wire.idle()
    job.run()  # and again, from a clean state


def test_absent_destination_ranks_do_not_hold_slots():
    """A job that stages one of two target ranks: broadcast buckets name both, only one will ever unpack."""
    specs = [TensorSpec("n", (4096,), mesh_of(0, [4]), (Shard(0),), mesh_of(4, [2]), (Replicate(),), torch.float32, seed=1)]
    job, ref = _jobs(specs, 512, 2, targets=[4])
    assert job.wire.absent_ranks == {5}
    _interpret(job, False)
    run_oracle(ref)
    _compare(job, ref, specs)
    # without that knowledge the wire waits for rank 5 forever, and says so
    job2, _ = _jobs(specs, 512, 2, targets=[4])
    job2.wire.absent_ranks.clear()
    job2.wire.on_launch = lambda *a: None
    with pytest.raises(RuntimeError, match="still waiting for a peer"):
        job2.run()


def test_release_returns_ring_slots():
    spec = TensorSpec("w", (256, 8), [0, 1], (Shard(0),), [2, 3], (Shard(1),), torch.float32)
    job, _ = _jobs([spec], 256, 2)
    job.wire.on_launch = lambda *a: None
    job.run()
    reserved = job.wire.pool.reserved_bytes
    assert reserved > 0
    for buckets in list(job.recv_buckets.values()) + list(job.send_buckets.values()):
        job.wire.release(buckets)
    job2 = ReshardJob([spec], device="cpu", bucket_size=256, fill=cpu_fill, wire=job.wire)
    job2.run()
    assert job.wire.pool.reserved_bytes == reserved  # the second plan reuses the released slots


def test_resident_pool_keeps_one_slot_per_bucket():
    specs, targets, _ = workloads.llama3_8b_fsdp8_to_tp2(n_layers=2, hidden=64, inter=224, kv=16, vocab=520)
    job, ref = _jobs(specs, 2048, 2, targets, pool="resident")
    _interpret(job, True)
    run_oracle(ref)
    _compare(job, ref, specs)
    assert job.wire.pool.reserved_bytes >= job.payload_bytes()
    empty = LoopbackWire("cpu", host_inspection=True).export_manifest()  # a ring can be exported too: nothing planned yet
    assert empty["pool"] == "ring" and empty["slots"] == {}


@pytest.mark.parametrize("depth", [1, 2, 3])
@pytest.mark.parametrize("zero_copy", [False, True], ids=["packed", "lent"])
def test_a_ring_whose_ends_live_in_different_processes(depth, zero_copy):
    """Producer and consumer each hold their own wire and trade "packed" / "unpacked" notifications over a pipe
    (LoopbackWire.exchange), as two processes on one GPU do; here the two ends are threads of this process and the
    launches go to the tile interpreter.  Two transfers; the pool stays within max_in_flight slots per channel;
    a notification that does not fit the hand-shake is refused."""
    import multiprocessing as mp
    import threading

    from test_random_layouts_cpu import _run_step
    from tile_interpreter import AbsoluteMemory

    src, tgt = list(range(4)), [4, 5]
    specs = [TensorSpec(f"w{i}", (128, 96 + 32 * i), src, (Shard(0),), tgt, (Shard(1),), torch.bfloat16, seed=i, std=1.0)
             for i in range(5)]
    specs.append(TensorSpec("n", (256,), src, (Shard(0),), tgt, (Replicate(),), torch.float32, torch.bfloat16, seed=9, std=1.0))
    specs.append(TensorSpec("big", (256, 512), src, (Shard(0),), tgt, (Shard(0),), torch.bfloat16, seed=10, std=1.0))
    producer, ref = _jobs(specs, 4096, depth, zero_copy=zero_copy)
    for buckets in producer.send_buckets.values():
        producer.wire.plan(buckets)
    manifest = producer.wire.export_manifest()
    assert manifest["pool"] == "ring"
    wire = LoopbackWire.from_manifest(manifest, "cpu")
    consumer = ReshardJob(specs, device="cpu", bucket_size=4096, keep_globals=True, fill=cpu_fill, wire=wire, max_in_flight=depth)
    assert producer.wire.pool.reserved_bytes <= _ring_bound(producer, depth)
    spans = []
    for job in (producer, consumer):
        for d in job.source_locals + job.target_locals:
            for t in d.values():
                st = t.untyped_storage()
                if st.nbytes():
                    spans.append((st.data_ptr(), st.data_ptr() + st.nbytes()))
    spans += [(s.data_ptr(), s.data_ptr() + s.numel()) for s in producer.wire.pool.segments]
    mem = AbsoluteMemory(min(s[0] for s in spans), max(s[1] for s in spans))
    lock = threading.Lock()

    def on_set(members, flags):
        with lock:
            for p, kind, first, count in members:
                _run_step(mem, p, kind, first, count, ordered=(kind, first, count) in p._ordered_ranges)

    producer.wire.on_set = consumer.wire.on_set = on_set
    a, b = mp.Pipe()
    errors = []

    def consume():
        try:
            consumer.run_recv(True, drive=False)
            consumer.wire.exchange(b, synchronize=lambda: None)
        except BaseException as e:  # noqa: BLE001
            errors.append(e)
            a.close()

    for round_ in range(4):
        if round_ == 3:  # the recordings can be switched off on one end only: the protocol does not change
            consumer.wire.replay_schedules = False
        if round_:
            for d, e in zip(producer.source_locals, ref.source_locals):
                for r, t in d.items():
                    t.mul_(-3.0)
                    e[r].copy_(t)
        th = threading.Thread(target=consume)
        th.start()
        producer.run_send(True, drive=False)
        producer.wire.exchange(a, synchronize=lambda: None)
        th.join(60)
        assert not th.is_alive() and not errors, errors
        assert producer.wire.idle() and consumer.wire.idle()
        run_oracle(ref)
        for i, spec in enumerate(specs):
            for r, t in consumer.target_locals[i].items():
                assert_bit_equal(t, ref.target_locals[i][r], f"round {round_} {spec.name} rank {r} vs oracle")
    assert consumer.wire.pool is None  # the consumer allocated no bucket memory
    # from the second transfer on both ends were served from what the first one recorded
    assert producer.wire.replays > 0 and consumer.wire.replays > 0
    # notifications that contradict the hand-shake are refused
    key, entries = next(iter(producer.wire._sent.items()))
    with pytest.raises(RuntimeError, match="was not sent"):
        producer.wire.apply_remote([("unpacked", key, min(entries), 4)])
    with pytest.raises(RuntimeError, match="not planned on this wire"):
        consumer.wire.apply_remote([("packed", key, 10_000)])
    with pytest.raises(ValueError, match="unknown wire notification"):
        consumer.wire.apply_remote([("sent", key, min(entries))])
