"""The worker-facing surface: TensorBusClient / BatchHandler against the hub agent."""

import json
import multiprocessing as mp
import os
import threading
import time

import pytest
import torch
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

from etha_amd.tensor_bus import TensorBusAgent, TensorBusClient, bootstrap_client

from bus_workers import inference_process, path_naming, run_ranks, trainer_process


@pytest.fixture
def agent_factory(tmp_path):
    agents = []

    def make(world_size, device="cpu"):
        a = TensorBusAgent(world_size, path_naming(str(tmp_path)), device=device, heartbeat_interval=0.05)
        a.start_in_thread()
        agents.append(a)
        return a, path_naming(str(tmp_path))

    yield make
    for a in agents:
        a.close()


def _client(naming, rank, **kw):
    cmd, state = naming(rank)
    return TensorBusClient(rank, cmd, state, **kw)


def test_connection_errors(tmp_path):
    with pytest.raises(ConnectionError, match="not found"):
        TensorBusClient(0, str(tmp_path / "c"), str(tmp_path / "missing_state"), connection_timeout=0.3)
    stale = tmp_path / "stale_state"
    stale.write_text(json.dumps({"agent:heartbeat": time.time() - 60}))
    with pytest.raises(ConnectionError, match="Heartbeat is too old"):
        TensorBusClient(0, str(tmp_path / "c"), str(stale), connection_timeout=0.3)
    with pytest.raises(ValueError):
        os.environ.pop("TENSOR_BUS_STATE_PATH", None)
        TensorBusClient(0)


def test_init_pair_register_and_errors_on_cpu(agent_factory):
    agent, naming = agent_factory(3)
    clients = {r: _client(naming, r, connection_timeout=5) for r in range(3)}
    # the remote side never joins: blocking init_pair times out like the reference's semaphore wait
    with pytest.raises(TimeoutError):
        clients[0].init_pair("lonely", "a", "b", 1, device_mesh=torch.arange(1), placements=(Replicate(),), timeout=0.3)

    src = {0: torch.arange(8.0).reshape(2, 4), 1: torch.arange(8.0, 16.0).reshape(2, 4)}
    tgt = {2: torch.zeros(4, 4)}

    def body(r):
        c = clients[r]
        if r < 2:
            c.init_pair("w", "trainer", "inference", 2, device_mesh=torch.arange(2), placements=(Shard(0),), timeout=10)
            return c.register_tensors("b0", [(src[r], "w")], bucket_size=None, timeout=10)
        c.init_pair("w", "inference", "trainer", 1, device_mesh=torch.arange(1), placements=(Replicate(),), timeout=10)
        return c.register_tensors("b0", [(tgt[2], "w")], timeout=10)

    handlers = run_ranks(body, range(3))
    assert handlers[0].pair_names == ["w"] and handlers[0].batch_id == "b0"
    state = json.load(open(naming(0)[1]))
    assert state["pairs"]["w"] == "matched"
    batch = agent.batches["b0"]
    assert batch.planned_ranks == {0, 1, 2} and len(batch.send_buckets[0]) == 1 and len(batch.recv_buckets[2]) == 2
    assert batch.send_buckets[1][0].chunks[0].dst_ranks == (2,)
    assert handlers[2].query_transfer_signal() is False
    with pytest.raises(ValueError, match="cannot be empty"):
        clients[0].register_tensors("b1", [])
    with pytest.raises(ValueError, match="unknown pair"):
        clients[0].register_tensors("b2", [(src[0], "nope")], timeout=5)
    with pytest.raises(ValueError, match="unknown batch"):
        clients[0].transfer("never_registered", "send", blocking=True, timeout=5)
    # the hot path has no CPU implementation: a transfer of host tensors fails loudly
    with pytest.raises(RuntimeError, match="no CPU path"):
        handlers[0].transfer("send", blocking=True, timeout=5)
    sem = handlers[2].transfer("recv", blocking=False)  # its sources never sent: stays pending
    with pytest.raises(Exception):
        sem.acquire(timeout=0.3)
    for h in handlers.values():
        h.close()
    assert "b0" not in agent.batches
    for c in clients.values():
        c.close()


def test_idle_and_broken_connections_do_not_stall_the_agent(agent_factory):
    """One thread of the agent serves every rank's socket: a connection that never sends its command, or goes away
    before it has, must not keep the others waiting."""
    import socket

    agent, naming = agent_factory(2)
    idle = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
    idle.connect(naming(0)[0])  # connected, silent
    gone = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
    gone.connect(naming(1)[0])
    gone.close()  # connected, closed without a command
    half = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
    half.connect(naming(1)[0])
    half.sendall(b"\x00\x00")  # two of the four bytes of a message header, then nothing
    half.close()
    stalled = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
    stalled.connect(naming(1)[0])
    stalled.sendall(b"\x00\x00")  # the same, but the sender stays: the agent gives such a read one second
    client = _client(naming, 0, connection_timeout=5)
    t0 = time.time()
    with pytest.raises(ValueError, match="unknown batch"):
        client.transfer("never_registered", "send", blocking=True, timeout=5)
    assert time.time() - t0 < 3.0
    idle.close()
    stalled.close()
    with pytest.raises(ValueError, match="unknown batch"):
        client.transfer("never_registered", "recv", blocking=True, timeout=5)
    client.close()


def test_the_agent_waits_for_the_ranks_of_one_direction_only(agent_factory):
    """A batch plans both directions of its pair.  The agent gathers the commands of one transfer - its senders and
    their receivers - before it queues them, and must not wait for commands of the opposite direction."""
    from etha_amd.tensor_bus.agent import _Entry
    from etha_amd.tensor_bus.commands import Transfer

    agent, naming = agent_factory(6)
    clients = {r: _client(naming, r, connection_timeout=5) for r in range(6)}
    src = {r: torch.zeros(8, 16) for r in range(2)}
    tgt = {r: torch.zeros(16, 4) for r in range(2, 6)}

    def body(r):
        c = clients[r]
        if r < 2:
            c.init_pair("w", "trainer", "inference", 2, device_mesh=torch.arange(2), placements=(Shard(0),), timeout=10)
            return c.register_tensors("b0", [(src[r], "w")], timeout=10)
        c.init_pair("w", "inference", "trainer", 4, device_mesh=torch.arange(4), placements=(Shard(1),), timeout=10)
        return c.register_tensors("b0", [(tgt[r], "w")], timeout=10)

    handlers = run_ranks(body, range(6))  # kept: a handler that goes away cleans its batch up
    agent._stop.set()
    agent._serve_thread.join()
    batch = agent.batches["b0"]
    assert all(batch.send_buckets[r] and batch.recv_buckets[r] for r in range(6))  # both directions are planned
    forward = [_Entry(rank=r, conn=None, command=Transfer(batch_id="b0", transfer_type="send" if r < 2 else "recv"))
               for r in range(6)]
    for n in range(1, 6):
        agent._pending = forward[:n]
        assert agent._siblings_missing(), n
    agent._pending = forward
    assert not agent._siblings_missing()
    backward = [_Entry(rank=r, conn=None, command=Transfer(batch_id="b0", transfer_type="recv" if r < 2 else "send"))
                for r in range(6)]
    agent._pending = backward[2:]
    assert agent._siblings_missing()
    agent._pending = backward
    assert not agent._siblings_missing()
    # a rank that is a generation ahead is not waited for
    batch.recv_count[5] = 1
    agent._pending = forward[:5]
    assert not agent._siblings_missing()
    agent._pending = []
    agent._stop.clear()
    agent.start_in_thread()
    for h in handlers.values():
        h.close()
    for c in clients.values():
        c.close()


def test_partial_target_direction_is_rejected(agent_factory):
    agent, naming = agent_factory(2)
    clients = {r: _client(naming, r, connection_timeout=5) for r in range(2)}
    t = {0: torch.zeros(4, 4), 1: torch.zeros(4, 4)}

    def body(r):
        c = clients[r]
        if r == 0:
            c.init_pair("p", "a", "b", 1, device_mesh=torch.arange(1), placements=(Partial(),), timeout=10)
        else:
            c.init_pair("p", "b", "a", 1, device_mesh=torch.arange(1), placements=(Replicate(),), timeout=10)
        return c.register_tensors("b", [(t[r], "p")], timeout=10)

    handlers = run_ranks(body, range(2))
    assert agent.pairs["p"].m2m[("b", "a")] is None and agent.pairs["p"].m2m[("a", "b")] is not None
    with pytest.raises(RuntimeError, match="Partial target"):
        handlers[1].transfer("send", blocking=True, timeout=5)  # b -> a would need a Partial target
    for c in clients.values():
        c.close()


def test_cleanup_unmaps_each_ranks_ipc_tensors(agent_factory, monkeypatch):
    """CleanupBatch from a rank closes the hipIPC mappings of the tensors that rank registered - every one, once -
    and the batch disappears with its last rank."""
    from etha_amd import _native
    from etha_amd.tensor_bus.agent import BatchState, _Entry
    from etha_amd.tensor_bus.commands import CleanupBatch
    from etha_amd.tensor_bus.ipc_tensor import IpcTensor

    agent, _ = agent_factory(2)
    agent._stop.set()  # drive the commands by hand
    closed = []
    monkeypatch.setattr(_native, "ipc_close", lambda ptr: closed.append(ptr))
    dev = torch.device("cpu")
    batch = BatchState("b", ["p"], None)
    batch.registrations = {
        0: [("p", IpcTensor(0x1000, (4,), (1,), torch.float32, dev, 0x1000, 16)),
            ("p", IpcTensor(0x2000, (4,), (1,), torch.float32, dev, 0x2000, 16))],
        1: [("p", IpcTensor(0x3000, (4,), (1,), torch.float32, dev, 0x3000, 16)), ("p", torch.zeros(4))],
    }
    batch.planned_ranks = {0, 1}
    agent.batches["b"] = batch
    assert agent._advance(_Entry(rank=0, conn=None, command=CleanupBatch(batch_id="b"))) == (True, None)
    assert sorted(closed) == [0x1000, 0x2000] and "b" in agent.batches and 0 not in batch.registrations
    assert agent._advance(_Entry(rank=1, conn=None, command=CleanupBatch(batch_id="b"))) == (True, None)
    assert sorted(closed) == [0x1000, 0x2000, 0x3000] and "b" not in agent.batches
    assert agent._advance(_Entry(rank=1, conn=None, command=CleanupBatch(batch_id="b"))) == (True, None)  # idempotent
    assert len(closed) == 3


def test_bootstrap_client_resolves_rank_and_paths(agent_factory, monkeypatch):
    agent, naming = agent_factory(3)
    monkeypatch.setenv("RANK", "1")
    monkeypatch.delenv("AGENT_RANK", raising=False)
    monkeypatch.setenv("AGENT_RANK_OFFSET", "1")
    client, info = bootstrap_client(naming, connection_timeout=5)
    assert (info.agent_rank, info.global_rank, info.rank_offset, info.method) == (2, 1, 1, "offset")
    assert info.command_queue_path == naming(2)[0] and client.agent_rank == 2
    client.close()
    monkeypatch.setenv("AGENT_RANK", "0")
    client, info = bootstrap_client(naming, connection_timeout=5)
    assert (info.agent_rank, info.rank_offset, info.method) == (0, None, "direct")
    client.close()


@pytest.mark.gpu
def test_in_process_agent_end_to_end(gpu_device, agent_factory):
    """Trainer ranks 0..3 (fp32, Shard(0)) -> inference ranks 4..5 (bf16, Shard(1)) through the bus."""
    agent, naming = agent_factory(6, device=gpu_device)
    g = torch.Generator().manual_seed(3)
    glob = torch.randn(64, 96, generator=g)
    src = {r: glob[16 * r : 16 * (r + 1)].clone().to(gpu_device) for r in range(4)}
    tgt = {4 + j: torch.zeros(64, 48, dtype=torch.bfloat16, device=gpu_device) for j in range(2)}
    clients = {r: _client(naming, r, connection_timeout=5) for r in range(6)}

    def body(r):
        c = clients[r]
        if r < 4:
            c.init_pair("w", "trainer", "inference", 4, device_mesh=torch.arange(4), placements=(Shard(0),))
            h = c.register_tensors("step", [(src[r], "w")], bucket_size=1 << 20)
            h.transfer("send", blocking=True)
        else:
            c.init_pair("w", "inference", "trainer", 2, device_mesh=torch.arange(2), placements=(Shard(1),))
            h = c.register_tensors("step", [(tgt[r], "w")], bucket_size=1 << 20)
            h.transfer("recv", blocking=True)
        return h

    handlers = run_ranks(body, range(6))
    torch.cuda.synchronize()
    for j in range(2):
        want = glob[:, 48 * j : 48 * (j + 1)].to(torch.bfloat16)
        assert torch.equal(tgt[4 + j].cpu(), want)
    assert handlers[4].query_transfer_signal() is False  # every receiver has caught up
    for h in handlers.values():
        h.close()
    for c in clients.values():
        c.close()


@pytest.mark.gpu
def test_two_process_hipipc_handoff(gpu_device, tmp_path):
    """Worker processes own the tensors; the agent (this process) maps them with hipIpcOpenMemHandle,
    packs and unpacks, twice, with new values the second time."""
    agent = TensorBusAgent(6, path_naming(str(tmp_path)), device=gpu_device, heartbeat_interval=0.05)
    agent.start_in_thread()
    ctx = mp.get_context("spawn")
    out_q = ctx.Queue()
    procs = [ctx.Process(target=trainer_process, args=(str(tmp_path), str(gpu_device), 2, out_q)),
             ctx.Process(target=inference_process, args=(str(tmp_path), str(gpu_device), 2, out_q))]
    try:
        for p in procs:
            p.start()
        results = {}
        deadline = time.time() + 150
        while len(results) < 2 and time.time() < deadline:
            try:
                who, status, detail = out_q.get(timeout=1.0)
                results[who] = (status, detail)
            except Exception:
                if any(p.exitcode not in (None, 0) for p in procs):
                    break
        for p in procs:
            p.join(20)
        assert results.get("trainer", ("missing", None))[0] == "ok", results.get("trainer")
        assert results.get("inference", ("missing", None))[0] == "ok", results.get("inference")
        # the agent really worked on hipIPC-mapped pointers: 3 tensors x (4 + 2) ranks, 2 rounds x 6 transfers
        assert agent.stats == {"ipc_tensors": 18, "in_process_tensors": 0, "transfers": 12}
        assert agent.batches == {} or all(not b.registrations for b in agent.batches.values())
    finally:
        for p in procs:
            if p.is_alive():
                p.kill()
        agent.close()


@pytest.mark.gpu
@pytest.mark.parametrize("pool,depth", [("resident", 2), ("ring", 1), ("ring", 2)], ids=["resident", "ring1", "ring2"])
@pytest.mark.parametrize("zero_copy", [False, True], ids=["packed", "lent"])
def test_bucket_pool_crosses_a_process_boundary(gpu_device, zero_copy, pool, depth):
    """The wire step as a same-GPU loopback between two processes: the producer packs into its pool, the
    consumer maps the pool with hipIpcOpenMemHandle and unpacks from it; two rounds with new values.  With a
    ring pool the producer owns max_in_flight slots per channel (asserted there) and the two processes trade
    "packed" / "unpacked" notifications while the transfer runs, each behind a host-side fence."""
    from bus_workers import consumer_process, producer_process

    ctx = mp.get_context("spawn")
    a, b = ctx.Pipe()
    out_q = ctx.Queue()
    procs = [ctx.Process(target=producer_process, args=(str(gpu_device), a, 2, zero_copy, pool, depth)),
             ctx.Process(target=consumer_process, args=(str(gpu_device), b, 2, out_q))]
    try:
        for p in procs:
            p.start()
        who, status, detail = out_q.get(timeout=150)
        for p in procs:
            p.join(30)
        assert (who, status) == ("consumer", "ok"), detail
        assert all(p.exitcode == 0 for p in procs)
    finally:
        for p in procs:
            if p.is_alive():
                p.kill()


@pytest.mark.gpu
def test_cleanup_returns_pool_slots(gpu_device, agent_factory):
    """Registering, transferring and closing the same batch repeatedly must not grow the bucket pool."""
    agent, naming = agent_factory(2, device=gpu_device)
    src = torch.arange(4096, dtype=torch.float32, device=gpu_device).reshape(64, 64)
    tgt = torch.zeros(64, 64, device=gpu_device)
    clients = {r: _client(naming, r, connection_timeout=5) for r in range(2)}

    def pair(r):
        clients[r].init_pair("w", "a" if r == 0 else "b", "b" if r == 0 else "a", 1, device_mesh=torch.arange(1),
                             placements=(Replicate(),))

    run_ranks(pair, range(2))
    reserved = []
    for it in range(3):
        src.add_(1.0)
        torch.cuda.synchronize()

        def body(r):
            h = clients[r].register_tensors(f"b{it}", [((src if r == 0 else tgt), "w")], bucket_size=1 << 20)
            h.transfer("send" if r == 0 else "recv", blocking=True)
            h.close()

        run_ranks(body, range(2))
        torch.cuda.synchronize()
        assert torch.equal(tgt, src)
        reserved.append((agent.wire.pool.reserved_bytes, agent.wire.pool._cursor, len(agent.wire._plans)))
    assert reserved[0] == reserved[1] == reserved[2], reserved
    for c in clients.values():
        c.close()


@pytest.mark.gpu
def test_agent_zero_copy_send_completes_only_after_receive(gpu_device, tmp_path):
    """With lent buckets the receiver reads the worker's tensor itself, so a blocking send may only return
    once the receiver has unpacked - otherwise the worker could overwrite bytes still to be read."""
    agent = TensorBusAgent(2, path_naming(str(tmp_path)), device=gpu_device, heartbeat_interval=0.05,
                           zero_copy_single_chunk=True)
    agent.start_in_thread()
    try:
        naming = path_naming(str(tmp_path))
        src = torch.arange(4096, dtype=torch.float32, device=gpu_device).reshape(64, 64)
        tgt = torch.zeros(64, 64, device=gpu_device)
        clients = {r: _client(naming, r, connection_timeout=5) for r in range(2)}

        def reg(r):
            clients[r].init_pair("w", "a" if r == 0 else "b", "b" if r == 0 else "a", 1, device_mesh=torch.arange(1),
                                 placements=(Replicate(),))
            return clients[r].register_tensors("b", [((src if r == 0 else tgt), "w")], bucket_size=None)

        handlers = run_ranks(reg, range(2))
        assert agent.wire.plan(agent.batches["b"].send_buckets[0]).lends_tensor_memory()
        sem = handlers[0].transfer("send", blocking=False)
        with pytest.raises(Exception):
            sem.acquire(timeout=0.5)  # nobody has received yet: the send must still be pending
        handlers[1].transfer("recv", blocking=True, timeout=20)
        sem.acquire(timeout=20)  # now it completes
        torch.cuda.synchronize()
        assert torch.equal(tgt, src)
        for h in handlers.values():
            h.close()
        for c in clients.values():
            c.close()
    finally:
        agent.close()


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["buckets", "zero_copy", "direct"])
def test_agent_many_rounds_two_batches_all_wire_modes(gpu_device, tmp_path, mode):
    """Two registered batches (one with a Partial source) alternate for several rounds with new values each
    time; senders never wait for receivers between rounds except where the wire lends their tensors.  Every
    round's result must be the closed form of that round's values, in every wire mode."""
    agent = TensorBusAgent(6, path_naming(str(tmp_path)), device=gpu_device, heartbeat_interval=0.05,
                           zero_copy_single_chunk=mode == "zero_copy", direct_same_device=mode == "direct")
    agent.start_in_thread()
    naming = path_naming(str(tmp_path))
    rounds = 4

    def values(batch, i, round_, r=None):
        g = torch.Generator().manual_seed(1000 * round_ + 10 * i + (0 if batch == "a" else 500) + (0 if r is None else 7 * r + 1))
        shape = {("a", 0): (64, 96), ("a", 1): (128,), ("a", 2): (32, 40), ("b", 0): (48, 64), ("b", 1): (16, 24)}[(batch, i)]
        return torch.randn(shape, generator=g)

    # batch a: Shard(0)@4 -> Shard(1)@2 / Replicate / Shard(0); batch b: tensor 0 Partial@4 -> Shard(0)@2, tensor 1 Shard(1)@4 -> Replicate
    src_a = {r: [values("a", 0, 0)[16 * r:16 * r + 16].clone().to(gpu_device), values("a", 1, 0)[32 * r:32 * r + 32].clone().to(gpu_device),
                 values("a", 2, 0)[8 * r:8 * r + 8].clone().to(gpu_device)] for r in range(4)}
    tgt_a = {4 + j: [torch.zeros(64, 48, device=gpu_device), torch.zeros(128, device=gpu_device), torch.zeros(16, 40, device=gpu_device)]
             for j in range(2)}
    src_b = {r: [values("b", 0, 0, r).to(gpu_device), values("b", 1, 0)[:, 6 * r:6 * r + 6].clone().to(gpu_device)] for r in range(4)}
    tgt_b = {4 + j: [torch.zeros(24, 64, device=gpu_device), torch.zeros(16, 24, device=gpu_device)] for j in range(2)}
    barrier = threading.Barrier(6)
    failures = []

    def body(r):
        c = _client(naming, r, connection_timeout=10)
        trainer = r < 4
        me, other, n = ("trainer", "inference", 4) if trainer else ("inference", "trainer", 2)
        mesh = torch.arange(n)
        pls = {"a0": ((Shard(0),), (Shard(1),)), "a1": ((Shard(0),), (Replicate(),)), "a2": ((Shard(0),), (Shard(0),)),
               "b0": ((Partial(),), (Shard(0),)), "b1": ((Shard(1),), (Replicate(),))}
        for name, (sp, tp) in pls.items():
            c.init_pair(name, me, other, n, device_mesh=mesh, placements=sp if trainer else tp, timeout=60)
        mine_a, mine_b = (src_a[r], src_b[r]) if trainer else (tgt_a[r], tgt_b[r])
        ha = c.register_tensors("a", [(t, f"a{i}") for i, t in enumerate(mine_a)], bucket_size=4096, timeout=60)
        hb = c.register_tensors("b", [(t, f"b{i}") for i, t in enumerate(mine_b)], bucket_size=1 << 20, timeout=60)
        for round_ in range(rounds):
            for batch, h in (("a", ha), ("b", hb)):
                if trainer:
                    if round_ > 0:  # new values in the registered tensors
                        if batch == "a":
                            src_a[r][0].copy_(values("a", 0, round_)[16 * r:16 * r + 16])
                            src_a[r][1].copy_(values("a", 1, round_)[32 * r:32 * r + 32])
                            src_a[r][2].copy_(values("a", 2, round_)[8 * r:8 * r + 8])
                        else:
                            src_b[r][0].copy_(values("b", 0, round_, r))
                            src_b[r][1].copy_(values("b", 1, round_)[:, 6 * r:6 * r + 6])
                        torch.cuda.synchronize()
                    h.transfer("send", blocking=True, timeout=60)
                else:
                    h.transfer("recv", blocking=True, timeout=60)
                    j = r - 4
                    if batch == "a":
                        want = [values("a", 0, round_)[:, 48 * j:48 * j + 48], values("a", 1, round_), values("a", 2, round_)[16 * j:16 * j + 16]]
                        got = tgt_a[r]
                    else:
                        acc = values("b", 0, round_, 0)
                        for m in (1, 2, 3):
                            acc = acc + values("b", 0, round_, m)
                        want = [acc[24 * j:24 * j + 24], values("b", 1, round_)]
                        got = tgt_b[r]
                    for i, (g_, w_) in enumerate(zip(got, want)):
                        if not torch.equal(g_.cpu(), w_):
                            failures.append((mode, round_, batch, i, r))
            barrier.wait(60)  # a new round only overwrites source values once every receiver has checked
        # the same registration also carries the reverse direction: inference ranks send, trainer ranks receive
        if not trainer:
            j = r - 4
            tgt_a[r][0].copy_(values("a", 0, 99)[:, 48 * j:48 * j + 48])
            tgt_a[r][1].copy_(values("a", 1, 99))
            tgt_a[r][2].copy_(values("a", 2, 99)[16 * j:16 * j + 16])
            torch.cuda.synchronize()
            ha.transfer("send", blocking=True, timeout=60)
        else:
            ha.transfer("recv", blocking=True, timeout=60)
            want = [values("a", 0, 99)[16 * r:16 * r + 16], values("a", 1, 99)[32 * r:32 * r + 32], values("a", 2, 99)[8 * r:8 * r + 8]]
            for i, (g_, w_) in enumerate(zip(src_a[r], want)):
                if not torch.equal(g_.cpu(), w_):
                    failures.append((mode, "reverse", "a", i, r))
        barrier.wait(60)
        ha.close(); hb.close(); c.close()

    try:
        run_ranks(body, range(6))
        assert not failures, failures[:5]
        assert agent.stats["transfers"] == 6 * 2 * rounds + 6
    finally:
        agent.close()


@pytest.mark.gpu
def test_ranks_of_one_batch_in_different_pairs(gpu_device, agent_factory):
    """One batch id, two pairs with different members: ranks 0-1 -> rank 4 over pair "p", ranks 2-3 -> rank 5 over
    pair "q"; rank 4 additionally receives from pair "q"'s broadcast.  Every rank registers only its own pairs and
    is planned as soon as those are complete."""
    agent, naming = agent_factory(6, device=gpu_device)
    g = torch.Generator().manual_seed(9)
    gp, gq = torch.randn(32, 16, generator=g), torch.randn(8, 24, generator=g)
    src_p = {r: gp[16 * r:16 * r + 16].clone().to(gpu_device) for r in (0, 1)}
    src_q = {r: gq[:, 12 * (r - 2):12 * (r - 2) + 12].clone().to(gpu_device) for r in (2, 3)}
    tgt_p = {4: torch.zeros(32, 16, device=gpu_device)}
    tgt_q = {4: torch.zeros(8, 24, device=gpu_device), 5: torch.zeros(8, 24, device=gpu_device)}

    def body(r):
        c = _client(naming, r, connection_timeout=5)
        regs = []
        if r in (0, 1):
            c.init_pair("p", "src", "dst", 2, device_mesh=torch.arange(2), placements=(Shard(0),), timeout=30)
            regs.append((src_p[r], "p"))
        if r in (2, 3):
            c.init_pair("q", "src", "dst", 2, device_mesh=torch.arange(2), placements=(Shard(1),), timeout=30)
            regs.append((src_q[r], "q"))
        if r == 4:
            c.init_pair("p", "dst", "src", 1, device_mesh=torch.arange(1), placements=(Replicate(),), timeout=30)
            regs.append((tgt_p[4], "p"))
        if r in (4, 5):
            c.init_pair("q", "dst", "src", 2, device_mesh=torch.arange(2), placements=(Replicate(),), timeout=30)
            regs.append((tgt_q[r], "q"))
        h = c.register_tensors("mixed", regs, bucket_size=1 << 20, timeout=30)
        h.transfer("send" if r < 4 else "recv", blocking=True, timeout=30)
        h.close()
        c.close()

    run_ranks(body, range(6))
    torch.cuda.synchronize()
    assert torch.equal(tgt_p[4].cpu(), gp)
    assert torch.equal(tgt_q[4].cpu(), gq) and torch.equal(tgt_q[5].cpu(), gq)
