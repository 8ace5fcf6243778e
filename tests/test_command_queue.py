"""The persistent command queue: the case list of the reference's tests/test_command_queue.py (single command,
empty queue, FIFO order, mixed command types, batches, peek, clear, a large queue, persistence across reopen,
destroy, capacity, wrap-around, blocking enqueue and its timeout, two openers of one file) on the stdlib-backed
queue.  No GPU."""

import multiprocessing as mp
import os
import threading
import time

import pytest

from etha_amd.tensor_bus.command_queue import PersistentCommandQueue, QueueFullError
from etha_amd.tensor_bus.commands import CleanupBatch, InitPair, QueryStatus, RegisterTensors, Transfer


@pytest.fixture
def path(tmp_path):
    return str(tmp_path / "queue.lmdb")


@pytest.fixture
def queue(path):
    q = PersistentCommandQueue(path)
    yield q
    q.close()


def _send(i, **kw):
    return Transfer(batch_id=f"t{i}", transfer_type="send", **kw)


def test_one_command_round_trip(queue):
    pos = queue.enqueue(Transfer(batch_id="b", transfer_type="recv", timestamp=3.5, semaphore_name="/s"))
    assert pos == 0 and queue.size() == 1 and not queue.is_empty()
    got = queue.dequeue()
    assert isinstance(got, Transfer) and (got.batch_id, got.transfer_type, got.timestamp, got.semaphore_name) == ("b", "recv", 3.5, "/s")
    assert queue.is_empty() and queue.dequeue() is None


def test_fifo_order_and_positions(queue):
    assert [queue.enqueue(_send(i)) for i in range(10)] == list(range(10))
    assert [queue.dequeue().batch_id for _ in range(10)] == [f"t{i}" for i in range(10)]


def test_every_command_type_keeps_its_type_and_fields(queue):
    sent = [
        Transfer(batch_id="a", transfer_type="send"),
        RegisterTensors(batch_id="a", tensors=[("pair", b"\x00\x01payload")], bucket_size=1 << 20),
        InitPair(pair_name="p", local_name="trainer", expected_world_size=4, remote_name="inference",
                 mesh_shape_payload=(2, 2), placements_payload=("S0", "R")),
        QueryStatus(batch_id="a", state_name="transfer_signal"),
        CleanupBatch(batch_id="a"),
    ]
    for m in sent:
        queue.enqueue(m)
    assert [queue.dequeue() for _ in sent] == sent


def test_batches(queue):
    for i in range(10):
        queue.enqueue(_send(i))
    first = queue.dequeue_batch(4)
    assert [m.batch_id for m in first] == ["t0", "t1", "t2", "t3"] and queue.size() == 6
    rest = queue.dequeue_batch(100)  # more than there is
    assert [m.batch_id for m in rest] == [f"t{i}" for i in range(4, 10)] and queue.is_empty()
    assert queue.dequeue_batch() == []


def test_peek_does_not_remove(queue):
    assert queue.peek() is None
    queue.enqueue(_send(0))
    queue.enqueue(_send(1))
    assert queue.peek().batch_id == "t0" and queue.peek().batch_id == "t0" and queue.size() == 2
    queue.dequeue()
    assert queue.peek().batch_id == "t1"


def test_clear(queue):
    for i in range(7):
        queue.enqueue(_send(i))
    queue.clear()
    assert queue.is_empty() and queue.dequeue() is None and queue.peek() is None
    assert queue.enqueue(_send(99)) == 0  # positions start afresh
    assert queue.dequeue().batch_id == "t99"


def test_large_queue_keeps_order(queue):
    n = 1000
    for i in range(n):
        queue.enqueue(_send(i))
    assert queue.size() == n
    got = []
    while not queue.is_empty():
        got += queue.dequeue_batch(64)
    assert [m.batch_id for m in got] == [f"t{i}" for i in range(n)]


def test_contents_survive_close_and_reopen(path):
    q1 = PersistentCommandQueue(path)
    q1.enqueue(_send(1, timestamp=1.0))
    q1.enqueue(Transfer(batch_id="t2", transfer_type="recv", timestamp=2.0))
    q1.close(destroy=False)
    assert os.path.exists(path)
    q2 = PersistentCommandQueue(path)
    assert q2.size() == 2
    assert (q2.dequeue().batch_id, q2.dequeue().transfer_type) == ("t1", "recv")
    assert q2.is_empty()
    q2.close()


def test_destroy_removes_the_files_and_may_be_repeated(path):
    q = PersistentCommandQueue(path)
    q.enqueue(_send(0))
    assert os.path.exists(path) and os.path.exists(path + "-lock")
    q.close(destroy=True)
    assert q.env is None and not os.path.exists(path) and not os.path.exists(path + "-lock")
    q.close(destroy=True)  # nothing left to remove: silent
    with pytest.raises(RuntimeError, match="closed"):
        q.size()


def test_capacity_is_a_hard_limit(path):
    q = PersistentCommandQueue(path, capacity=5)
    for i in range(5):
        q.enqueue(_send(i), block=False)
    assert q.size() == 5
    with pytest.raises(QueueFullError, match="capacity=5"):
        q.enqueue(_send(5), block=False)
    assert q.size() == 5
    q.close()


def test_wrap_around_keeps_order(path):
    q = PersistentCommandQueue(path, capacity=5)
    for i in range(5):
        q.enqueue(_send(i), block=False)
    q.dequeue(), q.dequeue()
    assert q.enqueue(_send(5), block=False) == 5 and q.enqueue(_send(6), block=False) == 6  # slots 0 and 1 again
    assert q.size() == 5
    assert [q.dequeue().batch_id for _ in range(5)] == [f"t{i}" for i in range(2, 7)]
    for lap in range(3):  # several laps round the ring
        for i in range(5):
            q.enqueue(_send(100 * lap + i), block=False)
        assert [m.batch_id for m in q.dequeue_batch(5)] == [f"t{100 * lap + i}" for i in range(5)]
    q.close()


def test_blocking_enqueue_waits_for_space(path):
    q = PersistentCommandQueue(path, capacity=3)
    for i in range(3):
        q.enqueue(_send(i), block=False)
    t = threading.Thread(target=lambda: (time.sleep(0.4), q.dequeue()))
    t.start()
    start = time.time()
    q.enqueue(_send(3), block=True, timeout=5)
    waited = time.time() - start
    t.join()
    assert 0.3 < waited < 10.0 and q.size() == 3
    q.close()


def test_blocking_enqueue_times_out(path):
    q = PersistentCommandQueue(path, capacity=2)
    q.enqueue(_send(0)), q.enqueue(_send(1))
    start = time.time()
    with pytest.raises(QueueFullError):
        q.enqueue(_send(2), block=True, timeout=0.3)
    assert 0.25 < time.time() - start < 10.0
    q.close()


def test_blocking_dequeue_waits_for_a_command(queue):
    assert queue.dequeue(block=True, timeout=0.1) is None
    t = threading.Thread(target=lambda: (time.sleep(0.2), queue.enqueue(_send(7))))
    t.start()
    got = queue.dequeue(block=True, timeout=5)
    t.join()
    assert got.batch_id == "t7"


def test_two_openers_share_one_queue(path):
    q1 = PersistentCommandQueue(path, capacity=5)
    q1.enqueue(_send(1), block=False)
    q2 = PersistentCommandQueue(path, capacity=5)
    assert q2.size() == 1 and q2.dequeue().batch_id == "t1"
    assert q1.size() == 0
    q1.close(destroy=False)
    assert os.path.exists(path) and os.path.exists(path + "-lock")
    q2.close()
    assert not os.path.exists(path) and not os.path.exists(path + "-lock")


def _producer(path, n):
    q = PersistentCommandQueue(path, capacity=8)
    for i in range(n):
        q.enqueue(_send(i), block=True, timeout=30)
    q.close(destroy=False)


def test_a_producer_process_and_a_consumer_process(path):
    """A small ring between two processes: the producer blocks on a full queue, nothing is lost or reordered."""
    consumer = PersistentCommandQueue(path, capacity=8)
    proc = mp.get_context("spawn").Process(target=_producer, args=(path, 50))
    proc.start()
    got = []
    deadline = time.time() + 60
    while len(got) < 50 and time.time() < deadline:
        m = consumer.dequeue(block=True, timeout=1.0)
        if m is not None:
            got.append(m.batch_id)
    proc.join(30)
    assert proc.exitcode == 0 and got == [f"t{i}" for i in range(50)]
    consumer.close()
