"""The worker -> agent control channel.

The reference uses an LMDB file as a circular command queue plus one named POSIX semaphore per
command for completion (``src/etha/tensor_bus/command_queue.py``, ``client.py:153-182``).  Those
packages are not available here and the channel is off the hot path, so this is a thin stand-in with
the same roles: the agent listens on a Unix socket at the queue *path*; ``enqueue`` opens one
connection per command, sends it, and returns a :class:`Completion`, which plays the semaphore:
``acquire(timeout)`` returns when the agent has finished the command (or raises ``BusyError``).
"""

from __future__ import annotations

import os
import pickle
import socket
import sqlite3
import struct
import threading
import time
from multiprocessing.connection import Client, Connection


class BusyError(Exception):
    """The completion was not signalled within the timeout (cf. ``posix_ipc.BusyError``)."""


class QueueFullError(Exception):
    """Raised by :meth:`PersistentCommandQueue.enqueue` when the queue is full and the call may not wait (or its
    wait timed out).  The socket channel below does not fill up."""


class Completion:
    """Semaphore-like handle of one in-flight command."""

    def __init__(self, conn: Connection, name: str):
        self._conn = conn
        self.name = name
        self.result = None
        self._done = False

    def acquire(self, timeout: float | None = None):
        if self._done:
            return
        if not self._conn.poll(timeout):
            raise BusyError(self.name)
        try:
            status, value = self._conn.recv()
        except EOFError as e:
            raise ConnectionError("agent closed the connection before completing the command") from e
        self._done = True
        if status == "error":
            exc_type, message = value
            raise {"ValueError": ValueError, "RuntimeError": RuntimeError, "KeyError": KeyError,
                   "NotImplementedError": NotImplementedError, "TimeoutError": TimeoutError}.get(exc_type, RuntimeError)(message)
        self.result = value

    def close(self) -> None:
        try:
            self._conn.close()
        except OSError:
            pass

    def unlink(self) -> None:  # posix_ipc.Semaphore API
        self.close()


class CommandQueue:
    """``CommandQueue(path)`` on the worker side enqueues; ``CommandQueue(path, serve=True)`` on the
    agent side accepts connections.  The serving side is a plain non-blocking listening socket: the agent waits on
    the sockets of all its ranks at once (``fileno``) and takes what has arrived (``accept_ready``)."""

    def __init__(self, path: str, serve: bool = False):
        if path is None:
            raise ValueError("command queue path is required")
        self.path = path
        self._socket: socket.socket | None = None
        if serve:
            if os.path.exists(path):
                os.unlink(path)
            self._socket = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM)
            self._socket.bind(path)
            self._socket.listen(128)
            self._socket.setblocking(False)

    # worker side
    def enqueue(self, command) -> Completion:
        deadline = time.time() + 5.0
        while True:
            try:
                conn = Client(address=self.path, family="AF_UNIX")
                break
            except (FileNotFoundError, ConnectionRefusedError) as e:
                if time.time() > deadline:
                    raise ConnectionError(f"agent command queue at {self.path} is not reachable") from e
                time.sleep(0.05)
        conn.send(command)
        return Completion(conn, getattr(command, "semaphore_name", None) or "command")

    # agent side
    def fileno(self) -> int:
        return self._socket.fileno()

    def accept_ready(self) -> list[Connection]:
        """The connections that are waiting to be accepted, without blocking (possibly none)."""
        out = []
        while self._socket is not None:
            try:
                s, _ = self._socket.accept()
            except (BlockingIOError, InterruptedError):
                break
            except OSError:
                break
            s.setblocking(True)
            # the agent reads a command only once part of it has arrived; a sender that stalls in mid-message holds
            # the agent's one serving thread for at most this long (the read then fails and the connection is dropped)
            s.setsockopt(socket.SOL_SOCKET, socket.SO_RCVTIMEO, struct.pack("ll", 1, 0))
            out.append(Connection(s.detach()))
        return out

    def close(self) -> None:
        if self._socket is not None:
            self._socket.close()
            self._socket = None
            if os.path.exists(self.path):
                try:
                    os.unlink(self.path)
                except OSError:
                    pass


class PersistentCommandQueue:
    """The reference's queue API (``src/etha/tensor_bus/command_queue.py:23-395``) on a file from the standard
    library: a persistent circular FIFO of commands with a fixed capacity that several processes can open.

    ``enqueue`` returns the command's position (a running count; its slot is ``position % capacity``), blocks while
    the queue is full unless ``block=False`` and raises :class:`QueueFullError` when it may not wait or its wait
    times out; ``dequeue`` returns ``None`` on an empty queue (after waiting up to ``timeout`` with ``block=True``);
    ``dequeue_batch``, ``peek``, ``size``, ``is_empty``, ``clear`` as in the reference.  ``close(destroy=True)``
    removes the file, ``close(destroy=False)`` leaves it for the next opener (``command_queue.py:308-393``).
    Where the reference keeps an LMDB environment and counts free slots with POSIX semaphores, this keeps an
    SQLite file and polls: every operation is one ``BEGIN IMMEDIATE`` transaction, so openers in different
    processes see one queue.  The agent's live channel is the socket of :class:`CommandQueue`; this class is the
    queue as a data structure.
    """

    _POLL_S = 0.005

    def __init__(self, lmdb_path: str = "/tmp/tensor_bus.lmdb", capacity: int = 50000):
        if capacity < 1:
            raise ValueError("capacity must be positive")
        self.lmdb_path = str(lmdb_path)
        self.capacity = int(capacity)
        self._lock = threading.Lock()  # one connection, used by several threads: one transaction at a time
        self.env: sqlite3.Connection | None = sqlite3.connect(self.lmdb_path, timeout=30.0, isolation_level=None,
                                                              check_same_thread=False)
        with open(self.lmdb_path + "-lock", "a"):  # the companion file the reference's store keeps beside the data
            pass
        self._tx("CREATE TABLE IF NOT EXISTS slots (slot INTEGER PRIMARY KEY, data BLOB)")
        self._tx("CREATE TABLE IF NOT EXISTS pointers (name TEXT PRIMARY KEY, value INTEGER)")
        self._tx("INSERT OR IGNORE INTO pointers VALUES ('head', 0), ('tail', 0)")

    # -- transactions ----------------------------------------------------------------------------
    def _tx(self, sql: str, args: tuple = ()):
        with self._lock:
            env = self._env()
            env.execute("BEGIN IMMEDIATE")
            try:
                out = env.execute(sql, args).fetchall()
                env.execute("COMMIT")
                return out
            except BaseException:
                env.execute("ROLLBACK")
                raise

    def _env(self) -> sqlite3.Connection:
        if self.env is None:
            raise RuntimeError("queue is closed")
        return self.env

    def _pointers(self, env) -> tuple[int, int]:
        got = dict(env.execute("SELECT name, value FROM pointers").fetchall())
        return int(got["head"]), int(got["tail"])

    # -- producer --------------------------------------------------------------------------------
    def enqueue(self, msg, *, block: bool = True, timeout: float | None = None) -> int:
        deadline = None if timeout is None else time.monotonic() + timeout
        data = pickle.dumps(msg, protocol=pickle.HIGHEST_PROTOCOL)
        while True:
            with self._lock:
                env = self._env()
                env.execute("BEGIN IMMEDIATE")
                try:
                    head, tail = self._pointers(env)
                    if tail - head < self.capacity:
                        env.execute("INSERT OR REPLACE INTO slots VALUES (?, ?)", (tail % self.capacity, data))
                        env.execute("UPDATE pointers SET value = ? WHERE name = 'tail'", (tail + 1,))
                        env.execute("COMMIT")
                        return tail
                    env.execute("ROLLBACK")
                except BaseException:
                    if env.in_transaction:
                        env.execute("ROLLBACK")
                    raise
            if not block or (deadline is not None and time.monotonic() >= deadline):
                raise QueueFullError(f"Queue is full (capacity={self.capacity})")
            time.sleep(self._POLL_S)

    # -- consumer --------------------------------------------------------------------------------
    def _take(self, max_count: int, remove: bool = True) -> list:
        with self._lock:
            return self._take_locked(max_count, remove)

    def _take_locked(self, max_count: int, remove: bool) -> list:
        env = self._env()
        env.execute("BEGIN IMMEDIATE")
        try:
            head, tail = self._pointers(env)
            count = max(0, min(max_count, tail - head))
            out = []
            for pos in range(head, head + count):
                row = env.execute("SELECT data FROM slots WHERE slot = ?", (pos % self.capacity,)).fetchone()
                if row is not None:
                    out.append(pickle.loads(row[0]))
                    if remove:
                        env.execute("DELETE FROM slots WHERE slot = ?", (pos % self.capacity,))
            if remove and count:
                env.execute("UPDATE pointers SET value = ? WHERE name = 'head'", (head + count,))
            env.execute("COMMIT")
            return out
        except BaseException:
            env.execute("ROLLBACK")
            raise

    def dequeue(self, *, block: bool = False, timeout: float | None = None):
        deadline = None if timeout is None else time.monotonic() + timeout
        while True:
            got = self._take(1)
            if got:
                return got[0]
            if not block or (deadline is not None and time.monotonic() >= deadline):
                return None
            time.sleep(self._POLL_S)

    def dequeue_batch(self, max_count: int = 32) -> list:
        return self._take(max_count)

    def peek(self):
        got = self._take(1, remove=False)
        return got[0] if got else None

    def size(self) -> int:
        with self._lock:
            head, tail = self._pointers(self._env())
        return tail - head

    def is_empty(self) -> bool:
        return self.size() == 0

    def clear(self, delete_commands: bool = True) -> None:
        with self._lock:
            env = self._env()
            env.execute("BEGIN IMMEDIATE")
            try:
                env.execute("UPDATE pointers SET value = 0")
                if delete_commands:
                    env.execute("DELETE FROM slots")
                env.execute("COMMIT")
            except BaseException:
                env.execute("ROLLBACK")
                raise

    def close(self, destroy: bool = True) -> None:
        """``destroy=True`` (the default, as in the reference) removes the queue's files; ``destroy=False`` only
        closes this opener's handle.  Safe to call more than once."""
        with self._lock:
            if self.env is not None:
                self.env.close()
                self.env = None
        if destroy:
            for suffix in ("", "-lock", "-journal", "-wal", "-shm"):
                try:
                    os.unlink(self.lmdb_path + suffix)
                except OSError:
                    pass

    def __repr__(self) -> str:
        if self.env is None:
            return f"PersistentCommandQueue({self.lmdb_path!r}, closed)"
        return f"PersistentCommandQueue({self.lmdb_path!r}, size={self.size()}, capacity={self.capacity})"
