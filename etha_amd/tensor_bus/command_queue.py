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
import time
from multiprocessing.connection import Client, Connection, Listener


class BusyError(Exception):
    """The completion was not signalled within the timeout (cf. ``posix_ipc.BusyError``)."""


class QueueFullError(Exception):
    """Kept for API compatibility; a socket queue does not fill up."""


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
    agent side accepts connections."""

    def __init__(self, path: str, serve: bool = False):
        if path is None:
            raise ValueError("command queue path is required")
        self.path = path
        self._listener: Listener | None = None
        if serve:
            if os.path.exists(path):
                os.unlink(path)
            self._listener = Listener(address=path, family="AF_UNIX")

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
    @property
    def listener(self) -> Listener:
        return self._listener

    def accept(self) -> Connection:
        return self._listener.accept()

    def close(self) -> None:
        if self._listener is not None:
            self._listener.close()
            self._listener = None
            if os.path.exists(self.path):
                try:
                    os.unlink(self.path)
                except OSError:
                    pass
