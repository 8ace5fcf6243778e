"""Worker-side tensor bus client.

Same surface as ``src/etha/tensor_bus/client.py``: ``TensorBusClient(agent_rank,
lmdb_command_queue_path=None, agent_state_lmdb_path=None, connection_timeout=30.0)`` with
``init_pair`` / ``register_tensors`` / ``transfer`` / ``query_transfer_signal`` / ``close``, and
``BatchHandler.transfer`` / ``query_transfer_signal`` / ``close``.  The two paths name the agent's
command socket and its state/heartbeat file (the reference's two LMDB files).  Tensors are handed to
the agent as hipIPC handles (:mod:`etha_amd.tensor_bus.ipc_tensor`).
"""

from __future__ import annotations

import json
import logging
import os
import time
import uuid
import weakref
from typing import Literal

import torch

from .command_queue import BusyError, CommandQueue, Completion
from .commands import CleanupBatch, InitPair, QueryStatus, RegisterTensors, Transfer
from .ipc_tensor import export_tensor, release_local

logger = logging.getLogger(__name__)

HEARTBEAT_MAX_AGE = 5.0  # seconds (client.py:374)


class BatchHandler:
    """Handle of one registered batch (``client.py:30-107``)."""

    def __init__(self, client: "TensorBusClient", batch_id: str, pair_names: list[str]):
        self._client_ref = weakref.ref(client)
        self.batch_id = batch_id
        self.pair_names = pair_names
        self._closed = False

    @property
    def client(self) -> "TensorBusClient":
        client = self._client_ref()
        if client is None:
            raise RuntimeError("TensorBusClient has been garbage collected. BatchHandler is no longer valid.")
        return client

    def transfer(self, transfer_type: Literal["send", "recv"], blocking: bool = False, timeout: float = 30.0) -> Completion:
        msg = Transfer(batch_id=self.batch_id, transfer_type=transfer_type)
        return self.client._execute_command_with_semaphore(
            msg, "transfer", context_id=f"batch_{self.batch_id}_{transfer_type}", blocking=blocking, timeout=timeout)

    def query_transfer_signal(self, blocking: bool = True, timeout: float = 30.0) -> bool:
        return self.client.query_transfer_signal(self.batch_id, blocking=blocking, timeout=timeout)

    def close(self, blocking: bool = True, timeout: float = 30.0):
        if self._closed:
            return
        self._closed = True
        msg = CleanupBatch(batch_id=self.batch_id)
        self.client._execute_command_with_semaphore(
            msg, "cleanup_batch", context_id=f"batch_{self.batch_id}", blocking=blocking, timeout=timeout)

    def __del__(self):
        try:
            self.close(blocking=False)
        except Exception:
            pass


def generate_semaphore_name(command_type: str, context_id: str) -> str:
    safe = context_id.replace("/", "_").replace(":", "_")
    return f"/command_{command_type}_{safe}_{os.getpid()}_{uuid.uuid4().hex}"


class TensorBusClient:
    """Host-side tensor bus client."""

    def __init__(self, agent_rank: int, lmdb_command_queue_path: str | None = None,
                 agent_state_lmdb_path: str | None = None, connection_timeout: float = 30.0):
        self.agent_rank = agent_rank
        if agent_state_lmdb_path is None:
            agent_state_lmdb_path = os.environ.get("TENSOR_BUS_STATE_PATH")
        if agent_state_lmdb_path is None:
            raise ValueError("agent_state_lmdb_path is required (or set TENSOR_BUS_STATE_PATH)")
        self.agent_state_lmdb_path = agent_state_lmdb_path
        self._connect_agent(agent_state_lmdb_path, timeout=connection_timeout)
        if lmdb_command_queue_path is None:
            lmdb_command_queue_path = os.environ.get("TENSOR_BUS_COMMAND_QUEUE_PATH")
        self.command_queue = CommandQueue(lmdb_command_queue_path)

    # ---- plumbing ---------------------------------------------------------------------------
    def _read_state(self) -> dict | None:
        try:
            with open(self.agent_state_lmdb_path) as f:
                return json.load(f)
        except (OSError, ValueError):
            return None

    def _connect_agent(self, path: str, timeout: float) -> None:
        deadline = time.time() + timeout
        while not os.path.exists(path):
            if time.time() > deadline:
                raise ConnectionError(
                    f"Agent state not found at {path} after {timeout}s. Please ensure the agent process is running. "
                    "Check AGENT_RANK environment variable is correct."
                )
            time.sleep(0.05)
        while time.time() <= deadline:
            state = self._read_state()
            if state is not None and time.time() - float(state.get("agent:heartbeat", 0.0)) < HEARTBEAT_MAX_AGE:
                return
            time.sleep(0.05)
        raise ConnectionError(
            f"Agent at {path} is not responding after {timeout}s. Heartbeat is too old or missing. Agent may have crashed."
        )

    def _execute_command_with_semaphore(self, command, command_type: str, context_id: str, blocking: bool = False,
                                        timeout: float = 30.0) -> Completion:
        command.semaphore_name = generate_semaphore_name(command_type, context_id)
        command.timestamp = time.time()
        command.agent_rank = self.agent_rank
        sem = self.command_queue.enqueue(command)
        if blocking:
            try:
                sem.acquire(timeout=timeout)
            except BusyError as e:
                raise TimeoutError(
                    f"TensorBusClient[{self.agent_rank}]: {command_type} timeout for context '{context_id}' "
                    f"with semaphore {command.semaphore_name}"
                ) from e
            finally:
                sem.close()
        return sem

    # ---- API ----------------------------------------------------------------------------------
    def init_pair(self, pair_name: str, local_name: str, remote_name: str, expected_world_size: int,
                  device_mesh=None, placements=None, blocking: bool = True, timeout: float = 30.0) -> None:
        """Register this rank as part of ``local_name`` in a pair; blocks until both sides are complete.

        ``device_mesh`` may be a ``DeviceMesh`` or anything with a shape (array, tensor, nested list);
        only its shape travels, as in the reference (``client.py:220-222``).
        """
        mesh_shape = None
        if device_mesh is not None:
            mesh = device_mesh.mesh if hasattr(device_mesh, "mesh") else device_mesh
            mesh_shape = tuple(int(s) for s in (mesh.shape if hasattr(mesh, "shape") else torch.as_tensor(mesh).shape))
        msg = InitPair(pair_name=pair_name, local_name=local_name, expected_world_size=expected_world_size,
                       remote_name=remote_name, mesh_shape_payload=mesh_shape,
                       placements_payload=tuple(placements) if placements is not None else None)
        sem = self._execute_command_with_semaphore(msg, "register", context_id=pair_name, blocking=blocking, timeout=timeout)
        if blocking and sem.result != "matched":
            raise RuntimeError(f"Pair '{pair_name}' is not matched")

    def transfer(self, batch_id: str, transfer_type: Literal["send", "recv"], blocking: bool = False,
                 timeout: float = 30.0) -> Completion:
        msg = Transfer(batch_id=batch_id, transfer_type=transfer_type)
        return self._execute_command_with_semaphore(msg, "transfer", context_id=batch_id, blocking=blocking, timeout=timeout)

    def query_transfer_signal(self, batch_id: str, blocking: bool = True, timeout: float = 30.0) -> bool:
        msg = QueryStatus(batch_id=batch_id, state_name="transfer_signal")
        sem = self._execute_command_with_semaphore(msg, "query", context_id=f"batch_{batch_id}", blocking=blocking, timeout=timeout)
        if blocking:
            return bool(sem.result)
        state = self._read_state() or {}
        return bool(state.get("batches", {}).get(batch_id, {}).get("transfer_signal", False))

    def register_tensors(self, batch_id: str, tensors: list[tuple[torch.Tensor, str]], bucket_size: int | None = None,
                         timeout: float = 30.0) -> BatchHandler:
        """Register tensors across pairs; always blocks until every rank of the batch has registered."""
        if not tensors:
            raise ValueError("tensors list cannot be empty")
        for t, _ in tensors:
            if t.device.type == "cuda":
                torch.cuda.current_stream(t.device).synchronize()  # the agent works on its own stream
        payloads = [(pair_name, export_tensor(tensor)) for tensor, pair_name in tensors]
        msg = RegisterTensors(batch_id=batch_id, tensors=payloads, bucket_size=bucket_size)
        try:
            self._execute_command_with_semaphore(msg, "register_tensors", context_id=f"batch_{batch_id}", blocking=True,
                                                 timeout=timeout)
        finally:
            # An agent in this process has taken the tensor objects by now; an agent in another process maps the
            # memory and, as in the reference, the worker keeps its tensors alive for as long as the batch lives.
            for _, p in payloads:
                release_local(p)
        unique_pair_names = list(dict.fromkeys(pair_name for _, pair_name in tensors))
        return BatchHandler(client=self, batch_id=batch_id, pair_names=unique_pair_names)

    def close(self):
        self.command_queue.close()
