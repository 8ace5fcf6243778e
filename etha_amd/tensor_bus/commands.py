"""Commands a worker sends to the agent.

Same names and fields as ``src/etha/tensor_bus/commands.py`` (``Transfer``, ``RegisterTensors``,
``InitPair``, ``QueryStatus``, ``CleanupBatch`` with ``timestamp`` and ``semaphore_name``).  They are
plain dataclasses pickled over a Unix socket instead of msgpack structs in an LMDB queue; the mesh
shape and placements travel as values instead of pickled payloads.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Literal


@dataclass(kw_only=True)
class BaseCommand:
    timestamp: float | None = None
    semaphore_name: str | None = None
    agent_rank: int | None = None  # which virtual agent rank the command is addressed to


@dataclass(kw_only=True)
class Transfer(BaseCommand):
    batch_id: str
    transfer_type: Literal["send", "recv"]


@dataclass(kw_only=True)
class RegisterTensors(BaseCommand):
    batch_id: str
    tensors: list[tuple[str, bytes]] = field(default_factory=list)  # (pair_name, tensor payload)
    bucket_size: int | None = None


@dataclass(kw_only=True)
class InitPair(BaseCommand):
    pair_name: str
    local_name: str
    expected_world_size: int
    remote_name: str
    mesh_shape_payload: tuple | None = None
    placements_payload: tuple | None = None


@dataclass(kw_only=True)
class QueryStatus(BaseCommand):
    batch_id: str
    state_name: str


@dataclass(kw_only=True)
class CleanupBatch(BaseCommand):
    batch_id: str


Message = Transfer | RegisterTensors | InitPair | QueryStatus | CleanupBatch
