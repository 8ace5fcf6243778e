"""Worker-side bootstrap (``src/etha/tensor_bus/bootstrap.py``): resolve the agent rank from the
environment, derive the two paths, create the client."""

from __future__ import annotations

import ctypes
import logging
import os
from collections.abc import Callable
from dataclasses import dataclass

from .agent import default_path_naming
from .client import TensorBusClient

logger = logging.getLogger(__name__)


def setup_ptrace() -> None:
    """Allow another process (the agent) to open this process's device allocations."""
    PR_SET_PTRACER, PR_SET_PTRACER_ANY = 0x59616D61, -1
    libc = ctypes.CDLL("libc.so.6", use_errno=True)
    if libc.prctl(PR_SET_PTRACER, PR_SET_PTRACER_ANY, 0, 0, 0) != 0:
        logger.error("[Bootstrap] ptrace setup failed")


@dataclass
class BootstrapInfo:
    agent_rank: int
    global_rank: int
    rank_offset: int | None
    command_queue_path: str
    state_path: str
    method: str


def bootstrap_client(path_naming_fn: Callable[[int], tuple[str, str]] | None = None,
                     connection_timeout: float = 30.0) -> tuple[TensorBusClient, BootstrapInfo]:
    """``AGENT_RANK`` wins; otherwise ``RANK + AGENT_RANK_OFFSET`` (``bootstrap.py:84-100``)."""
    setup_ptrace()
    global_rank = int(os.environ["RANK"])
    if "AGENT_RANK" in os.environ:
        rank_offset, agent_rank, method = None, int(os.environ["AGENT_RANK"]), "direct"
    else:
        rank_offset = int(os.environ.get("AGENT_RANK_OFFSET", 0))
        agent_rank, method = global_rank + rank_offset, "offset"
    command_queue_path, state_path = (path_naming_fn or default_path_naming)(agent_rank)
    client = TensorBusClient(agent_rank=agent_rank, lmdb_command_queue_path=command_queue_path,
                             agent_state_lmdb_path=state_path, connection_timeout=connection_timeout)
    info = BootstrapInfo(agent_rank=agent_rank, global_rank=global_rank, rank_offset=rank_offset,
                         command_queue_path=command_queue_path, state_path=state_path, method=method)
    return client, info
