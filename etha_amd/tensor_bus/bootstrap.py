"""Worker-side bootstrap (``src/etha/tensor_bus/bootstrap.py``): resolve the agent rank from the
environment, derive the two paths, create the client."""

from __future__ import annotations

import ctypes
import errno
import logging
import os
from collections.abc import Callable
from dataclasses import dataclass

from .agent import default_path_naming
from .client import TensorBusClient

logger = logging.getLogger(__name__)


def setup_ptrace() -> None:
    """Allow another process (the agent) to open this process's device allocations."""
    PR_SET_PTRACER = 0x59616D61
    pr_set_ptracer_any = ctypes.c_ulong(-1)  # (unsigned long)-1: a plain -1 would travel as a 32-bit int
    libc = ctypes.CDLL("libc.so.6", use_errno=True)
    libc.prctl.argtypes = [ctypes.c_int, ctypes.c_ulong, ctypes.c_ulong, ctypes.c_ulong, ctypes.c_ulong]
    if libc.prctl(PR_SET_PTRACER, pr_set_ptracer_any, 0, 0, 0) != 0:
        err = ctypes.get_errno()
        if err == errno.EINVAL:
            # a kernel without the Yama module does not know the option: there is no ptrace restriction to lift,
            # and another process can open this one's allocations anyway
            logger.info("[Bootstrap] prctl(PR_SET_PTRACER) is not known to this kernel (no ptrace restriction to lift)")
        else:
            logger.warning("[Bootstrap] prctl(PR_SET_PTRACER, ANY) failed: errno %d (%s)", err, os.strerror(err))


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
