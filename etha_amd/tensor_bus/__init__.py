"""Tensor bus: the worker-facing API (same public names as ``etha.tensor_bus``)."""

from .agent import BatchState, PairState, TensorBusAgent
from .bootstrap import BootstrapInfo, bootstrap_client
from .client import BatchHandler, TensorBusClient
from .command_queue import CommandQueue
from .commands import CleanupBatch, InitPair, Message, QueryStatus, RegisterTensors, Transfer

__all__ = [
    "Message", "Transfer", "InitPair", "RegisterTensors", "QueryStatus", "CleanupBatch", "PairState",
    "BatchState", "CommandQueue", "TensorBusAgent", "TensorBusClient", "BatchHandler", "bootstrap_client",
    "BootstrapInfo",
]
