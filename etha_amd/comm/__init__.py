"""Planner + executor of the redistribute path (same public names as ``etha.comm``)."""

from .comm_methods import TransferPlan, bucket_comm
from .get_buckets import chunk_to_bucket_ops
from .get_chunks import m2m_to_chunks
from .get_m2m_map import get_m2m_map
from .ir import Bucket, Chunk, Endpoint, M2MMap, PartialGroup, Route
from .loopback import LoopbackWire, default_wire, reset_default_wire
from .transfer import Transport

__all__ = [
    "get_m2m_map",
    "m2m_to_chunks",
    "chunk_to_bucket_ops",
    "bucket_comm",
    "TransferPlan",
    "Bucket",
    "Chunk",
    "Endpoint",
    "M2MMap",
    "PartialGroup",
    "Route",
    "Transport",
    "LoopbackWire",
    "default_wire",
    "reset_default_wire",
]
