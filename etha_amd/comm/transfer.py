"""Transport kinds of a chunk.

Mirrors the ``Transport`` enum of the reference (``src/etha/comm/transfer.py:11-17``).  The wire
operations themselves (``isend/irecv/broadcast``, ``transfer.py:20-41``) are replaced by the
same-GPU loopback in :mod:`etha_amd.comm.loopback`.
"""

from enum import Enum


class Transport(Enum):
    """How a chunk's bytes cross ranks (independent of its produce/consume role)."""

    P2P = "p2p"
    BROADCAST = "broadcast"
    LOCAL = "local"  # source and target live on the same rank: direct copy, no wire
    NONE = "none"  # reduce-only member of a Partial group: contributes, ships nothing
