"""The agent side of the tensor bus, as one hub process for all ranks of one GPU.

In the reference every rank runs its own ``TensorBusAgent`` process inside a torchrun world and the
agents rendezvous through a KV store and NCCL (``src/etha/tensor_bus/agent.py``).  That control plane
is outside this build.  What the hot path needs from it is kept, in one process that plays every
agent rank of the GPU:

* one command queue and one state/heartbeat file per agent rank (``bootstrap.py:105-106`` naming);
* ``InitPair``: a pair matches when ``expected_world_size`` ranks of both sides have registered;
  meshes are rebuilt as ``arange`` from each side's first rank and the M2M map is planned in both
  directions, skipping a direction whose target is Partial (``agent.py:203-436``);
* ``RegisterTensors``: tensors arrive as hipIPC handles; a rank is planned once every pair it named
  is complete in the batch (all ranks of both sides have registered tensors for it): chunks and
  buckets with the transfer-dtype rule (``agent.py:543-687``), compiled into device tile programs;
* ``Transfer``: runs that rank's send or recv buckets through the HIP path (``agent.py:438-507``).
  The reference brackets a transfer with barriers over both sides; here a send waits until its
  previous generation has been consumed and a recv waits for its sources' sends, which gives the
  same lock step.  The sends of the members of a Partial reduction form a collective (the primary's
  kernel reads every member's tensor), and a send whose tensors are lent to the receivers completes
  only after they have run.  Commands that are ready are handled in one sweep: enqueue every launch,
  synchronise the device once, publish state once, reply;
* ``QueryStatus`` (``transfer_signal``) and ``CleanupBatch``.

A failing command is reported back to the worker as an exception of the same type; the reference
logs it, releases the semaphore and lets the agent die (``agent.py:196-201``).
"""

from __future__ import annotations

import json
import logging
import os
import threading
import time
from dataclasses import dataclass, field
from multiprocessing.connection import wait as mp_wait

import numpy as np
import torch
from torch.distributed.tensor.placement_types import Partial

from ..comm import LoopbackWire, bucket_comm, chunk_to_bucket_ops, get_m2m_map, m2m_to_chunks
from ..comm.transfer import Transport
from ..world import create_partial_groups, transfer_dtype_rule
from .command_queue import CommandQueue
from .commands import CleanupBatch, InitPair, QueryStatus, RegisterTensors, Transfer
from .ipc_tensor import IpcTensor, import_tensor

logger = logging.getLogger(__name__)


def default_path_naming(rank: int) -> tuple[str, str]:
    return f"/tmp/agent_rank{rank}_command.lmdb", f"/tmp/agent_rank{rank}_state.lmdb"


@dataclass
class PairState:
    pair_name: str
    sides: dict = field(default_factory=dict)  # name -> {"expected": n, "ranks": {rank: (mesh_shape, placements)}}
    matched: bool = False
    ranks: dict = field(default_factory=dict)  # name -> sorted ranks
    meshes: dict = field(default_factory=dict)  # name -> (mesh ndarray, placements)
    m2m: dict = field(default_factory=dict)  # (source name, target name) -> M2MMap | None


@dataclass
class BatchState:
    batch_id: str
    pair_names: list[str]
    bucket_size: int | None
    registrations: dict = field(default_factory=dict)  # rank -> [(pair_name, tensor)]
    planned_ranks: set = field(default_factory=set)  # ranks whose bucket lists exist
    send_compiled: set = field(default_factory=set)  # ranks whose send / receive tile programs exist
    recv_compiled: set = field(default_factory=set)
    send_buckets: dict = field(default_factory=dict)
    recv_buckets: dict = field(default_factory=dict)
    send_count: dict = field(default_factory=dict)
    siblings: dict = field(default_factory=dict)  # (kind, rank) -> (senders, receivers) of that rank's transfer
    recv_count: dict = field(default_factory=dict)
    owed: dict = field(default_factory=dict)  # destination rank -> number of receives its sources have asked of it
    send_arrived: dict = field(default_factory=dict)  # rank -> number of send commands it has issued so far
    partial_members: dict = field(default_factory=dict)  # rank -> other ranks of its Partial reductions (cached)
    transfer_signal: bool = False


@dataclass
class _Entry:
    rank: int
    conn: object
    command: object
    started: bool = False
    result: object = None


class TensorBusAgent:
    """Hub agent: serves ``world_size`` agent ranks on one device."""

    def __init__(self, world_size: int, path_naming_fn=None, device: str | torch.device = "cuda:0",
                 heartbeat_interval: float = 0.2, zero_copy_single_chunk: bool = False,
                 direct_same_device: bool = False, pool: str = "ring", max_in_flight: int = 2,
                 gather_window: float = 0.001):
        self.world_size = world_size
        # The ranks of a batch issue their transfer commands together (the reference brackets a transfer with a
        # barrier over all of them, agent.py:457).  When the first one arrives the agent waits up to this long for
        # the others, so that it can queue every rank's pipeline in rank order and step them in one go: the same
        # sequence every transfer, which the wire then serves from its recording (LoopbackWire.replay_schedules).
        self.gather_window = gather_window
        self.device = torch.device(device)
        self.path_naming_fn = path_naming_fn or default_path_naming
        self.heartbeat_interval = heartbeat_interval
        # bucket buffers: a ring of max_in_flight slots per channel (the reference's bound, comm_methods.py:53-119),
        # or pool="resident" for a slot per bucket
        self.wire = LoopbackWire(self.device if self.device.type == "cuda" else None, pool=pool, max_in_flight=max_in_flight)
        # lent buckets are read from the worker's tensor at receive time, so a send that lends memory only
        # completes once its receivers have unpacked (the reference's transfers end with a barrier as well)
        self.wire.zero_copy_single_chunk = zero_copy_single_chunk
        # no bucket buffers for plain buckets: a recv copies straight from the sending worker's tensors
        self.wire.direct_same_device = direct_same_device
        self.pairs: dict[str, PairState] = {}
        self.batches: dict[str, BatchState] = {}
        self._opened: list = []  # (rank, connection) accepted, command not read yet
        self._rank_of_queue: dict[int, int] = {}
        self._pending: list[_Entry] = []
        self._stop = threading.Event()
        self._queues: dict[int, CommandQueue] = {}
        self._state_paths: dict[int, str] = {}
        self._last_heartbeat = 0.0
        self._last_core: dict | None = None
        self._moved = False  # set by a command that changed shared state without completing
        self._unsynced: list[tuple[dict, float, str]] = []  # (result, start time, label) of transfers enqueued, not yet synchronised
        self._queued = False  # pipelines were queued on the wire in this pass and have not been stepped yet
        self.stats = {"ipc_tensors": 0, "in_process_tensors": 0, "transfers": 0}
        # host time of the passes that launched transfers, in ms: waiting for the other ranks' commands, walking the
        # commands and issuing launches, waiting for the device, publishing state and replying
        self.timing = {"passes": 0, "gather_ms": 0.0, "issue_ms": 0.0, "device_ms": 0.0, "reply_ms": 0.0}
        for rank in range(world_size):
            cmd_path, state_path = self.path_naming_fn(rank)
            self._queues[rank] = CommandQueue(cmd_path, serve=True)
            self._rank_of_queue[id(self._queues[rank])] = rank
            self._state_paths[rank] = state_path
        self._write_state(force=True)

    # ---- plumbing ---------------------------------------------------------------------------
    def _receive(self, timeout: float) -> int:
        """Wait up to ``timeout`` for commands on any rank's socket and append what has arrived to the pending list;
        returns how many.  One thread waits on every socket: ten ranks that issue their commands together are taken
        in one go, without a hand-over between threads per command."""
        opened = list(self._opened)
        try:
            ready = mp_wait(list(self._queues.values()) + [c for _, c in opened], timeout)
        except OSError:  # a socket was closed under the wait (close() from another thread)
            return 0
        got = 0
        for obj in ready:
            if isinstance(obj, CommandQueue):
                rank = self._rank_of_queue[id(obj)]
                for conn in obj.accept_ready():
                    self._opened.append((rank, conn))
        # a worker sends its command right after connecting: most new connections can be read at once
        for item in list(self._opened):
            rank, conn = item
            try:
                if not conn.poll(0):
                    continue
                command = conn.recv()
            except (EOFError, OSError):
                self._opened.remove(item)
                conn.close()
                continue
            self._opened.remove(item)
            self._pending.append(_Entry(rank=rank, conn=conn, command=command))
            got += 1
        return got

    def _write_state(self, force: bool = False) -> None:
        """Publish heartbeat and pair/batch state.  ``force`` asks for the current state to be visible on
        return; files are rewritten only if the state differs from what they hold or the heartbeat is due."""
        now = time.time()
        core = {
            "pairs": {name: ("matched" if p.matched else "pending") for name, p in self.pairs.items()},
            "batches": {bid: {"transfer_signal": b.transfer_signal} for bid, b in self.batches.items()},
        }
        due = now - self._last_heartbeat >= self.heartbeat_interval
        if not due and (not force or core == self._last_core):
            return
        self._last_heartbeat = now
        self._last_core = core
        blob = json.dumps({"agent:heartbeat": now, **core})
        for path in self._state_paths.values():
            tmp = f"{path}.tmp{os.getpid()}"
            with open(tmp, "w") as f:
                f.write(blob)
            os.replace(tmp, path)

    def run(self) -> None:
        """Serve until :meth:`close` is called (the reference's ``TensorBusAgent.run``)."""
        while not self._stop.is_set():
            self.step(0.02)

    def start_in_thread(self) -> threading.Thread:
        t = threading.Thread(target=self.run, daemon=True, name="etha-agent")
        self._serve_thread = t
        t.start()
        return t

    def step(self, timeout: float = 0.0) -> None:
        self._write_state()
        self._receive(timeout)
        # ranks of one batch issue their commands from threads that take turns: wait while commands keep coming
        # (the window restarts at every arrival), but never longer than eight windows in all
        start = time.perf_counter()
        deadline, limit = start + self.gather_window, start + 8 * self.gather_window
        while self._siblings_missing():
            left = min(deadline, limit) - time.perf_counter()
            if left <= 0:
                break
            if self._receive(left):
                deadline = time.perf_counter() + self.gather_window
        # Sweep until nothing moves.  Commands that complete are answered only after the sweep: the device
        # work of every transfer that became ready is enqueued first, then the stream is synchronised once
        # and the state files are written once, instead of once per rank.
        finished: list[tuple[_Entry, tuple]] = []
        progressed = True
        t_gathered = time.perf_counter()
        while progressed:
            progressed, self._moved = False, False
            for entry in self._in_rank_order(self._pending):
                try:
                    done, value = self._advance(entry)
                except Exception as e:  # report to the worker, keep serving
                    logger.exception("agent rank %s: %s failed", entry.rank, type(entry.command).__name__)
                    finished.append((entry, ("error", (type(e).__name__, str(e)))))
                    self._pending.remove(entry)
                    progressed = True
                    continue
                if done:
                    finished.append((entry, ("ok", value)))
                    self._pending.remove(entry)
                    progressed = True
            if self._queued:  # every pipeline queued in this pass is stepped now, together
                self._queued = False
                self.wire.drive()
                progressed = True
            # a command that changed shared state without completing (a send that lends its tensors and now
            # waits for its receivers) may have unblocked commands examined earlier in this pass
            progressed = progressed or self._moved
        timed = bool(self._unsynced)
        t_issued = time.perf_counter()
        if self._unsynced:
            # a worker may overwrite its tensors as soon as its send returns, and read them as soon as its
            # recv returns: both replies wait for the device
            if self.device.type == "cuda":
                torch.cuda.current_stream(self.device).synchronize()
            now = time.perf_counter()
            for result, t0, label in self._unsynced:
                result["ms"] = (now - t0) * 1e3
                logger.info("%s: %.3f ms (enqueue to device completion)", label, result["ms"])
            self._unsynced.clear()
        if finished:
            # the state file must show the new state before a worker is released
            self._write_state(force=True)
            for entry, message in finished:
                self._reply(entry, message)
        if timed:
            t_end = time.perf_counter()
            self.timing["passes"] += 1
            self.timing["gather_ms"] += (t_gathered - start) * 1e3
            self.timing["issue_ms"] += (t_issued - t_gathered) * 1e3
            self.timing["device_ms"] += (now - t_issued) * 1e3
            self.timing["reply_ms"] += (t_end - now) * 1e3

    @staticmethod
    def _in_rank_order(pending: list) -> list:
        """Commands in arrival order, except that the transfer commands among them are taken batch by batch, sends
        before receives, ranks ascending - whichever order their threads happened to deliver them in."""
        transfers = sorted((e for e in pending if isinstance(e.command, Transfer)),
                           key=lambda e: (e.command.batch_id, e.command.transfer_type != "send", e.rank))
        return [e for e in pending if not isinstance(e.command, Transfer)] + transfers

    def _ranks_of_transfer(self, batch: BatchState, kind: str, rank: int) -> tuple[frozenset, frozenset]:
        """(senders, receivers) of the transfer that ``rank``'s command of ``kind`` belongs to: the ranks its buckets
        go to or come from, their other sources, the members of Partial sources, and so on until nothing is added.
        A batch plans both directions of its pairs; the opposite direction is a different transfer."""
        key = (kind, rank)
        if key not in batch.siblings:
            senders, receivers = ({rank}, set()) if kind == "send" else (set(), {rank})
            grown = True
            while grown:
                before = len(senders) + len(receivers)
                for s in list(senders):
                    receivers |= self._peers(batch.send_buckets.get(s) or (), "dst")
                    senders |= self._partial_members(batch, s)
                for d in list(receivers):
                    senders |= self._peers(batch.recv_buckets.get(d) or (), "src")
                grown = len(senders) + len(receivers) != before
            batch.siblings[key] = (frozenset(senders), frozenset(receivers))
        return batch.siblings[key]

    def _siblings_missing(self) -> bool:
        """True while some rank has issued a transfer command that is not under way yet and another rank of the same
        transfer has not issued its command of that generation (a rank that both sends and receives counts as
        present with either command: it issues them one after the other)."""
        waiting: dict = {}
        for e in self._pending:
            if isinstance(e.command, Transfer) and not e.started:
                waiting.setdefault(e.command.batch_id, []).append((e.command.transfer_type, e.rank))
        for batch_id, entries in waiting.items():
            batch = self.batches.get(batch_id)
            if batch is None:
                continue
            present = {r for _, r in entries}
            for kind, rank in entries:
                if rank not in batch.planned_ranks:
                    continue
                gen = (batch.send_count if kind == "send" else batch.recv_count).get(rank, 0)
                senders, receivers = self._ranks_of_transfer(batch, kind, rank)
                if any(r not in present and batch.send_count.get(r, 0) <= gen for r in senders):
                    return True
                if any(r not in present and batch.recv_count.get(r, 0) <= gen for r in receivers):
                    return True
        return False

    @staticmethod
    def _reply(entry: _Entry, message) -> None:
        try:
            entry.conn.send(message)
        except (OSError, BrokenPipeError):
            pass
        finally:
            try:
                entry.conn.close()
            except OSError:
                pass

    def close(self) -> None:
        self._stop.set()
        serving = getattr(self, "_serve_thread", None)
        if serving is not None and serving is not threading.current_thread():
            serving.join(timeout=5.0)  # let the current sweep finish before its plans are released
        for q in self._queues.values():
            q.close()
        for b in list(self.batches.values()):
            self._release_batch(b)
        self.batches.clear()
        for path in self._state_paths.values():
            if os.path.exists(path):
                os.unlink(path)

    # ---- commands ---------------------------------------------------------------------------
    def _advance(self, entry: _Entry):
        cmd = entry.command
        if isinstance(cmd, InitPair):
            return self._init_pair(entry, cmd)
        if isinstance(cmd, RegisterTensors):
            return self._register_tensors(entry, cmd)
        if isinstance(cmd, Transfer):
            return self._transfer(entry, cmd)
        if isinstance(cmd, QueryStatus):
            batch = self.batches.get(cmd.batch_id)
            if batch is None or cmd.state_name != "transfer_signal":
                return True, False
            return True, batch.transfer_signal
        if isinstance(cmd, CleanupBatch):
            batch = self.batches.get(cmd.batch_id)
            if batch is not None:
                # this rank is done with the batch (its transfers have returned, so the device has been
                # synchronised since): drop its plans, then the mappings of its tensors
                self._release_rank(batch, entry.rank)
                if not batch.registrations:
                    self._release_batch(batch)
                    del self.batches[cmd.batch_id]
            return True, None
        raise ValueError(f"unknown command {type(cmd).__name__}")

    def _init_pair(self, entry: _Entry, cmd: InitPair):
        pair = self.pairs.setdefault(cmd.pair_name, PairState(pair_name=cmd.pair_name))
        if not entry.started:
            entry.started = True
            side = pair.sides.setdefault(cmd.local_name, {"expected": cmd.expected_world_size, "ranks": {}, "remote": cmd.remote_name})
            if side["expected"] != cmd.expected_world_size:
                raise ValueError(f"pair {cmd.pair_name}: ranks of '{cmd.local_name}' disagree on expected_world_size")
            side["ranks"][entry.rank] = (cmd.mesh_shape_payload, cmd.placements_payload)
        if pair.matched:
            return True, "matched"
        local, remote = pair.sides.get(cmd.local_name), pair.sides.get(cmd.remote_name)
        if local is None or remote is None:
            return False, None
        if len(local["ranks"]) < local["expected"] or len(remote["ranks"]) < remote["expected"]:
            return False, None
        self._match_pair(pair)
        return True, "matched"

    def _match_pair(self, pair: PairState) -> None:
        for name, side in pair.sides.items():
            infos = list(side["ranks"].values())
            if any(i != infos[0] for i in infos):
                raise ValueError(f"pair {pair.pair_name}: ranks of '{name}' disagree on mesh shape or placements")
            ranks = sorted(side["ranks"])
            pair.ranks[name] = ranks
            mesh_shape, placements = infos[0]
            if mesh_shape is not None and placements is not None:
                n = int(np.prod(mesh_shape))
                if n != len(ranks):
                    raise ValueError(f"pair {pair.pair_name}: mesh {mesh_shape} does not hold {len(ranks)} ranks")
                # same rebuild as the reference: consecutive ranks from the side's first rank
                pair.meshes[name] = (np.arange(ranks[0], ranks[0] + n).reshape(mesh_shape), tuple(placements))
        names = sorted(pair.sides)
        if len(names) == 2 and all(n in pair.meshes for n in names):
            for a, b in ((names[0], names[1]), (names[1], names[0])):
                (mesh_a, pl_a), (mesh_b, pl_b) = pair.meshes[a], pair.meshes[b]
                if any(isinstance(p, Partial) for p in pl_b):
                    pair.m2m[(a, b)] = None  # a Partial target is not supported: that direction is skipped
                else:
                    pair.m2m[(a, b)] = get_m2m_map(mesh_a, pl_a, mesh_b, pl_b)
        pair.matched = True

    def _side_of(self, pair: PairState, rank: int) -> str:
        for name, ranks in pair.ranks.items():
            if rank in ranks:
                return name
        raise ValueError(f"rank {rank} is not part of pair {pair.pair_name}")

    def _register_tensors(self, entry: _Entry, cmd: RegisterTensors):
        if not entry.started:
            entry.started = True
            pair_names = list(dict.fromkeys(p for p, _ in cmd.tensors))
            for p in pair_names:
                if p not in self.pairs or not self.pairs[p].matched:
                    raise ValueError(f"RegisterTensors for unknown pair: {p}")
                self._side_of(self.pairs[p], entry.rank)  # raises if the rank is not part of the pair
            batch = self.batches.setdefault(cmd.batch_id, BatchState(cmd.batch_id, [], cmd.bucket_size))
            if entry.rank in batch.registrations:
                raise ValueError(f"batch {cmd.batch_id} is already registered by rank {entry.rank}")
            for p in pair_names:
                if p not in batch.pair_names:
                    batch.pair_names.append(p)
            index = self.device.index if self.device.type == "cuda" else None
            batch.registrations[entry.rank] = [(p, import_tensor(payload, index)) for p, payload in cmd.tensors]
            for _, t in batch.registrations[entry.rank]:
                self.stats["ipc_tensors" if isinstance(t, IpcTensor) else "in_process_tensors"] += 1
            self._plan_ready_ranks(batch)
        batch = self.batches[cmd.batch_id]
        return (True, None) if entry.rank in batch.planned_ranks else (False, None)

    def _pair_complete(self, batch: BatchState, pair_name: str) -> bool:
        """Has every rank of the pair registered tensors for it in this batch?"""
        pair = self.pairs[pair_name]
        return all(r in batch.registrations and any(p == pair_name for p, _ in batch.registrations[r])
                   for ranks in pair.ranks.values() for r in ranks)

    def _plan_ready_ranks(self, batch: BatchState) -> None:
        """Plan every registered rank whose pairs have all become complete (each rank is planned once; ranks of
        one batch may take part in different pairs, as each rank's own agent would plan only its own pairs)."""
        for rank in sorted(batch.registrations):
            if rank in batch.planned_ranks:
                continue
            mine = list(dict.fromkeys(p for p, _ in batch.registrations[rank]))
            if all(self._pair_complete(batch, p) for p in mine):
                self._plan_rank(batch, rank, mine)
                batch.planned_ranks.add(rank)
                batch.siblings.clear()
        # tile programs: a receive list pairs with send lists, so it is compiled once all its sources' lists are
        for rank in sorted(batch.planned_ranks - batch.send_compiled):
            self._plan_if_device(batch.send_buckets.get(rank), batch.batch_id)
            batch.send_compiled.add(rank)
        for rank in sorted(batch.planned_ranks - batch.recv_compiled):
            buckets = batch.recv_buckets.get(rank)
            if all(s in batch.send_compiled for s in self._peers(buckets or [], "src")):
                self._plan_if_device(buckets, batch.batch_id)
                batch.recv_compiled.add(rank)

    def _plan_rank(self, batch: BatchState, rank: int, pair_names: list[str]) -> None:
        send_chunks: list = []
        recv_chunks: list = []
        for pair_name in pair_names:
            pair = self.pairs[pair_name]
            per_rank = {r: [t for p, t in regs if p == pair_name] for r, regs in batch.registrations.items()}
            names = sorted(pair.sides)
            counts = {len(per_rank[r]) for name in names for r in pair.ranks[name]}
            if len(counts) != 1:
                raise ValueError(f"batch {batch.batch_id}: ranks registered different numbers of tensors for '{pair_name}'")
            for i in range(counts.pop()):
                for a, b in ((names[0], names[1]), (names[1], names[0])):
                    m2m = pair.m2m.get((a, b))
                    if m2m is None:
                        continue
                    src = {r: per_rank[r][i] for r in pair.ranks[a]}
                    tgt = {r: per_rank[r][i] for r in pair.ranks[b]}
                    wire_dtype = transfer_dtype_rule(next(iter(src.values())).dtype, next(iter(tgt.values())).dtype)
                    if rank in src:
                        groups = create_partial_groups(pair.meshes[a][0], m2m.source_partial_reductions, rank, src) or None
                        send_chunks.extend(m2m_to_chunks(m2m, rank, source_tensor=src[rank], transfer_dtype=wire_dtype,
                                                         source_partial_groups=groups))
                    if rank in tgt:
                        recv_chunks.extend(m2m_to_chunks(m2m, rank, target_tensor=tgt[rank], transfer_dtype=wire_dtype))
        size = batch.bucket_size or 1
        batch.send_buckets[rank] = chunk_to_bucket_ops(send_chunks, size)
        batch.recv_buckets[rank] = chunk_to_bucket_ops(recv_chunks, size)
        batch.send_count[rank] = 0
        batch.recv_count[rank] = 0

    def _plan_if_device(self, buckets, scope) -> None:
        if buckets and buckets[0].chunks[0].tensor.device.type == "cuda":
            self.wire.plan(buckets, scope=scope)

    @staticmethod
    def _partial_members(batch: BatchState, rank: int) -> set[int]:
        """The other ranks whose tensors this rank's send reads, or whose sends read this rank's tensors."""
        if rank not in batch.partial_members:
            members: set[int] = set()
            for b in batch.send_buckets.get(rank, []):
                for c in b.chunks:
                    for group, _ in c.source_partial_groups or ():
                        members.update(int(r) for r in group.ranks)
            members.discard(rank)
            batch.partial_members[rank] = members
        return batch.partial_members[rank]

    @staticmethod
    def _peers(buckets, attr: str) -> set[int]:
        out: set[int] = set()
        for b in buckets:
            if b.transport in (Transport.P2P, Transport.BROADCAST):
                out.update(b.dst_ranks if attr == "dst" else (b.src_rank,))
        return out

    def _transfer(self, entry: _Entry, cmd: Transfer):
        batch = self.batches.get(cmd.batch_id)
        if batch is None:
            raise ValueError(f"Transfer for unknown batch: {cmd.batch_id}")
        rank = entry.rank
        if rank not in batch.planned_ranks:
            return False, None
        table = batch.send_buckets if cmd.transfer_type == "send" else batch.recv_buckets
        other = batch.recv_buckets if cmd.transfer_type == "send" else batch.send_buckets
        buckets = table.get(rank)
        if not buckets:
            if any(other.values()) or any(table.values()):
                raise RuntimeError(
                    f"Batch {cmd.batch_id}: no {cmd.transfer_type} chunks. The pair's {cmd.transfer_type} direction "
                    "has a Partial target, which is not supported. Partial is only valid as a source placement."
                )
            return True, None
        if cmd.transfer_type == "send":
            members = self._partial_members(batch, rank)
            if not entry.started:
                gen = batch.send_count[rank]
                for d in self._peers(buckets, "dst"):
                    if d in batch.recv_count and batch.recv_count[d] < gen:
                        return False, None  # the previous generation has not been consumed yet
                if batch.send_arrived.get(rank, 0) <= gen:
                    batch.send_arrived[rank] = gen + 1
                    self._moved = True
                # A Partial source is a collective among its members, as the all-reduce is in the reference:
                # the primary's reduce reads every member's tensor, so it starts only once all of them have
                # called send for this generation ...
                if any(batch.send_arrived.get(m, 0) <= gen for m in members):
                    return False, None
                batch.transfer_signal = True
                entry.result = {"ms": 0.0}
                self._unsynced.append((entry.result, time.perf_counter(), f"batch {cmd.batch_id} rank {rank} send #{gen}"))
                bucket_comm(buckets, wire=self.wire, merge_launches=True, synchronize=False, scope=batch.batch_id, drive=False)
                self._queued = True
                batch.send_count[rank] = gen + 1
                for d in self._peers(buckets, "dst"):
                    batch.owed[d] = max(batch.owed.get(d, 0), gen + 1)
                entry.started = True
                self._moved = True
                self.stats["transfers"] += 1
            done_gen = batch.send_count[rank]
            # ... and no member's send returns before every member's launch is enqueued (the sweep synchronises
            # the device before it replies), because a member's tensor is read by another member's kernel
            if any(batch.send_count.get(m, 0) < done_gen for m in members):
                return False, None
            # with a ring pool a send has only packed as far as its slots reach; the rest follows as its receivers
            # unpack, so it completes with them - as a sender's bucket_comm does in the reference
            if self.wire.in_progress(buckets):
                return False, None
            # a send whose tensors are lent to receivers - its own buckets, or a Partial reduction that another
            # member ships and the receiver computes - waits for those receivers to have run
            for m in members | {rank}:
                theirs = batch.send_buckets.get(m)
                if theirs and self.wire.plan(theirs).lends_tensor_memory() and not all(
                        batch.recv_count.get(d, done_gen) >= done_gen for d in self._peers(theirs, "dst")):
                    return False, None
            return True, entry.result
        else:
            gen = batch.recv_count[rank]
            for s in self._peers(buckets, "src"):
                if batch.send_count.get(s, 0) <= gen:
                    return False, None  # wait for the source's send of this generation
            result = {"ms": 0.0}
            self._unsynced.append((result, time.perf_counter(), f"batch {cmd.batch_id} rank {rank} recv #{gen}"))
            bucket_comm(buckets, wire=self.wire, merge_launches=True, synchronize=False, scope=batch.batch_id, drive=False)
            self._queued = True
            batch.recv_count[rank] = gen + 1
            if all(batch.recv_count.get(d, 0) >= n for d, n in batch.owed.items()):
                batch.transfer_signal = False  # every destination of every send so far has received
        self.stats["transfers"] += 1
        return True, result

    def _release_rank(self, batch: BatchState, rank: int) -> None:
        """Forget one rank of a batch: its compiled bucket lists (receive side first: it only references slots
        that send lists own) and the hipIPC mappings of the tensors it registered."""
        for table in (batch.recv_buckets, batch.send_buckets):
            buckets = table.pop(rank, None)
            if buckets:
                self.wire.release(buckets)
        for _, t in batch.registrations.pop(rank, ()):
            if isinstance(t, IpcTensor):
                try:
                    t.close()
                except Exception:
                    logger.exception("closing an IPC mapping failed")
        batch.planned_ranks.discard(rank)
        batch.siblings.clear()

    def _release_batch(self, batch: BatchState) -> None:
        # receivers first: their plans only reference slots, the senders' plans own them
        for buckets in list(batch.recv_buckets.values()) + list(batch.send_buckets.values()):
            self.wire.release(buckets)
        for regs in batch.registrations.values():
            for _, t in regs:
                if isinstance(t, IpcTensor):
                    try:
                        t.close()
                    except Exception:
                        logger.exception("closing an IPC mapping failed")
        batch.registrations.clear()
        batch.send_buckets.clear()
        batch.recv_buckets.clear()
