"""A replica-group cluster inside one process: quorum service and process group for
replicas that run as threads and share one GPU.

The reference tests its fault-tolerance logic "multi-node without a cluster": a real
(Rust) lighthouse in-process, one thread per replica group, Gloo over localhost
(torchft/manager_integ_test.py:340-665).  Neither the Rust servers nor a network
backend are rebuilt here.  This module gives the same experiment its two missing
pieces for the one-GPU setting:

* :class:`InProcessLighthouse` - decides quorums for the replicas that are currently
  alive and answers like the reference's lighthouse + manager server pair
  (``src/lighthouse.rs`` quorum formation reduced to "every live replica has asked and
  there are at least ``min_replicas``"; the per-replica answer follows
  ``compute_quorum_results``, src/manager.rs:357-480: ranks by sorted replica id,
  max-step cohort, round-robin recovery assignment, initial sync from the primary at
  step 0).  Its per-replica :meth:`client` objects sit in the Manager's
  ``quorum_client`` seat.
* :class:`ProcessGroupThreads` - ``allreduce`` among the thread-replicas of the current
  quorum: every rank deposits its tensor and gets a future, the last one to arrive runs
  ONE reduction kernel over all of them plus one copy launch that writes the result back
  into every rank's tensor.  The Manager's time-out turns a dead peer into an error
  instead of a hang.
"""

from __future__ import annotations

import threading
import time
from dataclasses import dataclass
from datetime import timedelta
from typing import Dict, List, Optional, Tuple

import torch
from torch.distributed import ReduceOp
from torch.distributed.distributed_c10d import AllreduceOptions, Work

from . import ops
from .manager import QuorumClient, QuorumResult
from .process_group import ProcessGroup, _DummyWork


@dataclass
class _Member:
    replica_id: str
    step: int
    metadata: str


@dataclass
class _Quorum:
    quorum_id: int
    members: List[_Member]


def compute_quorum_result(replica_id: str, rank: int, quorum: _Quorum) -> QuorumResult:
    """One replica's view of a quorum (src/manager.rs:357-480)."""
    members = sorted(quorum.members, key=lambda m: m.replica_id)
    ids = [m.replica_id for m in members]
    if replica_id not in ids:
        raise KeyError(f"replica {replica_id} not participating in returned quorum")
    replica_rank = ids.index(replica_id)
    max_step = max(m.step for m in members)
    at_max = [m for m in members if m.step == max_step]
    max_ids = [m.replica_id for m in at_max]
    max_rank = max_ids.index(replica_id) if replica_id in max_ids else None
    primary = at_max[rank % len(at_max)]
    # recovering: behind the newest step, or - before the first step - everyone but the primary
    recovering = [
        i for i, m in enumerate(members)
        if m.step != max_step or (max_step == 0 and m.replica_id != primary.replica_id)
    ]
    up_to_date = [i for i in range(len(members)) if i not in set(recovering)]
    assignments: Dict[int, List[int]] = {}
    recover_src_rank: Optional[int] = None
    for i, dst in enumerate(recovering):
        src = up_to_date[(i + rank) % len(up_to_date)]
        assignments.setdefault(src, []).append(dst)
        if dst == replica_rank:
            recover_src_rank = src
    return QuorumResult(
        quorum_id=quorum.quorum_id,
        replica_rank=replica_rank,
        replica_world_size=len(members),
        recover_src_manager_address=(
            members[recover_src_rank].replica_id if recover_src_rank is not None else ""
        ),
        recover_src_rank=recover_src_rank,
        recover_dst_ranks=assignments.get(replica_rank, []),
        store_address=f"inprocess/{primary.replica_id}",
        max_step=max_step,
        max_rank=max_rank,
        max_world_size=len(at_max),
        heal=recover_src_rank is not None,
    )


class InProcessLighthouse:
    """Quorum service for replicas living in this process."""

    def __init__(self, min_replicas: int) -> None:
        self.min_replicas = min_replicas
        self._cv = threading.Condition()
        self._alive: Dict[str, bool] = {}
        self._requests: Dict[str, _Member] = {}
        self._metadata: Dict[str, str] = {}
        self._generation = 0
        self._latest: Optional[_Quorum] = None
        self._quorum_id = 0

    def client(self, replica_id: str) -> "LighthouseClient":
        with self._cv:
            self._alive[replica_id] = True
            self._cv.notify_all()
        return LighthouseClient(self, replica_id)

    def leave(self, replica_id: str) -> None:
        """A replica that dies (or shuts down) stops counting towards quorums."""
        with self._cv:
            self._alive.pop(replica_id, None)
            self._requests.pop(replica_id, None)
            self._try_form()
            self._cv.notify_all()

    def _try_form(self) -> None:
        alive = set(self._alive)
        if len(alive) < self.min_replicas or not alive.issubset(self._requests):
            return
        members = [self._requests[r] for r in sorted(alive)]
        # Every quorum gets a fresh id, so the Manager re-configures its process group for
        # every step.  In-process that costs nothing, and it keeps the collectives of
        # different steps apart even after a step in which some replica skipped its
        # all-reduces because of an error.
        self._quorum_id += 1
        self._latest = _Quorum(self._quorum_id, members)
        self._requests.clear()
        self._generation += 1

    def _quorum(self, replica_id: str, rank: int, step: int, metadata: str,
                timeout: timedelta) -> QuorumResult:
        deadline = time.monotonic() + timeout.total_seconds()
        with self._cv:
            self._metadata[replica_id] = metadata
            self._requests[replica_id] = _Member(replica_id, step, metadata)
            wanted = self._generation + 1
            self._try_form()
            self._cv.notify_all()
            while self._generation < wanted:
                left = deadline - time.monotonic()
                if left <= 0 or not self._cv.wait(timeout=left):
                    self._requests.pop(replica_id, None)
                    raise TimeoutError(f"quorum did not form within {timeout}")
                self._try_form()
            assert self._latest is not None
            return compute_quorum_result(replica_id, rank, self._latest)

    def _checkpoint_metadata(self, replica_id: str) -> str:
        with self._cv:
            return self._metadata[replica_id]


class LighthouseClient(QuorumClient):
    """One replica group's connection to the in-process lighthouse (single-rank groups:
    the commit vote of the group is the vote of its only rank, src/manager.rs:295-347)."""

    def __init__(self, lighthouse: InProcessLighthouse, replica_id: str) -> None:
        self._lighthouse = lighthouse
        self.replica_id = replica_id

    def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout) -> QuorumResult:
        return self._lighthouse._quorum(self.replica_id, rank, step, checkpoint_metadata, timeout)

    def should_commit(self, rank, step, should_commit, timeout) -> bool:
        return should_commit

    def checkpoint_metadata(self, address, rank, timeout) -> str:
        return self._lighthouse._checkpoint_metadata(address)

    def leave(self) -> None:
        self._lighthouse.leave(self.replica_id)


# ---------------------------------------------------------------------------
# Process group among threads
# ---------------------------------------------------------------------------


@dataclass
class _Deposit:
    tensor: torch.Tensor
    participating: bool
    divisor: int
    future: torch.futures.Future
    stream: Optional["torch.cuda.Stream"]
    ready: Optional["torch.cuda.Event"]


class _FutureWork(Work):
    def __init__(self, fut: torch.futures.Future) -> None:
        super().__init__()
        self._fut = fut

    def wait(self, timeout: Optional[timedelta] = None) -> bool:
        self._fut.wait()
        return True

    def get_future(self) -> torch.futures.Future:
        return self._fut


class ThreadWorld:
    """Shared rendezvous for the :class:`ProcessGroupThreads` of one process.

    Collectives never block the calling thread: a rank deposits its tensor and gets a
    future; the rank that completes the round runs the reduction and resolves everybody's
    future.  (Blocking would deadlock thread-replicas that share a GPU as soon as the
    call comes from the autograd engine, which runs all backward passes of one device on
    a single thread.)"""

    def __init__(self) -> None:
        self._lock = threading.Lock()
        self._rounds: Dict[Tuple[str, int], Dict[int, _Deposit]] = {}

    def forget(self, epoch: str) -> None:
        """Drops rounds of other epochs that never completed (a replica died mid-step)."""
        with self._lock:
            for key in [k for k in self._rounds if k[0] != epoch]:
                del self._rounds[key]

    def reduce_async(self, key: Tuple[str, int], rank: int, world: int, tensor: torch.Tensor,
                     participating: bool, divisor: int) -> torch.futures.Future:
        """After every rank of ``world`` has deposited, each deposited tensor holds
        (sum of the participating tensors) / divisor and its future resolves."""
        stream = ready = None
        if tensor.is_cuda:
            stream = torch.cuda.current_stream(tensor.device)
            ready = torch.cuda.Event()
            ready.record(stream)
        fut: torch.futures.Future = torch.futures.Future()
        with self._lock:
            rnd = self._rounds.setdefault(key, {})
            rnd[rank] = _Deposit(tensor, participating, divisor, fut, stream, ready)
            if len(rnd) < world:
                return fut
            del self._rounds[key]
        try:
            self._run(rnd, world)
        except BaseException as e:  # every rank of the round sees the failure
            for d in rnd.values():
                d.future.set_exception(e)
        else:
            for d in rnd.values():
                d.future.set_result([d.tensor])
        return fut

    @staticmethod
    def _run(rnd: Dict[int, _Deposit], world: int) -> None:
        ordered = [rnd[r] for r in range(world)]
        first = ordered[0].tensor
        mask = sum(1 << r for r, d in enumerate(ordered) if d.participating)
        mine = torch.cuda.current_stream(first.device) if first.is_cuda else None
        if mine is not None:
            for d in ordered:
                mine.wait_event(d.ready)
        result = torch.empty_like(first)
        ops.reduce_avg_(result, [d.tensor for d in ordered], mask, ordered[0].divisor)
        ops.mt_copy([d.tensor for d in ordered], [result] * world)
        if mine is not None:
            done = torch.cuda.Event()
            done.record(mine)
            for d in ordered:  # whatever a rank enqueues next comes after the result
                d.stream.wait_event(done)


class ProcessGroupThreads(ProcessGroup):
    """``allreduce`` among replicas that are threads of this process (all tensors on one
    GPU).  ``configure`` is called by the Manager with the rank / world size of each new
    quorum; collectives of different quorums never meet because the quorum's store
    address is part of the rendezvous key.  A peer that never shows up leaves the future
    pending; the Manager's timeout turns that into a latched error.

    With torch's DistributedDataParallel the Reducer waits for the hook's future on the
    autograd engine's per-device thread, which all thread-replicas of one GPU share: use
    PureDistributedDataParallel (or CPU tensors, or one process per replica) for DDP
    among thread-replicas of the same GPU."""

    fails_only_at_launch = False

    def __init__(self, world: ThreadWorld) -> None:
        super().__init__(0, 1)
        self._shared = world
        self._rank = 0
        self._size = 1
        self._epoch = ""
        self._seq = 0
        self.configure_count = 0

    def configure(self, store_addr: str, rank: int, world_size: int) -> None:
        self.configure_count += 1
        self._rank, self._size = rank, world_size
        # ".../torchft/<quorum_id>/<local rank>": identical on every replica of the quorum
        self._epoch = store_addr
        self._seq = 0
        self._shared.forget(store_addr)

    def size(self) -> int:
        return self._size

    def getBackendName(self) -> str:
        return "torchft-threads"

    def _collective(self, tensors, participating: bool, divisor: int) -> Work:
        futs = []
        for t in tensors:
            self._seq += 1
            futs.append(self._shared.reduce_async(
                (self._epoch, self._seq), self._rank, self._size, t, participating, divisor))
        if len(futs) == 1:
            return _FutureWork(futs[0])
        return _FutureWork(torch.futures.collect_all(futs).then(lambda _f: list(tensors)))

    def allreduce(self, tensors, opts) -> Work:  # type: ignore[override]
        op = opts.reduceOp if isinstance(opts, AllreduceOptions) else opts
        if op != ReduceOp.SUM:
            raise NotImplementedError(f"only ReduceOp.SUM is supported, got {op}")
        return self._collective(tensors, True, 1)

    def allreduce_avg(self, tensors, participating: bool, num_participants: int) -> Work:
        """Zeroing of non-participants, SUM and division in the one reduction kernel."""
        return self._collective(tensors, participating, num_participants)

    def broadcast(self, tensor_list, opts) -> Work:  # type: ignore[override]
        return _DummyWork(tensor_list)
