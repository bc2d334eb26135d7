"""Manager: the caller contract of the replica-sync path.

The reference's Manager (torchft/manager.py) is mostly control plane: a Rust
gRPC client/server pair, a TCPStore rendezvous and live checkpoint recovery.
None of that is rebuilt here.  What the hot path needs from a Manager is kept
with the reference's names, arguments and error behaviour:

* ``allreduce(tensor) -> Future[tensor]``  (torchft/manager.py:242-303)
* ``num_participants`` / ``is_participating`` / ``WorldSizeMode``
  (torchft/manager.py:55-70, 452-468, 655-679)
* ``start_quorum`` / ``wait_quorum`` / ``should_commit``  (:365-415, 545-598)
* ``report_error`` / ``errored`` / ``wrap_future``  (:305-363)
* ``state_dict`` / ``load_state_dict`` / ``current_step`` / ``batches_committed``

The quorum itself comes from a :class:`QuorumClient`; :class:`StaticQuorum` is
an in-process one for a fixed set of replicas (what the reference's unit tests
get by patching ``ManagerClient``).  A deployment would plug a client that talks
to a real lighthouse in the same seat.

The arithmetic of ``allreduce`` runs in HIP kernels: with a process group that
offers ``allreduce_avg`` (ProcessGroupLocalReplicas) zeroing, sum and division
are one pass; with any other ``ProcessGroup`` the zeroing and the division are
each one kernel around the backend's collective.  In addition
``allreduce_tensors`` / ``pseudograd_allreduce`` give LocalSGD / DiLoCo one
launch for the whole model instead of one collective per parameter.
"""

from __future__ import annotations

import concurrent.futures
import logging
import os
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass, field
from datetime import timedelta
from enum import Enum
from typing import Callable, Dict, Generic, List, Optional, Sequence, TypeVar, cast

import torch
from torch.distributed import ReduceOp

from . import ops
from .checkpointing import CheckpointServer, CheckpointTransport
from .futures import future_timeout
from .multi_tensor import TensorTable

T = TypeVar("T")

logger: logging.Logger = logging.getLogger(__name__)


class WorldSizeMode(Enum):
    """How many replicas count in the average when more than ``min_replica_size`` are up
    (torchft/manager.py:55-70): DYNAMIC uses all of them; FIXED_WITH_SPARES keeps the
    first ``min_replica_size`` active and has the spares contribute zeros."""

    DYNAMIC = 0
    FIXED_WITH_SPARES = 1


@dataclass
class QuorumResult:
    """Fields of the control plane's answer (torchft/torchft.pyi:25-36)."""

    quorum_id: int = 0
    replica_rank: int = 0
    replica_world_size: int = 1
    recover_src_manager_address: str = ""
    recover_src_rank: Optional[int] = None
    recover_dst_ranks: List[int] = field(default_factory=list)
    store_address: str = ""
    max_step: int = 0
    max_rank: Optional[int] = 0
    max_world_size: int = 1
    heal: bool = False


class QuorumClient:
    """Seat of the reference's ``ManagerClient`` (torchft/torchft.pyi:4-23)."""

    def quorum(
        self, rank: int, step: int, checkpoint_metadata: str, shrink_only: bool, timeout: timedelta
    ) -> QuorumResult:
        raise NotImplementedError

    def should_commit(self, rank: int, step: int, should_commit: bool, timeout: timedelta) -> bool:
        raise NotImplementedError

    def checkpoint_metadata(self, address: str, rank: int, timeout: timedelta) -> str:
        raise NotImplementedError("this quorum client cannot reach other managers")


class StaticQuorum(QuorumClient):
    """A fixed replica group: every quorum has the same members and nobody heals;
    the commit vote is this replica's own."""

    def __init__(self, replica_rank: int = 0, replica_world_size: int = 1) -> None:
        self.replica_rank = replica_rank
        self.replica_world_size = replica_world_size
        self.quorum_count = 0
        self.commit_votes: List[bool] = []

    def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout) -> QuorumResult:
        self.quorum_count += 1
        return QuorumResult(
            quorum_id=1,
            replica_rank=self.replica_rank,
            replica_world_size=self.replica_world_size,
            max_step=step,
            max_rank=self.replica_rank,
            max_world_size=self.replica_world_size,
            heal=False,
        )

    def should_commit(self, rank, step, should_commit, timeout) -> bool:
        self.commit_votes.append(should_commit)
        return should_commit


class ManagerClientAdapter(QuorumClient):
    """Puts a client with the reference's ``ManagerClient`` interface
    (torchft/torchft.pyi:4-23: ``quorum``, ``should_commit``, ``checkpoint_metadata(rank,
    timeout)``) into the ``QuorumClient`` seat.  ``connect(address)`` must return such a
    client for another replica group's manager (torchft: ``ManagerClient(address,
    connect_timeout=...)``, torchft/manager.py:497-502)."""

    def __init__(self, client: object, connect: Optional[Callable[[str], object]] = None) -> None:
        self._client = client
        self._connect = connect

    def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
        return self._client.quorum(
            rank=rank, step=step, checkpoint_metadata=checkpoint_metadata,
            shrink_only=shrink_only, timeout=timeout,
        )

    def should_commit(self, rank, step, should_commit, timeout):
        return self._client.should_commit(rank, step, should_commit, timeout=timeout)

    def checkpoint_metadata(self, address, rank, timeout):
        if self._connect is None:
            raise NotImplementedError("no way to connect to other managers was given")
        return self._connect(address).checkpoint_metadata(rank, timeout=timeout)


def _done_future(value: object) -> torch.futures.Future:
    fut: torch.futures.Future = torch.futures.Future()
    fut.set_result(value)
    return fut


class Manager(Generic[T]):
    """Fault-tolerant step bookkeeping plus the averaged all-reduce.

    The constructor takes the reference's arguments in the reference's order
    (torchft/manager.py:87-108), so a call written for torchft binds the same way.
    What the arguments *do* differs for the control plane, which is not part of
    this package: ``store_addr`` / ``store_port`` / ``lighthouse_addr`` / ``port`` /
    ``hostname`` / ``heartbeat_interval`` / ``connect_timeout`` / ``world_size``
    describe the reference's TCPStore rendezvous and its Rust manager server.
    Here the quorum comes from ``quorum_client`` (an extra, keyword-only seat for
    the reference's ``ManagerClient``); a call that names a lighthouse, a store or
    a server port without giving a ``quorum_client`` is refused with one clear
    error instead of silently training without fault tolerance.  With neither,
    the manager runs a static single-group quorum over ``pg.size()`` replicas.
    """

    def __init__(
        self,
        pg,
        load_state_dict: Optional[Callable[[T], None]],
        state_dict: Optional[Callable[[], T]],
        min_replica_size: int,
        use_async_quorum: bool = True,
        timeout: timedelta = timedelta(seconds=60),
        quorum_timeout: timedelta = timedelta(seconds=60),
        connect_timeout: timedelta = timedelta(seconds=60),
        rank: Optional[int] = None,
        world_size: Optional[int] = None,
        world_size_mode: WorldSizeMode = WorldSizeMode.DYNAMIC,
        store_addr: Optional[str] = None,
        store_port: Optional[int] = None,
        lighthouse_addr: Optional[str] = None,
        replica_id: Optional[str] = None,
        port: Optional[int] = None,
        hostname: Optional[str] = None,
        heartbeat_interval: timedelta = timedelta(milliseconds=100),
        checkpoint_transport: Optional[CheckpointTransport] = None,
        *,
        quorum_client: Optional[QuorumClient] = None,
    ) -> None:
        if quorum_client is None:
            named = {
                "lighthouse_addr": lighthouse_addr,
                "store_addr": store_addr,
                "store_port": store_port,
                "port": port,
                "TORCHFT_LIGHTHOUSE (environment)": os.environ.get("TORCHFT_LIGHTHOUSE"),
            }
            given = [k for k, v in named.items() if v is not None]
            if given:
                raise NotImplementedError(
                    "control plane not built; pass quorum_client=: this package has no lighthouse / "
                    "manager server / TCPStore rendezvous, and " + ", ".join(given) + " was given. "
                    "Seat a client with torchft's ManagerClient interface via "
                    "quorum_client=ManagerClientAdapter(client)."
                )
            quorum_client = StaticQuorum(0, pg.size())
        self._pg = pg
        self._load_state_dict = load_state_dict
        self._user_state_dict = state_dict
        self._min_replica_size = min_replica_size
        self._use_async_quorum = use_async_quorum
        self._timeout = timeout
        self._quorum_timeout = quorum_timeout
        self._connect_timeout = connect_timeout
        self._rank: int = rank if rank is not None else int(os.environ.get("RANK", 0))
        self._world_size_mode = world_size_mode
        self._replica_id = replica_id or ""
        if checkpoint_transport is None and not isinstance(quorum_client, StaticQuorum):
            # the reference's default (torchft/manager.py:155-158); a static quorum never
            # asks anybody to heal, so it gets no server thread
            checkpoint_transport = CheckpointServer(timeout=timeout)
        self._checkpoint_transport: Optional[CheckpointTransport] = checkpoint_transport
        self._client: QuorumClient = quorum_client

        self._executor = ThreadPoolExecutor(max_workers=1, thread_name_prefix="async_quorum")
        self._quorum_future: Optional[concurrent.futures.Future] = None
        self._pending_state_dict: Optional[Dict[str, object]] = None
        self._pending_work: List[torch.futures.Future] = []
        self._errored: Optional[Exception] = None
        self._healing = False
        self._step = 0
        self._batches_committed = 0
        self._quorum_id = -1
        self._participating_rank: Optional[int] = None
        self._participating_world_size = 0
        self._tables: Dict[str, TensorTable] = {}
        self._columns: Optional[tuple] = None  # replica_columns' previous answer and its key

    # ------------------------------------------------------------------ state
    def set_state_dict_fns(
        self, load_state_dict: Callable[[T], None], state_dict: Callable[[], T]
    ) -> None:
        self._load_state_dict = load_state_dict
        self._user_state_dict = state_dict

    def shutdown(self, wait: bool = True) -> None:
        if self._checkpoint_transport is not None:
            self._checkpoint_transport.shutdown(wait=wait)
        self._executor.shutdown(wait=wait)

    def state_dict(self) -> Dict[str, int]:
        return {"step": self._step, "batches_committed": self._batches_committed}

    def load_state_dict(self, state_dict: Dict[str, int]) -> None:
        self._step = state_dict["step"]
        self._batches_committed = state_dict["batches_committed"]

    def _manager_state_dict(self) -> Dict[str, object]:
        assert self._user_state_dict is not None, "user state_dict is not initialized."
        return {"user": self._user_state_dict(), "torchft": self.state_dict()}

    def current_step(self) -> int:
        return self._step

    def batches_committed(self) -> int:
        return self._batches_committed

    # ------------------------------------------------------------ participants
    def num_participants(self) -> int:
        """Replicas that count in this step's average (torchft/manager.py:655-665)."""
        assert self._participating_world_size >= 0, "internal error"
        return self._participating_world_size

    def is_participating(self) -> bool:
        """False for a spare or a replica that is still healing: its contribution is
        zeroed (torchft/manager.py:667-679)."""
        if self._participating_rank is None:
            return False
        if self._healing:
            assert self._use_async_quorum
            return False
        return True

    # ------------------------------------------------------------------ errors
    def report_error(self, e: Exception) -> None:
        """Latches an error: the step will not commit and later allreduces are no-ops."""
        self._errored = e

    def errored(self) -> Optional[Exception]:
        return self._errored

    def wrap_future(
        self, fut: torch.futures.Future, default: object, timeout: Optional[timedelta] = None
    ) -> torch.futures.Future:
        """Adds the manager timeout to ``fut`` and swallows its failure: the returned
        future resolves to ``default`` and the error is latched
        (torchft/manager.py:326-363)."""
        timed = future_timeout(fut, timeout or self._timeout)

        def swallow(f: torch.futures.Future) -> object:
            try:
                return f.value()
            except Exception as e:
                logger.exception("%s got exception in future -- skipping remaining: %s", self._tag(), e)
                self.report_error(e)
                return default

        wrapped = timed.then(swallow)
        self._pending_work.append(wrapped)
        return wrapped

    def _tag(self) -> str:
        return f"[{self._replica_id}/{self._rank} - step {self._step}]"

    # ------------------------------------------------------------------ quorum
    def start_quorum(
        self,
        allow_heal: bool = True,
        shrink_only: bool = False,
        timeout: Optional[timedelta] = None,
    ) -> None:
        """Starts the quorum for a new step and clears the error latch
        (torchft/manager.py:365-415).  Synchronous mode waits for it and applies a
        recovered state dict right away."""
        if self._quorum_future is not None:
            self._quorum_future.result()
        self._errored = None
        self._healing = False
        self._quorum_future = self._executor.submit(
            self._async_quorum,
            allow_heal=allow_heal,
            shrink_only=shrink_only,
            quorum_timeout=timeout or self._quorum_timeout,
        )
        if not self._use_async_quorum:
            self.wait_quorum()
            if self._healing:
                self._apply_pending_state_dict()
                self._healing = False

    def wait_quorum(self) -> None:
        assert self._quorum_future is not None, "must call start_quorum before wait_quorum"
        self._quorum_future.result()

    def applies_recovered_state_in_vote(self) -> bool:
        """After ``wait_quorum()``: True for a replica that is healing under an asynchronous
        quorum.  Its recovered state dict is loaded by ``should_commit()``
        (torchft/manager.py:572-575), over whatever a reduction has written before."""
        return self._healing

    def _async_quorum(self, allow_heal: bool, shrink_only: bool, quorum_timeout: timedelta) -> None:
        metadata = self._checkpoint_transport.metadata() if self._checkpoint_transport else ""
        q = self._client.quorum(
            rank=self._rank,
            step=self._step,
            checkpoint_metadata=metadata,
            shrink_only=shrink_only,
            timeout=quorum_timeout,
        )
        # torchft/manager.py:452-468: asynchronous quorums count only the replicas
        # at the newest step (the others are still recovering); synchronous ones
        # have healed everybody before the step, so all of them count.
        if self._use_async_quorum or not allow_heal:
            self._participating_rank, self._participating_world_size = q.max_rank, q.max_world_size
        else:
            self._participating_rank, self._participating_world_size = (
                q.replica_rank,
                q.replica_world_size,
            )
        if self._world_size_mode == WorldSizeMode.FIXED_WITH_SPARES:
            self._participating_world_size = min(
                self._participating_world_size, self._min_replica_size
            )
            if (
                self._participating_rank is not None
                and self._participating_rank >= self._min_replica_size
            ):
                self._participating_rank = None

        if q.quorum_id != self._quorum_id:
            self._pg.configure(
                f"{q.store_address}/torchft/{q.quorum_id}/{self._rank}",
                q.replica_rank,
                q.replica_world_size,
            )
            self._quorum_id = q.quorum_id

        if not allow_heal:
            return
        if q.recover_dst_ranks:
            assert self._checkpoint_transport is not None, "no checkpoint transport configured"
            self._checkpoint_transport.send_checkpoint(
                dst_ranks=q.recover_dst_ranks,
                step=q.max_step,
                state_dict=self._manager_state_dict(),
                timeout=self._timeout,
            )
        if q.heal:
            assert self._checkpoint_transport is not None, "no checkpoint transport configured"
            assert q.recover_src_rank is not None, "must have a recover rank when healing"
            self._healing = True
            remote = self._client.checkpoint_metadata(
                q.recover_src_manager_address, self._rank, timeout=self._timeout
            )
            self._pending_state_dict = self._checkpoint_transport.recv_checkpoint(
                src_rank=q.recover_src_rank,
                metadata=remote,
                step=q.max_step,
                timeout=self._timeout,
            )
            self.load_state_dict(cast(Dict[str, int], self._pending_state_dict["torchft"]))
            self._step = q.max_step

    def _apply_pending_state_dict(self) -> None:
        assert self._healing, "must be in healing state"
        assert self._quorum_future is not None, "must call step before should_commit"
        self._quorum_future.result()
        assert self._pending_state_dict is not None, "checkpoint was not staged"
        assert self._load_state_dict is not None, "user load_state_dict is not initialized."
        self._load_state_dict(cast(T, self._pending_state_dict["user"]))
        self._pending_state_dict = None

    def should_commit(self, timeout: Optional[timedelta] = None) -> bool:
        """Drains the pending all-reduces, votes and returns the group's decision; on
        commit the step counter advances (torchft/manager.py:545-598)."""
        for work in self._pending_work:
            if self._errored is not None:
                break
            work.wait()
        self._pending_work = []

        if self._healing:
            self._apply_pending_state_dict()

        enough_replicas = self.num_participants() >= self._min_replica_size
        local_should_commit = enough_replicas and self._errored is None
        decision = self._client.should_commit(
            self._rank, self._step, local_should_commit, timeout=timeout or self._timeout
        )
        logger.info(
            "%s should_commit=%s enough_replicas=%s, errored=%s",
            self._tag(), decision, enough_replicas, self._errored,
        )
        if self._checkpoint_transport is not None:
            self._checkpoint_transport.disallow_checkpoint()
        if decision:
            self._step += 1
            self._batches_committed += self.num_participants()
        return decision

    # --------------------------------------------------------------- allreduce
    def allreduce(self, tensor: torch.Tensor, *, divide: bool = True) -> torch.futures.Future:
        """In place: zero if this replica does not participate, SUM over the replicas,
        divide by ``num_participants()``; the future resolves to ``tensor`` itself.

        ``divide=False`` (not in the reference) leaves the sum in ``tensor``: for callers
        whose next kernel reads the buffer anyway and divides on the way in (the bucketised
        LocalSGD / DiLoCo sync), which saves a pass over the buffer.

        Never raises: a failure is latched (``errored()``), the future still
        completes with the (possibly corrupt) tensor and every later call is a no-op
        until the next ``start_quorum`` (torchft/manager.py:242-303).  That includes a
        tensor the kernels cannot take (not on a GPU, not contiguous, an integer dtype):
        it is reported and latched like any other failed all-reduce, so the step is
        discarded instead of the training loop being torn down.  There is no CPU
        arithmetic behind this method."""
        if self.errored():
            return _done_future(tensor)
        self.wait_quorum()
        try:
            ops.check_tensor(tensor, "Manager.allreduce")
            if hasattr(self._pg, "allreduce_avg"):
                work = self._pg.allreduce_avg(
                    [tensor], self.is_participating(), self.num_participants() if divide else 1
                )
                fut = work.get_future().then(lambda f: (f.value(), tensor)[1])
            else:
                if not self.is_participating():
                    ops.reduce_avg_(tensor, [], 0, 1)  # tensor.zero_()
                work = self._pg.allreduce([tensor], ReduceOp.SUM)

                def normalize(f: torch.futures.Future) -> torch.Tensor:
                    f.value()  # surfaces a failed collective
                    if divide:
                        ops.reduce_avg_(tensor, [tensor], 1, self.num_participants())
                    return tensor

                fut = work.get_future().then(normalize)
            return self.wrap_future(fut, tensor)
        except Exception as e:
            logger.exception("%s got exception in all reduce -- skipping remaining: %s", self._tag(), e)
            self.report_error(e)
            return _done_future(tensor)

    def _cached_table(self, key: str, columns: Sequence[Sequence[torch.Tensor]]) -> Optional[TensorTable]:
        table = self._tables.get(key)
        return table if table is not None and table.matches(columns) else None

    def supports_fused_sync(self) -> bool:
        """True when the process group exposes its peers' buffers, so a whole model can
        be reduced in one launch."""
        return hasattr(self._pg, "ordered")

    def allreduce_tensors(
        self, tensors: Sequence[torch.Tensor], also_write: Optional[Sequence[torch.Tensor]] = None
    ) -> torch.futures.Future:
        """``allreduce`` of every tensor in ONE launch (same arithmetic per element, same
        error behaviour).  ``also_write`` receives a second copy of the result (LocalSGD
        refreshes its backup with it).  Needs ``supports_fused_sync()``."""
        tensors = list(tensors)
        if self.errored():
            return _done_future(tensors)
        self.wait_quorum()
        try:
            replicas, mask = self.replica_columns(tensors)
            for idx in ops.dtype_groups(tensors):
                outs = [[tensors[i] for i in idx]]
                if also_write is not None:
                    outs.append([also_write[i] for i in idx])
                reps = [[rep[i] for i in idx] for rep in replicas]
                key = "allreduce_tensors/%d/%s" % (len(outs), tensors[idx[0]].dtype)
                self._tables[key] = ops.mt_reduce_avg(
                    outs, reps, mask, self.num_participants(),
                    table=self._cached_table(key, [*outs, *reps]),
                )
            return self.wrap_future(_done_future(tensors), tensors)
        except Exception as e:
            logger.exception("%s got exception in all reduce -- skipping remaining: %s", self._tag(), e)
            self.report_error(e)
            return _done_future(tensors)

    def pseudograd_allreduce(
        self,
        grads: Sequence[torch.Tensor],
        params: Sequence[torch.Tensor],
        backups: Sequence[torch.Tensor],
        restore_params: bool,
    ) -> torch.futures.Future:
        """DiLoCo phase 1 in one launch: ``grads = allreduce(params - backups)`` over all
        replicas (each replica subtracts the shared backup from its own parameters),
        optionally followed by ``params = backups``.  Needs ``supports_fused_sync()``."""
        grads, params, backups = list(grads), list(params), list(backups)
        if self.errored():
            return _done_future(grads)
        self.wait_quorum()
        try:
            replicas, mask = self.replica_columns(params)
            for idx in ops.dtype_groups(params):
                cols = [[col[i] for i in idx] for col in (grads, params, backups, *replicas)]
                key = "pseudograd/%s" % params[idx[0]].dtype
                self._tables[key] = ops.mt_pseudograd_avg(
                    cols[0], cols[1], cols[2], cols[3:], restore_params, mask,
                    self.num_participants(), table=self._cached_table(key, cols),
                )
            return self.wrap_future(_done_future(grads), grads)
        except Exception as e:
            logger.exception("%s got exception in all reduce -- skipping remaining: %s", self._tag(), e)
            self.report_error(e)
            return _done_future(grads)

    def replica_columns(self, tensors: Sequence[torch.Tensor], identity: object = None):
        """([replica][tensor] buffers in rank order, participation mask) for a tensor list.

        ``identity``: a hashable value by which the caller vouches for ``tensors`` (the same
        value means the same tensors at the same addresses).  With it, and with a process
        group whose peer buffers only change when it says so (``peers_generation``), the
        columns of the previous call are returned as the very same list objects instead of
        looking every tensor's peers up again; callers recognise an unchanged answer by
        ``is``."""
        participating = self.is_participating()
        generation = None
        if identity is not None:
            peers_generation = getattr(self._pg, "peers_generation", None)
            generation = peers_generation() if peers_generation is not None else None
        if generation is not None:
            key = (identity, generation, participating, len(tensors))
            kept = self._columns
            if kept is not None and kept[0] == key:
                return kept[1], kept[2]
        per_tensor = [self._pg.ordered(t, participating) for t in tensors]
        if not per_tensor:
            return [], 0
        n_rep = len(per_tensor[0][0])
        columns = [[pt[0][r] for pt in per_tensor] for r in range(n_rep)]
        mask = per_tensor[0][1]
        if generation is not None:
            self._columns = (key, columns, mask)
        return columns, mask

    def reduction_fails_only_at_launch(self) -> bool:
        return bool(getattr(self._pg, "fails_only_at_launch", False))
