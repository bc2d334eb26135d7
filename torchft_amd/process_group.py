"""Process-group plugins for the replica-sync path.

Only the part of the reference's plugin contract that the hot path uses is
mirrored (torchft/process_group.py:123-187): ``configure``, ``allreduce``
returning a ``Work`` with ``wait`` / ``get_future``, ``size`` and
``getBackendName``.  Backends that talk to other GPUs or hosts are out of scope
for this build; instead :class:`ProcessGroupLocalReplicas` runs the N-replica
reduction on one GPU over N replica buffers resident in its HBM.
"""

from __future__ import annotations

from datetime import timedelta
from typing import Callable, Dict, List, Optional, Sequence, Tuple, Union

import torch
import torch.distributed as dist
from torch.distributed import ReduceOp
from torch.distributed.distributed_c10d import AllreduceOptions, Work

from . import ops

PeerLookup = Callable[[torch.Tensor], Sequence[torch.Tensor]]


class ProcessGroup(dist.ProcessGroup):
    """Reconfigurable process group (torchft/process_group.py:123-187)."""

    def __init__(self, *args: object, **kwargs: object) -> None:
        super().__init__(*args, **kwargs)  # type: ignore[arg-type]

    def configure(self, store_addr: str, rank: int, world_size: int) -> None:
        """Re-targets the group at a new store / rank / world size; blocks until usable."""
        raise NotImplementedError("not implemented")

    def allreduce(  # type: ignore[override]
        self, tensors: List[torch.Tensor], opts: Union[AllreduceOptions, ReduceOp]
    ) -> Work:
        raise NotImplementedError("not implemented")

    def allgather(self, output_tensors, input_tensor, opts) -> Work:  # type: ignore[override]
        raise NotImplementedError("not implemented")

    def broadcast(self, tensor_list, opts) -> Work:  # type: ignore[override]
        raise NotImplementedError("not implemented")

    def broadcast_one(self, tensor: torch.Tensor, root: int) -> Work:
        opts = dist.BroadcastOptions()
        opts.rootRank = root
        return self.broadcast([tensor], opts)

    def size(self) -> int:
        raise NotImplementedError("not implemented")

    def getBackendName(self) -> str:
        raise NotImplementedError("not implemented")

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}()"


class _DummyWork(dist._Work):
    """An already completed ``Work`` (torchft/process_group.py:339-351)."""

    def __init__(self, result: object) -> None:
        super().__init__()
        self.result_ = result
        self.future_: torch.futures.Future = torch.futures.Future()
        self.future_.set_result(result)

    def wait(self, timeout: Optional[timedelta] = None) -> bool:
        return True

    def get_future(self) -> torch.futures.Future:
        return self.future_


class ProcessGroupDummy(ProcessGroup):
    """Discards every collective and reports success; world size 1 only
    (torchft/process_group.py:354-405).  The DDP wrapper hands it to torch's
    Reducer to soak up the constructor's collectives."""

    def __init__(self, rank: int, world: int) -> None:
        super().__init__(rank, world)
        assert rank == 0
        assert world == 1
        self._rank = rank
        self._world = world
        self.configure_count = 0

    def configure(self, store_addr: str, rank: int, world_size: int) -> None:
        self.configure_count += 1

    def broadcast(self, tensor_list, opts) -> Work:  # type: ignore[override]
        return _DummyWork(tensor_list)

    def allgather(self, output_tensors, input_tensor, opts) -> Work:  # type: ignore[override]
        for o, i in zip(output_tensors[0], input_tensor):
            o.copy_(i)
        return _DummyWork(output_tensors)

    def allreduce(self, tensors, opts) -> Work:  # type: ignore[override]
        return _DummyWork(tensors)

    def size(self) -> int:
        return self._world

    def getBackendName(self) -> str:
        return "torchft-dummy"


class _StreamWork(dist._Work):
    """Work whose result is ready in stream order on the launching stream.

    The kernels are enqueued on torch's current stream, so any later torch op on
    that stream sees the result; ``wait`` therefore has nothing to block on
    (the same convention as c10d's NCCL work objects).  ``synchronize`` is for
    callers that read the result from the host.
    """

    def __init__(self, result: List[torch.Tensor], device: torch.device) -> None:
        super().__init__()
        self._device = device
        self._event: Optional[torch.cuda.Event] = None
        if device.type == "cuda":
            self._event = torch.cuda.Event()
            self._event.record(torch.cuda.current_stream(device))
        self._future: torch.futures.Future = torch.futures.Future()
        self._future.set_result(result)

    def wait(self, timeout: Optional[timedelta] = None) -> bool:
        if self._event is not None:
            torch.cuda.current_stream(self._device).wait_event(self._event)
        return True

    def synchronize(self) -> None:
        if self._event is not None:
            self._event.synchronize()

    def get_future(self) -> torch.futures.Future:
        return self._future


class ProcessGroupLocalReplicas(ProcessGroup):
    """All-reduce over N replicas whose buffers all live on this GPU.

    This stands where ProcessGroupGloo / ProcessGroupNCCL stand in the reference:
    ``Manager(pg=...)`` drives it through ``allreduce([tensor], SUM)``.  The local
    replica has rank ``rank``; for each tensor it reduces, the buffers the other
    replicas would have contributed are found through ``peer_lookup(tensor)``
    (or tensors registered with :meth:`register_peers`), ordered by replica rank
    with the local replica left out.

    ``peer_participating[i]`` says whether peer i contributes its data or zeros
    (a healing or spare replica zeroes its tensor before the collective:
    torchft/manager.py:267-268).  The sum runs in replica-rank order.

    Besides the plain contract the group offers the fused forms the Manager and
    the LocalSGD / DiLoCo wrappers use when they find them: sum, zeroing and the
    division by ``num_participants`` in a single pass (``allreduce_avg``), and
    the same over a whole list of tensors in one launch.
    """

    #: the reduction is one kernel on the caller's stream: it cannot fail after launch
    fails_only_at_launch = True

    def __init__(
        self,
        rank: int = 0,
        world_size: int = 1,
        peer_lookup: Optional[PeerLookup] = None,
        peer_participating: Optional[Sequence[bool]] = None,
        peers_are_stable: bool = False,
    ) -> None:
        super().__init__(rank, world_size)
        if not 0 <= rank < world_size:
            raise ValueError(f"rank {rank} outside world of {world_size}")
        if world_size > ops.MAX_REPLICAS:
            raise ValueError(f"at most {ops.MAX_REPLICAS} local replicas, got {world_size}")
        self._rank = rank
        self._world = world_size
        self._lookup = peer_lookup
        self._lookup_is_stable = peers_are_stable
        self._generation = 0
        self._registry: Dict[Tuple[int, int], List[torch.Tensor]] = {}
        self._peer_participating = list(
            peer_participating if peer_participating is not None else [True] * (world_size - 1)
        )
        if len(self._peer_participating) != world_size - 1:
            raise ValueError("peer_participating needs one entry per peer")
        self.configure_count = 0

    # -- plugin contract ---------------------------------------------------
    def configure(self, store_addr: str, rank: int, world_size: int) -> None:
        """Membership of a local group is fixed at construction; a quorum change only
        has to agree with it."""
        self.configure_count += 1
        if world_size != self._world or rank != self._rank:
            raise ValueError(
                f"local replica group is rank {self._rank} of {self._world}; "
                f"cannot reconfigure to rank {rank} of {world_size}"
            )

    def size(self) -> int:
        return self._world

    def getBackendName(self) -> str:
        return "torchft-local-replicas"

    # -- peers -------------------------------------------------------------
    def set_peer_lookup(self, peer_lookup: Optional[PeerLookup], peers_are_stable: bool = False) -> None:
        self._lookup = peer_lookup
        self._lookup_is_stable = peers_are_stable
        self._generation += 1

    def set_peer_participating(self, flags: Sequence[bool]) -> None:
        if len(flags) != self._world - 1:
            raise ValueError("peer_participating needs one entry per peer")
        self._peer_participating = list(flags)
        self._generation += 1

    def invalidate_peers(self) -> None:
        """Says that the peers' buffers may have moved (for lookups declared stable)."""
        self._generation += 1

    def peers_generation(self) -> Optional[int]:
        """A counter that changes whenever the answer of :meth:`ordered` may change for a
        tensor that has not moved, or None if that cannot be known: a ``peer_lookup``
        callback may return different buffers from one call to the next unless it was
        declared stable (``peers_are_stable=True``: it returns the same buffers for the
        same tensor until ``invalidate_peers()`` / ``set_peer_lookup()``).  Registered peers
        (``register_peers``) only change through this object.  Callers that hold a whole
        model's peer columns use it to skip one lookup per tensor per sync."""
        if self._lookup is not None and not self._lookup_is_stable:
            return None
        return self._generation

    def register_peers(self, tensor: torch.Tensor, peers: Sequence[torch.Tensor]) -> None:
        """Declares the peers' buffers for ``tensor`` (matched by address and size)."""
        if len(peers) != self._world - 1:
            raise ValueError(f"{len(peers)} peer tensors for a world of {self._world}")
        self._registry[(tensor.data_ptr(), tensor.numel())] = list(peers)
        self._generation += 1

    def peers_of(self, tensor: torch.Tensor) -> List[torch.Tensor]:
        if self._world == 1:
            return []
        found = self._registry.get((tensor.data_ptr(), tensor.numel()))
        if found is None and self._lookup is not None:
            found = list(self._lookup(tensor))
        if found is None:
            raise KeyError(
                f"no peer buffers known for tensor at {tensor.data_ptr():#x} "
                f"({tuple(tensor.shape)}, {tensor.dtype})"
            )
        if len(found) != self._world - 1:
            raise ValueError(f"{len(found)} peer tensors for a world of {self._world}")
        return found

    def ordered(
        self, local: torch.Tensor, local_participating: bool = True
    ) -> Tuple[List[torch.Tensor], int]:
        """(replica buffers in rank order, participation mask) for one tensor."""
        peers = self.peers_of(local)
        replicas = peers[: self._rank] + [local] + peers[self._rank :]
        flags = (
            self._peer_participating[: self._rank]
            + [local_participating]
            + self._peer_participating[self._rank :]
        )
        mask = sum(1 << r for r, f in enumerate(flags) if f)
        return replicas, mask

    # -- collectives ---------------------------------------------------------
    def allreduce(self, tensors, opts) -> Work:  # type: ignore[override]
        """In-place SUM over the replicas (the c10d contract Manager.allreduce uses)."""
        op = opts.reduceOp if isinstance(opts, AllreduceOptions) else opts
        if op != ReduceOp.SUM:
            raise NotImplementedError(f"only ReduceOp.SUM is supported, got {op}")
        for t in tensors:
            replicas, mask = self.ordered(t)
            ops.reduce_avg_(t, replicas, mask, 1)
        return _StreamWork(list(tensors), tensors[0].device)

    def allreduce_avg(
        self, tensors: List[torch.Tensor], participating: bool, num_participants: int
    ) -> Work:
        """Zero-if-not-participating, SUM and divide in one pass per tensor."""
        for t in tensors:
            replicas, mask = self.ordered(t, participating)
            ops.reduce_avg_(t, replicas, mask, num_participants)
        return _StreamWork(list(tensors), tensors[0].device)

    def broadcast(self, tensor_list, opts) -> Work:  # type: ignore[override]
        return _DummyWork(tensor_list)

    def allgather(self, output_tensors, input_tensor, opts) -> Work:  # type: ignore[override]
        raise NotImplementedError("allgather is not on the replica-sync path")
