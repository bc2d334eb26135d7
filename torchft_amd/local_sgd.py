"""LocalSGD and DiLoCo with the synchronisation step fused into multi-tensor HIP launches.

Same classes, constructor arguments, hooks and attributes as the reference
(torchft/local_sgd.py:26-239): a context manager that counts optimizer steps and
every ``sync_every`` steps starts a quorum, synchronises the replicas through the
Manager and commits or rolls back.  What differs is how the work is issued:

* the reference runs five Python loops with one or more kernels per parameter
  tensor (subtract, all-reduce, divide, restore, SGD, save); here each of those
  loops is one launch over a tensor table, and with this package's Manager on a
  process group that exposes the replicas' buffers the whole DiLoCo step (all
  loops) is a single launch;
* the backup copy defaults to the parameters' own GPU instead of pinned host
  memory (``backup_device=None``): the kernels need it in HBM, and 288 GB holds
  it.  ``backup_device=torch.device("cpu")`` is still accepted by LocalSGD (plain
  DMA copies); DiLoCo needs the backup on the device, as the reference's
  ``p.data - backup`` does for GPU parameters.

With this package's Manager on any other process group (one real collective per call) the
model is bucketised: the pseudo-gradients (DiLoCo) or a flattened copy of the weights
(LocalSGD) live in ONE flat buffer per dtype and a single ``manager.allreduce`` covers the
whole model, instead of the reference's one collective per parameter
(``torchft/local_sgd.py:170`` "TODO: bucketize parameters").

With a Manager that is not this package's (for instance a mock) the per-parameter
``manager.allreduce`` contract is kept call for call.
"""

from __future__ import annotations

import logging
import operator
from dataclasses import dataclass
from types import TracebackType
from typing import Dict, List, Optional, Sequence, Tuple, Type

import torch
from torch import nn, optim
from torch.utils.hooks import RemovableHandle

from . import _native, hbm_placement, ops
from .manager import Manager
from .multi_tensor import TensorTable

logger: logging.Logger = logging.getLogger(__name__)


_KERNEL_DTYPES = (torch.float32, torch.bfloat16, torch.float16)   # every kernel
_AVERAGE_DTYPES = _KERNEL_DTYPES + (torch.float64,)                # the replica average and the copies

_DATA_PTR = torch.Tensor.data_ptr
_NUMEL = torch.Tensor.numel
_MOMENTUM_OF = operator.itemgetter("momentum_buffer")


@dataclass
class _Bound:
    """The tensors a wrapper synchronises, gathered once and re-validated on every sync by
    address and size alone (C-level maps over the parameter objects), so that a sync does
    not walk the module tree or create 2 x T tensor objects again.  ``generation`` changes
    whenever the lists are rebuilt; everything derived from them is keyed on it."""

    generation: int
    names: List[str]
    params: List[torch.Tensor]       # p.data of every parameter
    backups: List[torch.Tensor]
    backup_dict: Dict[str, torch.Tensor]
    param_key: Tuple
    backup_key: Tuple
    on_device: bool = False          # parameters and backups all on one GPU


@dataclass
class _SgdPlan:
    """What ``_fusable_sgd`` found, and what it has to be compared with to still hold."""

    entries: Optional[List[Tuple[List[int], "ops.OuterSGD", bool]]]
    state: object                    # the optimizer's state mapping itself
    n_state: int
    groups_key: Tuple
    bufs: Optional[List[Optional[torch.Tensor]]]   # momentum buffers found, by parameter index
    slots: Optional[List[dict]]      # optimizer.state[p] of every parameter (steady state)


def _is_native_manager(manager: object) -> bool:
    # a create_autospec(Manager) double passes isinstance() but is not a subclass instance
    return issubclass(type(manager), Manager)


class _PackedHostBackup:
    """Backup of GPU parameters in pinned host memory, moved as ONE transfer.

    The reference copies tensor by tensor into pinned host tensors on the compute
    stream (torchft/local_sgd.py:121-131, with a TODO to use a separate stream).  Here
    the parameters are gathered into a device staging buffer by one launch and the
    staging buffer crosses PCIe as a single copy on a side stream, so the save overlaps
    the next inner steps; restore is the same path backwards.  The tensors handed out
    as ``_backup_parameters`` are views into the one pinned buffer.
    """

    ALIGN = 256

    def __init__(self, named_params, pin_memory: bool) -> None:
        params = [p for _, p in named_params]
        self.device = params[0].device
        offsets, off = [], 0
        for p in params:
            offsets.append(off)
            off += -(-(p.numel() * p.element_size()) // self.ALIGN) * self.ALIGN
        self.total = max(off, self.ALIGN)
        self.host = torch.empty(self.total, dtype=torch.uint8, pin_memory=pin_memory)
        self.staging = torch.empty(self.total, dtype=torch.uint8, device=self.device)
        self.host_views = [
            self.host[o : o + p.numel() * p.element_size()].view(p.dtype).view(p.shape)
            for o, p in zip(offsets, params)
        ]
        self.staging_views = [
            self.staging[o : o + p.numel() * p.element_size()] for o, p in zip(offsets, params)
        ]
        # the staging buffer seen as the parameters' device-side backup: the sync kernels read
        # and write these, the staging buffer then crosses PCIe as it does after a save
        self.device_views = [
            v.view(p.dtype).view(p.shape) for v, p in zip(self.staging_views, params)
        ]
        self.stream = torch.cuda.Stream(device=self.device)
        self.host_ready: Optional[torch.cuda.Event] = None  # the last save has reached the host
        self._tables: Dict[str, TensorTable] = {}

    def owns(self, backups: Sequence[torch.Tensor]) -> bool:
        return len(backups) == len(self.host_views) and all(
            b.data_ptr() == v.data_ptr() for b, v in zip(backups, self.host_views)
        )

    def save(self, params: List[torch.Tensor]) -> None:
        current = torch.cuda.current_stream(self.device)
        if self.host_ready is not None:
            current.wait_event(self.host_ready)  # staging is free again
        self._tables["pack"] = ops.mt_copy(self.staging_views, params, table=self._tables.get("pack"))
        self.publish()

    def reserve(self) -> List[torch.Tensor]:
        """``device_views`` for a kernel on the current stream to WRITE: waits (on the stream)
        until the previous transfer has left the staging buffer."""
        if self.host_ready is not None:
            torch.cuda.current_stream(self.device).wait_event(self.host_ready)
        return self.device_views

    def publish(self) -> None:
        """Sends the staging buffer, as the current stream leaves it, to the host on the side
        stream (the tail of a save; also after a sync kernel has written ``device_views``)."""
        current = torch.cuda.current_stream(self.device)
        packed = torch.cuda.Event()
        packed.record(current)
        self.stream.wait_event(packed)
        with torch.cuda.stream(self.stream):
            self.host.copy_(self.staging, non_blocking=True)
            self.host_ready = torch.cuda.Event()
            self.host_ready.record(self.stream)

    def load(self) -> List[torch.Tensor]:
        """Brings the host backup into the staging buffer (one transfer on the current stream)
        and returns it as ``device_views``: the backup as the kernels read it.  The host
        tensors are the user's to change between syncs, so this is done for every sync that
        reads the backup (the reference moves every tensor with ``.to(p.device)`` instead,
        torchft/local_sgd.py:214)."""
        self.wait()
        self.staging.copy_(self.host, non_blocking=True)
        return self.device_views

    def wait(self) -> None:
        """Blocks until the host copy is complete (before anything reads the backup)."""
        if self.host_ready is not None:
            self.host_ready.synchronize()

    def restore(self, params: List[torch.Tensor]) -> None:
        self.wait()
        current = torch.cuda.current_stream(self.device)
        self.staging.copy_(self.host, non_blocking=True)
        self._tables["unpack"] = ops.mt_copy(params, self.staging_views, table=self._tables.get("unpack"))
        current.synchronize()  # the reference's restore is blocking


class LocalSGD:
    """Periodic weight averaging across replicas (https://arxiv.org/pdf/1805.09767),
    fault tolerant: if anything fails between two syncs the parameters roll back to
    the backup taken at the last successful sync (torchft/local_sgd.py:26-175)."""

    _DTYPES = _AVERAGE_DTYPES

    def __init__(
        self,
        manager: Manager,
        model: nn.Module,
        optimizer: optim.Optimizer,
        sync_every: int,
        backup_device: Optional[torch.device] = None,
        pin_memory: bool = True,
    ) -> None:
        super().__init__()
        self._manager = manager
        self._model = model
        self._local_optimizer = optimizer
        self._local_step = 0
        self._sync_every = sync_every
        assert sync_every >= 1, "sync_every must be greater than or equal to 1"
        self._backup_parameters: Dict[str, torch.Tensor] = {}
        self._host_backup: Optional[_PackedHostBackup] = None
        self._hooks: List[RemovableHandle] = []
        self._tables: Dict[str, TensorTable] = {}
        self._launches: Dict[str, tuple] = {}  # prepared launches, with what they were prepared for
        self._flat: Dict[str, tuple] = {}
        self._placed_momentum: Optional[List[Optional[torch.Tensor]]] = None
        self._placed_grads: Optional[List[torch.Tensor]] = None
        named = list(self._model.named_parameters())
        # like an optimizer, the wrapper binds to the parameters the model has now
        self._param_names: List[str] = [name for name, _ in named]
        self._param_objs: List[nn.Parameter] = [p for _, p in named]
        self._bound: Optional[_Bound] = None
        self._generation = 0
        if (
            backup_device is not None
            and torch.device(backup_device).type == "cpu"
            and named
            and all(p.is_cuda and p.device == named[0][1].device for _, p in named)
        ):
            # GPU parameters with a host backup: one pinned buffer, one transfer per save
            self._host_backup = _PackedHostBackup(named, pin_memory)
            for (name, _), view in zip(named, self._host_backup.host_views):
                self._backup_parameters[name] = view
        elif (
            named
            and all(p.is_cuda and p.device == named[0][1].device for _, p in named)
            and (backup_device is None or torch.device(backup_device) == named[0][1].device)
        ):
            # backup in HBM next to the parameters.  On MI355X concurrent write streams slow
            # each other down inside one HBM bank group, so models of some size get
            # per-tensor buffers (the backup and, if there will be one, the outer momentum)
            # in a group their parameter does not occupy; otherwise views into one
            # allocation per dtype
            datas = [p.data for _, p in named]
            placed = hbm_placement.allocate_apart(datas, self._placed_copies())
            if placed is not None:
                views = placed[0]
                self._keep_placed(placed[1:])
            else:
                _, views = self._flat_like("backup", datas)
            for (name, _), view in zip(named, views):
                self._backup_parameters[name] = view
        else:
            for name, p in named:
                device = backup_device if backup_device is not None else p.device
                t = torch.empty(*tuple(p.shape), dtype=p.dtype, device=device)
                if pin_memory and t.device == torch.device("cpu") and torch.cuda.is_available():
                    t = t.pin_memory()
                self._backup_parameters[name] = t
        if named and any(p.is_cuda for _, p in named):
            _native.lib()  # GPU parameters need the kernels: fail now, loudly, if they are missing
            # a dtype the kernels do not have is a configuration error: say so here, once,
            # instead of latching it as a failed all-reduce on every sync
            bad = sorted({str(p.dtype) for _, p in named if p.is_cuda and p.dtype not in self._DTYPES})
            if bad:
                raise TypeError(
                    f"{type(self).__name__}: GPU parameters of {', '.join(bad)}; its kernels take "
                    + ", ".join(str(d).replace("torch.", "") for d in self._DTYPES)
                )
            strided = [name for name, p in named if p.is_cuda and not p.is_contiguous()]
            if strided:
                raise ValueError(
                    f"{type(self).__name__}: parameters that are not contiguous in memory "
                    f"({', '.join(strided[:4])}{', ...' if len(strided) > 4 else ''}): the kernels "
                    "stream whole tensors; make them contiguous before wrapping the model"
                )
        # the first sync needs a valid backup
        self._save_parameters()

    def _placed_copies(self) -> int:
        """Model-sized device buffers this wrapper will keep: the backup."""
        return 1

    def _keep_placed(self, extra: Sequence[List[torch.Tensor]]) -> None:
        """Receives the copies allocated together with the backup (none for LocalSGD)."""

    # -- context manager / hook ---------------------------------------------
    def __enter__(self) -> "LocalSGD":
        self._hooks.append(self._local_optimizer.register_step_post_hook(self._step_post_hook))
        return self

    def __exit__(
        self,
        exc_type: Optional[Type[BaseException]],
        exc_value: Optional[BaseException],
        traceback: Optional[TracebackType],
    ) -> bool:
        if exc_type is not None:
            # discard the local steps since the last sync
            self._restore_parameters()
        for hook in self._hooks:
            hook.remove()
        self._hooks.clear()
        return False  # exceptions propagate

    def _step_post_hook(
        self, _optim: optim.Optimizer, _args: List[object], _kwargs: Dict[str, object]
    ) -> None:
        self._local_step += 1
        if self._local_step >= self._sync_every:
            self.sync()

    # -- tensors -------------------------------------------------------------
    def _named(self) -> Tuple[List[str], List[torch.Tensor], List[torch.Tensor]]:
        """(names, parameter data, backups) in ``named_parameters()`` order.  The lists are
        kept between syncs and only rebuilt when a parameter or a backup tensor has moved
        (``p.data`` reassigned, ``_backup_parameters`` replaced or refilled by the user)."""
        objs = self._param_objs
        backup_dict = self._backup_parameters
        param_key = (tuple(map(_DATA_PTR, objs)), tuple(map(_NUMEL, objs)))
        backup_key = tuple(map(_DATA_PTR, backup_dict.values()))
        bound = self._bound
        if (
            bound is not None
            and bound.param_key == param_key
            and bound.backup_dict is backup_dict
            and bound.backup_key == backup_key
        ):
            return bound.names, bound.params, bound.backups
        names = self._param_names
        backups = []
        for name in names:
            assert name in backup_dict
            backups.append(backup_dict[name])
        self._generation += 1
        params = [p.data for p in objs]
        self._bound = _Bound(
            self._generation, names, params, backups, backup_dict, param_key, backup_key,
            self._on_device(params, backups),
        )
        return names, params, backups

    @staticmethod
    def _on_device(params: Sequence[torch.Tensor], backups: Sequence[torch.Tensor]) -> bool:
        return bool(params) and all(
            p.is_cuda and b.device == p.device and p.device == params[0].device
            for p, b in zip(params, backups)
        )

    def _copy(self, key: str, dsts: List[torch.Tensor], srcs: List[torch.Tensor], blocking: bool) -> None:
        if self._on_device(dsts, srcs):
            cached = self._tables.get(key)
            self._tables[key] = ops.mt_copy(dsts, srcs, table=cached)
            return
        for d, s in zip(dsts, srcs):  # host-resident backup: plain DMA, no arithmetic
            d.copy_(s, non_blocking=not blocking)

    def _flat_like(self, key: str, tensors: Sequence[torch.Tensor]):
        """One flat buffer per dtype with the sizes of ``tensors`` back to back, plus a view
        per tensor (in the order of ``tensors``).  Kept across syncs."""
        cached = self._flat.get(key)
        sig = tuple((t.dtype, t.device, tuple(t.shape)) for t in tensors)
        if cached is not None and cached[0] == sig:
            return cached[1], cached[2]
        flats: Dict[torch.dtype, torch.Tensor] = {}
        for dtype in {t.dtype for t in tensors}:
            n = sum(t.numel() for t in tensors if t.dtype == dtype)
            flats[dtype] = torch.empty(n, dtype=dtype, device=tensors[0].device)
        offsets = {dtype: 0 for dtype in flats}
        views = []
        for t in tensors:
            off = offsets[t.dtype]
            views.append(flats[t.dtype][off : off + t.numel()].view(t.shape))
            offsets[t.dtype] = off + t.numel()
        self._flat[key] = (sig, flats, views)
        return flats, views

    def _save_parameters(self) -> None:
        """backup <- parameters (torchft/local_sgd.py:121-125), one launch."""
        with torch.no_grad():
            _, params, backups = self._named()
            if self._host_backup is not None and self._host_backup.owns(backups):
                self._host_backup.save(params)
                return
            self._copy("save", backups, params, blocking=False)

    def _restore_parameters(self) -> None:
        """parameters <- backup (torchft/local_sgd.py:127-131), one launch."""
        with torch.no_grad():
            _, params, backups = self._named()
            if self._host_backup is not None:
                if self._host_backup.owns(backups):
                    self._host_backup.restore(params)
                    return
                self._host_backup.wait()  # the user swapped the backup tensors: plain copies
            self._copy("restore", params, backups, blocking=True)

    # -- sync ------------------------------------------------------------------
    def sync(self) -> None:
        """Averages the model weights across the replicas of the current quorum."""
        self._manager.start_quorum()
        self._perform_sync()
        self._local_step = 0

    def _fused(self, params: Sequence[torch.Tensor], backups: Sequence[torch.Tensor]) -> bool:
        return (
            self._together(params, backups)
            and _is_native_manager(self._manager)
            and self._manager.supports_fused_sync()
        )

    def _together(self, params: Sequence[torch.Tensor], backups: Sequence[torch.Tensor]) -> bool:
        """``_on_device``, remembered for the bound lists."""
        bound = self._bound
        if bound is not None and bound.params is params and bound.backups is backups:
            return bound.on_device
        return self._on_device(params, backups)

    @staticmethod
    def _on_one_gpu(params: Sequence[torch.Tensor]) -> bool:
        return bool(params) and all(p.is_cuda and p.device == params[0].device for p in params)

    def _perform_sync(self) -> None:
        """Average, then keep the result (commit) or roll back (torchft/local_sgd.py:151-162)."""
        _, params, backups = self._named()
        hb = self._host_backup
        if _is_native_manager(self._manager):
            self._manager.wait_quorum()
            if self._manager.applies_recovered_state_in_vote():
                # Healing under an asynchronous quorum: the vote loads the recovered state
                # dict over whatever the reduction has written (torchft/manager.py:572-575).
                # Only the reference's own order of steps - average into the parameters, vote,
                # save or restore - ends where the reference ends, so this (rare) sync takes it.
                if self._fused(params, backups):
                    self._manager.allreduce_tensors(params).wait()
                elif self._on_one_gpu(params):
                    self._average_bucketized(params)
                else:
                    self._average()
                if self._manager.should_commit():
                    self._save_parameters()
                else:
                    self._restore_parameters()
                return
        if (
            hb is not None
            and hb.owns(backups)
            and self._fused(params, hb.device_views)
            and self._manager.reduction_fails_only_at_launch()
        ):
            # backup in pinned host memory: the launch writes the average to the parameters and
            # to the backup's device-side staging buffer, which then crosses PCIe once
            if self._average_single_launch(params, hb.reserve()):
                hb.publish()
            return
        if self._fused(params, backups):
            if self._manager.reduction_fails_only_at_launch():
                self._average_single_launch(params, backups)
                return
            self._manager.allreduce_tensors(params).wait()
        elif _is_native_manager(self._manager) and self._on_one_gpu(params):
            self._sync_bucketized(params, backups)  # wherever the backup is kept
            return
        else:
            self._average()
        if self._manager.should_commit():
            self._save_parameters()
        else:
            self._restore_parameters()

    def _average_single_launch(self, params: List[torch.Tensor], backups: List[torch.Tensor]) -> bool:
        """A local reduction cannot fail once launched, so the commit decision is taken
        first and the sync is ONE launch: the average written to the parameters and the
        backup together, or (no commit) a plain restore.  Everything that can fail for a
        reason other than the launch itself (the quorum, finding the peers' buffers,
        building and validating the tensor table) happens before the vote and is latched
        like a failed all-reduce; a launch that fails after the vote raises, because the
        group has already counted the step as committed.

        The prepared launches are kept: as long as the parameters, the backups and the
        peers' buffers are the ones of the previous sync, nothing is rebuilt or compared
        tensor by tensor.  Returns whether the step was committed (``backups`` written)."""
        manager = self._manager
        manager.wait_quorum()  # should_commit reads the quorum's results (async quorum)
        launches = []
        mask = 0
        if manager.errored() is None:
            try:
                generation = self._generation
                replicas, mask = manager.replica_columns(params, identity=(id(self), generation))
                kept = self._launches.get("average")
                if kept is not None and kept[0] == generation and kept[1] is replicas:
                    launches = kept[2]
                else:
                    for idx in ops.dtype_groups(params):
                        outs = [[params[i] for i in idx], [backups[i] for i in idx]]
                        reps = [[rep[i] for i in idx] for rep in replicas]
                        key = f"average/{params[idx[0]].dtype}"
                        table = self._tables.get(key)
                        if table is None or not table.matches([*outs, *reps]):
                            table = ops.reduce_avg_table(outs, reps)
                        launches.append((key, outs, reps, table))
                    self._launches["average"] = (generation, replicas, launches)
            except Exception as e:  # same latch as Manager.allreduce
                logger.exception("got exception preparing the fused sync -- skipping: %s", e)
                manager.report_error(e)
                launches = []
        if manager.should_commit():
            assert launches, "a replica that failed to prepare cannot have voted to commit"
            for key, outs, reps, table in launches:
                self._tables[key] = ops.mt_reduce_avg(
                    outs, reps, mask, manager.num_participants(), table=table, table_is_current=True
                )
            return True
        self._restore_parameters()
        return False

    def _average_bucketized(self, params: List[torch.Tensor]) -> None:
        """Flatten (one launch), ONE ``manager.allreduce`` per dtype, unflatten (one launch): the
        average is in the parameters before the vote, as in the reference."""
        flats, views = self._flat_like("weights", params)
        self._tables["flatten"] = ops.mt_copy(views, params, table=self._tables.get("flatten"))
        works = [self._manager.allreduce(flat) for flat in flats.values()]
        for work in works:
            work.wait()
        if self._manager.errored() is None:
            self._tables["unflatten"] = ops.mt_copy(params, views, table=self._tables.get("unflatten"))

    def _sync_bucketized(self, params: List[torch.Tensor], backups: List[torch.Tensor]) -> None:
        """Through an ordinary process group: flatten (one launch), ONE collective per dtype
        that leaves the SUM in the flat buffer, and then, if the step is committed, ONE
        launch that divides by the number of participants and writes the average to the
        parameters and to the backup (what the reference does in four passes: divide,
        copy back, save; torchft/manager.py:287, torchft/local_sgd.py:121-125).  A step that
        is not committed only restores the parameters."""
        manager = self._manager
        flats, views = self._flat_like("weights", params)
        self._tables["flatten"] = ops.mt_copy(views, params, table=self._tables.get("flatten"))
        works = [manager.allreduce(flat, divide=False) for flat in flats.values()]
        for work in works:
            work.wait()
        if not manager.should_commit():
            self._restore_parameters()
            return
        hb = self._host_backup
        packed = hb is not None and hb.owns(backups)
        if self._together(params, backups):
            outs = [params, backups]
        elif packed:
            outs = [params, hb.reserve()]  # the backup's device-side staging buffer
        else:
            outs = [params]               # a backup kept elsewhere: saved below, tensor by tensor
        for idx in ops.dtype_groups(params):
            key = f"unflatten/{params[idx[0]].dtype}"
            self._tables[key] = ops.mt_reduce_avg(
                [[col[i] for i in idx] for col in outs], [[views[i] for i in idx]],
                1, manager.num_participants(), table=self._tables.get(key),
            )
        if packed:
            hb.publish()
        elif len(outs) == 1:
            self._save_parameters()

    def _average(self) -> None:
        works = []
        for p in self._param_objs:
            works.append(self._manager.allreduce(p.data.detach()))
        for work in works:
            work.wait()


def _fusable_sgd(
    optimizer: optim.Optimizer, params: Sequence[torch.Tensor]
) -> Optional[List[Tuple[List[int], ops.OuterSGD, bool]]]:
    """If ``optimizer`` is a plain ``torch.optim.SGD`` over exactly ``params``, returns one
    entry per (parameter group, dtype): (indices into ``params``, hyper-parameters,
    first_step); else None.  fp32, bf16 and fp16 parameters are fused (16-bit storage
    with fp32 arithmetic); the momentum buffer has the parameter's dtype, as torch's has."""
    if type(optimizer) is not optim.SGD:
        return None
    index = {p.data_ptr(): i for i, p in enumerate(params)}
    plan = []
    covered = 0
    for group in optimizer.param_groups:
        if group.get("maximize") or group.get("differentiable"):
            return None
        lr = group["lr"]
        if isinstance(lr, torch.Tensor):
            return None
        sgd = ops.OuterSGD(
            lr=float(lr),
            momentum=float(group["momentum"]),
            dampening=float(group["dampening"]),
            weight_decay=float(group["weight_decay"]),
            nesterov=bool(group["nesterov"]),
        )
        by_dtype: Dict[torch.dtype, Tuple[List[int], List[bool]]] = {}
        for p in group["params"]:
            i = index.get(p.data_ptr())
            if i is None or p.dtype not in _KERNEL_DTYPES:
                return None
            buf = optimizer.state.get(p, {}).get("momentum_buffer")
            if buf is not None and (buf.dtype != p.dtype or buf.device != p.device):
                return None
            idx, have_buf = by_dtype.setdefault(p.dtype, ([], []))
            idx.append(i)
            have_buf.append(buf is not None)
        for idx, have_buf in by_dtype.values():
            if any(have_buf) != all(have_buf):
                return None
            covered += len(idx)
            plan.append((idx, sgd, not all(have_buf)))
    if covered != len(params):
        return None
    return plan


_GROUP_FIELDS = ("momentum", "dampening", "weight_decay", "nesterov", "maximize", "differentiable")


def _groups_key(optimizer: optim.Optimizer) -> Tuple:
    """What ``_fusable_sgd`` reads from the parameter groups (an lr schedule changes it)."""
    return tuple(
        (id(g["params"]), len(g["params"]),
         g["lr"] if not isinstance(g["lr"], torch.Tensor) else id(g["lr"]),
         *[g.get(name) for name in _GROUP_FIELDS])
        for g in optimizer.param_groups
    )


class DiLoCo(LocalSGD):
    """DiLoCo (https://arxiv.org/pdf/2311.08105): the replicas average their
    pseudo-gradients ``params - backup`` and an outer optimizer applies the average
    to the parameters restored from the backup (torchft/local_sgd.py:177-239)."""

    _DTYPES = _KERNEL_DTYPES  # the outer step's arithmetic is fp32

    def __init__(
        self,
        manager: Manager,
        model: nn.Module,
        inner_optimizer: optim.Optimizer,
        outer_optimizer: optim.Optimizer,
        sync_every: int,
        backup_device: Optional[torch.device] = None,
        pin_memory: bool = True,
    ) -> None:
        if manager._use_async_quorum:
            raise ValueError(
                "Using DiLoCo require synchronous quorum to be enabled. "
                "Ensure that the manager is initialized with use_async_quorum=False"
            )
        self._outer_optimizer = outer_optimizer  # before super().__init__: see _placed_copies
        self._grads: Optional[List[torch.Tensor]] = None
        self._plan: Optional[_SgdPlan] = None
        super().__init__(manager, model, inner_optimizer, sync_every, backup_device, pin_memory)

    # -- buffers allocated with the backup ---------------------------------------
    def _wants_momentum(self) -> bool:
        opt = self._outer_optimizer
        return type(opt) is optim.SGD and any(g.get("momentum", 0) != 0 for g in opt.param_groups)

    def _wants_grad_buffers(self) -> bool:
        """Whether a sync will materialise the averaged pseudo-gradients per parameter: not
        when the whole step is one launch (they stay in registers), and not when the model
        is bucketised into one flat buffer per dtype."""
        manager = self._manager
        if not _is_native_manager(manager):
            return True  # the per-parameter manager.allreduce contract
        if not manager.supports_fused_sync():
            return False  # bucketised
        return not (manager.reduction_fails_only_at_launch() and type(self._outer_optimizer) is optim.SGD)

    def _placed_copies(self) -> int:
        """The backup, plus the outer momentum when a fusable SGD with momentum will create it,
        plus the pseudo-gradients where a sync needs them in memory: all found in ONE search
        at construction, none inside a sync."""
        return 1 + int(self._wants_momentum()) + int(self._wants_grad_buffers())

    def _keep_placed(self, extra: Sequence[List[torch.Tensor]]) -> None:
        extra = list(extra)
        if self._wants_momentum() and extra:
            self._placed_momentum = list(extra.pop(0))
        if self._wants_grad_buffers() and extra:
            self._placed_grads = extra.pop(0)

    def _grad_buffers(self, params: Sequence[torch.Tensor]) -> List[torch.Tensor]:
        """Pseudo-gradient storage, kept across syncs (the reference allocates it anew
        with every ``p.data - backup``)."""
        if self._grads is None or len(self._grads) != len(params) or any(
            g.shape != p.shape or g.device != p.device or g.dtype != p.dtype
            for g, p in zip(self._grads, params)
        ):
            placed, self._placed_grads = self._placed_grads, None
            if placed is not None and len(placed) == len(params) and all(
                g.shape == p.shape and g.device == p.device and g.dtype == p.dtype
                for g, p in zip(placed, params)
            ):
                # allocated with the backup, outside the parameters' HBM bank group (they are
                # written next to the parameters by the pseudo-gradient launch)
                self._grads = placed
            else:
                self._grads = [torch.empty_like(p) for p in params]
        return self._grads

    # -- the outer optimizer -------------------------------------------------------
    def _sgd_plan(self, params: Sequence[torch.Tensor]) -> Optional[List[Tuple[List[int], ops.OuterSGD, bool]]]:
        """``_fusable_sgd`` of the outer optimizer, recomputed only when something it depends
        on has changed: the parameters (generation), the groups' hyper-parameters, the
        optimizer's state mapping (replaced by ``load_state_dict``, grown or cleared), or a
        momentum buffer in it."""
        opt = self._outer_optimizer
        plan = self._plan
        groups_key = (self._generation, _groups_key(opt))
        if (
            plan is not None
            and plan.state is opt.state
            and plan.n_state == len(opt.state)
            and plan.groups_key == groups_key
            and (
                plan.slots is None
                or all(map(operator.is_, map(_MOMENTUM_OF, plan.slots), plan.bufs))
            )
        ):
            return plan.entries
        entries = _fusable_sgd(opt, params)
        bufs = slots = None
        if entries is not None and opt.state and not any(first for _, _, first in entries) and any(
            sgd.momentum != 0.0 for _, sgd, _ in entries
        ):
            try:
                slots = [opt.state[p] for p in self._param_objs]
                bufs = [slot["momentum_buffer"] for slot in slots]
            except KeyError:
                slots = bufs = None
        self._plan = _SgdPlan(entries, opt.state, len(opt.state), groups_key, bufs, slots)
        if entries is None:
            # the outer optimizer runs its own step(): buffers set aside for a fused one are
            # not going to be used
            self._placed_momentum = None
        return entries

    def _momentum_buffers(self, idx: Sequence[int], first: bool) -> List[torch.Tensor]:
        """The outer SGD's momentum buffers; on the first step fresh tensors that are
        not yet part of the optimizer state (see ``_attach_momentum``)."""
        live = self._param_objs
        placed = self._placed_momentum
        if first:
            if placed is not None and all(
                placed[i] is not None
                and placed[i].shape == live[i].shape
                and placed[i].dtype == live[i].dtype for i in idx
            ):
                return [placed[i] for i in idx]
            key = "momentum/" + ",".join(map(str, idx[:4])) + f"/{len(idx)}"
            return self._flat_like(key, [live[i].data for i in idx])[1]
        plan = self._plan
        if plan is not None and plan.bufs is not None:
            bufs = [plan.bufs[i] for i in idx]
        else:
            bufs = [self._outer_optimizer.state[live[i]]["momentum_buffer"] for i in idx]
        if placed is not None:
            # where the optimizer state was replaced (a load_state_dict after healing) the
            # buffer set aside for it at construction is not in use any more: let it go
            for b, i in zip(bufs, idx):
                if placed[i] is not None and b.data_ptr() != placed[i].data_ptr():
                    placed[i] = None
            if all(t is None for t in placed):
                self._placed_momentum = None
        return bufs

    def _attach_momentum(self, idx: Sequence[int], bufs: Sequence[torch.Tensor]) -> None:
        """After a committed first step the buffers become optimizer state, exactly where
        torch.optim.SGD keeps them."""
        live = self._param_objs
        for i, buf in zip(idx, bufs):
            self._outer_optimizer.state[live[i]]["momentum_buffer"] = buf
        self._plan = None  # the next sync is a steady-state step

    def _outer_step(
        self,
        params: List[torch.Tensor],
        backups: List[torch.Tensor],
        grads: List[torch.Tensor],
        plan: Optional[List[Tuple[List[int], ops.OuterSGD, bool]]],
        grads_are_sums_of: Optional[int] = None,
    ) -> None:
        """Committed: apply the outer optimizer to the restored parameters and refresh the
        backup (torchft/local_sgd.py:221-224).  ``grads_are_sums_of=n`` (fusable SGD only): the
        gradient buffers hold sums over n participants, divided inside the launch."""
        if plan is None:
            assert grads_are_sums_of is None
            self._outer_optimizer.step()
            self._save_parameters()
            return
        for gi, (idx, sgd, first) in enumerate(plan):
            bufs = self._momentum_buffers(idx, first) if sgd.momentum != 0.0 else None
            key = f"outer_sgd/{gi}"
            self._tables[key] = ops.mt_outer_sgd(
                [params[i] for i in idx],
                [backups[i] for i in idx],
                bufs,
                [grads[i] for i in idx],
                sgd,
                first,
                table=self._tables.get(key),
                grads_are_sums_of=grads_are_sums_of,
            )
            if first and bufs is not None:
                self._attach_momentum(idx, bufs)

    def _perform_sync(self) -> None:
        """Pseudo-gradients, their average over the replicas, restore, and (on commit)
        the outer step plus backup refresh (torchft/local_sgd.py:205-225)."""
        _, params, backups = self._named()
        if self._together(params, backups):
            self._sync_with(params, backups)
            return
        if not self._on_one_gpu(params):
            raise RuntimeError(
                "DiLoCo needs its parameters on one GPU (the kernels have no CPU path)"
            )
        # The backup is kept elsewhere: in host memory (``backup_device="cpu"``) or in tensors
        # the user has put in place.  The reference moves every backup tensor to the
        # parameter's device for the subtraction (torchft/local_sgd.py:214); here the backup
        # is brought into device buffers once per sync, the kernels work on those, and after a
        # committed step they are written back.
        hb = self._host_backup
        packed = hb is not None and hb.owns(backups)
        if packed:
            mirror = hb.load()
        else:
            mirror = self._flat_like("backup_mirror", params)[1]
            for m, b in zip(mirror, backups):
                m.copy_(b, non_blocking=True)
        if self._sync_with(params, mirror):
            if packed:
                hb.publish()
            else:
                for b, m in zip(backups, mirror):
                    b.copy_(m, non_blocking=True)
                if any(not b.is_cuda for b in backups):
                    torch.cuda.current_stream(params[0].device).synchronize()

    def _sync_with(self, params: List[torch.Tensor], backups: List[torch.Tensor]) -> bool:
        """One sync over device-resident ``backups``.  Returns whether the kernels have
        rewritten them (a committed step with a fusable outer SGD); any other outer optimizer
        refreshes ``_backup_parameters`` itself through ``_save_parameters``."""
        live = self._param_objs
        plan = self._sgd_plan(params)
        fused = self._fused(params, backups)

        if fused and plan is not None and self._manager.reduction_fails_only_at_launch():
            committed = self._sync_single_launch(params, backups, plan)
            self._outer_optimizer.zero_grad()
            return committed

        bucketized = not fused and _is_native_manager(self._manager)
        grads = self._flat_like("grads", params)[1] if bucketized else self._grad_buffers(params)
        # The reference restores the parameters before the vote (torchft/local_sgd.py:219) because
        # its optimizer then steps on them.  The fused outer SGD computes the new parameters from
        # the backup and the averaged pseudo-gradient and overwrites the parameters without
        # reading them, so on a committed step the restore would be written for nothing (one
        # model-sized stream): with a fusable optimizer it is done only when the step is NOT
        # committed.  Any other optimizer gets its restore first, as in the reference.
        restore_first = plan is None
        restored = False
        sums_of: Optional[int] = None  # -1: the gradient buffers hold sums over the participants
        if fused:
            # pseudo-gradient, replica sum and divide (and the restore, if it comes first): one launch
            for p, g in zip(live, grads):
                p.grad = g
            self._manager.pseudograd_allreduce(grads, params, backups, restore_params=restore_first).wait()
            restored = restore_first and self._manager.errored() is None
        elif bucketized:
            # pseudo-gradients written straight into one flat buffer by one launch, then ONE
            # collective for the whole model
            self._local_pseudograd(grads, params, backups, restore_params=restore_first)
            restored = restore_first
            for p, g in zip(live, grads):
                p.grad = g
            # with a fusable SGD the collective leaves the SUM in the buffer and the outer
            # step divides on the way in (no pass of its own over the buffer for the division)
            sums_of = -1 if plan is not None else None
            works = [self._manager.allreduce(flat, divide=plan is None)
                     for flat in self._flat_like("grads", params)[0].values()]
            for work in works:
                work.wait()
        else:
            # pseudo-gradients in one launch, then the Manager contract per parameter
            self._local_pseudograd(grads, params, backups, restore_params=False)
            for p, g in zip(live, grads):
                p.grad = g
            self._average_grads()
        if restore_first and not restored:
            self._restore_from(params, backups)
            restored = True

        committed = self._manager.should_commit()
        if committed:
            if sums_of is not None:
                sums_of = self._manager.num_participants()
            self._outer_step(params, backups, grads, plan, grads_are_sums_of=sums_of)
        elif not restored:
            self._restore_from(params, backups)
        self._outer_optimizer.zero_grad()
        return committed and plan is not None

    def _restore_from(self, params: List[torch.Tensor], backups: List[torch.Tensor]) -> None:
        """``_restore_parameters`` from the device-resident form of the backup this sync works
        on (the bound backup itself, or its mirror)."""
        bound = self._bound
        if bound is not None and bound.backups is backups:
            self._restore_parameters()
        else:
            self._copy("restore_mirror", params, backups, blocking=True)

    def _local_pseudograd(
        self,
        grads: List[torch.Tensor],
        params: List[torch.Tensor],
        backups: List[torch.Tensor],
        restore_params: bool,
    ) -> None:
        """This replica's own pseudo-gradients ``params - backups`` (torchft/local_sgd.py:212-215),
        one launch per dtype; optionally restores the parameters in the same pass."""
        for idx in ops.dtype_groups(params):
            key = f"pseudograd/{params[idx[0]].dtype}"
            sub = [[col[i] for i in idx] for col in (grads, params, backups)]
            self._tables[key] = ops.mt_pseudograd_avg(
                sub[0], sub[1], sub[2], [sub[1]], restore_params=restore_params,
                table=self._tables.get(key),
            )

    def _sync_single_launch(
        self,
        params: List[torch.Tensor],
        backups: List[torch.Tensor],
        plan: List[Tuple[List[int], ops.OuterSGD, bool]],
    ) -> bool:
        """The reduction is local and cannot fail once launched, so the commit decision
        can be taken first and the whole sync becomes one launch per parameter group:
        either the fully fused step, or (no commit) a plain restore.  The prepared launches
        (tensor lists and their validated table) are kept for as long as the parameters,
        the backups, the plan and the peers' buffers are those of the previous sync.  Returns
        whether the step was committed."""
        manager = self._manager
        manager.wait_quorum()
        launches = []
        mask = 0
        if manager.errored() is None:
            try:
                generation = self._generation
                replicas, mask = manager.replica_columns(params, identity=(id(self), generation))
                kept = self._launches.get("fused")
                if (
                    kept is not None
                    and kept[0] == generation
                    and kept[1] is replicas
                    and kept[2] is plan
                ):
                    launches = kept[3]
                else:
                    for gi, (idx, sgd, first) in enumerate(plan):
                        bufs = self._momentum_buffers(idx, first) if sgd.momentum != 0.0 else None
                        cols = dict(
                            params=[params[i] for i in idx],
                            backups=[backups[i] for i in idx],
                            bufs=bufs,
                            replicas=[[rep[i] for i in idx] for rep in replicas],
                        )
                        key = f"fused/{gi}"
                        # built (and validated) before the vote: after it only the launch is left
                        table = ops.diloco_outer_table(
                            cols["params"], cols["backups"], bufs, cols["replicas"],
                            table=self._tables.get(key),
                        )
                        launches.append((key, idx, cols, sgd, first, table))
                    if not any(first for _, _, first in plan):
                        # a first step is prepared once only (its buffers become state)
                        self._launches["fused"] = (generation, replicas, plan, launches)
            except Exception as e:  # same latch as Manager.allreduce
                logger.exception("got exception preparing the fused sync -- skipping: %s", e)
                manager.report_error(e)
                launches = []
        if manager.should_commit():
            assert launches or not params, "a replica that failed to prepare cannot have voted to commit"
            for key, idx, cols, sgd, first, table in launches:
                self._tables[key] = ops.mt_diloco_outer(
                    cols["params"], cols["backups"], cols["bufs"], cols["replicas"], sgd, first,
                    mask, manager.num_participants(), table=table, table_is_current=True,
                )
                if first and cols["bufs"] is not None:
                    self._attach_momentum(idx, cols["bufs"])
            return True
        self._restore_from(params, backups)
        return False

    def _average_grads(self) -> None:
        """One ``manager.allreduce`` per pseudo-gradient (torchft/local_sgd.py:227-239)."""
        works = []
        for p in self._param_objs:
            assert p.grad is not None
            works.append(self._manager.allreduce(p.grad))
        for work in works:
            work.wait()
