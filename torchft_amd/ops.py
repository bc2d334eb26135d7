"""Tensor-level wrappers over the C ABI (one kernel launch each).

Every function validates shapes on the host before anything is launched and
enqueues on torch's current stream of the tensors' device.  None of them
allocates, synchronises or falls back to torch arithmetic.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from . import _native
from .multi_tensor import (
    TensorTable,
    current_stream_handle,
    dtype_code,
    require_device_tensor,
)

MAX_REPLICAS = _native.MAX_REPLICAS


@dataclass(frozen=True)
class OuterSGD:
    """Hyper-parameters of the outer torch.optim.SGD (reference: local_sgd_test.py:112-114)."""

    lr: float
    momentum: float = 0.0
    dampening: float = 0.0
    weight_decay: float = 0.0
    nesterov: bool = False

    def to_struct(self, first_step: bool) -> _native.SgdParams:
        return _native.SgdParams(
            self.lr,
            self.momentum,
            self.dampening,
            self.weight_decay,
            1 if self.nesterov else 0,
            1 if first_step else 0,
        )


def check_tensor(t: torch.Tensor, what: str) -> None:
    """Raises for a tensor the replica average cannot take: not on a GPU, not contiguous, or
    of a dtype other than fp32 / bf16 / fp16 / fp64."""
    require_device_tensor(t, what)
    dtype_code(t.dtype)


def full_mask(n_replicas: int) -> int:
    return (1 << n_replicas) - 1


def _check_reduce_args(n_replicas: int, participate_mask: int, num_participants: int) -> None:
    if n_replicas > MAX_REPLICAS:
        raise ValueError(f"{n_replicas} replicas; one launch takes at most {MAX_REPLICAS}")
    if participate_mask < 0 or participate_mask >> n_replicas:
        raise ValueError(f"participate_mask {participate_mask:#x} names replicas >= {n_replicas}")
    if num_participants < 1:
        raise ValueError(f"num_participants must be >= 1, got {num_participants}")


def reduce_avg_(
    out: torch.Tensor,
    replicas: Sequence[torch.Tensor],
    participate_mask: Optional[int] = None,
    num_participants: Optional[int] = None,
) -> torch.Tensor:
    """out = (sum of participating replicas) / num_participants over one flat buffer.

    ``out`` may be one of ``replicas`` (the in-place form Manager.allreduce needs).
    """
    n = len(replicas)
    mask = full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    _check_reduce_args(n, mask, nump)
    require_device_tensor(out, "reduce_avg_: out")
    code = dtype_code(out.dtype)
    for r, x in enumerate(replicas):
        require_device_tensor(x, f"reduce_avg_: replica {r}")
        if x.dtype != out.dtype or x.numel() != out.numel() or x.device != out.device:
            raise ValueError(
                f"reduce_avg_: replica {r} is {x.dtype}[{x.numel()}] on {x.device}, "
                f"out is {out.dtype}[{out.numel()}] on {out.device}"
            )
    ptrs = (ctypes.c_void_p * max(n, 1))(*[x.data_ptr() for x in replicas])
    with torch.cuda.device(out.device):
        rc = _native.lib().tft_reduce_avg(
            out.data_ptr(), ptrs, n, mask, nump, out.numel(), code, current_stream_handle(out.device)
        )
    _native.check(rc, "tft_reduce_avg")
    return out


def _launch(table: TensorTable, fn_name: str, *args) -> None:
    if table.total_chunks == 0:
        return
    with torch.cuda.device(table.device):
        rc = getattr(_native.lib(), fn_name)(table.ref(), *args, current_stream_handle(table.device))
    _native.check(rc, fn_name)


def reduce_avg_table(
    outs: Sequence[Sequence[torch.Tensor]], replicas: Sequence[Sequence[torch.Tensor]]
) -> TensorTable:
    if len(outs) not in (1, 2):
        raise ValueError("one or two output columns")
    return TensorTable([*outs, *replicas], what="mt_reduce_avg")


def mt_reduce_avg(
    outs: Sequence[Sequence[torch.Tensor]],
    replicas: Sequence[Sequence[torch.Tensor]],
    participate_mask: Optional[int] = None,
    num_participants: Optional[int] = None,
    table: Optional[TensorTable] = None,
    table_is_current: bool = False,
) -> TensorTable:
    """outs[j][t] = (sum_r replicas[r][t]) / n for every tensor t, in one launch.
    ``table_is_current``: the caller has just built or matched ``table`` against exactly
    these tensors, so it is not compared with them again."""
    n = len(replicas)
    mask = full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    _check_reduce_args(n, mask, nump)
    if table is None or not (table_is_current or table.matches([*outs, *replicas])):
        table = reduce_avg_table(outs, replicas)
    _launch(table, "tft_mt_reduce_avg", len(outs), n, mask, nump, table.dtype_code)
    return table


def diloco_outer_table(
    params: Sequence[torch.Tensor],
    backups: Sequence[torch.Tensor],
    bufs: Optional[Sequence[torch.Tensor]],
    replicas: Sequence[Sequence[torch.Tensor]],
    table: Optional[TensorTable] = None,
) -> TensorTable:
    """The tensor table of :func:`mt_diloco_outer` (validates devices, dtypes and sizes;
    ``table`` is returned as is when it still describes the same tensors)."""
    cols = [params, backups, bufs if bufs is not None else backups, *replicas]
    if table is not None and table.matches(cols):
        return table
    return TensorTable(cols, what="mt_diloco_outer")


def mt_diloco_outer(
    params: Sequence[torch.Tensor],
    backups: Sequence[torch.Tensor],
    bufs: Optional[Sequence[torch.Tensor]],
    replicas: Sequence[Sequence[torch.Tensor]],
    sgd: OuterSGD,
    first_step: bool,
    participate_mask: Optional[int] = None,
    num_participants: Optional[int] = None,
    table: Optional[TensorTable] = None,
    table_is_current: bool = False,
) -> TensorTable:
    """Fused DiLoCo outer step (pseudo-gradient, average, Nesterov SGD, backup refresh);
    fp32, or bf16 / fp16 storage with fp32 arithmetic and one rounding on store.
    ``table_is_current``: ``table`` comes from :func:`diloco_outer_table` for exactly these
    tensors and is not compared with them again."""
    n = len(replicas)
    mask = full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    _check_reduce_args(n, mask, nump)
    if sgd.momentum != 0.0 and bufs is None:
        raise ValueError("momentum != 0 needs momentum buffers")
    if table is None or not table_is_current:
        table = diloco_outer_table(params, backups, bufs, replicas, table)
    _launch(
        table, "tft_mt_diloco_outer", n, mask, nump, table.dtype_code,
        ctypes.byref(sgd.to_struct(first_step)),
    )
    return table


def mt_pseudograd_avg(
    grads: Sequence[torch.Tensor],
    params: Sequence[torch.Tensor],
    backups: Sequence[torch.Tensor],
    replicas: Sequence[Sequence[torch.Tensor]],
    restore_params: bool,
    participate_mask: Optional[int] = None,
    num_participants: Optional[int] = None,
    table: Optional[TensorTable] = None,
) -> TensorTable:
    """grads = (sum_r (replica_r - backup)) / n; optionally params = backup."""
    n = len(replicas)
    mask = full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    _check_reduce_args(n, mask, nump)
    cols = [grads, params, backups, *replicas]
    if table is None or not table.matches(cols):
        table = TensorTable(cols, what="mt_pseudograd_avg")
    _launch(
        table, "tft_mt_pseudograd_avg", n, mask, nump, table.dtype_code, 1 if restore_params else 0
    )
    return table


def mt_outer_sgd(
    params: Sequence[torch.Tensor],
    backups: Sequence[torch.Tensor],
    bufs: Optional[Sequence[torch.Tensor]],
    grads: Sequence[torch.Tensor],
    sgd: OuterSGD,
    first_step: bool,
    table: Optional[TensorTable] = None,
    grads_are_sums_of: Optional[int] = None,
) -> TensorTable:
    """SGD update from backups with grads; writes params, backups (and momentum buffers).
    ``grads_are_sums_of=n``: ``grads`` holds the sum a collective left in it, and every
    element is divided by n (rounded to the storage dtype) on the way into the update -
    the division ``Manager.allreduce`` otherwise does in a pass of its own."""
    if sgd.momentum != 0.0 and bufs is None:
        raise ValueError("momentum != 0 needs momentum buffers")
    cols = [params, backups, bufs if bufs is not None else backups, grads]
    if table is None or not table.matches(cols):
        table = TensorTable(cols, what="mt_outer_sgd")
    if grads_are_sums_of is None:
        _launch(
            table, "tft_mt_outer_sgd", table.dtype_code, ctypes.byref(sgd.to_struct(first_step))
        )
    else:
        if grads_are_sums_of < 1:
            raise ValueError("grads_are_sums_of must be at least 1")
        _launch(
            table, "tft_mt_outer_sgd_of_sum", int(grads_are_sums_of), table.dtype_code,
            ctypes.byref(sgd.to_struct(first_step)),
        )
    return table


def mt_copy(
    dsts: Sequence[torch.Tensor],
    srcs: Sequence[torch.Tensor],
    table: Optional[TensorTable] = None,
) -> TensorTable:
    """dsts[t] <- srcs[t] byte for byte, all tensors in one launch."""
    cols = [dsts, srcs]
    if table is None or not table.matches(cols):
        table = TensorTable(cols, as_bytes=True, what="mt_copy")
    _launch(table, "tft_mt_copy_bytes")
    return table


def dtype_groups(tensors: Sequence[torch.Tensor]) -> List[List[int]]:
    """Indices of ``tensors`` grouped by dtype, groups in order of first appearance.  One
    launch covers one dtype (the kernels are instantiated per element type), so a model
    with bf16 weights and fp32 norms synchronises in two launches."""
    groups: dict = {}
    for i, t in enumerate(tensors):
        groups.setdefault(t.dtype, []).append(i)
    return list(groups.values())


def flat_views(flat: torch.Tensor, like: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    """Views of ``flat`` laid out back to back with the sizes of ``like`` (no padding)."""
    views = []
    offset = 0
    for t in like:
        views.append(flat[offset : offset + t.numel()].view(t.shape))
        offset += t.numel()
    if offset != flat.numel():
        raise ValueError(f"flat buffer has {flat.numel()} elements, tensors need {offset}")
    return views
