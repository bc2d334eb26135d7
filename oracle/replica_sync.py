"""TEST INFRASTRUCTURE - not part of the product.

CPU restatement of torchft's replica-sync path with the same stock torch ops
the reference calls, tensor by tensor, in the reference's own loop order.  Only
``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg may
import this module; the product (``torchft_amd``) never does.

The reference is Python whose arithmetic lives in torch (an unpinned
dependency, ``pyproject.toml:14-16``; this image has torch 2.10).  Nothing of
the reference is imported here: every function restates the cited lines over
explicit tensors, with the N replicas of a real job simulated by N tensor
lists in one process and the all-reduce taken as a sequential sum in replica
order.

How each function is pinned (tests/test_oracle.py):
  manager_allreduce_     reference-held known answers: 1.0 with n=5 -> 0.2 and
                         healing -> 0.0 (torchft/manager_test.py:520-543),
                         [1]+[2]=[3] (torchft/process_group_test.py:185-203);
                         float64 brute force
  sgd_step_              torch.optim.SGD itself (library routine), closed forms
  diloco_perform_sync    composition check against torch.optim.SGD fed with a
                         float64-checked pseudo-gradient; fixed point; N=1
                         special case; cross-replica identity
                         (torchft/manager_integ_test.py:553-562); the
                         fp32-arithmetic variant for bf16 / fp16 storage against
                         a float64 evaluation (within one rounding of the storage
                         dtype) and against the dtype-native form (the stated
                         tolerance rtol 1e-2)
  localsgd_perform_sync  closed form mean; commit / no-commit invariants
                         (torchft/local_sgd_test.py:65-67, 98-101)
  bucket_assignment      torch's dist._compute_bucket_assignment_by_size and a
                         real DDP comm-hook probe
  ddp_bucket_average     torch.cat / split identities
  state-dict round trip  torch.save -> torch.load of the same dict
The plain-C twin (replica_sync_c.c) is checked against this module bit for bit.
"""

from __future__ import annotations

import ctypes
import io
import os
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

# ---------------------------------------------------------------------------
# Manager.allreduce arithmetic
# ---------------------------------------------------------------------------


def manager_allreduce_(
    contributions: Sequence[torch.Tensor],
    participating: Sequence[bool],
    num_participants: int,
    accumulate_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """What every replica holds after ``Manager.allreduce`` (torchft/manager.py:242-303).

    ``contributions[r]`` is the tensor replica r passes in.  Follows
    manager.py:267-268 (a non-participating replica zeroes its tensor first),
    :274 (all-reduce SUM; here r = 0..N-1 in order) and :287
    (``tensor /= num_participants()``, a true divide).

    ``accumulate_dtype=None`` sums in the tensors' own dtype, which is what a
    c10d backend does (bf16 sums in bf16).  ``torch.float32`` widens first and
    rounds once at the end: the fp32-accumulate variant the kernels implement.
    Returns a new tensor; inputs are not modified.
    """
    assert len(contributions) == len(participating)
    first = contributions[0]
    acc_dtype = accumulate_dtype or first.dtype
    total: Optional[torch.Tensor] = None
    for x, part in zip(contributions, participating):
        x = x.detach().to(acc_dtype, copy=True)
        if not part:
            x.zero_()  # manager.py:268
        total = x if total is None else total.add_(x)  # manager.py:274
    assert total is not None
    total /= num_participants  # manager.py:287
    return total.to(first.dtype)


# ---------------------------------------------------------------------------
# Outer optimizer: torch.optim.SGD, single-tensor form
# ---------------------------------------------------------------------------


def sgd_step_(
    param: torch.Tensor,
    grad: torch.Tensor,
    buf: Optional[torch.Tensor],
    lr: float,
    momentum: float = 0.0,
    dampening: float = 0.0,
    weight_decay: float = 0.0,
    nesterov: bool = False,
) -> Optional[torch.Tensor]:
    """One ``torch.optim.SGD`` update of ``param`` in place; returns the momentum buffer.

    This is the optimizer the reference drives at torchft/local_sgd.py:223
    (configured at torchft/local_sgd_test.py:112-114).  ``buf is None`` means
    the state does not exist yet (first step): the buffer becomes a clone of
    the gradient.
    """
    g = grad
    if weight_decay != 0:
        g = g.add(param, alpha=weight_decay)
    if momentum != 0:
        if buf is None:
            buf = g.detach().clone()
        else:
            buf.mul_(momentum).add_(g, alpha=1 - dampening)
        g = g.add(buf, alpha=momentum) if nesterov else buf
    param.add_(g, alpha=-lr)
    return buf


# ---------------------------------------------------------------------------
# DiLoCo / LocalSGD sync
# ---------------------------------------------------------------------------


def diloco_perform_sync(
    replica_params: Sequence[Sequence[torch.Tensor]],
    backup: Sequence[torch.Tensor],
    momentum_bufs: Optional[Sequence[Optional[torch.Tensor]]],
    participating: Sequence[bool],
    num_participants: int,
    commit: bool,
    lr: float,
    momentum: float = 0.0,
    dampening: float = 0.0,
    weight_decay: float = 0.0,
    nesterov: bool = False,
    accumulate_dtype: Optional[torch.dtype] = None,
    grads_through_storage: bool = False,
) -> Dict[str, List[Optional[torch.Tensor]]]:
    """``DiLoCo._perform_sync`` (torchft/local_sgd.py:205-225) for one replica group.

    Because every replica ends with identical params/backup/momentum
    (torchft/manager_integ_test.py:553-562) one result set is returned:
    ``{"params", "backup", "momentum", "grads"}``; ``grads`` is the averaged
    pseudo-gradient the reference stores in ``p.grad`` before ``zero_grad``.

    ``accumulate_dtype=None`` is the reference itself: every torch op runs in the
    tensors' own dtype (for bf16 parameters each subtraction, sum, division and
    optimizer op rounds to bf16).  ``accumulate_dtype=torch.float32`` is the
    fp32-arithmetic variant the kernels implement for 16-bit storage: the same
    ops in the same order on values widened to fp32, each output rounded to the
    storage dtype once.  ``grads_through_storage`` additionally rounds the
    averaged pseudo-gradient to the storage dtype before the optimizer reads it
    (the two-launch form, where it passes through memory between the launches).
    """
    n_tensors = len(backup)
    params: List[torch.Tensor] = []
    new_backup: List[torch.Tensor] = []
    new_bufs: List[Optional[torch.Tensor]] = []
    grads: List[torch.Tensor] = []
    for t in range(n_tensors):
        store = backup[t].dtype
        work = accumulate_dtype or store
        b = backup[t].detach().to(work)
        # local_sgd.py:212-215, on every replica
        pseudo = [rp[t].detach().to(work) - b for rp in replica_params]
        # local_sgd.py:227-239 -> manager.py:267-287
        g = manager_allreduce_(pseudo, participating, num_participants)
        if grads_through_storage:
            g = g.to(store).to(work)
        p = b.clone()  # local_sgd.py:219 (_restore_parameters)
        buf = None if momentum_bufs is None or momentum_bufs[t] is None else momentum_bufs[t].to(work, copy=True)
        nb = b.clone()
        if commit:  # local_sgd.py:221-224
            buf = sgd_step_(p, g, buf, lr, momentum, dampening, weight_decay, nesterov)
            nb = p.clone()
        params.append(p.to(store))
        new_backup.append(nb.to(store))
        new_bufs.append(None if buf is None else buf.to(store))
        grads.append(g.to(store))
    return {"params": params, "backup": new_backup, "momentum": new_bufs, "grads": grads}


def localsgd_perform_sync(
    replica_params: Sequence[Sequence[torch.Tensor]],
    backup: Sequence[torch.Tensor],
    participating: Sequence[bool],
    num_participants: int,
    commit: bool,
) -> Dict[str, List[torch.Tensor]]:
    """``LocalSGD._perform_sync`` (torchft/local_sgd.py:151-174): average the weights
    themselves; commit -> backup <- params (:157-158), else params <- backup (:160-162)."""
    params: List[torch.Tensor] = []
    new_backup: List[torch.Tensor] = []
    for t in range(len(backup)):
        avg = manager_allreduce_(
            [rp[t].detach() for rp in replica_params], participating, num_participants
        )
        if commit:
            params.append(avg)
            new_backup.append(avg.clone())
        else:
            params.append(backup[t].clone())
            new_backup.append(backup[t].clone())
    return {"params": params, "backup": new_backup}


# ---------------------------------------------------------------------------
# DDP buckets
# ---------------------------------------------------------------------------

DEFAULT_FIRST_BUCKET_BYTES = 1024 * 1024
DEFAULT_BUCKET_CAP_BYTES = 25 * 1024 * 1024


def bucket_assignment(
    numels: Sequence[int],
    element_size: int,
    first_cap: int = DEFAULT_FIRST_BUCKET_BYTES,
    cap: int = DEFAULT_BUCKET_CAP_BYTES,
) -> List[List[int]]:
    """Parameter indices per DDP bucket, in the order the Reducer fires them.

    Rule of torch's Reducer as driven from torchft/ddp.py:52-63 (one dtype, one
    device): walk parameters in declaration order, append to the open bucket, close
    it once its byte size reaches the current cap (first bucket ``first_cap``,
    later ones ``cap``); a tensor is never split; the resulting list is reversed
    because gradients become ready back to front.
    """
    buckets: List[List[int]] = []
    current: List[int] = []
    size = 0
    limit = first_cap
    for i, n in enumerate(numels):
        current.append(i)
        size += n * element_size
        if size >= limit:
            buckets.append(current)
            current, size, limit = [], 0, cap
    if current:
        buckets.append(current)
    return list(reversed(buckets))


def bucket_offsets(numels: Sequence[int], bucket: Sequence[int]) -> List[int]:
    """Element offset of each parameter inside its flat bucket: running numel, no padding."""
    offs, off = [], 0
    for i in bucket:
        offs.append(off)
        off += numels[i]
    return offs


def ddp_bucket_average(
    replica_grads: Sequence[Sequence[torch.Tensor]],
    participating: Sequence[bool],
    num_participants: int,
    buckets: Sequence[Sequence[int]],
    accumulate_dtype: Optional[torch.dtype] = None,
) -> List[torch.Tensor]:
    """Flatten -> ``Manager.allreduce`` -> unflatten, bucket by bucket
    (torchft/ddp.py:65-71 inside torch's Reducer copy-in / copy-out)."""
    out: List[Optional[torch.Tensor]] = [None] * len(replica_grads[0])
    for bucket in buckets:
        flats = [torch.cat([g[i].reshape(-1) for i in bucket]) for g in replica_grads]
        avg = manager_allreduce_(flats, participating, num_participants, accumulate_dtype)
        off = 0
        for i in bucket:
            n = replica_grads[0][i].numel()
            out[i] = avg[off : off + n].view(replica_grads[0][i].shape).clone()
            off += n
    return out  # type: ignore[return-value]


# ---------------------------------------------------------------------------
# Checkpoint transport
# ---------------------------------------------------------------------------


def state_dict_round_trip(state_dict: object) -> object:
    """What the receiving replica ends up with: ``torch.save`` on the sender
    (torchft/checkpointing.py:164) and ``torch.load(weights_only=False)`` on the
    receiver (:197-203).  Only ever applied to dicts built by the caller."""
    buf = io.BytesIO()
    torch.save(state_dict, buf)
    buf.seek(0)
    return torch.load(buf, weights_only=False)


def gather_bytes(tensors: Sequence[torch.Tensor], offsets: Sequence[int], total: int) -> np.ndarray:
    """Byte image of a staging buffer holding each tensor's raw bytes at its offset
    (zero elsewhere): the layout check for the device-side pack."""
    out = np.zeros(total, dtype=np.uint8)
    for t, off in zip(tensors, offsets):
        raw = t.detach().cpu().contiguous().reshape(-1).view(torch.uint8).numpy()
        out[off : off + raw.size] = raw
    return out


# ---------------------------------------------------------------------------
# The plain-C twin
# ---------------------------------------------------------------------------

_C_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_build", "liboracle.so")


class _SgdC(ctypes.Structure):
    _fields_ = [
        ("lr", ctypes.c_float),
        ("momentum", ctypes.c_float),
        ("dampening", ctypes.c_float),
        ("weight_decay", ctypes.c_float),
        ("nesterov", ctypes.c_int32),
        ("first_step", ctypes.c_int32),
    ]


def c_lib() -> ctypes.CDLL:
    if not os.path.exists(_C_LIB_PATH):
        raise RuntimeError(f"{_C_LIB_PATH} missing: run `make -C oracle`")
    return ctypes.CDLL(_C_LIB_PATH)


def _ptr_array(tensors: Sequence[torch.Tensor]):
    return (ctypes.c_void_p * max(len(tensors), 1))(*[t.data_ptr() for t in tensors])


def c_reduce_avg(
    replicas: Sequence[torch.Tensor], mask: int, num_participants: int
) -> torch.Tensor:
    out = torch.empty_like(replicas[0])
    fn = c_lib().oracle_reduce_avg_f32 if out.dtype == torch.float32 else c_lib().oracle_reduce_avg_bf16
    fn(
        ctypes.c_void_p(out.data_ptr()),
        _ptr_array(replicas),
        ctypes.c_uint32(len(replicas)),
        ctypes.c_uint32(mask),
        ctypes.c_uint32(num_participants),
        ctypes.c_uint64(out.numel()),
    )
    return out


def c_diloco_outer(
    backup: torch.Tensor,
    buf: Optional[torch.Tensor],
    replicas: Sequence[torch.Tensor],
    mask: int,
    num_participants: int,
    lr: float,
    momentum: float,
    dampening: float,
    weight_decay: float,
    nesterov: bool,
    first_step: bool,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Returns (params, backup, momentum) after the fused step; inputs untouched."""
    p = torch.empty_like(backup)
    b = backup.clone()
    m = buf.clone() if buf is not None else (torch.zeros_like(backup) if momentum != 0 else None)
    k = _SgdC(lr, momentum, dampening, weight_decay, int(nesterov), int(first_step))
    c_lib().oracle_diloco_outer_f32(
        ctypes.c_void_p(p.data_ptr()),
        ctypes.c_void_p(b.data_ptr()),
        ctypes.c_void_p(m.data_ptr() if m is not None else None),
        _ptr_array(replicas),
        ctypes.c_uint32(len(replicas)),
        ctypes.c_uint32(mask),
        ctypes.c_uint32(num_participants),
        ctypes.byref(k),
        ctypes.c_uint64(p.numel()),
    )
    return p, b, m


# ---------------------------------------------------------------------------
# The reference loop as a timed CPU baseline
# ---------------------------------------------------------------------------


def make_gloo_world1():
    """A ``ProcessGroupGloo`` of world size 1 over an in-process store: the backend the
    reference's own tests run this path on (torchft/process_group.py:303-317)."""
    import datetime

    import torch.distributed as dist

    store = dist.HashStore()
    return dist.ProcessGroupGloo(store, 0, 1, datetime.timedelta(seconds=60))


def diloco_reference_loop_(
    pg,
    params: Sequence[torch.Tensor],
    backup: Sequence[torch.Tensor],
    peers: Sequence[Sequence[torch.Tensor]],
    outer_optimizer: torch.optim.Optimizer,
    num_participants: int,
) -> None:
    """One committed DiLoCo sync written as the reference writes it: five per-tensor
    loops of stock torch ops (torchft/local_sgd.py:205-239, torchft/manager.py:274-287),
    in place on ``params`` / ``backup``; ``outer_optimizer`` must own ``params``.

    ``pg`` is a world-size-1 process group (its all-reduce is the identity on this
    replica's tensor); the other replicas of the job are the parameter lists in
    ``peers``, whose pseudo-gradients are added in order, as a ring step would.
    """
    import torch.distributed as dist

    # local_sgd.py:212-215
    for p, b in zip(params, backup):
        p.grad = p.data - b
    # local_sgd.py:227-239 -> manager.py:274, 287
    works = []
    for t, p in enumerate(params):
        for peer in peers:
            p.grad.add_(peer[t] - backup[t])
        opts = dist.AllreduceOptions()
        opts.reduceOp = dist.ReduceOp.SUM
        works.append(pg.allreduce([p.grad], opts))
    for p, w in zip(params, works):
        w.wait()
        p.grad /= num_participants
    # local_sgd.py:219
    for p, b in zip(params, backup):
        p.data.copy_(b)
    # local_sgd.py:221-225
    outer_optimizer.step()
    for p, b in zip(params, backup):
        b.copy_(p.data)
    outer_optimizer.zero_grad()
