"""CPU stand-in for ``torchft_amd.ops`` so that host logic (hooks, commit gate, error
latching, optimizer-state handling) can be tested without a GPU.

It computes with the checker under ``oracle/`` and exists only inside the test-suite:
the product never imports it and has no CPU path of its own.  Use the ``cpu_ops``
fixture, which monkeypatches the functions below over ``torchft_amd.ops``.
"""

from typing import List

import torch

from oracle import replica_sync as O
from torchft_amd import ops as real_ops

calls: List[str] = []


class FakeTable:
    def matches(self, columns) -> bool:
        return True


def _flags(mask: int, n: int) -> List[bool]:
    return [bool((mask >> r) & 1) for r in range(n)]


def reduce_avg_(out, replicas, participate_mask=None, num_participants=None):
    calls.append("reduce_avg_")
    n = len(replicas)
    mask = real_ops.full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    real_ops._check_reduce_args(n, mask, nump)
    if n == 0:
        out.zero_()
        return out
    out.copy_(O.manager_allreduce_(list(replicas), _flags(mask, n), nump, torch.float32))
    return out


def check_tensor(t, what):
    pass  # the stand-in computes on CPU tensors of any dtype


def reduce_avg_table(outs, replicas):
    return FakeTable()


def mt_reduce_avg(outs, replicas, participate_mask=None, num_participants=None, table=None,
                  table_is_current=False):
    calls.append("mt_reduce_avg")
    n = len(replicas)
    mask = real_ops.full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    for t in range(len(outs[0])):
        avg = O.manager_allreduce_([rep[t] for rep in replicas], _flags(mask, n), nump, torch.float32)
        for col in outs:
            col[t].copy_(avg)
    return FakeTable()


def _pseudograd_f32(t, backups, replicas, mask, nump):
    n = len(replicas)
    b = backups[t].float()
    pseudo = [rep[t].float() - b for rep in replicas]
    return O.manager_allreduce_(pseudo, _flags(mask, n), nump)


def mt_pseudograd_avg(grads, params, backups, replicas, restore_params, participate_mask=None,
                      num_participants=None, table=None):
    calls.append("mt_pseudograd_avg")
    n = len(replicas)
    mask = real_ops.full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    for t in range(len(grads)):
        grads[t].copy_(_pseudograd_f32(t, backups, replicas, mask, nump))  # one rounding on store
        if restore_params:
            params[t].copy_(backups[t])
    return FakeTable()


def _sgd_from_backup(t, params, backups, bufs, g32, sgd, first_step):
    p = backups[t].float()
    buf = None if (first_step or bufs is None) else bufs[t].float()
    buf = O.sgd_step_(p, g32, buf, sgd.lr, sgd.momentum, sgd.dampening, sgd.weight_decay,
                      sgd.nesterov)
    if bufs is not None and buf is not None:
        bufs[t].copy_(buf)
    params[t].copy_(p)
    backups[t].copy_(p)


def mt_outer_sgd(params, backups, bufs, grads, sgd, first_step, table=None, grads_are_sums_of=None):
    calls.append("mt_outer_sgd")
    for t in range(len(params)):
        g32 = grads[t].float()
        if grads_are_sums_of is not None:
            # what Manager.allreduce's own division would have stored in the buffer
            g32 = (g32 / float(grads_are_sums_of)).to(grads[t].dtype).float()
        _sgd_from_backup(t, params, backups, bufs, g32, sgd, first_step)
    return FakeTable()


def diloco_outer_table(params, backups, bufs, replicas, table=None):
    return FakeTable()


def mt_diloco_outer(params, backups, bufs, replicas, sgd, first_step, participate_mask=None,
                    num_participants=None, table=None, table_is_current=False):
    calls.append("mt_diloco_outer")
    n = len(replicas)
    mask = real_ops.full_mask(n) if participate_mask is None else participate_mask
    nump = n if num_participants is None else num_participants
    for t in range(len(params)):
        g32 = _pseudograd_f32(t, backups, replicas, mask, nump)  # stays in fp32 registers
        _sgd_from_backup(t, params, backups, bufs, g32, sgd, first_step)
    return FakeTable()


def mt_copy(dsts, srcs, table=None):
    calls.append("mt_copy")
    for d, s in zip(dsts, srcs):
        d.view(torch.uint8).reshape(-1).copy_(s.contiguous().view(torch.uint8).reshape(-1))
    return FakeTable()


PATCHED = ["check_tensor", "reduce_avg_", "reduce_avg_table", "mt_reduce_avg", "mt_pseudograd_avg", "mt_outer_sgd",
           "mt_diloco_outer", "diloco_outer_table", "mt_copy"]
