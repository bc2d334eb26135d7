"""The allocation-free entry point against the table-based one, through the C ABI."""

import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_bits_equal
from oracle import replica_sync as O
from torchft_amd import _native, ops, workloads

pytestmark = pytest.mark.gpu


def _call_noalloc(cols, sgd, first_step, mask, nump, dtype_code):
    """cols: [p, b, buf, replica_0 ..], each a list of device tensors (empty ones dropped)."""
    keep = [t for t in range(len(cols[0])) if cols[0][t].numel() > 0]
    n_t = len(keep)
    ptrs = (ctypes.c_void_p * (len(cols) * n_t))()
    for c, col in enumerate(cols):
        for i, t in enumerate(keep):
            ptrs[c * n_t + i] = col[t].data_ptr() if col is not None else None
    numel = np.asarray([cols[0][t].numel() for t in keep], dtype=np.uint64)
    lib = _native.lib()
    stream = torch.cuda.current_stream()
    rc = lib.tft_mt_diloco_outer_noalloc(
        ptrs, numel.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64)), n_t, len(cols) - 3, mask, nump,
        dtype_code, ctypes.byref(sgd.to_struct(first_step)), ctypes.c_void_p(stream.cuda_stream))
    _native.check(rc, "tft_mt_diloco_outer_noalloc")


def _workload(shapes, n_rep, dtype, device, seed):
    wl = workloads.make_diloco_workload(shapes, n_rep, torch.device("cpu"))
    g = torch.Generator().manual_seed(seed)
    backup = [t.to(dtype) for t in wl.backup]
    bufs = [(1e-3 * torch.randn(t.shape, generator=g)).to(dtype) for t in backup]
    reps = [[(b.float() + 1e-3 * torch.randn(b.shape, generator=g)).to(dtype) for b in backup]
            for _ in range(n_rep)]
    dev = lambda ts: [t.to(device) for t in ts]
    return backup, bufs, reps, dev


@pytest.mark.parametrize("dtype,code", [(torch.float32, _native.TFT_F32), (torch.bfloat16, _native.TFT_BF16)])
def test_noalloc_matches_the_table_entry_point_twice(device, dtype, code):
    """Two calls in a row on the same GPU, the second with a smaller input (fewer and
    smaller tensors, so stale table entries of the first call lie behind the second's):
    outputs must equal those of tft_mt_diloco_outer, and the checker's, bit for bit."""
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    big = workloads.mlp_shapes() + [("odd", (7, 3)), ("one", (1,)), ("wide", (3, 70_001))]
    small = [("w", (300, 33)), ("v", (5,))]
    for shapes, n_rep, mask, nump, first in ((big, 3, 0b101, 2, False), (small, 2, 0b11, 2, True)):
        backup, bufs, reps, dev = _workload(shapes, n_rep, dtype, device, seed=len(shapes))
        flags = [bool((mask >> r) & 1) for r in range(n_rep)]
        want = O.diloco_perform_sync(reps, backup, None if first else bufs, flags, nump, True, lr=0.7,
                                     momentum=0.9, nesterov=True, accumulate_dtype=torch.float32)
        # existing entry point
        b1, m1, r1 = dev(backup), dev(bufs), [dev(r) for r in reps]
        p1 = [torch.empty_like(t) for t in b1]
        ops.mt_diloco_outer(p1, b1, m1, r1, sgd, first, mask, nump)
        # allocation-free entry point
        b2, m2, r2 = dev(backup), dev(bufs), [dev(r) for r in reps]
        p2 = [torch.empty_like(t) for t in b2]
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        _call_noalloc([p2, b2, m2, *r2], sgd, first, mask, nump, code)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        for i, (name, _) in enumerate(shapes):
            for got, ref, exp, what in ((p2[i], p1[i], want["params"][i], "params"),
                                        (b2[i], b1[i], want["backup"][i], "backup"),
                                        (m2[i], m1[i], want["momentum"][i], "momentum")):
                assert_bits_equal(got, ref.cpu(), f"{what} {name} vs table entry point")
                assert_bits_equal(got, exp, f"{what} {name} vs checker")
        for r in range(n_rep):
            for i in range(len(shapes)):
                assert_bits_equal(r2[r][i], reps[r][i], "replica buffers are read-only")


def test_noalloc_rejects_what_does_not_fit(device):
    lib = _native.lib()
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True).to_struct(False)
    x = torch.zeros(16, device=device)
    n_t = _native.NOALLOC_MAX_TENSORS + 1
    ptrs = (ctypes.c_void_p * (4 * n_t))(*([x.data_ptr()] * (4 * n_t)))
    numel = (ctypes.c_uint64 * n_t)(*([16] * n_t))
    assert lib.tft_mt_diloco_outer_noalloc(ptrs, numel, n_t, 1, 1, 1, 0, ctypes.byref(sgd), None) == -2
    assert b"at most 4096" in lib.tft_last_error()
    # one tensor whose chunk list alone exceeds the array (sizes are only looked at on the host)
    numel = (ctypes.c_uint64 * 1)(3 * 2 ** 37)
    assert lib.tft_mt_diloco_outer_noalloc(ptrs, numel, 1, 1, 1, 1, 0, ctypes.byref(sgd), None) == -2
    assert b"built-in array holds" in lib.tft_last_error()
    numel = (ctypes.c_uint64 * 1)(0)
    assert lib.tft_mt_diloco_outer_noalloc(ptrs, numel, 1, 1, 1, 1, 0, ctypes.byref(sgd), None) == -1
    ptrs[1] = None
    numel = (ctypes.c_uint64 * 1)(16)
    assert lib.tft_mt_diloco_outer_noalloc(ptrs, numel, 1, 1, 1, 1, 0, ctypes.byref(sgd), None) == -1
    assert b"NULL" in lib.tft_last_error()
