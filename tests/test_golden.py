"""Frozen vectors (tests/golden/replica_sync_vectors.npz, made by library routines only)
against the CPU checker here and against the kernels on the GPU."""

import os

import numpy as np
import pytest
import torch

from helpers import assert_bits_equal
from oracle import replica_sync as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "replica_sync_vectors.npz")
KW = dict(lr=0.7, momentum=0.9, nesterov=True)


@pytest.fixture(scope="module")
def vec():
    data = np.load(PATH, allow_pickle=False)
    return {k: data[k] for k in data.files}


def f32(a):
    return torch.from_numpy(np.ascontiguousarray(a))


def bf16(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)


def test_checker_reproduces_the_golden_vectors(vec):
    backup, bufs = [f32(vec["backup"])], None
    for step in range(2):
        reps = [[f32(vec[f"diloco_step{step}_replica{r}"])] for r in range(3)]
        res = O.diloco_perform_sync(reps, backup, bufs, [True, False, True], 2, True, **KW)
        assert_bits_equal(res["grads"][0], f32(vec[f"diloco_step{step}_grad"]))
        assert_bits_equal(res["params"][0], f32(vec[f"diloco_step{step}_params"]))
        assert_bits_equal(res["momentum"][0], f32(vec[f"diloco_step{step}_momentum"]))
        backup, bufs = res["backup"], res["momentum"]
    got = O.manager_allreduce_([f32(vec[f"allreduce_f32_in{r}"]) for r in range(4)],
                               [True, True, True, False], 3)
    assert_bits_equal(got, f32(vec["allreduce_f32_out"]))
    got = O.manager_allreduce_([bf16(vec[f"allreduce_bf16_in{r}"]) for r in range(4)],
                               [True, True, True, False], 3, torch.float32)
    assert_bits_equal(got, bf16(vec["allreduce_bf16_out"]))
    got = O.c_reduce_avg([bf16(vec[f"allreduce_bf16_in{r}"]) for r in range(4)], 0b0111, 3)
    assert_bits_equal(got, bf16(vec["allreduce_bf16_out"]))


@pytest.mark.gpu
def test_kernels_reproduce_the_golden_vectors(vec, device):
    from torchft_amd import ops

    sgd = ops.OuterSGD(**KW)
    b = [f32(vec["backup"]).to(device)]
    p = [torch.empty_like(b[0])]
    m = [torch.empty_like(b[0])]
    g = [torch.empty_like(b[0])]
    for step in range(2):
        reps = [[f32(vec[f"diloco_step{step}_replica{r}"]).to(device)] for r in range(3)]
        # two-phase form exposes the averaged pseudo-gradient, fused form must agree with it
        b2, m2, p2 = [b[0].clone()], [m[0].clone()], [torch.empty_like(b[0])]
        ops.mt_pseudograd_avg(g, p2, b2, reps, True, 0b101, 2)
        assert_bits_equal(g[0], f32(vec[f"diloco_step{step}_grad"]))
        ops.mt_outer_sgd(p2, b2, m2, g, sgd, step == 0)
        ops.mt_diloco_outer(p, b, m, reps, sgd, step == 0, 0b101, 2)
        for got in (p, p2, b, b2):
            assert_bits_equal(got[0], f32(vec[f"diloco_step{step}_params"]))
        for got in (m, m2):
            assert_bits_equal(got[0], f32(vec[f"diloco_step{step}_momentum"]))
    xs = [f32(vec[f"allreduce_f32_in{r}"]).to(device) for r in range(4)]
    ops.reduce_avg_(xs[0], xs, 0b0111, 3)
    assert_bits_equal(xs[0], f32(vec["allreduce_f32_out"]))
    bs = [bf16(vec[f"allreduce_bf16_in{r}"]).to(device) for r in range(4)]
    ops.reduce_avg_(bs[0], bs, 0b0111, 3)
    assert_bits_equal(bs[0], bf16(vec["allreduce_bf16_out"]))
