"""Pins the CPU checker (oracle/) before anything is compared with it.

Every check here is independent of the checker's own formulas: known answers held by
the reference's tests, torch library routines (torch.optim.SGD, the DDP Reducer's bucket
assignment, torch.save/torch.load), closed forms, float64 brute force and invariants.
"""

import pytest
import torch
import torch.distributed as dist
from torch import nn

from helpers import assert_bits_equal
from oracle import replica_sync as O
from torchft_amd import workloads


# ---------------------------------------------------------------------------
# Manager.allreduce arithmetic
# ---------------------------------------------------------------------------

def test_known_answers_from_reference_tests():
    # torchft/manager_test.py:520-543 (test_manager_numerics): one contribution of 1.0,
    # five participants -> 1/5; a healing (non-participating) replica -> 0
    out = O.manager_allreduce_([torch.tensor([1.0])], [True], 5)
    torch.testing.assert_close(out, torch.tensor([1.0 / 5]))
    out = O.manager_allreduce_([torch.tensor([1.0])], [False], 5)
    torch.testing.assert_close(out, torch.tensor([0.0]))
    # torchft/manager_test.py:256-258, 316-318: healing => the gradient is zeroed
    out = O.manager_allreduce_([torch.tensor([1.0])], [False], 1)
    torch.testing.assert_close(out, torch.zeros(1))
    # torchft/process_group_test.py:185-203 (two ranks): [1] + [2] == [3]
    out = O.manager_allreduce_([torch.tensor([1.0]), torch.tensor([2.0])], [True, True], 1)
    torch.testing.assert_close(out, torch.tensor([3.0]))
    # torchft/manager_test.py:407-442: FIXED_WITH_SPARES, world of 3 with 2 active: the
    # spare's data does not count and the divisor is 2
    out = O.manager_allreduce_([torch.tensor([4.0]), torch.tensor([6.0]), torch.tensor([100.0])],
                               [True, True, False], 2)
    torch.testing.assert_close(out, torch.tensor([5.0]))


@pytest.mark.parametrize("n,mask,nump", [(2, 0b11, 2), (4, 0b1011, 3), (8, 0xFF, 8), (3, 0b010, 5)])
def test_allreduce_against_float64_brute_force(n, mask, nump):
    g = torch.Generator().manual_seed(n)
    xs = [torch.randn(257, generator=g) for _ in range(n)]
    flags = [bool((mask >> r) & 1) for r in range(n)]
    got = O.manager_allreduce_(xs, flags, nump)
    want = sum(x.double() for x, f in zip(xs, flags) if f) / nump
    # n fp32 additions and one division: a few ulp of the largest partial sum
    torch.testing.assert_close(got.double(), want, rtol=0, atol=float(n) * 2 ** -22 * 4)
    # inputs are untouched, every replica would hold the same result
    assert all(torch.equal(x, y) for x, y in zip(xs, [x.clone() for x in xs]))


def test_allreduce_bf16_fp32_accumulate_rounds_once():
    # 1 + 1.0078125 + 1.0078125 = 3.015625 exactly, and every term is a bf16 number.
    # Running sums in bf16 round twice (2.0078125 -> 2.0, then 3.0078125 -> 3.0);
    # fp32 accumulation keeps the exact sum and rounds once at the end.
    xs = [torch.tensor([v], dtype=torch.bfloat16) for v in (1.0, 1.0078125, 1.0078125)]
    assert [float(x) for x in xs] == [1.0, 1.0078125, 1.0078125]
    acc32 = O.manager_allreduce_(xs, [True] * 3, 1, torch.float32)
    native = O.manager_allreduce_(xs, [True] * 3, 1)
    assert float(acc32) == 3.015625
    assert float(native) == 3.0
    # and the two variants stay within the bf16 tolerance the path is specified with
    g = torch.Generator().manual_seed(0)
    xs = [(torch.randn(4096, generator=g) * 1e-2).bfloat16() for _ in range(4)]
    a = O.manager_allreduce_(xs, [True, True, False, True], 3, torch.float32)
    b = O.manager_allreduce_(xs, [True, True, False, True], 3)
    torch.testing.assert_close(a.float(), b.float(), rtol=1e-2, atol=1e-4)


# ---------------------------------------------------------------------------
# Outer optimizer
# ---------------------------------------------------------------------------

SGD_CASES = [
    dict(lr=0.7, momentum=0.9, nesterov=True),
    dict(lr=0.7, momentum=0.9),
    dict(lr=0.3, momentum=0.8, dampening=0.1, weight_decay=0.01),
    dict(lr=0.5),
    dict(lr=0.5, weight_decay=0.1),
]


@pytest.mark.parametrize("kw", SGD_CASES)
def test_sgd_step_is_torch_optim_sgd(kw):
    """Library routine: three consecutive steps of torch.optim.SGD, bit for bit."""
    g = torch.Generator().manual_seed(1)
    p0 = torch.randn(1000, generator=g) * 0.02
    param = nn.Parameter(p0.clone())
    opt = torch.optim.SGD([param], **kw)
    mine, buf = p0.clone(), None
    for step in range(3):
        grad = torch.randn(1000, generator=g) * 1e-3
        param.grad = grad.clone()
        opt.step()
        buf = O.sgd_step_(mine, grad, buf, **kw)
        assert_bits_equal(mine, param.data, f"step {step}")
        if kw.get("momentum"):
            assert_bits_equal(buf, opt.state[param]["momentum_buffer"], f"step {step} momentum")
        else:
            assert buf is None and "momentum_buffer" not in opt.state[param]


def test_sgd_closed_forms():
    g = torch.tensor([1e-3, -2e-3, 0.0, 5e-4], dtype=torch.float64)
    b = torch.tensor([0.02, -0.01, 0.3, 0.0], dtype=torch.float64)
    # first Nesterov step: buf = g, p = b - lr * (g + mu * g) = b - 0.7 * 1.9 * g
    p = b.float().clone()
    buf = O.sgd_step_(p, g.float(), None, lr=0.7, momentum=0.9, nesterov=True)
    torch.testing.assert_close(p.double(), b - 0.7 * 1.9 * g, rtol=1e-6, atol=1e-9)
    torch.testing.assert_close(buf.double(), g, rtol=1e-7, atol=0)
    # second step with the same gradient: buf = 1.9 g, p -= 0.7 * (g + 0.9 * 1.9 g)
    buf = O.sgd_step_(p, g.float(), buf, lr=0.7, momentum=0.9, nesterov=True)
    torch.testing.assert_close(buf.double(), 1.9 * g, rtol=1e-6, atol=0)
    torch.testing.assert_close(
        p.double(), b - 0.7 * 1.9 * g - 0.7 * (1 + 0.9 * 1.9) * g, rtol=1e-6, atol=1e-9)
    # zero gradient is a fixed point; momentum == 0 is plain SGD
    p = b.float().clone()
    O.sgd_step_(p, torch.zeros(4), None, lr=0.7, momentum=0.9, nesterov=True)
    assert torch.equal(p, b.float())
    p = b.float().clone()
    assert O.sgd_step_(p, g.float(), None, lr=0.5) is None
    torch.testing.assert_close(p.double(), b - 0.5 * g, rtol=1e-6, atol=1e-9)


# ---------------------------------------------------------------------------
# DiLoCo / LocalSGD
# ---------------------------------------------------------------------------

def _tiny_workload(n_replicas, seed=0):
    shapes = [("w", (33, 7)), ("b", (7,)), ("s", (1,))]
    return workloads.make_diloco_workload(shapes, n_replicas, torch.device("cpu"))


def test_diloco_against_torch_optim_and_float64():
    """Composition: the pseudo-gradient average is checked against float64 brute force,
    the update against torch.optim.SGD stepping real Parameters with that gradient."""
    wl = _tiny_workload(4)
    flags, nump = [True, False, True, True], 3
    res = O.diloco_perform_sync(wl.replicas, wl.backup, None, flags, nump, True,
                                lr=0.7, momentum=0.9, nesterov=True)
    params = [nn.Parameter(b.clone()) for b in wl.backup]
    opt = torch.optim.SGD(params, lr=0.7, momentum=0.9, nesterov=True)
    for t, b in enumerate(wl.backup):
        want_g = sum((rep[t].double() - b.double()) for rep, f in zip(wl.replicas, flags) if f) / nump
        # subtract-then-sum in fp32 against exact: a few ulp of |p| (~0.02..0.1)
        torch.testing.assert_close(res["grads"][t].double(), want_g, rtol=0, atol=4 * 2 ** -24 * 0.1)
        params[t].grad = res["grads"][t].clone()
    opt.step()
    for t in range(len(params)):
        assert_bits_equal(res["params"][t], params[t].data)
        assert_bits_equal(res["backup"][t], params[t].data)  # committed: backup == params
        assert_bits_equal(res["momentum"][t], opt.state[params[t]]["momentum_buffer"])


def test_diloco_special_cases():
    wl = _tiny_workload(2)
    kw = dict(lr=0.7, momentum=0.9, nesterov=True)
    # every replica equal to the backup: fixed point, zero momentum
    same = [[b.clone() for b in wl.backup] for _ in range(2)]
    res = O.diloco_perform_sync(same, wl.backup, None, [True, True], 2, True, **kw)
    for t, b in enumerate(wl.backup):
        assert torch.equal(res["params"][t], b) and torch.equal(res["backup"][t], b)
        assert torch.count_nonzero(res["momentum"][t]) == 0
    # one replica, one participant: the pseudo-gradient is exactly p - b
    res = O.diloco_perform_sync([wl.replicas[0]], wl.backup, None, [True], 1, True, **kw)
    for t, b in enumerate(wl.backup):
        assert_bits_equal(res["grads"][t], wl.replicas[0][t] - b)
    # no commit: params return to the previous backup, backup and momentum untouched
    # (torchft/local_sgd.py:219-225)
    bufs = [torch.full_like(b, 0.5) for b in wl.backup]
    res = O.diloco_perform_sync(wl.replicas, wl.backup, bufs, [True, True], 2, False, **kw)
    for t, b in enumerate(wl.backup):
        assert torch.equal(res["params"][t], b) and torch.equal(res["backup"][t], b)
        assert torch.equal(res["momentum"][t], bufs[t])
    # the order replicas are listed in only matters through fp32 summation order
    a = O.diloco_perform_sync(wl.replicas, wl.backup, None, [True, True], 2, True, **kw)
    b_ = O.diloco_perform_sync(wl.replicas[::-1], wl.backup, None, [True, True], 2, True, **kw)
    for x, y in zip(a["params"], b_["params"]):
        assert_bits_equal(x, y)  # two terms: addition commutes exactly


def test_diloco_reference_loop_matches_restatement():
    """The timed baseline loop (real ProcessGroupGloo + torch.optim.SGD, written loop by
    loop like torchft/local_sgd.py:205-239) and the functional restatement agree for
    two consecutive syncs."""
    wl = _tiny_workload(3)
    params = [nn.Parameter(t.clone()) for t in wl.replicas[0]]
    backup = [t.clone() for t in wl.backup]
    opt = torch.optim.SGD(params, lr=0.7, momentum=0.9, nesterov=True)
    pg = O.make_gloo_world1()
    cur_backup, bufs = wl.backup, None
    replicas = wl.replicas
    for step in range(2):
        want = O.diloco_perform_sync(replicas, cur_backup, bufs, [True] * 3, 3, True,
                                     lr=0.7, momentum=0.9, nesterov=True)
        O.diloco_reference_loop_(pg, params, backup, replicas[1:], opt, 3)
        for t in range(len(params)):
            assert_bits_equal(params[t].data, want["params"][t])
            assert_bits_equal(backup[t], want["backup"][t])
            assert_bits_equal(opt.state[params[t]]["momentum_buffer"], want["momentum"][t])
            assert params[t].grad is None  # zero_grad(set_to_none)
        cur_backup, bufs = want["backup"], want["momentum"]
        replicas = [workloads.drifted_replica(cur_backup, 1e-3, 50 + r) for r in range(3)]
        for p, r in zip(params, replicas[0]):
            p.data.copy_(r)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_diloco_fp32_arithmetic_for_16_bit_storage(dtype):
    """The fp32-arithmetic variant for bf16 / fp16 parameters (what the kernels compute):
    (1) for values that are exact in the storage dtype the whole step evaluated in float64
    and rounded once differs from it by at most one unit in the last place of the storage
    dtype (fp32 error is far below half a 16-bit ulp, so only ties can differ);
    (2) it stays within the stated rtol 1e-2 (atol for near-zero values) of the reference
    form, where torch rounds to the storage dtype after every op
    (torchft/local_sgd.py:212-215 on bf16 parameters);
    (3) passing the averaged pseudo-gradient through memory in the storage dtype (the
    two-launch form) changes results by no more than that same tolerance."""
    shapes = [("w", (257, 5)), ("b", (9,))]
    wl = workloads.make_diloco_workload(shapes, 3, torch.device("cpu"))
    backup = [t.to(dtype) for t in wl.backup]
    reps = [[t.to(dtype) for t in rep] for rep in wl.replicas]
    bufs = [(1e-3 * torch.randn(t.shape, generator=torch.Generator().manual_seed(5))).to(dtype)
            for t in backup]
    flags, nump = [True, True, False], 2
    kw = dict(lr=0.7, momentum=0.9, nesterov=True)
    for first in (True, False):
        mb = None if first else bufs
        got = O.diloco_perform_sync(reps, backup, mb, flags, nump, True, **kw,
                                    accumulate_dtype=torch.float32)
        native = O.diloco_perform_sync(reps, backup, mb, flags, nump, True, **kw)
        two = O.diloco_perform_sync(reps, backup, mb, flags, nump, True, **kw,
                                    accumulate_dtype=torch.float32, grads_through_storage=True)
        for t, b in enumerate(backup):
            assert got["params"][t].dtype == dtype and got["momentum"][t].dtype == dtype
            # (1) float64 evaluation of the same formulas
            b64 = b.double()
            g64 = sum((rep[t].double() - b64) for rep, f in zip(reps, flags) if f) / nump
            buf64 = g64 if first else 0.9 * bufs[t].double() + g64
            p64 = b64 - 0.7 * (g64 + 0.9 * buf64)
            for name, exact in (("params", p64), ("backup", p64), ("momentum", buf64), ("grads", g64)):
                rounded = exact.to(dtype)
                ulp_apart = (got[name][t].view(torch.int16).int() - rounded.view(torch.int16).int()).abs()
                assert int(ulp_apart.max()) <= 1, (name, first)
                assert float((ulp_apart > 0).float().mean()) < 0.02, (name, first)
            # (2) and (3)
            for name in ("params", "backup", "momentum", "grads"):
                torch.testing.assert_close(got[name][t].float(), native[name][t].float(), rtol=1e-2, atol=2e-4)
                torch.testing.assert_close(got[name][t].float(), two[name][t].float(), rtol=1e-2, atol=2e-4)
    # fp32 storage: the option changes nothing
    a = O.diloco_perform_sync(wl.replicas, wl.backup, None, flags, nump, True, **kw)
    b_ = O.diloco_perform_sync(wl.replicas, wl.backup, None, flags, nump, True, **kw,
                               accumulate_dtype=torch.float32, grads_through_storage=True)
    for name in ("params", "backup", "momentum", "grads"):
        for x, y in zip(a[name], b_[name]):
            assert_bits_equal(x, y)


def test_localsgd_closed_form_and_invariants():
    wl = _tiny_workload(2)
    res = O.localsgd_perform_sync(wl.replicas, wl.backup, [True, True], 2, True)
    for t in range(len(wl.backup)):
        want = (wl.replicas[0][t].double() + wl.replicas[1][t].double()) / 2
        torch.testing.assert_close(res["params"][t].double(), want, rtol=1e-7, atol=1e-9)
        assert torch.equal(res["backup"][t], res["params"][t])  # local_sgd_test.py:65-67
    res = O.localsgd_perform_sync(wl.replicas, wl.backup, [True, True], 2, False)
    for t, b in enumerate(wl.backup):
        assert torch.equal(res["params"][t], b)  # local_sgd_test.py:98-101
    # world size 1 is the identity
    res = O.localsgd_perform_sync([wl.replicas[0]], wl.backup, [True], 1, True)
    for t in range(len(wl.backup)):
        assert torch.equal(res["params"][t], wl.replicas[0][t])


# ---------------------------------------------------------------------------
# The plain-C twin
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("kw", SGD_CASES)
@pytest.mark.parametrize("first", [True, False])
def test_c_twin_matches_torch_restatement(kw, first):
    g = torch.Generator().manual_seed(7)
    n = 10_007
    b = torch.randn(n, generator=g) * 0.02
    reps = [b + torch.randn(n, generator=g) * 1e-3 for _ in range(4)]
    buf = None if first else torch.randn(n, generator=g) * 1e-3
    full = dict(lr=kw["lr"], momentum=kw.get("momentum", 0.0), dampening=kw.get("dampening", 0.0),
                weight_decay=kw.get("weight_decay", 0.0), nesterov=kw.get("nesterov", False))
    want = O.diloco_perform_sync([[r] for r in reps], [b], None if first else [buf],
                                 [True, True, False, True], 3, True, **full)
    p, nb, m = O.c_diloco_outer(b, buf, reps, 0b1011, 3, first_step=first, **full)
    assert_bits_equal(p, want["params"][0])
    assert_bits_equal(nb, want["backup"][0])
    if full["momentum"]:
        assert_bits_equal(m, want["momentum"][0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_c_twin_reduce_avg(dtype):
    g = torch.Generator().manual_seed(3)
    xs = [torch.randn(5001, generator=g).to(dtype) for _ in range(5)]
    want = O.manager_allreduce_(xs, [True, False, True, True, False], 4, torch.float32)
    assert_bits_equal(O.c_reduce_avg(xs, 0b01101, 4), want)


# ---------------------------------------------------------------------------
# DDP buckets
# ---------------------------------------------------------------------------

def _torch_bucket_assignment(params, first_cap, cap):
    idx, _ = dist._compute_bucket_assignment_by_size(params, [first_cap, cap], [False] * len(params))
    return list(reversed(idx))


@pytest.mark.parametrize("shapes_fn,dtype", [
    (workloads.mlp_shapes, torch.float32),
    (workloads.gpt2_small_shapes, torch.float32),
    (workloads.gpt2_small_shapes, torch.bfloat16),
])
def test_bucket_assignment_is_torchs(shapes_fn, dtype):
    shapes = shapes_fn()
    metas = [torch.empty(s, dtype=dtype, device="meta") for _, s in shapes]
    want = _torch_bucket_assignment(metas, O.DEFAULT_FIRST_BUCKET_BYTES, O.DEFAULT_BUCKET_CAP_BYTES)
    got = O.bucket_assignment([m.numel() for m in metas], metas[0].element_size())
    assert got == want


def test_bucket_assignment_llama_matches_torch_and_known_count():
    shapes = workloads.llama3_8b_shapes()
    metas = [torch.empty(s, dtype=torch.bfloat16, device="meta") for _, s in shapes]
    want = _torch_bucket_assignment(metas, O.DEFAULT_FIRST_BUCKET_BYTES, O.DEFAULT_BUCKET_CAP_BYTES)
    got = O.bucket_assignment([m.numel() for m in metas], 2)
    assert got == want
    assert len(got) == 162  # probed with torch's rule for Llama-3-8B bf16 gradients


def test_bucket_layout_against_a_real_reducer():
    """A real DDP Reducer on the MLP: bucket membership, order and in-bucket offsets."""
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(1024, 2048), nn.ReLU(), nn.Linear(2048, 2048), nn.ReLU(),
                          nn.Linear(2048, 10))
    from torchft_amd.process_group import ProcessGroupDummy

    pg = ProcessGroupDummy(0, 1)  # soaks up the constructor's collectives, as in torchft/ddp.py:50
    ddp = nn.parallel.DistributedDataParallel(model, process_group=pg, find_unused_parameters=True)
    seen = []

    def hook(state, bucket: dist.GradBucket) -> torch.futures.Future[torch.Tensor]:
        base = bucket.buffer().data_ptr()
        esize = bucket.buffer().element_size()
        seen.append((bucket.index(), [p.data_ptr() for p in bucket.parameters()],
                     [(g.data_ptr() - base) // esize for g in bucket.gradients()],
                     bucket.buffer().numel()))
        fut = torch.futures.Future()
        fut.set_result(bucket.buffer())
        return fut

    ddp.register_comm_hook(None, hook)
    ddp(torch.randn(2, 1024)).sum().backward()
    params = list(model.parameters())
    numels = [p.numel() for p in params]
    buckets = O.bucket_assignment(numels, 4)
    assert len(seen) == len(buckets) == 2
    by_ptr = {p.data_ptr(): i for i, p in enumerate(params)}
    for index, ptrs, offsets, total in sorted(seen):
        members = [by_ptr[x] for x in ptrs]
        assert members == buckets[index]
        assert offsets == O.bucket_offsets(numels, buckets[index])
        assert total == sum(numels[i] for i in members)
    # the bucket sizes torch produces for this model (4 218 890 and 2 097 152 elements)
    assert sorted(s[3] for s in seen) == [2_097_152, 4_218_890]


def test_ddp_bucket_average_identities():
    shapes = [("a", (300, 7)), ("b", (5,)), ("c", (1000,)), ("d", (3, 3))]
    grads = workloads.make_grad_replicas(shapes, 3, torch.device("cpu"), torch.float32)
    numels = [workloads.numel(s) for _, s in shapes]
    buckets = O.bucket_assignment(numels, 4, first_cap=4000, cap=8000)
    assert sorted(i for b in buckets for i in b) == list(range(len(shapes)))
    got = O.ddp_bucket_average(grads, [True, True, True], 3, buckets)
    # bucketing must not change the numbers: same as averaging tensor by tensor
    for t in range(len(shapes)):
        want = O.manager_allreduce_([g[t] for g in grads], [True] * 3, 3)
        assert_bits_equal(got[t], want)
        assert got[t].shape == grads[0][t].shape


# ---------------------------------------------------------------------------
# Checkpoint state
# ---------------------------------------------------------------------------

def test_state_dict_round_trip_is_identity():
    state = workloads.make_training_state([("w", (17, 5)), ("b", (5,))], torch.device("cpu"), step=7)
    back = O.state_dict_round_trip(state)
    assert back["torchft"] == state["torchft"]
    assert back["user"]["optim"]["param_groups"] == state["user"]["optim"]["param_groups"]
    for name, t in state["user"]["model"].items():
        assert_bits_equal(back["user"]["model"][name], t)
        assert back["user"]["model"][name].dtype == torch.bfloat16
    for i, st in state["user"]["optim"]["state"].items():
        for k, t in st.items():
            assert_bits_equal(back["user"]["optim"]["state"][i][k], t)
    # torchft/checkpointing_test.py:17-37: a plain dict comes back equal
    assert O.state_dict_round_trip({"state": "dict"}) == {"state": "dict"}


def test_gather_bytes_layout():
    a = torch.arange(5, dtype=torch.int16)
    b = torch.tensor([1.5], dtype=torch.float32)
    img = O.gather_bytes([a, b], [0, 256], 512)
    assert img[:10].tobytes() == a.numpy().tobytes()
    assert img[256:260].tobytes() == b.numpy().tobytes()
    assert not img[10:256].any() and not img[260:].any()


def test_workload_shapes_match_the_named_configs():
    assert workloads.total_params(workloads.mlp_shapes()) == 6_316_042
    assert len(workloads.gpt2_small_shapes()) == 148
    assert workloads.total_params(workloads.gpt2_small_shapes()) == 124_439_808
    assert len(workloads.llama3_8b_shapes()) == 291
    assert workloads.total_params(workloads.llama3_8b_shapes()) == 8_030_261_248
