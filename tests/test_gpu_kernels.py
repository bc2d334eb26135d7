"""GPU parity: every kernel, called through the C ABI, against the CPU checker.

The kernels and the checker perform the same IEEE operations in the same order
(sequential replica sum, true divide, the fused multiply-adds torch's
add(alpha=) kernels use), so these comparisons are bit-exact, which is stricter
than the rtol 1e-6 (fp32) / 1e-2 (bf16) bars the path is specified with.
"""

import itertools

import pytest
import torch

from helpers import assert_bits_equal, assert_bits_equal_up_to_nan_payload
from oracle import replica_sync as O
from torchft_amd import ops, workloads

pytestmark = pytest.mark.gpu

SIZES = [1, 3, 4, 5, 255, 1023, 1024, 1025, 4099, 32768, 32769, 65536 + 7, 200_003]


def mask_to_list(mask, n):
    return [bool((mask >> r) & 1) for r in range(n)]


def draw(n, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n_replicas,mask,nump", [
    (1, 0b1, 1), (1, 0b1, 5), (1, 0b0, 5), (2, 0b11, 2), (3, 0b101, 2), (4, 0b1011, 3),
    (4, 0b1111, 4), (8, 0xFF, 8), (8, 0b10110101, 2), (0, 0, 3),
])
def test_reduce_avg_flat(device, dtype, n_replicas, mask, nump):
    for numel in SIZES:
        reps = [draw(numel, dtype, 10 * r + numel % 7) for r in range(n_replicas)]
        if n_replicas:
            want = O.manager_allreduce_(reps, mask_to_list(mask, n_replicas), nump, torch.float32)
        else:
            want = torch.zeros(numel, dtype=dtype)
        out = torch.full((numel,), 7.0, dtype=dtype, device=device)
        ops.reduce_avg_(out, [r.to(device) for r in reps], mask, nump)
        assert_bits_equal(out, want, f"numel={numel}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_reduce_avg_in_place_and_misaligned(device, dtype):
    # out aliases replica 1; all buffers start 1 element past a 16-byte boundary
    numel = 70_001
    reps = [draw(numel + 1, dtype, 50 + r) for r in range(3)]
    want = O.manager_allreduce_([r[1:] for r in reps], [True, True, True], 3, torch.float32)
    dev = [r.to(device) for r in reps]
    out = dev[1][1:]
    ops.reduce_avg_(out, [d[1:] for d in dev], 0b111, 3)
    assert_bits_equal(out, want)
    # the guard element in front is untouched
    assert_bits_equal(dev[1][:1], reps[1][:1])
    # mixed: only one operand misaligned
    dev2 = [r.to(device) for r in reps]
    out2 = torch.empty(numel, dtype=dtype, device=device)
    ops.reduce_avg_(out2, [dev2[0][1:], dev2[1][:-1], dev2[2][1:]], 0b111, 3)
    want2 = O.manager_allreduce_([reps[0][1:], reps[1][:-1], reps[2][1:]], [True] * 3, 3, torch.float32)
    assert_bits_equal(out2, want2)


# ---------------------------------------------------------------------------
# fp64: the replica average is dtype-generic in the reference (torchft/manager.py:267-287)
# ---------------------------------------------------------------------------

def draw64(n, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, generator=g, dtype=torch.float64) * scale


@pytest.mark.parametrize("n_replicas,mask,nump", [
    (1, 0b1, 1), (1, 0b1, 5), (1, 0b0, 5), (2, 0b11, 2), (3, 0b101, 2), (4, 0b1011, 3),
    (4, 0b1111, 4), (8, 0xFF, 8), (8, 0b10110101, 2), (0, 0, 3),
])
def test_reduce_avg_flat_fp64(device, n_replicas, mask, nump):
    """fp64 buffers are summed and divided in fp64, exactly as torch does on the host: the
    mantissa bits beyond fp32 must survive (values drawn in fp64, scaled apart)."""
    for numel in SIZES:
        reps = [draw64(numel, 10 * r + numel % 7, 10.0 ** (r % 3)) for r in range(n_replicas)]
        if n_replicas:
            want = O.manager_allreduce_(reps, mask_to_list(mask, n_replicas), nump)
        else:
            want = torch.zeros(numel, dtype=torch.float64)
        out = torch.full((numel,), 7.0, dtype=torch.float64, device=device)
        ops.reduce_avg_(out, [r.to(device) for r in reps], mask, nump)
        assert_bits_equal(out, want, f"numel={numel}")
    # not merely fp32 arithmetic widened: 1 + 2^-40 is not representable in fp32
    a = torch.tensor([1.0, 3.0], dtype=torch.float64, device=device)
    b = torch.tensor([2.0 ** -40, 2.0 ** -45], dtype=torch.float64, device=device)
    out = torch.empty_like(a)
    ops.reduce_avg_(out, [a, b], 0b11, 3)
    assert_bits_equal(out, (torch.tensor([1.0 + 2.0 ** -40, 3.0 + 2.0 ** -45], dtype=torch.float64)) / 3)


def test_reduce_avg_fp64_in_place_misaligned_and_multi_tensor(device):
    numel = 70_001
    reps = [draw64(numel + 1, 50 + r) for r in range(3)]
    want = O.manager_allreduce_([r[1:] for r in reps], [True, True, True], 3)
    dev = [r.to(device) for r in reps]
    out = dev[1][1:]                      # 8 bytes past a 16-byte boundary, aliases replica 1
    ops.reduce_avg_(out, [d[1:] for d in dev], 0b111, 3)
    assert_bits_equal(out, want)
    assert_bits_equal(dev[1][:1], reps[1][:1])
    # columns misaligned differently from each other: the scalar path
    dev2 = [r.to(device) for r in reps]
    out2 = torch.empty(numel, dtype=torch.float64, device=device)
    ops.reduce_avg_(out2, [dev2[0][1:], dev2[1][:-1], dev2[2][1:]], 0b110, 2)
    want2 = O.manager_allreduce_([reps[0][1:], reps[1][:-1], reps[2][1:]], [False, True, True], 2)
    assert_bits_equal(out2, want2)
    # a table of ragged tensors, two outputs (LocalSGD: parameters and backup together)
    sizes = [1, 0, 5, 1023, 1025, 40_000, 66_000, 131_073]
    cols = [[draw64(n, 300 + 17 * r + i) for i, n in enumerate(sizes)] for r in range(2)]
    dev_cols = [[t.to(device) for t in col] for col in cols]
    p = dev_cols[0]                       # in place on replica 0
    bkp = [torch.full_like(t, 5.0) for t in p]
    ops.mt_reduce_avg([p, bkp], dev_cols, 0b11, 2)
    for i, n in enumerate(sizes):
        want = O.manager_allreduce_([cols[0][i], cols[1][i]], [True, True], 2)
        assert_bits_equal(p[i], want, f"tensor {i} ({n})")
        assert_bits_equal(bkp[i], want, f"backup {i} ({n})")


def test_fp64_over_the_whole_encoding(device):
    """Random bit patterns (denormals, infinities, NaNs, values next to overflow) through the
    fp64 average: bit-equal wherever the checker has a number, NaN wherever it has a NaN."""
    g = torch.Generator().manual_seed(11)
    n = 300_000
    reps = [torch.randint(-2 ** 63, 2 ** 63 - 1, (n,), generator=g, dtype=torch.int64).view(torch.float64)
            for _ in range(3)]
    for mask, nump in ((0b111, 3), (0b111, 4), (0b101, 2)):
        want = O.manager_allreduce_(reps, mask_to_list(mask, 3), nump)
        out = torch.empty(n, dtype=torch.float64, device=device)
        ops.reduce_avg_(out, [r.to(device) for r in reps], mask, nump)
        assert_bits_equal_up_to_nan_payload(out, want, f"mask {mask:#b} n {nump}")


def test_reference_known_answers(device):
    # torchft/manager_test.py:520-543: 1.0 with 5 participants -> 0.2; healing -> 0.0
    t = torch.tensor([1.0], device=device)
    ops.reduce_avg_(t, [t], 0b1, 5)
    torch.testing.assert_close(t.cpu(), torch.tensor([1.0 / 5]))
    t = torch.tensor([1.0], device=device)
    ops.reduce_avg_(t, [t], 0b0, 5)
    torch.testing.assert_close(t.cpu(), torch.tensor([0.0]))
    # torchft/process_group_test.py:185-203: [1] + [2] == [3]
    a, b = torch.tensor([1.0], device=device), torch.tensor([2.0], device=device)
    ops.reduce_avg_(a, [a, b], 0b11, 1)
    torch.testing.assert_close(a.cpu(), torch.tensor([3.0]))


def _mlp_workload(n_replicas, seed_shift=0):
    shapes = workloads.mlp_shapes() + [("odd", (7, 3)), ("empty", (0,)), ("one", (1,))]
    wl = workloads.make_diloco_workload(shapes, n_replicas, torch.device("cpu"))
    return wl


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n_outs", [1, 2])
def test_mt_reduce_avg(device, dtype, n_outs):
    wl = _mlp_workload(3)
    reps = [[t.to(dtype) for t in rep] for rep in wl.replicas]
    want = [
        O.manager_allreduce_([rep[t] for rep in reps], [True, False, True], 2, torch.float32)
        for t in range(len(wl.backup))
    ]
    dev = [[t.to(device) for t in rep] for rep in reps]
    outs = [dev[0]] + ([[torch.empty_like(t) for t in dev[0]]] if n_outs == 2 else [])
    ops.mt_reduce_avg(outs, dev, 0b101, 2)
    for col in outs:
        for got, w, name in zip(col, want, wl.names):
            assert_bits_equal(got, w, name)
    # replica 1 (not participating) was not written
    for got, src in zip(dev[1], reps[1]):
        assert_bits_equal(got, src)


SGD_CASES = [
    dict(lr=0.7, momentum=0.9, nesterov=True),
    dict(lr=0.7, momentum=0.9, nesterov=False),
    dict(lr=0.3, momentum=0.8, dampening=0.1, weight_decay=0.01),
    dict(lr=0.5),
    dict(lr=0.5, weight_decay=0.1),
]


@pytest.mark.parametrize("sgd_kw", SGD_CASES)
@pytest.mark.parametrize("n_replicas,mask,nump", [(1, 1, 1), (2, 0b11, 2), (4, 0b1011, 3), (8, 0xFF, 8)])
def test_diloco_fused_two_steps(device, sgd_kw, n_replicas, mask, nump):
    """First step (no momentum state) then a steady-state step, against the checker."""
    wl = _mlp_workload(n_replicas)
    sgd = ops.OuterSGD(**sgd_kw)
    kw = dict(lr=sgd.lr, momentum=sgd.momentum, dampening=sgd.dampening,
              weight_decay=sgd.weight_decay, nesterov=sgd.nesterov)
    part = mask_to_list(mask, n_replicas)
    b_dev = [t.to(device) for t in wl.backup]
    p_dev = [torch.empty_like(t) for t in b_dev]
    m_dev = [torch.full_like(t, float("nan")) for t in b_dev] if sgd.momentum else None
    backup, bufs = wl.backup, None
    table = None
    for step in range(2):
        reps = [workloads.drifted_replica(backup, 1e-3, 77 + 10 * step + r) for r in range(n_replicas)]
        want = O.diloco_perform_sync(reps, backup, bufs, part, nump, True, **kw)
        reps_dev = [[t.to(device) for t in rep] for rep in reps]
        ops.mt_diloco_outer(p_dev, b_dev, m_dev, reps_dev, sgd, step == 0, mask, nump)
        for i, name in enumerate(wl.names):
            assert_bits_equal(p_dev[i], want["params"][i], f"step {step} params {name}")
            assert_bits_equal(b_dev[i], want["backup"][i], f"step {step} backup {name}")
            if sgd.momentum:
                assert_bits_equal(m_dev[i], want["momentum"][i], f"step {step} momentum {name}")
        backup, bufs = want["backup"], (want["momentum"] if sgd.momentum else None)


def test_diloco_two_phase_matches_fused_and_checker(device):
    wl = _mlp_workload(2)
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    bufs = workloads.normal_tensors([(n, tuple(t.shape)) for n, t in zip(wl.names, wl.backup)],
                                    1e-3, 5, torch.device("cpu"))
    want = O.diloco_perform_sync(wl.replicas, wl.backup, bufs, [True, True], 2, True,
                                 lr=0.7, momentum=0.9, nesterov=True)
    b = [t.to(device) for t in wl.backup]
    m = [t.to(device) for t in bufs]
    reps = [[t.to(device) for t in rep] for rep in wl.replicas]
    p = reps[0]  # live params of "this" replica: in place
    g = [torch.empty_like(t) for t in b]
    ops.mt_pseudograd_avg(g, p, b, reps, restore_params=True)
    for i, name in enumerate(wl.names):
        assert_bits_equal(g[i], want["grads"][i], f"grad {name}")
        assert_bits_equal(p[i], wl.backup[i], f"restored {name}")
    ops.mt_outer_sgd(p, b, m, g, sgd, first_step=False)
    for i, name in enumerate(wl.names):
        assert_bits_equal(p[i], want["params"][i], f"params {name}")
        assert_bits_equal(b[i], want["backup"][i], f"backup {name}")
        assert_bits_equal(m[i], want["momentum"][i], f"momentum {name}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [1, 2, 3, 4, 7])
def test_outer_sgd_of_a_sum_divides_like_the_pass_it_replaces(device, dtype, n):
    """The gradient buffer holds the SUM a collective left in it.  Two ways to the same bits:
    Manager.allreduce's own division over the buffer (``reduce_avg_`` with one replica and
    ``num_participants = n``), then the outer SGD; or the outer SGD that divides on the way in.
    Sums over the whole encoding of the storage type, ragged sizes, misaligned views."""
    gen = torch.Generator().manual_seed(100 * n + int(dtype.itemsize))
    sizes = [1, 7, 1023, 4096, 65536 + 3, 300001]
    esize = dtype.itemsize

    def make(scale):
        out = []
        for i, size in enumerate(sizes):
            flat = torch.empty(size + 8, dtype=dtype, device=device)
            t = flat[(i % 3):(i % 3) + size]  # some views start off a 16-byte boundary
            t.copy_((scale * torch.randn(size, generator=gen)).to(dtype).to(device))
            out.append(t)
        return out

    def sums():
        out = []
        for i, size in enumerate(sizes):
            bits = torch.randint(0, 2 ** (8 * esize) - 1, (size,), generator=gen, dtype=torch.int64)
            raw = bits.to(torch.int32 if esize == 4 else torch.int16)
            flat = torch.empty(size + 8, dtype=dtype, device=device)
            t = flat[(i % 3):(i % 3) + size]
            t.copy_(raw.view(dtype).to(device))
            out.append(t)
        return out

    for sgd in (ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True),
                ops.OuterSGD(lr=0.1, momentum=0.5, dampening=0.1, weight_decay=0.01, nesterov=False),
                ops.OuterSGD(lr=0.3)):
        for first in (True, False):
            g = sums()
            b1, m1 = make(0.02), (make(1e-3) if sgd.momentum else None)
            b2 = [t.clone() for t in b1]
            m2 = [t.clone() for t in m1] if m1 is not None else None
            # the same misalignment on both sides: clone() re-aligns, so carve again
            def like(ts):
                out = []
                for i, t in enumerate(ts):
                    flat = torch.empty(t.numel() + 8, dtype=dtype, device=device)
                    v = flat[(i % 3):(i % 3) + t.numel()]
                    v.copy_(t)
                    out.append(v)
                return out
            b2, m2 = like(b2), (like(m2) if m2 is not None else None)
            p1, p2 = like(b1), like(b1)
            g_avg = like(g)
            for t in g_avg:
                ops.reduce_avg_(t, [t], 1, n)            # the pass Manager.allreduce makes
            ops.mt_outer_sgd(p1, b1, m1, g_avg, sgd, first)
            g_before = [t.clone() for t in g]
            ops.mt_outer_sgd(p2, b2, m2, g, sgd, first, grads_are_sums_of=n)
            for i in range(len(sizes)):
                assert_bits_equal(g[i], g_before[i], f"sum buffer {i} is only read")
                assert_bits_equal_up_to_nan_payload(p2[i], p1[i], f"params {i} n={n} first={first}")
                assert_bits_equal_up_to_nan_payload(b2[i], b1[i], f"backup {i}")
                if m1 is not None:
                    assert_bits_equal_up_to_nan_payload(m2[i], m1[i], f"momentum {i}")


def test_diloco_no_commit_leaves_state(device):
    """Phase 1 only (should_commit() false): params == backup, backup and momentum untouched."""
    wl = _mlp_workload(2)
    want = O.diloco_perform_sync(wl.replicas, wl.backup, None, [True, True], 2, False, lr=0.7,
                                 momentum=0.9, nesterov=True)
    b = [t.to(device) for t in wl.backup]
    reps = [[t.to(device) for t in rep] for rep in wl.replicas]
    g = [torch.empty_like(t) for t in b]
    ops.mt_pseudograd_avg(g, reps[0], b, reps, restore_params=True)
    for i, name in enumerate(wl.names):
        assert_bits_equal(reps[0][i], want["params"][i], name)
        assert_bits_equal(b[i], want["backup"][i], name)
        assert_bits_equal(g[i], want["grads"][i], name)


def test_localsgd_average_with_backup_refresh(device):
    wl = _mlp_workload(2)
    want = O.localsgd_perform_sync(wl.replicas, wl.backup, [True, True], 2, True)
    reps = [[t.to(device) for t in rep] for rep in wl.replicas]
    b = [t.to(device) for t in wl.backup]
    ops.mt_reduce_avg([reps[0], b], reps)
    for i, name in enumerate(wl.names):
        assert_bits_equal(reps[0][i], want["params"][i], name)
        assert_bits_equal(b[i], want["backup"][i], name)


@pytest.mark.parametrize("src_off,dst_off", [(0, 0), (16, 32), (4, 8), (4, 0), (1, 1), (3, 6), (2, 2)])
def test_mt_copy_bytes_alignments(device, src_off, dst_off):
    sizes = [0, 1, 5, 16, 17, 4096, 262144, 262144 + 33, 1_000_003]
    g = torch.Generator().manual_seed(3)
    srcs_cpu = [torch.randint(0, 256, (n + src_off,), dtype=torch.uint8, generator=g) for n in sizes]
    srcs = [t.to(device)[src_off:] for t in srcs_cpu]
    dst_full = [torch.full((n + dst_off + 5,), 0xAB, dtype=torch.uint8, device=device) for n in sizes]
    dsts = [t[dst_off:dst_off + n] for t, n in zip(dst_full, sizes)]
    ops.mt_copy(dsts, srcs)
    for full, src, n in zip(dst_full, srcs_cpu, sizes):
        want = torch.full((n + dst_off + 5,), 0xAB, dtype=torch.uint8)
        want[dst_off:dst_off + n] = src[src_off:]
        assert_bits_equal(full, want, f"n={n}")


def test_mt_copy_mixed_dtypes(device):
    srcs_cpu = [torch.randn(1000).bfloat16(), torch.randn(333), torch.arange(7, dtype=torch.int64)]
    srcs = [t.to(device) for t in srcs_cpu]
    dsts = [torch.empty_like(t) for t in srcs]
    ops.mt_copy(dsts, srcs)
    for d, s in zip(dsts, srcs_cpu):
        assert_bits_equal(d, s)


def variant_bits(unroll=0, plain=0, run_log2=None, lds_kib=None):
    return (unroll | (plain << 4) | ((run_log2 + 1) << 8 if run_log2 is not None else 0)
            | ((lds_kib // 8 + 1) << 12 if lds_kib is not None else 0))


def test_launch_variants_agree(device, launch_variant):
    """Every launch shape computes the same bits: slab size, plain / non-temporal accesses,
    per-XCD run length (a permutation of the slab order with a padded grid) and the
    residency cap."""
    wl = _mlp_workload(2)
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    want = O.diloco_perform_sync(wl.replicas, wl.backup, None, [True, True], 2, True, lr=0.7,
                                 momentum=0.9, nesterov=True)
    shapes = [variant_bits(u, pl) for u, pl in itertools.product([1, 2, 4], [0, 1])]
    shapes += [variant_bits(u, 0, r, lds) for u in (1, 2, 4) for r, lds in
               ((0, 0), (3, 0), (6, 64), (7, 32), (12, 0))]
    for bits in shapes:
        launch_variant(bits)
        b = [t.to(device) for t in wl.backup]
        m = [torch.empty_like(t) for t in b]
        p = [torch.empty_like(t) for t in b]
        reps = [[t.to(device) for t in rep] for rep in wl.replicas]
        ops.mt_diloco_outer(p, b, m, reps, sgd, True)
        for i, name in enumerate(wl.names):
            assert_bits_equal(p[i], want["params"][i], f"variant {bits:#x} {name}")
            assert_bits_equal(b[i], want["backup"][i], f"variant {bits:#x} {name}")
            assert_bits_equal(m[i], want["momentum"][i], f"variant {bits:#x} {name}")
        # the flat form and the byte copy take the same shapes
        x = [torch.randn(300_001, generator=torch.Generator().manual_seed(r)) for r in range(3)]
        out = torch.empty(300_001, device=device)
        ops.reduce_avg_(out, [t.to(device) for t in x], 0b101, 2)
        assert_bits_equal(out, O.manager_allreduce_(x, [True, False, True], 2), f"variant {bits:#x}")
        src = torch.arange(1_000_003, dtype=torch.int32, device=device).view(torch.uint8)[3:]
        dst = torch.zeros(src.numel() + 16, dtype=torch.uint8, device=device)
        ops.mt_copy([dst[7:7 + src.numel()]], [src])
        assert torch.equal(dst[7:7 + src.numel()], src) and int(dst[:7].sum()) == 0 \
            and int(dst[7 + src.numel():].sum()) == 0, f"variant {bits:#x}"


def test_fp16_rounding_and_overflow(device):
    """fp16 goes through fp32: one rounding to nearest even, overflow to inf, NaN stays NaN."""
    vals = [65504.0, 65504.0, 1.0, 1.0009765625, float("nan"), 6.0e-8, -0.0]
    a = torch.tensor(vals, dtype=torch.float16)
    b = torch.tensor([65504.0, -65504.0, 1.0009765625, 1.0009765625, 1.0, 6.0e-8, 0.0], dtype=torch.float16)
    want = O.manager_allreduce_([a, b], [True, True], 1, torch.float32)
    out = torch.empty_like(a).to(device)
    ops.reduce_avg_(out, [a.to(device), b.to(device)], 0b11, 1)
    out = out.cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(out), nan)  # the NaN payload is not part of the contract
    assert_bits_equal(out[~nan], want[~nan])
    assert torch.isinf(out[0]) and float(out[1]) == 0.0 and torch.isnan(out[4])


def test_argument_errors(device):
    x = torch.zeros(8, device=device)
    with pytest.raises(ValueError):
        ops.reduce_avg_(x, [x] * 9)
    with pytest.raises(ValueError):
        ops.reduce_avg_(x, [x], 0b10, 1)
    with pytest.raises(ValueError):
        ops.reduce_avg_(x, [x], 0b1, 0)
    with pytest.raises(ValueError):
        ops.reduce_avg_(x, [torch.zeros(9, device=device)])
    with pytest.raises(RuntimeError):
        ops.reduce_avg_(torch.zeros(8), [torch.zeros(8)])
    with pytest.raises(TypeError):
        ops.reduce_avg_(x.long(), [x.long()])
    with pytest.raises(ValueError):
        ops.reduce_avg_(torch.zeros(4, 4, device=device).t(), [x[:16]])


# ---------------------------------------------------------------------------
# Alignment: a common misalignment of all columns keeps the 128-bit body
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype,shift", [(torch.float32, 1), (torch.float32, 3), (torch.bfloat16, 1),
                                         (torch.bfloat16, 5), (torch.float16, 7)])
def test_diloco_on_views_behind_an_odd_sized_tensor(device, dtype, shift):
    """All columns start ``shift`` elements past a 16-byte boundary (what views into flat
    buffers look like behind an odd-sized tensor): head elements scalar, 128-bit body, scalar
    tail; several tensors per table, sizes around the slab and head boundaries; guard
    elements in front of and behind every view must stay untouched."""
    sizes = [1, 2, 3, 4, 7, 8, 9, 2047, 2048, 2049, 8191, 8192, 8193, 65536 + 3, 300_007]
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    g = torch.Generator().manual_seed(11)

    def host(scale):
        return [(torch.randn(n + shift + 1, generator=g) * scale).to(dtype) for n in sizes]

    backup_h, buf_h = host(0.02), host(1e-3)
    reps_h = [[(b.float() + 1e-3 * torch.randn(b.shape, generator=g)).to(dtype) for b in backup_h]
              for _ in range(3)]
    view = lambda ts: [t[shift:-1] for t in ts]
    want = O.diloco_perform_sync([view(r) for r in reps_h], view(backup_h), view(buf_h),
                                 [True, False, True], 2, True, lr=0.7, momentum=0.9, nesterov=True,
                                 accumulate_dtype=torch.float32)
    b_d, m_d = [t.to(device) for t in backup_h], [t.to(device) for t in buf_h]
    p_d = [torch.full_like(t, 7.0) for t in b_d]
    r_d = [[t.to(device) for t in rep] for rep in reps_h]
    ops.mt_diloco_outer(view(p_d), view(b_d), view(m_d), [view(r) for r in r_d], sgd, False, 0b101, 2)
    for i, n in enumerate(sizes):
        for got, exp, src, what in ((p_d[i], want["params"][i], None, "params"),
                                    (b_d[i], want["backup"][i], backup_h[i], "backup"),
                                    (m_d[i], want["momentum"][i], buf_h[i], "momentum")):
            assert_bits_equal(got[shift:-1], exp, f"{what} n={n}")
            guard = torch.full((1,), 7.0, dtype=dtype) if src is None else None
            for sl in (slice(0, shift), slice(-1, None)):
                assert_bits_equal(got[sl], guard.expand(got[sl].shape) if src is None else src[sl],
                                  f"{what} guard n={n}")
        for r in (0, 2):
            assert_bits_equal(r_d[r][i], reps_h[r][i], f"replica {r} n={n} was modified")


@pytest.mark.parametrize("dtype,shift_bytes", [(torch.float32, 4), (torch.bfloat16, 2)])
def test_large_misaligned_tensor_against_the_checker(device, dtype, shift_bytes):
    """50 M elements starting 4 bytes (fp32) / 2 bytes (bf16) past a 16-byte boundary, all
    columns alike: in-place average of three contributions, held to the checker bit for bit
    (and the same data aligned must give the same values)."""
    n = 50_000_000
    shift = shift_bytes // torch.empty(0, dtype=dtype).element_size()
    g = torch.Generator().manual_seed(3)
    reps_h = [(torch.randn(n + shift, generator=g) * 0.01).to(dtype) for _ in range(3)]
    want = O.manager_allreduce_([r[shift:] for r in reps_h], [True, True, True], 3, torch.float32)
    dev = [r.to(device) for r in reps_h]
    assert all(d[shift:].data_ptr() % 16 == shift_bytes for d in dev)
    ops.reduce_avg_(dev[0][shift:], [d[shift:] for d in dev], 0b111, 3)
    assert_bits_equal(dev[0][shift:], want)
    assert_bits_equal(dev[0][:shift], reps_h[0][:shift])
    aligned = [r[shift:].clone().to(device) for r in reps_h]
    ops.reduce_avg_(aligned[0], aligned, 0b111, 3)
    assert_bits_equal(aligned[0], want)


def test_copy_with_common_and_mixed_misalignment(device):
    """Byte copy: dst and src misaligned alike (vector body after a head of bytes), alike only
    modulo 4 (word path), and arbitrarily (byte path); guards around every destination."""
    g = torch.Generator().manual_seed(5)
    for n in (1, 5, 15, 16, 17, 4095, 4096, 4097, 70_001, 1_000_003):
        for d_off, s_off in ((3, 3), (13, 13), (1, 17), (2, 6), (5, 9), (0, 1), (7, 2), (0, 0)):
            src = torch.randint(0, 256, (n + 64,), dtype=torch.uint8, generator=g)
            dst = torch.full((n + 64,), 0xAB, dtype=torch.uint8)
            s_d, d_d = src.to(device), dst.to(device)
            ops.mt_copy([d_d[d_off:d_off + n]], [s_d[s_off:s_off + n]])
            want = dst.clone()
            want[d_off:d_off + n] = src[s_off:s_off + n]
            assert torch.equal(d_d.cpu(), want), f"n={n} dst+{d_off} src+{s_off}"


# ---------------------------------------------------------------------------
# DiLoCo on bf16 / fp16 parameters (torchft/local_sgd.py:212-215 is dtype-generic)
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sgd_kw", SGD_CASES)
def test_diloco_16_bit_storage(device, dtype, sgd_kw):
    """Fused and two-launch forms on 16-bit parameters: fp32 arithmetic, one rounding per
    stored value.  Bit-exact against the checker's fp32-arithmetic variant; within the stated
    rtol 1e-2 of the reference form that rounds after every torch op."""
    wl = _mlp_workload(3)
    sgd = ops.OuterSGD(**sgd_kw)
    kw = dict(lr=sgd.lr, momentum=sgd.momentum, dampening=sgd.dampening,
              weight_decay=sgd.weight_decay, nesterov=sgd.nesterov)
    flags, mask, nump = [True, True, False], 0b011, 2
    backup = [t.to(dtype) for t in wl.backup]
    bufs = None
    for step in range(2):
        first = step == 0
        reps = [[(b.float() + 1e-3 * torch.randn(b.shape, generator=torch.Generator().manual_seed(
            100 * step + 10 * r + i))).to(dtype) for i, b in enumerate(backup)] for r in range(3)]
        want = O.diloco_perform_sync(reps, backup, bufs, flags, nump, True, **kw,
                                     accumulate_dtype=torch.float32)
        want2 = O.diloco_perform_sync(reps, backup, bufs, flags, nump, True, **kw,
                                      accumulate_dtype=torch.float32, grads_through_storage=True)
        native = O.diloco_perform_sync(reps, backup, bufs, flags, nump, True, **kw)
        to_dev = lambda ts: [t.to(device) for t in ts]
        for form in ("fused", "two_launch"):
            b_d, r_d = to_dev(backup), [to_dev(r) for r in reps]
            m_d = None
            if sgd.momentum:
                m_d = [torch.full_like(t, float("nan")) for t in b_d] if first else to_dev(bufs)
            p_d = r_d[0]  # in place on replica 0, as the API path runs it
            if form == "fused":
                ops.mt_diloco_outer(p_d, b_d, m_d, r_d, sgd, first, mask, nump)
                exp = want
            else:
                g_d = [torch.empty_like(t) for t in b_d]
                ops.mt_pseudograd_avg(g_d, p_d, b_d, r_d, True, mask, nump)
                for i in range(len(backup)):
                    assert_bits_equal(g_d[i], want2["grads"][i], f"{form} grads {wl.names[i]}")
                    assert_bits_equal(p_d[i], backup[i], f"{form} restore {wl.names[i]}")
                ops.mt_outer_sgd(p_d, b_d, m_d, g_d, sgd, first)
                exp = want2
            for i, name in enumerate(wl.names):
                assert_bits_equal(p_d[i], exp["params"][i], f"{form} step {step} params {name}")
                assert_bits_equal(b_d[i], exp["backup"][i], f"{form} step {step} backup {name}")
                if sgd.momentum:
                    assert_bits_equal(m_d[i], exp["momentum"][i], f"{form} step {step} momentum {name}")
                    torch.testing.assert_close(m_d[i].cpu().float(), native["momentum"][i].float(),
                                               rtol=1e-2, atol=2e-4)
                torch.testing.assert_close(p_d[i].cpu().float(), native["params"][i].float(),
                                           rtol=1e-2, atol=2e-4)
        backup, bufs = want["backup"], (want["momentum"] if sgd.momentum else None)


def test_fp16_result_is_rounded_from_the_fp32_value(device):
    """An element whose fp32 result lies exactly on the tie between two fp16 values
    (0x3a3f5000: the low 13 bits are 0x1000).  The update's last fused multiply-add must
    first round to fp32 and only then to fp16 (ties to even: 0x11fa); folding both into one
    mixed-precision instruction rounds the exact product-sum instead and gives 0x11fb."""
    vals = dict(b=0.001712799072265625, m=0.0012683868408203125, x0=0.0028934478759765625,
                x2=0.0009288787841796875)
    n = 5000
    mk = lambda v: torch.full((n,), v, dtype=torch.float16)
    b, m, x0, x1, x2 = mk(vals["b"]), mk(vals["m"]), mk(vals["x0"]), mk(123.0), mk(vals["x2"])
    want = O.diloco_perform_sync([[x0], [x1], [x2]], [b], [m], [True, False, True], 2, True,
                                 lr=0.7, momentum=0.9, nesterov=True, accumulate_dtype=torch.float32)
    assert int(want["params"][0][0].view(torch.int16)) == 0x11fa
    d = lambda t: t.to(device)
    p_d, b_d, m_d = torch.empty(n, dtype=torch.float16, device=device), d(b), d(m)
    ops.mt_diloco_outer([p_d], [b_d], [m_d], [[d(x0)], [d(x1)], [d(x2)]],
                        ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True), False, 0b101, 2)
    assert_bits_equal(p_d, want["params"][0])
    assert_bits_equal(b_d, want["backup"][0])
    assert_bits_equal(m_d, want["momentum"][0])


def _bit_patterns(n, dtype, seed):
    """Values over the whole encoding: random bit patterns, plus runs confined to the
    smallest exponents (denormal and barely normal), the largest ones (next to overflow,
    infinities, NaNs) and ordinary magnitudes."""
    g = torch.Generator().manual_seed(seed)
    if dtype == torch.float32:
        raw = torch.randint(-2**31, 2**31, (n,), generator=g, dtype=torch.int64).to(torch.int32)
        mant, sign, shift, top = 0x007fffff, -2**31, 23, 0xff
    else:
        raw = torch.randint(-2**15, 2**15, (n,), generator=g, dtype=torch.int64).to(torch.int16)
        shift = 7 if dtype == torch.bfloat16 else 10
        mant, sign, top = (1 << shift) - 1, -2**15, 0xff if dtype == torch.bfloat16 else 0x1f
    kind = torch.randint(0, 4, (n,), generator=g)
    low = torch.randint(0, 3, (n,), generator=g, dtype=torch.int64)
    high = top - torch.randint(0, 3, (n,), generator=g, dtype=torch.int64)
    r64 = raw.to(torch.int64)
    keep = r64 & (mant | sign)
    r64 = torch.where(kind == 1, keep | (low << shift), r64)
    r64 = torch.where(kind == 2, keep | (high << shift), r64)
    out = r64.to(raw.dtype).view(dtype)
    ordinary = torch.randn(n, generator=g).to(dtype)
    return torch.where(kind == 3, ordinary, out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n_replicas,mask,nump", [(2, 0b11, 2), (2, 0b11, 1), (4, 0b1111, 4), (3, 0b111, 3),
                                                 (2, 0b01, 2), (8, 0xFF, 8), (2, 0b11, 64)])
def test_reduce_avg_over_the_whole_encoding(device, dtype, n_replicas, mask, nump):
    """Denormals, values next to overflow, infinities and NaNs through the reduction, for
    divisors that are powers of two (multiplied by the exact reciprocal when everybody
    participates) and divisors that are not (IEEE division), on full and ragged slabs."""
    numel = 3 * 65536 + 1234
    reps = [_bit_patterns(numel, dtype, 900 + r) for r in range(n_replicas)]
    want = O.manager_allreduce_(reps, mask_to_list(mask, n_replicas), nump, torch.float32)
    out = torch.empty(numel, dtype=dtype, device=device)
    ops.reduce_avg_(out, [r.to(device) for r in reps], mask, nump)
    assert_bits_equal_up_to_nan_payload(out, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sgd_kw", [SGD_CASES[0], SGD_CASES[2]])
@pytest.mark.parametrize("n_replicas,mask,nump", [(2, 0b11, 2), (2, 0b11, 3), (4, 0b0111, 4)])
def test_diloco_over_the_whole_encoding(device, dtype, sgd_kw, n_replicas, mask, nump):
    """The fused step and the two-launch form on inputs drawn over the whole encoding, in
    the common configuration (everybody participates, power-of-two divisor, Nesterov
    momentum) and outside it."""
    numel = 2 * 65536 + 777
    sgd = ops.OuterSGD(**sgd_kw)
    kw = dict(lr=sgd.lr, momentum=sgd.momentum, dampening=sgd.dampening,
              weight_decay=sgd.weight_decay, nesterov=sgd.nesterov)
    flags = mask_to_list(mask, n_replicas)
    backup = [_bit_patterns(numel, dtype, 1)]
    bufs = [_bit_patterns(numel, dtype, 2)]
    reps = [[_bit_patterns(numel, dtype, 10 + r)] for r in range(n_replicas)]
    extra = {} if dtype == torch.float32 else dict(accumulate_dtype=torch.float32)
    want = O.diloco_perform_sync(reps, backup, bufs, flags, nump, True, **kw, **extra)
    to_dev = lambda ts: [t.to(device) for t in ts]
    b_d, m_d, r_d = to_dev(backup), to_dev(bufs), [to_dev(r) for r in reps]
    p_d = [torch.empty_like(b_d[0])]
    ops.mt_diloco_outer(p_d, b_d, m_d, r_d, sgd, False, mask, nump)
    assert_bits_equal_up_to_nan_payload(p_d[0], want["params"][0], "params")
    assert_bits_equal_up_to_nan_payload(b_d[0], want["backup"][0], "backup")
    assert_bits_equal_up_to_nan_payload(m_d[0], want["momentum"][0], "momentum")
    if dtype == torch.float32:  # two launches, the pseudo-gradient passing through memory
        b_d, m_d = to_dev(backup), to_dev(bufs)
        g_d = [torch.empty_like(b_d[0])]
        ops.mt_pseudograd_avg(g_d, p_d, b_d, r_d, True, mask, nump)
        assert_bits_equal_up_to_nan_payload(g_d[0], want["grads"][0], "grads")
        ops.mt_outer_sgd(p_d, b_d, m_d, g_d, sgd, False)
        assert_bits_equal_up_to_nan_payload(p_d[0], want["params"][0], "two-launch params")
        assert_bits_equal_up_to_nan_payload(m_d[0], want["momentum"][0], "two-launch momentum")
