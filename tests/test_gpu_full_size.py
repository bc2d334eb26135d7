"""Full-size runs of the named configurations on the GPU.

The CPU checker cannot process 8 billion parameters in seconds, so these tests lean on
what does not depend on size: every kernel is elementwise, hence windows of the full-size
result (head, tail and seeded random positions of every tensor, which is where indexing
mistakes live) must equal the checker run on the same windows; plus invariants
(backup == parameters after a committed step, fixed point when all replicas equal the
backup, idempotent restore, pack -> unpack identity with device-side comparison).
"""

import gc

import pytest
import torch

from helpers import assert_bits_equal
from oracle import replica_sync as O
from torchft_amd import GradBucketAverager, ops, state_pack, workloads

pytestmark = pytest.mark.gpu

WINDOW = 4096


def windows(numel: int, gen: torch.Generator, k: int = 3):
    """Element ranges to compare: head, tail and k random windows (whole tensor if small)."""
    if numel <= 4 * WINDOW:
        return [(0, numel)]
    spans = [(0, WINDOW), (numel - WINDOW, numel)]
    for _ in range(k):
        lo = int(torch.randint(0, numel - WINDOW, (1,), generator=gen))
        spans.append((lo, lo + WINDOW))
    # chunk and slab boundaries of the kernels (65536 / 2048 elements)
    spans.append((65536 - 100, 65536 + 100))
    return spans


def take(t: torch.Tensor, spans):
    flat = t.reshape(-1)
    return torch.cat([flat[lo:hi] for lo, hi in spans]).cpu()


@pytest.fixture(autouse=True)
def free_memory():
    yield
    gc.collect()
    torch.cuda.empty_cache()


def test_diloco_llama3_8b_full_size(device):
    """DiLoCo outer step, fp32, all 291 Llama-3-8B tensors (8 030 261 248 parameters), 2
    replicas, Nesterov SGD lr 0.7 momentum 0.9: a first step and a steady-state step."""
    shapes = workloads.llama3_8b_shapes()
    wl = workloads.make_diloco_workload(shapes, 2, device)
    assert wl.n_params == 8_030_261_248
    params = [torch.empty_like(t) for t in wl.backup]
    bufs = [torch.empty_like(t) for t in wl.backup]
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    gen = torch.Generator().manual_seed(11)
    spans = [windows(t.numel(), gen) for t in wl.backup]
    table = None
    for step in range(2):
        before_b = [take(t, s) for t, s in zip(wl.backup, spans)]
        before_m = [take(t, s) for t, s in zip(bufs, spans)] if step else None
        reps = [[take(t, s) for t, s in zip(rep, spans)] for rep in wl.replicas]
        table = ops.mt_diloco_outer(params, wl.backup, bufs, wl.replicas, sgd, step == 0, table=table)
        want = O.diloco_perform_sync(reps, before_b, before_m, [True, True], 2, True,
                                     lr=0.7, momentum=0.9, nesterov=True)
        for i, (name, _) in enumerate(shapes):
            assert_bits_equal(take(params[i], spans[i]), want["params"][i], f"step {step} {name}")
            assert_bits_equal(take(bufs[i], spans[i]), want["momentum"][i], f"step {step} momentum {name}")
        # committed step: backup == parameters everywhere (compared on the device)
        assert all(torch.equal(p, b) for p, b in zip(params, wl.backup))
    # fixed point: replicas equal to the backup and zero momentum leave everything in place
    for m in bufs:
        m.zero_()
    snapshot = [take(t, s) for t, s in zip(wl.backup, spans)]
    ops.mt_diloco_outer(params, wl.backup, bufs, [wl.backup, wl.backup], sgd, False)
    for i in range(len(shapes)):
        assert_bits_equal(take(wl.backup[i], spans[i]), snapshot[i])
    assert all(int(torch.count_nonzero(m)) == 0 for m in bufs[:5])


def test_diloco_llama3_8b_full_size_bf16_in_place(device):
    """The same step on bf16 storage (fp32 arithmetic, one rounding per stored value), updated
    in place on replica 0 as ``DiLoCo.sync()`` runs it: windows of every tensor against the
    checker, backup == parameters everywhere, and the peer replica untouched."""
    shapes = workloads.llama3_8b_shapes()
    wl = workloads.make_diloco_workload(shapes, 2, device, torch.bfloat16)
    bufs = [torch.zeros_like(t) for t in wl.backup]
    params = wl.replicas[0]
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    gen = torch.Generator().manual_seed(13)
    spans = [windows(t.numel(), gen) for t in wl.backup]
    peer_before = [take(t, s) for t, s in zip(wl.replicas[1], spans)]
    table = None
    for step in range(2):
        before_b = [take(t, s) for t, s in zip(wl.backup, spans)]
        before_m = [take(t, s) for t, s in zip(bufs, spans)] if step else None
        reps = [[take(t, s) for t, s in zip(rep, spans)] for rep in wl.replicas]
        table = ops.mt_diloco_outer(params, wl.backup, bufs, wl.replicas, sgd, step == 0, table=table)
        want = O.diloco_perform_sync(reps, before_b, before_m, [True, True], 2, True,
                                     lr=0.7, momentum=0.9, nesterov=True, accumulate_dtype=torch.float32)
        for i, (name, _) in enumerate(shapes):
            assert_bits_equal(take(params[i], spans[i]), want["params"][i], f"step {step} {name}")
            assert_bits_equal(take(bufs[i], spans[i]), want["momentum"][i], f"step {step} momentum {name}")
        assert all(torch.equal(p, b) for p, b in zip(params, wl.backup))
    for i in range(len(shapes)):
        assert_bits_equal(take(wl.replicas[1][i], spans[i]), peer_before[i])


def test_diloco_sync_llama3_8b_full_size_fp32_through_the_api(device):
    """Config 4 through the reference's own seat: ``DiLoCo.sync()`` on a module with the 291
    fp32 Llama-3-8B parameters, this package's Manager on a local replica group of 2, outer
    ``torch.optim.SGD`` (Nesterov).  The parameters are replica 0 and are updated in place;
    backup and momentum are the library's own (placed) buffers.  A first sync and two
    steady-state syncs: windows of every tensor of the parameters, the backup and
    ``outer_optimizer.state[p]["momentum_buffer"]`` against the checker, backup == parameters
    everywhere, the peer untouched, ``id(param)`` and the inner optimizer's state intact."""
    from torch import nn, optim

    from torchft_amd import DiLoCo, Manager, ProcessGroupLocalReplicas, StaticQuorum

    shapes = workloads.llama3_8b_shapes()

    class Bag(nn.Module):
        def __init__(self) -> None:
            super().__init__()
            self.ps = nn.ParameterList(
                [nn.Parameter(t) for t in workloads.normal_tensors(shapes, 0.02, workloads.SEED_BACKUP, device)])

    model = Bag()
    params = list(model.parameters())
    assert sum(p.numel() for p in params) == 8_030_261_248
    peer = workloads.drifted_replica([p.data for p in params], 1e-3, workloads.SEED_REPLICA + 1)
    index = {p.data_ptr(): i for i, p in enumerate(params)}
    pg = ProcessGroupLocalReplicas(0, 2, peer_lookup=lambda t: [peer[index[t.data_ptr()]]],
                                   peers_are_stable=True)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                      use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(params, lr=0.1, momentum=0.5)
    outer = optim.SGD(params, lr=0.7, momentum=0.9, nesterov=True)
    ids = [id(p) for p in params]
    gen = torch.Generator().manual_seed(17)
    spans = [windows(p.numel(), gen) for p in params]
    peer_before = [take(t, s) for t, s in zip(peer, spans)]
    with DiLoCo(manager, model, inner, outer, sync_every=10 ** 9) as diloco:
        backups = list(diloco._backup_parameters.values())
        assert outer.state_dict()["state"] == {}
        bufs_before = None
        for step in range(3):
            # the replica has drifted since the last sync (inner steps): here one known shift
            with torch.no_grad():
                torch._foreach_add_([p.data for p in params], 1e-3 * (step + 1))
            local = [take(p.data, s) for p, s in zip(params, spans)]
            before_b = [take(b, s) for b, s in zip(backups, spans)]
            diloco.sync()
            want = O.diloco_perform_sync([local, peer_before], before_b, bufs_before, [True, True], 2,
                                         True, lr=0.7, momentum=0.9, nesterov=True)
            for i, (name, _) in enumerate(shapes):
                assert_bits_equal(take(params[i].data, spans[i]), want["params"][i], f"sync {step} {name}")
                assert_bits_equal(take(backups[i], spans[i]), want["backup"][i], f"sync {step} backup {name}")
                assert_bits_equal(take(outer.state[params[i]]["momentum_buffer"], spans[i]),
                                  want["momentum"][i], f"sync {step} momentum {name}")
            assert all(torch.equal(p.data, b) for p, b in zip(params, backups))
            assert all(p.grad is None for p in params)
            bufs_before = want["momentum"]
        assert len(outer.state_dict()["state"]) == len(params)
    assert manager.current_step() == 3
    assert [id(p) for p in model.parameters()] == ids
    assert list(diloco._backup_parameters.values())[0] is backups[0]
    for i in range(len(shapes)):
        assert_bits_equal(take(peer[i], spans[i]), peer_before[i])
    manager.shutdown(wait=False)


def test_ddp_buckets_llama3_8b_full_size(device):
    """bf16 gradients of Llama-3-8B, 162 buckets by torch's rule, 4 contributions of which
    3 participate, fp32 accumulation, result written over replica 0's gradients."""
    shapes = workloads.llama3_8b_shapes()
    grads = workloads.make_grad_replicas(shapes, 4, device, torch.bfloat16)
    gen = torch.Generator().manual_seed(12)
    spans = [windows(t.numel(), gen) for t in grads[0]]
    before = [[take(t, s) for t, s in zip(rep, spans)] for rep in grads]
    averager = GradBucketAverager(grads[0], grads)
    assert len(averager.buckets) == 162
    assert averager.buckets == O.bucket_assignment([g.numel() for g in grads[0]], 2)
    averager.average_all(0b0111, 3)
    for i, (name, _) in enumerate(shapes):
        want = O.manager_allreduce_([before[r][i] for r in range(4)], [True, True, True, False], 3,
                                    torch.float32)
        assert_bits_equal(take(grads[0][i], spans[i]), want, name)
        native = O.manager_allreduce_([before[r][i] for r in range(4)], [True, True, True, False], 3)
        torch.testing.assert_close(want.float(), native.float(), rtol=1e-2, atol=2e-4)
        for r in (1, 2, 3):  # contributions are read-only
            assert_bits_equal(take(grads[r][i], spans[i]), before[r][i])


def test_checkpoint_llama3_8b_full_size(device):
    """80 GB training state (bf16 params, fp32 AdamW moments, int64 steps): pack into one
    staging buffer, scatter back into fresh tensors; both directions compared on the device
    tensor by tensor, plus a slice of the staging buffer through pinned host memory."""
    shapes = workloads.llama3_8b_shapes()
    state = workloads.make_training_state(shapes, device)
    packed = state_pack.pack(state)
    plan = packed.plan
    assert len(plan.entries) == 4 * 291 and plan.total_bytes > 80e9
    for e, src in zip(plan.entries, plan.tensors):
        view = packed.staging[e.offset:e.offset + e.nbytes]
        assert torch.equal(view, src.reshape(-1).view(torch.uint8)), f"packed bytes at {e.offset}"
    header, staging = packed.header, packed.staging
    del packed, plan
    # free the source, then unpack by scattering into new tensors (80 GB + 80 GB resident)
    fingerprint = {n: t.view(torch.int16).sum(dtype=torch.int64).item()
                   for n, t in state["user"]["model"].items()}
    moments = {i: (st["exp_avg"].view(torch.int32).sum(dtype=torch.int64).item(),
                   st["exp_avg_sq"].view(torch.int32).sum(dtype=torch.int64).item(),
                   int(st["step"]))
               for i, st in state["user"]["optim"]["state"].items()}
    meta = (state["torchft"], state["user"]["optim"]["param_groups"])
    del state
    gc.collect()
    torch.cuda.empty_cache()
    out = state_pack.unpack(header, staging, copy=True)
    assert (out["torchft"], out["user"]["optim"]["param_groups"]) == meta
    for n, t in out["user"]["model"].items():
        assert t.dtype == torch.bfloat16
        assert t.view(torch.int16).sum(dtype=torch.int64).item() == fingerprint[n], n
    for i, st in out["user"]["optim"]["state"].items():
        got = (st["exp_avg"].view(torch.int32).sum(dtype=torch.int64).item(),
               st["exp_avg_sq"].view(torch.int32).sum(dtype=torch.int64).item(), int(st["step"]))
        assert got == moments[i], i
    # every scattered tensor equals the view of the staging buffer it came from (the staging
    # buffer itself was compared with the source tensors above), element for element
    views = state_pack.unpack(header, staging, copy=False)
    for n, t in out["user"]["model"].items():
        assert torch.equal(t, views["user"]["model"][n]), n
    for i, st in out["user"]["optim"]["state"].items():
        ref = views["user"]["optim"]["state"][i]
        for key in ("exp_avg", "exp_avg_sq", "step"):
            got, want = st[key], ref[key]
            assert got.dtype == want.dtype and got.shape == want.shape, (i, key)
            assert torch.equal(got.view(torch.uint8) if got.dim() else got, 
                               want.view(torch.uint8) if want.dim() else want), (i, key)
    del out, views
    gc.collect()
    torch.cuda.empty_cache()
    # the PCIe legs of the configuration: the WHOLE staging buffer to pinned host memory and
    # back into a second device buffer, through two 1 GiB pinned bounce buffers
    total = staging.numel()
    back = torch.empty(total, dtype=torch.uint8, device=device)
    chunk = 1 << 30
    bounce = [torch.empty(chunk, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
    for k, lo in enumerate(range(0, total, chunk)):
        n = min(chunk, total - lo)
        bounce[k % 2][:n].copy_(staging[lo:lo + n], non_blocking=True)   # same stream: ordered
        back[lo:lo + n].copy_(bounce[k % 2][:n], non_blocking=True)
    torch.cuda.synchronize()
    assert torch.equal(back, staging)


def test_more_than_2_31_work_items_in_one_launch(device, launch_variant):
    """A launch whose slab count exceeds what one grid dimension can hold (40 GiB through
    the byte copy is 5.2 M workgroups of 8 KiB, 10.5 M at 4 KiB) must still cover
    everything: the grid is split in two dimensions."""
    n = 40 << 30
    src = torch.empty(n, dtype=torch.uint8, device=device)
    src.view(torch.int64).copy_(torch.arange(n // 8, dtype=torch.int64, device=device))
    dst = torch.zeros(n, dtype=torch.uint8, device=device)
    for variant in (1, 2, 1 | (8 << 8)):  # 4 KiB slabs, 8 KiB slabs, 4 KiB with per-XCD runs of 128
        launch_variant(variant)
        dst.zero_()
        ops.mt_copy([dst], [src])
        assert torch.equal(dst, src), f"variant {variant:#x}"
