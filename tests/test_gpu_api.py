"""GPU parity through the reference-shaped API: Manager.allreduce, LocalSGD, DiLoCo, the DDP
communication hook, the bucket averager and the checkpoint transport, each against the
CPU checker on the same seeded inputs.  fp32 results are compared bit for bit (same IEEE
operations in the same order); the bf16 path additionally against the bf16-accumulating
form a c10d backend would compute, at the specified rtol of 1e-2.
"""

import copy
import io
from datetime import timedelta
from unittest.mock import MagicMock, create_autospec

import pytest
import torch
from torch import nn, optim
from torch.futures import Future

from helpers import assert_bits_equal
from oracle import replica_sync as O
from torchft_amd import (
    CheckpointServer,
    DiLoCo,
    DistributedDataParallel,
    GradBucketAverager,
    PureDistributedDataParallel,
    LocalSGD,
    Manager,
    ProcessGroup,
    ProcessGroupLocalReplicas,
    QuorumResult,
    StaticQuorum,
    WorldSizeMode,
    state_pack,
    workloads,
)
from torchft_amd.manager import QuorumClient
from torchft_amd.process_group import _DummyWork

pytestmark = pytest.mark.gpu

RTOL_F32 = 1e-6   # specified bar for fp32 outputs
RTOL_BF16 = 1e-2  # specified bar for bf16 outputs after fp32 accumulation


class MLP(nn.Module):
    """The 3-layer MLP of the CPU-runnable configuration (6 316 042 parameters)."""

    def __init__(self) -> None:
        super().__init__()
        self.net = nn.Sequential(nn.Linear(1024, 2048), nn.ReLU(), nn.Linear(2048, 2048), nn.ReLU(),
                                 nn.Linear(2048, 10))
        for p in self.parameters():
            nn.init.normal_(p, 0.0, 0.02)

    def forward(self, x):
        return self.net(x)


class Tiny(nn.Module):
    def __init__(self) -> None:
        super().__init__()
        self.net = nn.Sequential(nn.Linear(3, 4), nn.ReLU(), nn.Linear(4, 5), nn.Sigmoid())

    def forward(self, x):
        return self.net(x)


class Scripted(QuorumClient):
    def __init__(self, result, commit=True):
        self.result, self.commit = result, commit

    def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
        return self.result

    def should_commit(self, rank, step, should_commit, timeout):
        return should_commit and self.commit


def cpu(tensors):
    return [t.detach().cpu().clone() for t in tensors]


def peer_world(model, n):
    """n-1 deep copies of ``model`` on its device and a lookup pairing their parameters
    (and gradients) with the local model's."""
    peers = [copy.deepcopy(model) for _ in range(n - 1)]

    def lookup(t):
        for k, p in enumerate(model.parameters()):
            for is_grad, local in ((False, p.data), (True, p.grad)):
                if local is not None and local.data_ptr() == t.data_ptr():
                    out = []
                    for peer in peers:
                        q = list(peer.parameters())[k]
                        out.append(q.grad if is_grad else q.data)
                    return out
        raise KeyError("unknown tensor")

    return peers, lookup


# ---------------------------------------------------------------------------
# Manager.allreduce
# ---------------------------------------------------------------------------

def test_manager_numerics_generic_process_group(device):
    """torchft/manager_test.py:520-543 on the GPU with a mocked backend: zeroing and
    division are this package's kernels around the backend's (no-op) collective."""
    m = Manager(pg=create_autospec(ProcessGroup), load_state_dict=None, state_dict=None, min_replica_size=2)
    m._quorum_future = MagicMock()
    m._participating_rank, m._participating_world_size = 1, 5
    m._pg.allreduce.return_value = _DummyWork(None)
    t = torch.tensor([1.0], device=device)
    assert m.allreduce(t).value() is t
    torch.testing.assert_close(t.cpu(), torch.tensor([1.0 / 5]))
    m._healing = True
    t = torch.tensor([1.0], device=device)
    m.allreduce(t).value()
    torch.testing.assert_close(t.cpu(), torch.tensor([0.0]))
    m.shutdown(wait=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_manager_allreduce_local_replicas(device, dtype):
    """4 contributors, the last one a spare (FIXED_WITH_SPARES, 3 active): config-3 style."""
    n = 1_000_003
    g = torch.Generator().manual_seed(5)
    xs = [(torch.randn(n, generator=g) * 1e-2).to(dtype) for _ in range(4)]
    dev = [x.to(device) for x in xs]
    pg = ProcessGroupLocalReplicas(rank=1, world_size=4, peer_participating=[True, True, False])
    pg.register_peers(dev[1], [dev[0], dev[2], dev[3]])
    q = QuorumResult(quorum_id=1, replica_rank=1, replica_world_size=4, max_rank=1, max_world_size=4)
    m = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=3, world_size_mode=WorldSizeMode.FIXED_WITH_SPARES,
                quorum_client=Scripted(q))
    m.start_quorum()
    fut = m.allreduce(dev[1])
    assert fut.wait() is dev[1]
    assert m.num_participants() == 3 and m.is_participating()
    want = O.manager_allreduce_(xs, [True, True, True, False], 3, torch.float32)
    assert_bits_equal(dev[1], want)
    if dtype == torch.bfloat16:
        native = O.manager_allreduce_(xs, [True, True, True, False], 3)
        torch.testing.assert_close(dev[1].cpu().float(), native.float(), rtol=RTOL_BF16, atol=1e-4)
    for i in (0, 2, 3):
        assert_bits_equal(dev[i], xs[i])  # peers' buffers are read-only
    assert m.should_commit()
    m.shutdown(wait=False)


def test_manager_error_latch_on_gpu(device):
    pg = ProcessGroupLocalReplicas(rank=0, world_size=2)  # no peers registered
    m = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1, quorum_client=StaticQuorum(0, 2))
    m.start_quorum()
    t = torch.ones(8, device=device)
    assert m.allreduce(t).wait() is t  # KeyError swallowed
    assert isinstance(m.errored(), KeyError)
    assert_bits_equal(t, torch.ones(8))
    assert not m.should_commit()
    m.shutdown(wait=False)


def test_manager_allreduce_is_dtype_generic_and_never_raises(device):
    """torchft/manager.py:242-303 reduces whatever floating tensor it is given and never raises.
    fp64 runs in fp64 (oracle bits); a tensor the kernels cannot take (integer, not contiguous,
    on the host) is latched like any failed all-reduce: the future completes with the tensor
    untouched, later calls are no-ops, the step does not commit, the next quorum clears it."""
    n = 100_003
    g = torch.Generator().manual_seed(3)
    xs = [torch.randn(n, generator=g, dtype=torch.float64) for _ in range(3)]
    dev = [x.to(device) for x in xs]
    pg = ProcessGroupLocalReplicas(rank=0, world_size=3, peer_participating=[True, False])
    pg.register_peers(dev[0], dev[1:])
    m = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                quorum_client=StaticQuorum(0, 3))
    m.start_quorum()
    assert m.allreduce(dev[0]).wait() is dev[0]
    assert m.errored() is None
    assert_bits_equal(dev[0], O.manager_allreduce_(xs, [True, True, False], 3))
    assert m.should_commit()

    for make, kind in (
        (lambda: torch.arange(8, device=device), TypeError),                   # integer
        (lambda: torch.ones(4, 6, device=device).t(), ValueError),             # not contiguous
        (lambda: torch.ones(8), RuntimeError),                                 # host memory
    ):
        m.start_quorum()
        t = make()
        before = t.clone()
        fut = m.allreduce(t)          # must not raise
        assert fut.wait() is t
        assert isinstance(m.errored(), kind), m.errored()
        assert torch.equal(t, before)
        other = torch.ones(8, device=device)
        assert m.allreduce(other).wait() is other  # a no-op until the next quorum
        assert_bits_equal(other, torch.ones(8))
        assert not m.should_commit()
    m.start_quorum()
    assert m.errored() is None
    m.shutdown(wait=False)


def test_localsgd_on_fp64_parameters(device):
    """LocalSGD is dtype-generic in the reference (torchft/local_sgd.py:97-174); fp64 parameters
    are averaged in fp64 and backed up byte for byte."""
    torch.manual_seed(0)
    model = Tiny().to(device=device, dtype=torch.float64)
    peers, lookup = peer_world(model, 2)
    for q in peers[0].parameters():
        q.data.add_(1e-9)  # below fp32 resolution of the values
    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                      use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    optimizer = optim.SGD(model.parameters(), lr=1e-3)
    with LocalSGD(manager, model, optimizer, sync_every=10 ** 9) as lsgd:
        backup0 = cpu(lsgd._backup_parameters.values())
        with torch.no_grad():
            for p in model.parameters():
                p.add_(3e-9)
        local = cpu(p.data for p in model.parameters())
        want = O.localsgd_perform_sync([local, cpu(q.data for q in peers[0].parameters())],
                                       backup0, [True, True], 2, True)
        lsgd.sync()
        for p, w, b in zip(model.parameters(), want["params"], lsgd._backup_parameters.values()):
            assert p.dtype == torch.float64
            assert_bits_equal(p.data, w)
            assert_bits_equal(b, w)
    # DiLoCo's outer step is fp32 arithmetic: fp64 parameters are refused at construction
    manager2 = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                       use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    with pytest.raises(TypeError, match="float64"):
        DiLoCo(manager2, model, optimizer, optim.SGD(model.parameters(), lr=0.7), sync_every=2)
    manager.shutdown(wait=False)
    manager2.shutdown(wait=False)


# ---------------------------------------------------------------------------
# LocalSGD / DiLoCo
# ---------------------------------------------------------------------------

def test_wrappers_refuse_what_the_kernels_cannot_stream(device):
    """A configuration error is raised where the wrapper is constructed, not latched as a failed
    all-reduce on every sync: integer parameters, and parameters that are strided views."""
    manager = create_autospec(Manager)
    manager._use_async_quorum = False
    model = nn.Linear(8, 8).to(device)
    model.weight = nn.Parameter(model.weight.data.t())  # a transposed view: not contiguous
    with pytest.raises(ValueError, match="not contiguous"):
        LocalSGD(manager, model, optim.SGD(model.parameters(), lr=0.1), sync_every=2)
    model = nn.Linear(8, 8).to(device)
    model.half()
    model.weight = nn.Parameter(model.weight.data.to(torch.float64))
    with pytest.raises(TypeError, match="float64"):
        DiLoCo(manager, model, optim.SGD(model.parameters(), lr=0.1), optim.SGD(model.parameters(), lr=0.7), sync_every=2)


def test_localsgd_mlp_two_replicas(device):
    """The CPU-runnable configuration: 3-layer MLP, 2 replicas = backup + N(0, 1e-3),
    sync_every=1, result written into the parameters; the average is done on the GPU."""
    torch.manual_seed(0)
    model = MLP().to(device)
    peers, lookup = peer_world(model, 2)
    g = torch.Generator(device="cpu").manual_seed(1001)
    for q in peers[0].parameters():
        q.data.add_((torch.randn(q.shape, generator=g) * 1e-3).to(device))
    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    optimizer = optim.SGD(model.parameters(), lr=1e-3)
    with LocalSGD(manager, model, optimizer, sync_every=1) as lsgd:
        backup0 = cpu(lsgd._backup_parameters.values())
        seen = {}
        perform = lsgd._perform_sync

        def recording_perform_sync():  # what the sync sees: the parameters after the local step
            seen["local"] = cpu(p.data for p in model.parameters())
            perform()

        lsgd._perform_sync = recording_perform_sync
        model(torch.randn(4, 1024, device=device)).square().mean().backward()
        optimizer.step()  # local step, then the sync fires from the post hook
        want = O.localsgd_perform_sync([seen["local"], cpu(q.data for q in peers[0].parameters())],
                                       backup0, [True, True], 2, True)
        for p, w, (name, b) in zip(model.parameters(), want["params"], lsgd._backup_parameters.items()):
            assert_bits_equal(p.data, w, f"params {name}")
            assert_bits_equal(b, p.data, f"backup {name} == params after commit")
    assert manager.current_step() == 1
    manager.shutdown(wait=False)


def _run_diloco(device, manager_factory, n_replicas, commits, fused_expected, backup_device=None, mutate_host_backup=False):
    torch.manual_seed(0)
    model = Tiny().to(device)
    peers, lookup = peer_world(model, n_replicas)
    manager, commit_flag = manager_factory(lookup)
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    backup = cpu(p.data for p in model.parameters())
    bufs = None
    gen = torch.Generator().manual_seed(9)
    with DiLoCo(manager, model, inner, outer, sync_every=1, backup_device=backup_device) as diloco:
        for step, commit in enumerate(commits):
            commit_flag[0] = commit
            for k, peer in enumerate(peers):
                for q, b in zip(peer.parameters(), backup):
                    q.data.copy_((b + 1e-3 * torch.randn(b.shape, generator=gen)).to(device))
            inner.zero_grad()
            model(torch.rand(2, 3, device=device)).mean().backward()
            # make the local step exact on both sides: apply it here, not through inner.step
            with torch.no_grad():
                for p in model.parameters():
                    p.data.copy_((p.data.cpu() - 0.1 * p.grad.cpu()).to(device))
                    p.grad.zero_()
            local = cpu(p.data for p in model.parameters())
            want = O.diloco_perform_sync(
                [local] + [cpu(q.data for q in peer.parameters()) for peer in peers], backup, bufs,
                [True] * n_replicas, n_replicas, commit, lr=0.7, momentum=0.9, nesterov=True)
            if mutate_host_backup and step == 2:
                # the backup tensors are the user's to write between syncs: the next sync reads them
                diloco._host_backup.wait()
                for b, old_b in zip(diloco._backup_parameters.values(), backup):
                    b.mul_(1.0009765625)
                    old_b.mul_(1.0009765625)
                want = O.diloco_perform_sync(
                    [local] + [cpu(q.data for q in peer.parameters()) for peer in peers], backup, bufs,
                    [True] * n_replicas, n_replicas, commit, lr=0.7, momentum=0.9, nesterov=True)
            inner.step()  # zero gradient: parameters unchanged, post hook runs the sync
            if diloco._host_backup is not None:
                diloco._host_backup.wait()  # the refreshed backup crosses PCIe on a side stream
            for p, w in zip(model.parameters(), want["params"]):
                assert_bits_equal(p.data, w, f"step {step} params")
            for (name, b), w in zip(diloco._backup_parameters.items(), want["backup"]):
                assert_bits_equal(b, w, f"step {step} backup {name}")
            if commit:
                for p, w in zip(model.parameters(), want["momentum"]):
                    assert_bits_equal(outer.state[p]["momentum_buffer"], w, f"step {step} momentum")
                backup, bufs = want["backup"], want["momentum"]
            assert all(p.grad is None for p in model.parameters())
            # cross-replica invariant of torchft/manager_integ_test.py:553-562 is implied:
            # every replica would compute these same bits from the same inputs
    return manager


def test_diloco_fused_local_replicas(device):
    flag = [True]

    def factory(lookup):
        pg = ProcessGroupLocalReplicas(rank=0, world_size=3, peer_lookup=lookup)

        class Vote(StaticQuorum):
            def should_commit(self, rank, step, should_commit, timeout):
                return should_commit and flag[0]

        return Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1, use_async_quorum=False, quorum_client=Vote(0, 3)), flag

    m = _run_diloco(device, factory, 3, [True, True, False, True], True)
    assert m.current_step() == 3
    m.shutdown(wait=False)


def test_diloco_two_launches_when_the_reduction_may_fail_late(device):
    """A group whose reduction can fail after the launch takes the vote between the two
    launches: pseudo-gradient average first (the parameters are left alone when the outer
    SGD is fusable), then outer step (commit) or restore (no commit)."""
    flag = [True]

    def factory(lookup):
        pg = ProcessGroupLocalReplicas(rank=0, world_size=3, peer_lookup=lookup)
        pg.fails_only_at_launch = False

        class Vote(StaticQuorum):
            def should_commit(self, rank, step, should_commit, timeout):
                return should_commit and flag[0]

        return Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1, use_async_quorum=False, quorum_client=Vote(0, 3)), flag

    m = _run_diloco(device, factory, 3, [True, False, False, True, True], True)
    assert m.current_step() == 3
    m.shutdown(wait=False)


@pytest.mark.parametrize("fails_only_at_launch", [True, False])
def test_diloco_with_the_backup_in_host_memory(device, fails_only_at_launch):
    """``backup_device="cpu"`` (torchft/local_sgd.py:185-203 takes it; :214 moves the backup to
    the parameter's device per tensor): the kernels work on the backup's device-side staging
    buffer, loaded from the pinned host buffer before every sync and sent back after a
    committed one.  Single launch and two launches, committed and not, and a backup the user
    has written between two syncs."""
    flag = [True]

    def factory(lookup):
        pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
        pg.fails_only_at_launch = fails_only_at_launch

        class Vote(StaticQuorum):
            def should_commit(self, rank, step, should_commit, timeout):
                return should_commit and flag[0]

        return Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1, use_async_quorum=False, quorum_client=Vote(0, 2)), flag

    m = _run_diloco(device, factory, 2, [True, False, True, True], True,
                    backup_device=torch.device("cpu"), mutate_host_backup=True)
    assert m.current_step() == 3
    m.shutdown(wait=False)


def test_diloco_with_backup_tensors_the_user_put_in_place(device):
    """``_backup_parameters`` replaced by plain host tensors (a load_state_dict after healing,
    torchft/manager_integ_test.py:279): every sync reads them and a committed one rewrites them."""
    torch.manual_seed(0)
    model = Tiny().to(device)
    peers, lookup = peer_world(model, 2)
    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    gen = torch.Generator().manual_seed(5)
    with DiLoCo(manager, model, inner, outer, sync_every=1) as diloco:
        mine = {n: (b.cpu() + 1e-3 * torch.randn(b.shape, generator=gen)) for n, b in diloco._backup_parameters.items()}
        diloco._backup_parameters = mine
        backup, bufs = [b.clone() for b in mine.values()], None
        for step in range(3):
            for q, b in zip(peers[0].parameters(), backup):
                q.data.copy_((b + 1e-3 * torch.randn(b.shape, generator=gen)).to(device))
            with torch.no_grad():
                for p, b in zip(model.parameters(), backup):
                    p.data.copy_((b + 2e-3 * torch.randn(b.shape, generator=gen)).to(device))
                    p.grad = torch.zeros_like(p)
            local = cpu(p.data for p in model.parameters())
            want = O.diloco_perform_sync([local, cpu(q.data for q in peers[0].parameters())], backup, bufs,
                                         [True, True], 2, True, lr=0.7, momentum=0.9, nesterov=True)
            inner.step()
            assert diloco._backup_parameters is mine
            for p, b, w, wb, wm in zip(model.parameters(), mine.values(), want["params"], want["backup"], want["momentum"]):
                assert b.device.type == "cpu"
                assert_bits_equal(p.data, w, f"step {step} params")
                assert_bits_equal(b, wb, f"step {step} backup")
                assert_bits_equal(outer.state[p]["momentum_buffer"], wm, f"step {step} momentum")
            backup, bufs = want["backup"], want["momentum"]
    manager.shutdown(wait=False)


def test_localsgd_with_the_backup_in_host_memory_is_one_launch_and_one_transfer(device):
    """Local replicas and a pinned host backup: the average goes to the parameters and to the
    backup's staging buffer in one launch; the checker's bits, committed and not."""
    torch.manual_seed(0)
    model = MLP().to(device)
    peers, lookup = peer_world(model, 2)
    flag = [True]

    class Vote(StaticQuorum):
        def should_commit(self, rank, step, should_commit, timeout):
            return should_commit and flag[0]

    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False, quorum_client=Vote(0, 2))
    optimizer = optim.SGD(model.parameters(), lr=1e-3)
    gen = torch.Generator().manual_seed(11)
    with LocalSGD(manager, model, optimizer, sync_every=1, backup_device=torch.device("cpu")) as lsgd:
        lsgd._host_backup.wait()
        backup = [b.clone() for b in lsgd._backup_parameters.values()]
        for step, commit in enumerate([True, False, True]):
            flag[0] = commit
            for q in peers[0].parameters():
                q.data.add_((1e-3 * torch.randn(q.shape, generator=gen)).to(device))
            with torch.no_grad():
                for p in model.parameters():
                    p.add_((1e-3 * torch.randn(p.shape, generator=gen)).to(device))
                    p.grad = torch.zeros_like(p)
            local = cpu(p.data for p in model.parameters())
            want = O.localsgd_perform_sync([local, cpu(q.data for q in peers[0].parameters())], backup,
                                           [True, True], 2, commit)
            optimizer.step()
            lsgd._host_backup.wait()
            for p, b, w, wb in zip(model.parameters(), lsgd._backup_parameters.values(), want["params"], want["backup"]):
                assert b.is_pinned()
                assert_bits_equal(p.data, w, f"step {step} params")
                assert_bits_equal(b, wb, f"step {step} backup")
            backup = want["backup"]
    manager.shutdown(wait=False)


def test_diloco_generic_manager_contract(device):
    """A foreign Manager (mock): per-parameter allreduce calls, kernels for the rest."""
    flag = [True]
    calls = []

    def factory(lookup):
        manager = create_autospec(Manager)
        manager._use_async_quorum = False
        manager.should_commit.side_effect = lambda *a, **k: flag[0]

        def allreduce(t):
            calls.append(t)
            peers = lookup_grad(t)
            from torchft_amd import ops
            ops.reduce_avg_(t, [t] + peers, None, 2)
            f = Future()
            f.set_result(t)
            return f

        manager.allreduce.side_effect = allreduce
        return manager, flag

    # peers' pseudo-gradients for the mock's allreduce: peer params - backup, made on demand
    state = {}

    def lookup_grad(t):
        model, peers, diloco = state["model"], state["peers"], state["diloco"]
        for (name, p), q in zip(model.named_parameters(), peers[0].parameters()):
            if p.grad is not None and p.grad.data_ptr() == t.data_ptr():
                return [q.data - diloco._backup_parameters[name]]
        raise KeyError

    torch.manual_seed(0)
    model = Tiny().to(device)
    peers, _ = peer_world(model, 2)
    manager, _ = factory(None)
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    backup = cpu(p.data for p in model.parameters())
    with DiLoCo(manager, model, inner, outer, sync_every=1) as diloco:
        state.update(model=model, peers=peers, diloco=diloco)
        for q, b in zip(peers[0].parameters(), backup):
            q.data.copy_((b + 1e-3).to(device))
        with torch.no_grad():
            for p in model.parameters():
                p.data.add_(2e-3)
                p.grad = torch.zeros_like(p)
        local = cpu(p.data for p in model.parameters())
        want = O.diloco_perform_sync([local, cpu(q.data for q in peers[0].parameters())], backup, None,
                                     [True, True], 2, True, lr=0.7, momentum=0.9, nesterov=True)
        inner.step()
        assert len(calls) == len(list(model.parameters()))
        for p, w in zip(model.parameters(), want["params"]):
            assert_bits_equal(p.data, w)
        for p, w in zip(model.parameters(), want["momentum"]):
            assert_bits_equal(outer.state[p]["momentum_buffer"], w)
        # a sync that is not committed: the local changes are discarded, nothing else moves
        flag[0] = False
        with torch.no_grad():
            for p in model.parameters():
                p.data.add_(3e-3)
                p.grad = torch.zeros_like(p)
        inner.step()
        for p, b, w, m in zip(model.parameters(), diloco._backup_parameters.values(), want["backup"], want["momentum"]):
            assert_bits_equal(b, w)
            assert_bits_equal(p.data, w)
            assert_bits_equal(outer.state[p]["momentum_buffer"], m)


def test_diloco_gpt2_small_four_replicas(device):
    """DiLoCo outer step, fp32, GPT-2-small-shaped parameters (148 tensors, 124 439 808
    parameters), 4 replicas = backup + N(0, 1e-3), Nesterov SGD lr 0.7 / momentum 0.9, zero
    initial momentum; first step and a steady-state step, whole tensors compared."""
    from torchft_amd import ops

    shapes = workloads.gpt2_small_shapes()
    wl = workloads.make_diloco_workload(shapes, 4, torch.device("cpu"))
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    b = [t.to(device) for t in wl.backup]
    p = [torch.empty_like(t) for t in b]
    m = [torch.empty_like(t) for t in b]
    backup, bufs, replicas = wl.backup, None, wl.replicas
    table = None
    for step in range(2):
        want = O.diloco_perform_sync(replicas, backup, bufs, [True] * 4, 4, True,
                                     lr=0.7, momentum=0.9, nesterov=True)
        reps = [[t.to(device) for t in rep] for rep in replicas]
        ops.mt_diloco_outer(p, b, m, reps, sgd, step == 0)
        for i, (name, _) in enumerate(shapes):
            assert_bits_equal(p[i], want["params"][i], f"step {step} {name}")
            assert_bits_equal(b[i], want["backup"][i], f"step {step} backup {name}")
            assert_bits_equal(m[i], want["momentum"][i], f"step {step} momentum {name}")
        backup, bufs = want["backup"], want["momentum"]
        replicas = [workloads.drifted_replica(backup, 1e-3, 1100 + r) for r in range(4)]
        del reps


# ---------------------------------------------------------------------------
# DDP
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("bucket_views", [False, True])
def test_ddp_comm_hook_on_gpu(device, bucket_views):
    """torch's Reducer flattens, the hook's Manager.allreduce averages the flat bucket with
    one kernel, the Reducer unflattens: gradients equal the checker's bucket average.  With
    ``gradient_as_bucket_view=True`` the gradients are views of the bucket, so the Reducer's
    two copies disappear and the kernel's pass is the only one."""
    torch.manual_seed(0)
    model = MLP().to(device)
    captured = {}

    def lookup(flat):
        # the peer's flat bucket: a deterministic function of the local one
        peer = flat * 0.5 + 0.25
        captured[flat.data_ptr()] = (flat.detach().cpu().clone(), peer.cpu().clone())
        return [peer]

    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, quorum_client=StaticQuorum(0, 2))
    ddp = DistributedDataParallel(manager, model, gradient_as_bucket_view=bucket_views)
    manager.start_quorum()
    ddp(torch.randn(4, 1024, device=device)).square().mean().backward()
    torch.cuda.synchronize()
    assert manager.should_commit()
    assert len(captured) == 2  # two buckets for this model (4 218 890 and 2 097 152 elements)
    if bucket_views:  # every gradient lies inside one of the two flat buffers the hook saw
        spans = [(ptr, ptr + 4 * v[0].numel()) for ptr, v in captured.items()]
        assert all(any(lo <= p.grad.data_ptr() < hi for lo, hi in spans) for p in model.parameters())
    params = list(model.parameters())
    numels = [p.numel() for p in params]
    buckets = O.bucket_assignment(numels, 4)
    sizes = sorted(sum(numels[i] for i in bkt) for bkt in buckets)
    assert sorted(v[0].numel() for v in captured.values()) == sizes
    for local, peer in captured.values():
        want = O.manager_allreduce_([local, peer], [True, True], 2)
        bucket = next(bkt for bkt in buckets if sum(numels[i] for i in bkt) == local.numel())
        off = 0
        for i in bucket:
            assert_bits_equal(params[i].grad.reshape(-1), want[off:off + numels[i]], f"param {i}")
            off += numels[i]
    manager.shutdown(wait=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pure_ddp_gradients_against_the_checker(device, dtype):
    """PureDistributedDataParallel (torchft/ddp.py:84-94): one ``manager.allreduce(p.grad)``
    per parameter from the post-accumulate hook.  Three replicas of which the third is a
    spare (FIXED_WITH_SPARES, min 2): every gradient must equal the checker's
    ``manager_allreduce_`` of the three raw gradients with flags [1, 1, 0] and n = 2."""
    torch.manual_seed(0)
    model = MLP().to(device=device, dtype=dtype)
    peers, _ = peer_world(model, 3)
    for k, peer in enumerate(peers):  # the peers' gradients exist before the local backward
        peer(torch.randn(4, 1024, device=device, generator=torch.Generator(device).manual_seed(k + 1))
             .to(dtype)).square().mean().backward()
    raw = {}

    def lookup(grad):
        for k, p in enumerate(model.parameters()):
            if p.grad is not None and p.grad.data_ptr() == grad.data_ptr():
                raw[k] = grad.detach().cpu().clone()  # the local gradient before averaging
                return [list(peer.parameters())[k].grad for peer in peers]
        raise KeyError("unknown tensor")

    pg = ProcessGroupLocalReplicas(rank=0, world_size=3, peer_lookup=lookup,
                                   peer_participating=[True, False])
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                      world_size_mode=WorldSizeMode.FIXED_WITH_SPARES,
                      quorum_client=StaticQuorum(0, 3))
    ddp = PureDistributedDataParallel(manager, model)
    manager.start_quorum()
    x = torch.randn(4, 1024, device=device, generator=torch.Generator(device).manual_seed(9)).to(dtype)
    ddp(x).square().mean().backward()
    torch.cuda.synchronize()
    assert manager.num_participants() == 2 and manager.is_participating()
    assert manager.should_commit()
    params = list(model.parameters())
    assert sorted(raw) == list(range(len(params)))  # one allreduce per parameter
    for k, p in enumerate(params):
        contributions = [raw[k]] + [list(peer.parameters())[k].grad.cpu() for peer in peers]
        want = O.manager_allreduce_(contributions, [True, True, False], 2, torch.float32)
        assert_bits_equal(p.grad, want, f"param {k}")
        if dtype == torch.bfloat16:
            native = O.manager_allreduce_(contributions, [True, True, False], 2)
            torch.testing.assert_close(p.grad.cpu().float(), native.float(), rtol=RTOL_BF16, atol=2e-4)
    # the peers' gradients were only read
    assert all(q.grad is not None and torch.isfinite(q.grad).all() for peer in peers for q in peer.parameters())
    manager.shutdown(wait=False)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_grad_bucket_averager(device, dtype):
    """Config-3 arithmetic at GPT-2 scale: 4 contributions, one zeroed, n=3; bucket layout
    by torch's rule; in place on replica 0's gradients."""
    shapes = workloads.gpt2_small_shapes()[:40] + [("odd", (77, 3)), ("one", (1,))]
    grads = workloads.make_grad_replicas(shapes, 4, torch.device("cpu"), dtype)
    numels = [g.numel() for g in grads[0]]
    buckets = O.bucket_assignment(numels, grads[0][0].element_size())
    want = O.ddp_bucket_average(grads, [True, True, True, False], 3, buckets, torch.float32)
    dev = [[t.to(device) for t in rep] for rep in grads]
    avg = GradBucketAverager(dev[0], dev)
    assert avg.buckets == buckets
    for b in range(len(buckets)):
        assert avg.bucket_offsets(b) == O.bucket_offsets(numels, buckets[b])
        avg.average_bucket(b, 0b0111, 3)
    for i, (name, _) in enumerate(shapes):
        assert_bits_equal(dev[0][i], want[i], name)
    for r in (1, 2, 3):
        for i in range(len(shapes)):
            assert_bits_equal(dev[r][i], grads[r][i])
    if dtype == torch.bfloat16:
        native = O.ddp_bucket_average(grads, [True, True, True, False], 3, buckets)
        for i in range(len(shapes)):
            torch.testing.assert_close(dev[0][i].cpu().float(), native[i].float(),
                                       rtol=RTOL_BF16, atol=2e-4)
    # the one-launch form gives the same bits
    dev2 = [[t.to(device) for t in rep] for rep in grads]
    out = [torch.empty_like(t) for t in dev2[0]]
    GradBucketAverager(out, dev2).average_whole_model(0b0111, 3)
    for i in range(len(shapes)):
        assert_bits_equal(out[i], want[i])


@pytest.mark.parametrize("streams", [1, 2, 3])
def test_grad_bucket_averager_all_buckets_over_side_streams(device, streams):
    """``average_all`` alternates its launches between side streams: it must see what the
    current stream wrote just before the call, and what it writes must be visible to the
    current stream right after it (no synchronisation by the caller)."""
    shapes = workloads.gpt2_small_shapes()[:60]
    grads = workloads.make_grad_replicas(shapes, 3, torch.device("cpu"), torch.bfloat16)
    numels = [g.numel() for g in grads[0]]
    buckets = O.bucket_assignment(numels, 2)
    assert len(buckets) > 3
    doubled = [[(t.float() * 2).to(torch.bfloat16) for t in rep] for rep in grads]
    want = O.ddp_bucket_average(doubled, [True, True, True], 3, buckets, torch.float32)
    dev = [[t.to(device) for t in rep] for rep in grads]
    out = [torch.empty_like(t) for t in dev[0]]
    avg = GradBucketAverager(out, dev)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):  # a non-default current stream, to make ordering matter
        for rep in dev:
            torch._foreach_mul_(rep, 2.0)  # producer on the current stream
        avg.average_all(streams=streams)
        sums = [t.float().sum() for t in out]  # consumer on the current stream
    side.synchronize()
    for i, (name, _) in enumerate(shapes):
        assert_bits_equal(out[i], want[i], name)
        assert float(sums[i]) == float(want[i].float().sum().to(torch.float32)) or torch.isclose(
            sums[i].cpu(), want[i].float().sum(), rtol=1e-3, atol=1e-3)


def test_flatten_unflatten_are_byte_exact(device):
    """Bucket flatten / unflatten as explicit copies (what the Reducer does around the hook):
    offsets are running element counts with no padding."""
    from torchft_amd import ops

    shapes = [("a", (300, 7)), ("b", (5,)), ("c", (1000,)), ("d", (3, 3)), ("e", (1,))]
    grads = workloads.make_grad_replicas(shapes, 1, torch.device("cpu"), torch.bfloat16)[0]
    dev = [t.to(device) for t in grads]
    flat = torch.zeros(sum(t.numel() for t in dev), dtype=torch.bfloat16, device=device)
    views = ops.flat_views(flat, dev)
    ops.mt_copy(views, dev)
    assert_bits_equal(flat, torch.cat([t.reshape(-1) for t in grads]))
    back = [torch.empty_like(t) for t in dev]
    ops.mt_copy(back, views)
    for a, b in zip(back, grads):
        assert_bits_equal(a, b)


# ---------------------------------------------------------------------------
# Checkpoint transport
# ---------------------------------------------------------------------------

def _assert_state_equal(got, want, path=""):
    if isinstance(want, torch.Tensor):
        assert isinstance(got, torch.Tensor), path
        assert got.dtype == want.dtype and got.shape == want.shape, path
        assert_bits_equal(got, want, path)
    elif isinstance(want, dict):
        assert type(got) is type(want) and list(got.keys()) == list(want.keys()), path
        for k in want:
            _assert_state_equal(got[k], want[k], f"{path}/{k}")
    elif isinstance(want, (list, tuple)):
        assert type(got) is type(want) and len(got) == len(want), path
        for i, (g, w) in enumerate(zip(got, want)):
            _assert_state_equal(g, w, f"{path}[{i}]")
    else:
        assert got == want, path


def _training_state(device):
    shapes = workloads.gpt2_small_shapes()[:14] + [("odd", (77, 3)), ("empty", (0, 4)), ("one", (1,))]
    state = workloads.make_training_state(shapes, device, step=321)
    state["user"]["extra"] = {
        "bools": torch.tensor([True, False, True], device=device),
        "bytes": torch.arange(37, dtype=torch.uint8, device=device),
        "f64": torch.linspace(0, 1, 11, dtype=torch.float64, device=device),
        "cpu_tensor": torch.arange(5),
        "text": "lr schedule", "tuple": (1, 2.5, None),
        "noncontig": torch.arange(12, dtype=torch.float32, device=device).view(3, 4).t(),
    }
    first = next(iter(state["user"]["model"].values()))
    state["user"]["tied"] = first  # the same tensor reachable twice
    return state


@pytest.mark.parametrize("copy_out", [True, False])
def test_pack_unpack_bit_exact(device, copy_out):
    state = _training_state(device)
    packed = state_pack.pack(state)
    # layout: every device tensor's raw bytes at its 256-byte aligned offset
    plan = packed.plan
    assert all(e.offset % 256 == 0 for e in plan.entries)
    offsets = [e.offset for e in plan.entries]
    image = O.gather_bytes(plan.tensors, offsets, plan.total_bytes)
    got = packed.staging.cpu().numpy()
    for e in plan.entries:
        assert bytes(got[e.offset:e.offset + e.nbytes]) == bytes(image[e.offset:e.offset + e.nbytes])
    out = state_pack.unpack(packed.header, packed.staging, copy=copy_out)
    # the checker: what torch.save -> torch.load hands the receiver
    want = O.state_dict_round_trip(state)
    _assert_state_equal(out, want)
    assert out["user"]["tied"] is out["user"]["model"][next(iter(out["user"]["model"]))]
    assert out["user"]["extra"]["cpu_tensor"].device.type == "cpu"
    assert out["user"]["model"]["wte.weight"].device == device


def test_wire_round_trip_through_pinned_host(device):
    state = _training_state(device)
    buf = io.BytesIO()
    state_pack.write_packed(state_pack.pack(state), buf, chunk_bytes=1 << 20)  # many chunks
    data = buf.getvalue()
    assert data[:8] == state_pack.MAGIC
    buf.seek(0)
    header, staging = state_pack.read_packed(buf, device, chunk_bytes=3 << 19)
    out = state_pack.unpack(header, staging)
    _assert_state_equal(out, O.state_dict_round_trip(state))
    with pytest.raises(ValueError, match="bad magic"):
        state_pack.read_packed(io.BytesIO(b"not a packed state"), device)
    with pytest.raises(EOFError):
        state_pack.read_packed(io.BytesIO(data[:len(data) // 2]), device)


@pytest.mark.parametrize("chunk_bytes", [4096, 1 << 20, 64 << 20])
def test_streamed_payload_equals_the_one_shot_pack(device, chunk_bytes):
    """stream_packed never holds the payload as a whole (three ring slots of chunk_bytes):
    what it writes must equal the layout of the one-launch pack at every tensor's bytes, for
    whole payloads and for byte ranges whose concatenation is the payload."""
    state = _training_state(device)
    plan = state_pack.plan_pack(state)
    offsets = [e.offset for e in plan.entries]
    image = O.gather_bytes(plan.tensors, offsets, plan.total_bytes)

    def payload_of(lo, hi):
        buf = io.BytesIO()
        state_pack.stream_packed(plan, buf, lo, hi, chunk_bytes=chunk_bytes)
        data = buf.getvalue()
        assert data[:8] == state_pack.MAGIC
        hlen = int.from_bytes(data[8:16], "little")
        assert data[16:16 + hlen] == plan.header()
        return data[16 + hlen:]

    whole = payload_of(0, plan.total_bytes)
    assert len(whole) == plan.total_bytes
    for e in plan.entries:
        assert whole[e.offset:e.offset + e.nbytes] == bytes(image[e.offset:e.offset + e.nbytes])
    if chunk_bytes >= 1 << 20:
        parts = [payload_of(*state_pack.split_range(plan.total_bytes, k, 3)) for k in range(3)]
        joined = b"".join(parts)
        assert len(joined) == plan.total_bytes
        for e in plan.entries:
            assert joined[e.offset:e.offset + e.nbytes] == whole[e.offset:e.offset + e.nbytes]
    # and the receiving side rebuilds the checker's state from it
    buf = io.BytesIO()
    state_pack.stream_packed(plan, buf, chunk_bytes=chunk_bytes)
    buf.seek(0)
    header, staging = state_pack.read_packed(buf, device, chunk_bytes=max(chunk_bytes, 1 << 16))
    _assert_state_equal(state_pack.unpack(header, staging), O.state_dict_round_trip(state))


def test_checkpoint_fetched_over_parallel_connections(device):
    """A payload above 256 MiB is fetched as byte ranges over several connections at once;
    the result is the sender's state bit for bit, and disallow_checkpoint waits for the
    requests in flight."""
    g = torch.Generator(device).manual_seed(1)
    state = {"user": {"model": {f"w{i}": torch.randn(23_000_000 + i, device=device, generator=g)
                                for i in range(4)},
                      "step": 3},
             "torchft": {"step": 9, "batches_committed": 18}}
    nbytes = sum(t.numel() * 4 for t in state["user"]["model"].values())
    assert nbytes > 256 << 20
    for streams in (1, 3, 4):
        server = CheckpointServer(timeout=timedelta(seconds=60), fetch_streams=streams)
        server.send_checkpoint([1], 9, state, timedelta(seconds=60))
        out = server.recv_checkpoint(0, server.metadata(), 9, timedelta(seconds=60))
        server.disallow_checkpoint()
        assert server._readers == 0
        assert out["torchft"] == state["torchft"] and out["user"]["step"] == 3
        for k, v in state["user"]["model"].items():
            assert torch.equal(out["user"]["model"][k], v), (streams, k)
        with pytest.raises(Exception):  # wrong step: HTTP 400
            server.allow_checkpoint(10)
            server.recv_checkpoint(0, server.metadata(), 9, timedelta(seconds=10))
        server.shutdown()


def test_checkpoint_server_with_device_tensors(device):
    """torchft/checkpointing_test.py:17-58 with a tensor payload: the recovering side gets
    the same state, on its GPU, bit for bit."""
    state = _training_state(device)
    server = CheckpointServer(timeout=timedelta(seconds=30), chunk_bytes=1 << 20)
    server.send_checkpoint(dst_ranks=[1], step=7, state_dict=state, timeout=timedelta(seconds=30))
    out = server.recv_checkpoint(src_rank=0, metadata=server.metadata(), step=7,
                                 timeout=timedelta(seconds=30))
    _assert_state_equal(out, O.state_dict_round_trip(state))
    assert out["user"]["model"]["wte.weight"].is_cuda
    # serving twice reuses the staging buffer; a mutated state is served as mutated
    state["user"]["model"]["wte.weight"].add_(1)
    server.disallow_checkpoint()
    server.send_checkpoint(dst_ranks=[1], step=8, state_dict=state, timeout=timedelta(seconds=30))
    out = server.recv_checkpoint(0, server.metadata(), 8, timedelta(seconds=30))
    _assert_state_equal(out, O.state_dict_round_trip(state))
    server.shutdown()


# ---------------------------------------------------------------------------
# Bucketised sync through an ordinary process group (one collective per model)
# ---------------------------------------------------------------------------

class _PlainLocalPG(ProcessGroup):
    """A process group that only offers the plain contract (``allreduce`` SUM): the flat
    buffer it is handed is summed with a peer's flat buffer supplied by the test."""

    def __init__(self, peer_flat):
        super().__init__(0, 2)
        self.peer_flat = peer_flat
        self.calls = []

    def configure(self, store_addr, rank, world_size):
        pass

    def allreduce(self, tensors, opts):
        from torchft_amd import ops

        for t in tensors:
            self.calls.append(t.numel())
            ops.reduce_avg_(t, [t, self.peer_flat(t)], 0b11, 1)
        return _DummyWork(tensors)

    def size(self):
        return 2

    def getBackendName(self):
        return "plain-local"


def test_diloco_bucketized_on_gpu(device):
    torch.manual_seed(0)
    model = MLP().to(device)
    backup = cpu(p.data for p in model.parameters())
    peer_params = [b + 1e-3 * torch.randn(b.shape) for b in backup]
    # what the peer contributes to the flat buffer: its pseudo-gradients, back to back
    peer_flat = torch.cat([(q - b).reshape(-1) for q, b in zip(peer_params, backup)]).to(device)
    pg = _PlainLocalPG(lambda t: peer_flat)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    with DiLoCo(manager, model, inner, outer, sync_every=1) as diloco:
        with torch.no_grad():
            for p in model.parameters():
                p.add_(2e-3 * torch.randn_like(p))
                p.grad = torch.zeros_like(p)
        local = cpu(p.data for p in model.parameters())
        want = O.diloco_perform_sync([local, peer_params], backup, None, [True, True], 2, True,
                                     lr=0.7, momentum=0.9, nesterov=True)
        inner.step()
        assert pg.calls == [sum(b.numel() for b in backup)]  # one collective for 6.3 M parameters
        for p, w, m in zip(model.parameters(), want["params"], want["momentum"]):
            assert_bits_equal(p.data, w)
            assert_bits_equal(outer.state[p]["momentum_buffer"], m)
        for b, w in zip(diloco._backup_parameters.values(), want["backup"]):
            assert_bits_equal(b, w)
        # a sync that is not committed: the local changes are discarded, nothing else moves
        manager._client.should_commit = lambda *a, **k: False
        with torch.no_grad():
            for p in model.parameters():
                p.add_(2e-3 * torch.randn_like(p))
                p.grad = torch.zeros_like(p)
        inner.step()
        for p, b, w, m in zip(model.parameters(), diloco._backup_parameters.values(), want["backup"], want["momentum"]):
            assert_bits_equal(b, w)
            assert_bits_equal(p.data, w)
            assert_bits_equal(outer.state[p]["momentum_buffer"], m)
    manager.shutdown(wait=False)


@pytest.mark.parametrize("backup_device", [None, torch.device("cpu")])
def test_local_sgd_bucketized_on_gpu(device, backup_device):
    torch.manual_seed(0)
    model = MLP().to(device)
    peer_params = [p.data.cpu() + 1e-3 * torch.randn(p.shape) for p in model.parameters()]
    peer_flat = torch.cat([q.reshape(-1) for q in peer_params]).to(device)
    pg = _PlainLocalPG(lambda t: peer_flat)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    optimizer = optim.SGD(model.parameters(), lr=0.1)
    with LocalSGD(manager, model, optimizer, sync_every=1, backup_device=backup_device) as lsgd:
        if lsgd._host_backup is not None:
            lsgd._host_backup.wait()
        backup = cpu(lsgd._backup_parameters.values())
        with torch.no_grad():
            for p in model.parameters():
                p.add_(2e-3 * torch.randn_like(p))
                p.grad = torch.zeros_like(p)
        local = cpu(p.data for p in model.parameters())
        want = O.localsgd_perform_sync([local, peer_params], backup, [True, True], 2, True)
        optimizer.step()
        if lsgd._host_backup is not None:
            lsgd._host_backup.wait()
        assert pg.calls == [sum(b.numel() for b in backup)]  # one collective wherever the backup is kept
        for p, w in zip(model.parameters(), want["params"]):
            assert_bits_equal(p.data, w)
        for b, w in zip(lsgd._backup_parameters.values(), want["backup"]):
            assert_bits_equal(b, w)
    manager.shutdown(wait=False)


# ---------------------------------------------------------------------------
# Host-resident backup (the reference's default placement), moved as one transfer
# ---------------------------------------------------------------------------

def test_localsgd_host_backup_one_transfer(device):
    torch.manual_seed(0)
    model = MLP().to(device)
    manager = create_autospec(Manager)
    manager.should_commit.return_value = True
    manager.allreduce.side_effect = lambda t: _done(t)
    optimizer = optim.SGD(model.parameters(), lr=0.1)
    with LocalSGD(manager, model, optimizer, sync_every=1, backup_device=torch.device("cpu")) as lsgd:
        for name, b in lsgd._backup_parameters.items():
            assert b.device.type == "cpu" and b.is_pinned(), name
        lsgd._host_backup.wait()
        for (name, p), b in zip(model.named_parameters(), lsgd._backup_parameters.values()):
            assert_bits_equal(b, p.data, f"initial backup {name}")
        before = cpu(p.data for p in model.parameters())
        with torch.no_grad():
            for p in model.parameters():
                p.add_(1.0)
        lsgd._restore_parameters()  # local changes discarded
        for p, w in zip(model.parameters(), before):
            assert_bits_equal(p.data, w)
        # a committed sync refreshes the host copy (asynchronously; wait before reading it)
        with torch.no_grad():
            for p in model.parameters():
                p.add_(0.5)
                p.grad = torch.zeros_like(p)
        optimizer.step()
        lsgd._host_backup.wait()
        for (name, p), b in zip(model.named_parameters(), lsgd._backup_parameters.values()):
            assert_bits_equal(b, p.data, f"backup after commit {name}")
        # refused commit: parameters come back from the host copy
        manager.should_commit.return_value = False
        want = cpu(p.data for p in model.parameters())
        with torch.no_grad():
            for p in model.parameters():
                p.add_(0.25)
        optimizer.step()
        for p, w in zip(model.parameters(), want):
            assert_bits_equal(p.data, w)
        # a user may replace the backup tensors (torchft/manager_integ_test.py:279)
        lsgd._backup_parameters = {n: torch.zeros_like(b) for n, b in lsgd._backup_parameters.items()}
        lsgd._restore_parameters()
        assert all(int(torch.count_nonzero(p.data)) == 0 for p in model.parameters())


def _done(t):
    f = Future()
    f.set_result(t)
    return f
