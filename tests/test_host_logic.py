"""Host logic without a GPU: the reference's own unit tests for this path, re-expressed
against torchft_amd's classes (torchft/local_sgd_test.py, ddp_test.py, optim_test.py,
checkpointing_test.py and the allreduce / participation tests of manager_test.py).

Where arithmetic is involved the ``cpu_ops`` fixture substitutes the kernels by the CPU
checker, so what is tested here is control flow: call counts, the commit gate, rollback,
error latching, optimizer-state handling, bucket bookkeeping.
"""

import threading
import urllib.error
from datetime import timedelta
from typing import Dict
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
    LocalSGD,
    Manager,
    OptimizerWrapper,
    ProcessGroup,
    ProcessGroupLocalReplicas,
    PureDistributedDataParallel,
    QuorumResult,
    StaticQuorum,
    WorldSizeMode,
    workloads,
)
from torchft_amd.checkpointing import _timed_acquire
from torchft_amd.ddp import compute_bucket_assignment
from torchft_amd.manager import QuorumClient
from torchft_amd.process_group import ProcessGroupDummy, _DummyWork


class SimpleModel(nn.Module):
    def __init__(self) -> None:
        super().__init__()
        self.model = nn.Sequential(nn.Linear(3, 4), nn.ReLU(), nn.Linear(4, 5), nn.Sigmoid())

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.model(x)


def _params_dict(m: nn.Module) -> Dict[str, torch.Tensor]:
    return {name: p.data for name, p in m.named_parameters()}


def _train_step(model, optimizer):
    loss = model(torch.rand(2, 3)).mean()
    loss.backward()
    optimizer.step()


# ---------------------------------------------------------------------------
# torchft/local_sgd_test.py
# ---------------------------------------------------------------------------

def test_local_sgd_healthy():
    model = SimpleModel()
    optimizer = optim.SGD(model.parameters())
    manager = create_autospec(Manager)
    with LocalSGD(manager, model, optimizer, sync_every=2) as local_sgd:
        assert local_sgd._local_step == 0
        torch.testing.assert_close(local_sgd._backup_parameters, _params_dict(model))
        _train_step(model, optimizer)
        assert local_sgd._local_step == 1
        assert manager.start_quorum.call_count == 0
        _train_step(model, optimizer)
        assert manager.start_quorum.call_count == 1
        manager.should_commit.return_value = True
        assert local_sgd._local_step == 0
        torch.testing.assert_close(local_sgd._backup_parameters, _params_dict(model))
        assert manager.should_commit.call_count == 1
        assert manager.allreduce.call_count == 4


def test_local_sgd_recovery():
    model = SimpleModel()
    optimizer = optim.SGD(model.parameters())
    manager = create_autospec(Manager)
    with LocalSGD(manager, model, optimizer, sync_every=2) as local_sgd:
        torch.testing.assert_close(local_sgd._backup_parameters, _params_dict(model))
        og = {k: v.clone() for k, v in model.state_dict().items()}
        _train_step(model, optimizer)
        for name, param in model.state_dict().items():
            assert not torch.equal(og[name], param), f"Parameter {name} did not change."
        assert local_sgd._local_step == 1
        local_sgd._restore_parameters()
        torch.testing.assert_close(local_sgd._backup_parameters, _params_dict(model))
        torch.testing.assert_close(dict(model.state_dict()), og)


def test_local_sgd_no_commit_and_exception_roll_back():
    model = SimpleModel()
    optimizer = optim.SGD(model.parameters())
    manager = create_autospec(Manager)
    manager.should_commit.return_value = False
    og = {k: v.clone() for k, v in model.state_dict().items()}
    with LocalSGD(manager, model, optimizer, sync_every=1):
        _train_step(model, optimizer)  # sync happens, commit refused
        torch.testing.assert_close(dict(model.state_dict()), og)
    with pytest.raises(RuntimeError, match="boom"):
        with LocalSGD(manager, model, optimizer, sync_every=5):
            _train_step(model, optimizer)
            raise RuntimeError("boom")
    torch.testing.assert_close(dict(model.state_dict()), og)  # torchft/local_sgd.py:111-113
    assert len(optimizer._optimizer_step_post_hooks) == 0  # hooks removed on exit


def test_diloco_healthy(cpu_ops):
    model = SimpleModel()
    inner = optim.AdamW(model.parameters(), lr=4e-4, weight_decay=0.1, betas=(0.9, 0.95))
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    manager = create_autospec(Manager)
    manager._use_async_quorum = False
    with DiLoCo(manager, model, inner, outer, sync_every=2) as diloco:
        parameter_count = len(list(model.parameters()))
        assert outer.state_dict()["state"] == {}
        assert diloco._local_step == 0
        torch.testing.assert_close(diloco._backup_parameters, _params_dict(model))
        _train_step(model, inner)
        assert diloco._local_step == 1
        assert manager.start_quorum.call_count == 0
        _train_step(model, inner)
        assert manager.start_quorum.call_count == 1
        manager.should_commit.return_value = True
        assert diloco._local_step == 0
        torch.testing.assert_close(diloco._backup_parameters, _params_dict(model))
        assert manager.should_commit.call_count == 1
        assert manager.allreduce.call_count == parameter_count
        assert len(outer.state_dict()["state"]) == parameter_count
        assert all(p.grad is None for p in model.parameters())


def test_diloco_requires_sync_quorum():
    manager = create_autospec(Manager)
    manager._use_async_quorum = True
    model = SimpleModel()
    with pytest.raises(ValueError, match="synchronous quorum"):
        DiLoCo(manager, model, optim.SGD(model.parameters()), optim.SGD(model.parameters()), 2)


@pytest.mark.parametrize("outer_kind", ["sgd_nesterov", "adam"])
def test_diloco_matches_reference_loop_with_identity_allreduce(cpu_ops, outer_kind):
    """One replica, allreduce = identity (a mocked Manager whose allreduce returns the
    tensor): the wrapper must leave the model exactly where the reference's loop would."""
    torch.manual_seed(3)
    model = SimpleModel()
    twin = SimpleModel()
    twin.load_state_dict(model.state_dict())

    def make_outer(m):
        if outer_kind == "adam":
            return optim.Adam(m.parameters(), lr=1e-2)  # not fusable: optimizer.step() path
        return optim.SGD(m.parameters(), lr=0.7, momentum=0.9, nesterov=True)

    manager = create_autospec(Manager)
    manager._use_async_quorum = False
    manager.should_commit.return_value = True

    def allreduce(t):
        f = Future()
        f.set_result(t)
        return f

    manager.allreduce.side_effect = allreduce
    inner, outer = optim.SGD(model.parameters(), lr=0.1), make_outer(model)
    twin_inner, twin_outer = optim.SGD(twin.parameters(), lr=0.1), make_outer(twin)
    twin_backup = [p.data.clone() for p in twin.parameters()]
    pg = O.make_gloo_world1()
    with DiLoCo(manager, model, inner, outer, sync_every=2):
        for step in range(6):
            x = torch.rand(2, 3)
            for m, o in ((model, inner), (twin, twin_inner)):
                o.zero_grad()
                m(x).mean().backward()
                o.step()
            if step % 2 == 1:
                O.diloco_reference_loop_(pg, list(twin.parameters()), twin_backup, [], twin_outer, 1)
            for a, b in zip(model.parameters(), twin.parameters()):
                assert_bits_equal(a.data, b.data, f"step {step}")
    fused_calls = [c for c in cpu_ops.calls if c == "mt_outer_sgd"]
    assert (len(fused_calls) == 3) == (outer_kind == "sgd_nesterov")


def test_diloco_no_commit_discards_the_step(cpu_ops):
    model = SimpleModel()
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    manager = create_autospec(Manager)
    manager._use_async_quorum = False
    manager.should_commit.return_value = False
    og = {k: v.clone() for k, v in model.state_dict().items()}
    with DiLoCo(manager, model, inner, outer, sync_every=1) as diloco:
        _train_step(model, inner)
        torch.testing.assert_close(dict(model.state_dict()), og)
        torch.testing.assert_close(diloco._backup_parameters, _params_dict(model))
        assert outer.state_dict()["state"] == {}  # no momentum state from a discarded step
        assert all(p.grad is None for p in model.parameters())


# ---------------------------------------------------------------------------
# Manager: torchft/manager_test.py (allreduce numerics, errors, participation)
# ---------------------------------------------------------------------------

class ScriptedQuorum(QuorumClient):
    def __init__(self, result: QuorumResult) -> None:
        self.result = result
        self.votes = []
        self.quorum_calls = []

    def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
        self.quorum_calls.append(dict(rank=rank, step=step, checkpoint_metadata=checkpoint_metadata))
        return self.result

    def should_commit(self, rank, step, should_commit, timeout):
        self.votes.append(should_commit)
        return should_commit


def _manager(pg=None, quorum=None, **kw) -> Manager:
    pg = pg if pg is not None else create_autospec(ProcessGroup)
    return Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=kw.pop("min_replica_size", 2),
                   quorum_client=quorum or ScriptedQuorum(QuorumResult(
                       quorum_id=123, replica_rank=1, replica_world_size=2, max_step=1,
                       max_rank=1, max_world_size=2)), **kw)


def test_manager_numerics(cpu_ops):
    """torchft/manager_test.py:520-543."""
    manager = _manager()
    manager._quorum_future = MagicMock()
    manager._participating_rank = 1
    manager._participating_world_size = 5
    assert manager.num_participants() == 5
    manager._pg.allreduce.return_value = _DummyWork(None)
    assert manager.is_participating()
    result = manager.allreduce(torch.tensor([1.0])).value()
    torch.testing.assert_close(result, torch.tensor([1.0 / 5]))
    manager._healing = True
    assert not manager.is_participating()
    result = manager.allreduce(torch.tensor([1.0])).value()
    torch.testing.assert_close(result, torch.tensor([0.0]))
    manager.shutdown(wait=False)


def test_allreduce_future_resolves_to_the_same_tensor(cpu_ops):
    manager = _manager()
    manager._pg.allreduce.return_value = _DummyWork(None)
    manager.start_quorum()
    t = torch.tensor([4.0, 8.0])
    fut = manager.allreduce(t)
    assert fut.wait() is t
    torch.testing.assert_close(t, torch.tensor([2.0, 4.0]))
    assert manager._pending_work == [fut]
    assert manager.should_commit()
    assert manager._pending_work == []
    manager.shutdown(wait=False)


def test_allreduce_error(cpu_ops):
    """torchft/manager_test.py:338-405: errors are swallowed, latched, block the commit
    and are cleared by the next start_quorum."""
    manager = _manager()
    manager._pg.allreduce.return_value = _DummyWork(None)
    assert manager._quorum_id == -1 and manager.current_step() == 0
    manager.start_quorum()
    manager.allreduce(torch.tensor([1.0])).wait()
    assert manager._pg.allreduce.call_count == 1
    assert manager._pg.configure.call_count == 1 and manager._quorum_id == 123

    manager._pg.allreduce.side_effect = RuntimeError("injected failure")
    manager.allreduce(torch.tensor([1.0])).wait()
    assert manager.errored()
    manager.allreduce(torch.tensor([1.0])).wait()  # skipped
    assert manager._pg.allreduce.call_count == 2
    assert not manager.should_commit()
    assert manager.errored()
    assert manager.current_step() == 0

    manager._pg.allreduce.side_effect = None
    manager.start_quorum()
    assert not manager.errored()
    bad = Future()
    bad.set_exception(RuntimeError("injected failure"))
    work = MagicMock()
    work.get_future.return_value = bad
    manager._pg.allreduce.return_value = work
    t = torch.tensor([1.0])
    assert manager.allreduce(t).wait() is t  # completes with the input tensor
    assert manager.errored()
    assert not manager.should_commit()

    manager._pg.allreduce.return_value = _DummyWork(None)
    manager.start_quorum()
    manager.allreduce(torch.tensor([1.0])).wait()
    assert manager.should_commit()
    assert manager.current_step() == 1 and manager.batches_committed() == 2
    manager.shutdown(wait=False)


@pytest.mark.parametrize("rank", [1, 2])
def test_quorum_fixed_world_size(cpu_ops, rank):
    """torchft/manager_test.py:407-442: spares beyond min_replica_size do not participate."""
    q = QuorumResult(quorum_id=123, replica_rank=rank, replica_world_size=3, max_step=1,
                     max_rank=rank, max_world_size=3)
    manager = _manager(quorum=ScriptedQuorum(q), min_replica_size=2,
                       world_size_mode=WorldSizeMode.FIXED_WITH_SPARES)
    manager._pg.allreduce.return_value = _DummyWork(None)
    manager.start_quorum()
    t = torch.tensor([1.0])
    manager.allreduce(t).wait()
    assert manager.is_participating() == (rank != 2)
    assert manager.num_participants() == 2
    torch.testing.assert_close(t, torch.tensor([0.5 if rank != 2 else 0.0]))
    assert manager.should_commit()
    assert manager.batches_committed() == 2 and manager.current_step() == 1
    manager.shutdown(wait=False)


def test_async_quorum_counts_only_up_to_date_replicas(cpu_ops):
    """torchft/manager.py:452-468: async quorum uses (max_rank, max_world_size); a replica
    that is behind (max_rank None) contributes zeros; sync quorum uses the whole group."""
    q = QuorumResult(quorum_id=1, replica_rank=1, replica_world_size=3, max_step=20,
                     max_rank=None, max_world_size=2)
    m = _manager(quorum=ScriptedQuorum(q), use_async_quorum=True, min_replica_size=1)
    m._pg.allreduce.return_value = _DummyWork(None)
    m.start_quorum(allow_heal=False)
    m.wait_quorum()
    assert not m.is_participating() and m.num_participants() == 2
    t = torch.tensor([1.0])
    m.allreduce(t).wait()
    torch.testing.assert_close(t, torch.zeros(1))
    m.shutdown(wait=False)
    m = _manager(quorum=ScriptedQuorum(q), use_async_quorum=False, min_replica_size=1)
    m.start_quorum()
    assert m.is_participating() and m.num_participants() == 3
    m.shutdown(wait=False)


def test_not_enough_participants_blocks_commit(cpu_ops):
    q = QuorumResult(quorum_id=1, replica_rank=0, replica_world_size=1, max_step=0, max_rank=0,
                     max_world_size=1)
    m = _manager(quorum=ScriptedQuorum(q), min_replica_size=2)
    m.start_quorum()
    assert not m.should_commit()
    assert m._client.votes == [False]
    m.shutdown(wait=False)


def test_manager_wrap_future_and_timeout():
    """torchft/manager_test.py:486-518."""
    manager = _manager()
    assert not manager.errored()
    fut = Future()
    wrapped = manager.wrap_future(fut, 2)
    fut.set_exception(RuntimeError("injected failure"))
    assert wrapped.value() == 2
    assert manager.errored() is not None
    assert manager._pending_work == [wrapped]
    manager.shutdown(wait=False)

    manager = _manager(timeout=timedelta(seconds=0.01))
    wrapped = manager.wrap_future(Future(), 2)
    wrapped.wait()
    error = manager.errored()
    assert isinstance(error, TimeoutError)
    assert "future did not complete within" in str(error) and "0.01" in str(error)
    manager.shutdown(wait=False)


def test_manager_state_dict_round_trip():
    m = _manager()
    m.load_state_dict({"step": 7, "batches_committed": 21})
    assert m.current_step() == 7 and m.batches_committed() == 21
    assert m.state_dict() == {"step": 7, "batches_committed": 21}
    m.set_state_dict_fns(lambda sd: None, lambda: {"w": 1})
    assert m._manager_state_dict() == {"user": {"w": 1}, "torchft": m.state_dict()}
    m.shutdown(wait=False)


def test_heal_applies_the_recovered_state(cpu_ops):
    """torchft/manager.py:492-543 with an in-process transport: a healing replica loads the
    peer's state dict and step before the step runs (sync quorum)."""
    server = CheckpointServer(timeout=timedelta(seconds=10))
    server.send_checkpoint([1], 20, {"user": {"w": 5}, "torchft": {"step": 20, "batches_committed": 40}},
                           timedelta(seconds=10))

    class Healing(ScriptedQuorum):
        def checkpoint_metadata(self, address, rank, timeout):
            assert address == "peer manager"
            return server.metadata()

    q = QuorumResult(quorum_id=5, replica_rank=1, replica_world_size=2, max_step=20, max_rank=None,
                     max_world_size=1, heal=True, recover_src_rank=0,
                     recover_src_manager_address="peer manager")
    loaded = []
    mine = CheckpointServer(timeout=timedelta(seconds=10))
    m = Manager(pg=create_autospec(ProcessGroup), load_state_dict=loaded.append, state_dict=lambda: {},
                min_replica_size=1, use_async_quorum=False, quorum_client=Healing(q),
                checkpoint_transport=mine)
    m.start_quorum()
    assert loaded == [{"w": 5}]
    assert m.current_step() == 20 and m.batches_committed() == 40
    assert not m._healing and m.is_participating()
    m.shutdown()
    server.shutdown()


def _reference_quorum(**kw) -> QuorumResult:
    """The quorum the reference's manager tests script (torchft/manager_test.py:134-145)."""
    base = dict(quorum_id=123, replica_rank=1, replica_world_size=2, max_step=1, max_rank=1,
                max_world_size=2, heal=False, recover_src_manager_address="manager address")
    base.update(kw)
    return QuorumResult(**base)


class _TimedQuorum(ScriptedQuorum):
    """Records the time-outs the Manager passes on."""

    def __init__(self, result):
        super().__init__(result)
        self.quorum_timeouts, self.commit_timeouts = [], []

    def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
        self.quorum_timeouts.append(timeout)
        return super().quorum(rank, step, checkpoint_metadata, shrink_only, timeout)

    def should_commit(self, rank, step, should_commit, timeout):
        self.commit_timeouts.append(timeout)
        return super().should_commit(rank, step, should_commit, timeout)


def _healing_manager(quorum: QuorumResult, **kw):
    """A Manager whose own checkpoint server also plays the healthy peer, as the
    reference's healing tests arrange it (torchft/manager_test.py:181-190)."""
    loaded = MagicMock()
    transport = CheckpointServer(timeout=timedelta(seconds=10))

    class Client(ScriptedQuorum):
        def checkpoint_metadata(self, address, rank, timeout):
            assert address == "manager address"
            return transport.metadata()

    m = Manager(pg=create_autospec(ProcessGroup), load_state_dict=loaded, state_dict=lambda: {},
                quorum_client=Client(quorum), checkpoint_transport=transport, **kw)
    m._pg.allreduce.return_value = _DummyWork(None)
    transport.send_checkpoint(dst_ranks=[], step=quorum.max_step, state_dict=m._manager_state_dict(),
                              timeout=timedelta(seconds=10))
    return m, loaded


def test_state_dict_and_user_state_dict():
    """torchft/manager_test.py:76-127."""
    load = MagicMock()
    m = Manager(pg=create_autospec(ProcessGroup), load_state_dict=load, state_dict=lambda: {},
                min_replica_size=2, quorum_client=ScriptedQuorum(_reference_quorum()))
    assert m.state_dict() == {"step": 0, "batches_committed": 0}
    assert m._manager_state_dict() == {"user": {}, "torchft": {"step": 0, "batches_committed": 0}}
    m.set_state_dict_fns(load, lambda: {"new_state": 1})
    assert m._manager_state_dict() == {"user": {"new_state": 1},
                                       "torchft": {"step": 0, "batches_committed": 0}}
    m.load_state_dict({"step": 1234, "batches_committed": 2345})
    assert m.current_step() == 1234 and m.batches_committed() == 2345
    m.shutdown(wait=False)


def test_quorum_happy(cpu_ops):
    """torchft/manager_test.py:129-163."""
    m = _manager(quorum=ScriptedQuorum(_reference_quorum()))
    m._pg.allreduce.return_value = _DummyWork(None)
    assert m._quorum_id == -1 and m.current_step() == 0 and m.batches_committed() == 0
    m.start_quorum()
    m.allreduce(torch.tensor([1.0])).wait()
    assert len(m._pending_work) == 1
    assert m.should_commit()
    assert len(m._pending_work) == 0
    assert m._quorum_id == 123 and m.current_step() == 1
    assert m._pg.allreduce.call_count == 1
    m.start_quorum()
    assert m.batches_committed() == 2
    m.shutdown(wait=False)


def test_quorum_heal_sync(cpu_ops):
    """torchft/manager_test.py:165-212: with a synchronous quorum the recovered state is
    applied before the step, and the healed replica takes part in it."""
    q = _reference_quorum(max_step=20, max_rank=None, heal=True, recover_src_rank=0)
    m, loaded = _healing_manager(q, min_replica_size=2, use_async_quorum=False)
    assert m._quorum_id == -1 and m.current_step() == 0
    m.start_quorum()
    m.allreduce(torch.tensor([1.0])).wait()
    assert not m._healing
    assert m.is_participating() and m.num_participants() == 2
    assert m.should_commit()
    assert m._quorum_id == 123 and m.current_step() == 21
    assert m._pg.allreduce.call_count == 1
    assert loaded.call_count == 1
    m.shutdown(wait=False)


def test_quorum_heal_async_not_enough_participants(cpu_ops):
    """torchft/manager_test.py:214-276: a healing replica contributes zeros, and a step
    with fewer up-to-date replicas than min_replica_size does not commit."""
    q = _reference_quorum(max_step=20, max_rank=None, max_world_size=1, heal=True, recover_src_rank=0)
    m, loaded = _healing_manager(q, min_replica_size=2, use_async_quorum=True)
    m.start_quorum()
    m._quorum_future.result()
    assert m._healing and not m.is_participating() and m.num_participants() == 1
    grad = torch.tensor([1.0])
    m.allreduce(grad).wait()
    torch.testing.assert_close(grad, torch.zeros_like(grad))
    assert not m.should_commit()
    assert m.current_step() == 20 and m._quorum_id == 123
    assert m._pg.allreduce.call_count == 1
    assert loaded.call_count == 1
    q.heal = False
    m.start_quorum()
    assert m.current_step() == 20 and m.batches_committed() == 0
    m.shutdown(wait=False)


def test_quorum_heal_async_zero_grad(cpu_ops):
    """torchft/manager_test.py:278-336."""
    q = _reference_quorum(max_step=20, max_rank=None, max_world_size=1, heal=True, recover_src_rank=0)
    m, loaded = _healing_manager(q, min_replica_size=1, use_async_quorum=True)
    m.start_quorum()
    m._quorum_future.result()
    assert m._healing
    grad = torch.tensor([1.0])
    m.allreduce(grad).wait()
    torch.testing.assert_close(grad, torch.zeros_like(grad))
    assert m.should_commit()
    assert m.num_participants() == 1 and m.current_step() == 21
    assert m._quorum_id == 123 and m._pg.allreduce.call_count == 1
    assert loaded.call_count == 1
    q.heal = False
    m.start_quorum()
    assert m.current_step() == 21 and m.batches_committed() == 1
    m.shutdown(wait=False)


def test_quorum_no_healing(cpu_ops):
    """torchft/manager_test.py:444-476: ``allow_heal=False`` neither fetches a checkpoint
    nor takes part, but the step is still counted with the up-to-date replicas."""
    q = _reference_quorum(replica_rank=0, replica_world_size=3, max_rank=None, max_world_size=2,
                          heal=True, recover_src_rank=1)
    client = ScriptedQuorum(q)
    client.checkpoint_metadata = MagicMock(side_effect=AssertionError("must not heal"))
    m = _manager(quorum=client, min_replica_size=2)
    m._pg.allreduce.return_value = _DummyWork(None)
    m.start_quorum(allow_heal=False)
    m.allreduce(torch.tensor([1.0])).wait()
    assert not m.is_participating() and m.num_participants() == 2
    assert m.should_commit()
    assert m.batches_committed() == 2 and m.current_step() == 1
    m.shutdown(wait=False)


def test_manager_report_error():
    """torchft/manager_test.py:478-485."""
    m = _manager()
    assert m.errored() is None
    e = RuntimeError("some error")
    m.report_error(e)
    assert m.errored() is e
    m.shutdown(wait=False)


def test_quorum_happy_timeouts(cpu_ops):
    """torchft/manager_test.py:545-575: per-call time-outs reach the quorum client."""
    client = _TimedQuorum(_reference_quorum())
    m = _manager(quorum=client, use_async_quorum=False, timeout=timedelta(seconds=10),
                 quorum_timeout=timedelta(seconds=60))
    m.start_quorum(timeout=timedelta(seconds=12))
    assert client.quorum_timeouts[-1] == timedelta(seconds=12)
    assert m.should_commit(timeout=timedelta(seconds=23))
    assert client.commit_timeouts[-1] == timedelta(seconds=23)
    m.start_quorum()
    assert client.quorum_timeouts[-1] == timedelta(seconds=60)
    assert m.should_commit()
    assert client.commit_timeouts[-1] == timedelta(seconds=10)
    m.shutdown(wait=False)


def test_quorum_timeout():
    """torchft/manager_integ_test.py:621-660: one replica of a two-replica lighthouse gives
    up after the time-out it was given, for the quorum and for the commit vote alike."""
    import time

    from torchft_amd import InProcessLighthouse

    lighthouse = InProcessLighthouse(min_replicas=2)
    m = Manager(pg=create_autospec(ProcessGroup), load_state_dict=lambda x: None, state_dict=lambda: None,
                min_replica_size=2, use_async_quorum=False, rank=0, world_size=2,
                quorum_client=lighthouse.client("lonely"))
    t0 = time.monotonic()
    with pytest.raises(TimeoutError, match="quorum did not form within"):
        m.start_quorum(timeout=timedelta(seconds=0.01))
    assert time.monotonic() - t0 < 1.0
    m.shutdown(wait=False)


# ---------------------------------------------------------------------------
# Local replica group
# ---------------------------------------------------------------------------

def test_local_replicas_order_and_masks(cpu_ops):
    pg = ProcessGroupLocalReplicas(rank=1, world_size=3, peer_participating=[True, False])
    mine = torch.tensor([10.0])
    peers = [torch.tensor([1.0]), torch.tensor([100.0])]
    pg.register_peers(mine, peers)
    replicas, mask = pg.ordered(mine, True)
    assert [float(r) for r in replicas] == [1.0, 10.0, 100.0]
    assert mask == 0b011
    _, mask = pg.ordered(mine, False)
    assert mask == 0b001
    pg.allreduce([mine], torch.distributed.ReduceOp.SUM).wait()
    torch.testing.assert_close(mine, torch.tensor([11.0]))  # peer 2 contributes zeros
    with pytest.raises(KeyError):
        pg.peers_of(torch.tensor([0.0]))
    with pytest.raises(ValueError):
        pg.configure("addr", 0, 3)
    pg.configure("addr", 1, 3)
    with pytest.raises(NotImplementedError):
        pg.allreduce([mine], torch.distributed.ReduceOp.MAX)
    assert pg.size() == 3 and pg.getBackendName() == "torchft-local-replicas"


def _replica_world(model: nn.Module, n: int):
    """n-1 peer models + the lookup that pairs their parameters with the local ones."""
    import copy

    peers = [copy.deepcopy(model) for _ in range(n - 1)]
    index = {}

    def refresh():
        index.clear()
        for k, p in enumerate(model.parameters()):
            for t in (p.data, p.grad):
                if t is not None:
                    index[t.data_ptr()] = (k, t is p.grad)

    def lookup(t):
        refresh()
        k, is_grad = index[t.data_ptr()]
        out = []
        for peer in peers:
            q = list(peer.parameters())[k]
            out.append(q.grad if is_grad else q.data)
        return out

    return peers, lookup


@pytest.mark.parametrize("commit", [True, False])
def test_diloco_fused_on_local_replicas(cpu_ops, commit):
    """This package's Manager + local replica group: the sync is ONE fused launch (or one
    restore when the commit is refused) and matches the checker."""
    torch.manual_seed(0)
    model = SimpleModel()
    peers, lookup = _replica_world(model, 3)
    pg = ProcessGroupLocalReplicas(rank=0, world_size=3, peer_lookup=lookup)

    class Vote(StaticQuorum):
        def should_commit(self, rank, step, should_commit, timeout):
            return should_commit and commit

    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1, use_async_quorum=False,
                      quorum_client=Vote(0, 3))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    backup = [p.data.clone() for p in model.parameters()]
    bufs = None
    with DiLoCo(manager, model, inner, outer, sync_every=1) as diloco:
        for step in range(2):
            for k, peer in enumerate(peers):  # peers drift on their own
                for q, b in zip(peer.parameters(), backup):
                    q.data.copy_(b + 1e-3 * (k + 1) * torch.randn_like(b))
            cpu_ops.calls.clear()
            with torch.no_grad():  # an exact local drift; inner.step() is then a no-op
                for p in model.parameters():
                    p.add_(1e-3 * torch.randn_like(p))
                    p.grad = torch.zeros_like(p)
            local = [p.data.clone() for p in model.parameters()]
            want = O.diloco_perform_sync(
                [local] + [[q.data.clone() for q in peer.parameters()] for peer in peers],
                backup, bufs, [True] * 3, 3, commit, lr=0.7, momentum=0.9, nesterov=True)
            inner.step()
            for p, w in zip(model.parameters(), want["params"]):
                assert_bits_equal(p.data, w, f"step {step}")
            for (name, b_), w in zip(diloco._backup_parameters.items(), want["backup"]):
                assert_bits_equal(b_, w, f"backup {name}")
            if commit:
                assert cpu_ops.calls.count("mt_diloco_outer") == 1
                assert "mt_pseudograd_avg" not in [c for c in cpu_ops.calls[:1]]
                for p, w in zip(model.parameters(), want["momentum"]):
                    assert_bits_equal(outer.state[p]["momentum_buffer"], w)
                backup, bufs = want["backup"], want["momentum"]
            else:
                assert "mt_diloco_outer" not in cpu_ops.calls
                assert outer.state_dict()["state"] == {}
            assert manager.current_step() == (step + 1 if commit else 0)
    manager.shutdown(wait=False)


def test_local_sgd_fused_on_local_replicas(cpu_ops):
    torch.manual_seed(1)
    model = SimpleModel()
    peers, lookup = _replica_world(model, 2)
    for peer in peers:
        for q in peer.parameters():
            q.data.add_(0.01)
    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    optimizer = optim.SGD(model.parameters(), lr=0.1)
    with LocalSGD(manager, model, optimizer, sync_every=1) as local_sgd:
        with torch.no_grad():
            for p in model.parameters():
                p.add_(1e-3 * torch.randn_like(p))
                p.grad = torch.zeros_like(p)
        local = [p.data.clone() for p in model.parameters()]
        want = O.localsgd_perform_sync(
            [local, [q.data.clone() for q in peers[0].parameters()]],
            [b.clone() for b in local_sgd._backup_parameters.values()], [True, True], 2, True)
        optimizer.step()
        for p, w in zip(model.parameters(), want["params"]):
            assert_bits_equal(p.data, w)
        torch.testing.assert_close(local_sgd._backup_parameters, _params_dict(model))
        assert cpu_ops.calls.count("mt_reduce_avg") == 1  # average + backup refresh, one launch
    manager.shutdown(wait=False)


# ---------------------------------------------------------------------------
# torchft/ddp_test.py, torchft/optim_test.py
# ---------------------------------------------------------------------------

def test_pure_ddp():
    manager = create_autospec(Manager)
    m = PureDistributedDataParallel(manager, nn.Linear(3, 4))
    m(torch.rand(2, 3)).mean().backward()
    for p in m.parameters():
        assert p.grad is not None
    assert manager.allreduce.call_count == len(list(m.parameters()))


def test_ddp():
    manager = create_autospec(Manager)
    call_count = 0

    def allreduce(tensor: torch.Tensor) -> Future:
        nonlocal call_count
        call_count += 1
        fut = Future()
        fut.set_result(tensor)
        return fut

    manager.allreduce = allreduce
    m = DistributedDataParallel(manager, nn.Linear(3, 4))
    m(torch.rand(2, 3)).mean().backward()
    for p in m.parameters():
        assert p.grad is not None
    assert call_count >= 1


def test_dummy_process_group_under_torch_ddp():
    """torchft/process_group_test.py:294-298: torch's own DDP wrapper accepts the dummy
    process group (parameter verification and the initial broadcast go through it)."""
    from torchft_amd import ProcessGroupDummy

    pg = ProcessGroupDummy(0, 1)
    m = torch.nn.parallel.DistributedDataParallel(nn.Linear(3, 4), process_group=pg)
    m(torch.rand(2, 3)).sum().backward()
    assert all(p.grad is not None for p in m.parameters())
    assert pg.size() == 1 and pg.getBackendName() == "torchft-dummy"
    assert pg.configure_count == 0
    pg.configure("store", 0, 1)
    assert pg.configure_count == 1


def test_ddp_buckets_follow_the_reducer_rule():
    sizes = [p * 4 for p in (2_097_152, 2_048, 4_194_304, 2_048, 20_480, 10)]
    assert compute_bucket_assignment(sizes) == [[1, 2, 3, 4, 5], [0]]
    assert compute_bucket_assignment(sizes) == O.bucket_assignment([s // 4 for s in sizes], 4)
    metas = [torch.empty(s, dtype=torch.bfloat16, device="meta") for _, s in workloads.llama3_8b_shapes()]
    got = compute_bucket_assignment([m.numel() * 2 for m in metas])
    idx, _ = torch.distributed._compute_bucket_assignment_by_size(
        metas, [1024 * 1024, 25 * 1024 * 1024], [False] * len(metas))
    assert got == list(reversed(idx))


def test_optimizer_wrapper():
    """torchft/optim_test.py:18-50."""
    manager = create_autospec(Manager)
    m = nn.Linear(3, 4)
    base = optim.AdamW(m.parameters())
    wrapped = OptimizerWrapper(manager, base)
    wrapped.add_param_group({"params": [nn.Parameter(torch.zeros(1))], "lr": 1})
    assert wrapped.state_dict() == base.state_dict()
    wrapped.zero_grad()
    assert manager.start_quorum.call_count == 1
    manager.should_commit.return_value = True
    wrapped.step()
    manager.should_commit.return_value = False
    wrapped.step()
    assert manager.should_commit.call_count == 2
    assert wrapped.param_groups is base.param_groups and wrapped.state is base.state


# ---------------------------------------------------------------------------
# torchft/checkpointing_test.py
# ---------------------------------------------------------------------------

def test_checkpoint_server():
    expected = {"state": "dict", "nested": {"step": 3, "lr": [0.1, (1, 2)]}}
    server = CheckpointServer(timeout=timedelta(seconds=10))
    server.send_checkpoint(dst_ranks=[], step=1234, state_dict=expected, timeout=timedelta(seconds=10))
    metadata = server.metadata()
    out = server.recv_checkpoint(src_rank=0, metadata=metadata, step=1234, timeout=timedelta(seconds=10))
    assert out == expected
    with pytest.raises(urllib.error.URLError, match="urlopen error"):
        server.recv_checkpoint(src_rank=0, metadata=metadata, step=1234, timeout=timedelta(seconds=0.0))
    server.send_checkpoint(dst_ranks=[], step=2345, state_dict=expected, timeout=timedelta(seconds=10))
    with pytest.raises(urllib.error.HTTPError, match="Error 400"):
        server.recv_checkpoint(src_rank=0, metadata=metadata, step=1234, timeout=timedelta(seconds=10))
    server.shutdown()


def test_checkpoint_server_cpu_tensors_travel_in_the_header():
    state = {"w": torch.arange(6, dtype=torch.float32).view(2, 3), "n": 3}
    server = CheckpointServer(timeout=timedelta(seconds=10))
    server.send_checkpoint([], 1, state, timedelta(seconds=10))
    out = server.recv_checkpoint(0, server.metadata(), 1, timedelta(seconds=10))
    assert out["n"] == 3 and torch.equal(out["w"], state["w"])
    server.shutdown()


def test_checkpoint_server_locking():
    server = CheckpointServer(timeout=timedelta(seconds=10))
    assert server._checkpoint_lock.locked() and server._disallowed and server._step == -1
    server.allow_checkpoint(1)
    assert not server._checkpoint_lock.locked() and not server._disallowed and server._step == 1
    server.allow_checkpoint(2)
    assert server._step == 2
    server.disallow_checkpoint()
    server.disallow_checkpoint()
    assert server._checkpoint_lock.locked() and server._disallowed
    server.shutdown()


def test_timed_acquire():
    lock = threading.Lock()
    with _timed_acquire(lock, timedelta(seconds=10)):
        assert lock.locked()
    assert not lock.locked()
    lock.acquire()
    with pytest.raises(TimeoutError, match=r"timed out acquiring lock after 0:00:00"):
        with _timed_acquire(lock, timedelta(seconds=0.0)):
            pass
    assert lock.locked()


# ---------------------------------------------------------------------------
# No CPU path
# ---------------------------------------------------------------------------

def test_kernels_refuse_cpu_tensors():
    from torchft_amd import ops

    x = torch.zeros(8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.reduce_avg_(x, [x])
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.mt_copy([x], [x.clone()])
    model = SimpleModel()
    manager = create_autospec(Manager)
    manager._use_async_quorum = False
    inner = optim.SGD(model.parameters(), lr=0.1)
    with DiLoCo(manager, model, inner, optim.SGD(model.parameters(), lr=0.7), sync_every=1):
        model(torch.rand(2, 3)).mean().backward()
        with pytest.raises(RuntimeError, match="no CPU path"):
            inner.step()


def test_manager_allreduce_latches_what_the_kernels_cannot_take():
    """torchft/manager.py:242-303 never raises; neither does this one.  A host tensor has no
    kernel to run on (and there is no CPU arithmetic to fall back to): the error is latched,
    the tensor comes back untouched and the step does not commit."""
    manager = Manager(pg=ProcessGroupDummy(0, 1), load_state_dict=None, state_dict=None,
                      min_replica_size=1)
    manager.start_quorum()
    t = torch.tensor([1.0, 2.0])
    fut = manager.allreduce(t)
    assert fut.wait() is t
    assert isinstance(manager.errored(), RuntimeError) and "no CPU path" in str(manager.errored())
    assert torch.equal(t, torch.tensor([1.0, 2.0]))
    assert not manager.should_commit()
    manager.start_quorum()
    assert manager.errored() is None
    manager.shutdown(wait=False)


# ---------------------------------------------------------------------------
# Bucketised sync through an ordinary process group
# ---------------------------------------------------------------------------

class _DoublingPG(ProcessGroup):
    """A fake 2-replica backend: the peer's contribution equals ours, so SUM doubles."""

    def __init__(self):
        super().__init__(0, 2)
        self.calls = []

    def configure(self, store_addr, rank, world_size):
        pass

    def allreduce(self, tensors, opts):
        self.calls.append([t.numel() for t in tensors])
        for t in tensors:
            t.mul_(2)
        return _DummyWork(tensors)

    def size(self):
        return 2

    def getBackendName(self):
        return "doubling"


def test_diloco_bucketized_one_collective_per_sync(cpu_ops):
    torch.manual_seed(0)
    model = SimpleModel()
    pg = _DoublingPG()
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    backup = [p.data.clone() for p in model.parameters()]
    n_total = sum(p.numel() for p in model.parameters())
    with DiLoCo(manager, model, inner, outer, sync_every=1) as diloco:
        with torch.no_grad():  # an exact local drift; the inner step itself is then a no-op
            for p in model.parameters():
                p.add_(1e-3 * torch.randn_like(p))
                p.grad = torch.zeros_like(p)
        local = [p.data.clone() for p in model.parameters()]
        # both replicas hold the same parameters => the average equals the local pseudo-gradient
        want = O.diloco_perform_sync([local, local], backup, None, [True, True], 2, True,
                                     lr=0.7, momentum=0.9, nesterov=True)
        inner.step()
        assert pg.calls == [[n_total]]  # the whole model in one collective
        for p, w in zip(model.parameters(), want["params"]):
            assert_bits_equal(p.data, w)
        for b, w in zip(diloco._backup_parameters.values(), want["backup"]):
            assert_bits_equal(b, w)
        assert cpu_ops.calls.count("mt_pseudograd_avg") == 1 and cpu_ops.calls.count("mt_outer_sgd") == 1
    manager.shutdown(wait=False)


@pytest.mark.parametrize("outer_kind", ["sgd", "adam"])
def test_diloco_bucketized_failed_collective_discards_the_step(cpu_ops, outer_kind):
    """The collective fails: the error is latched, the vote is no, and the parameters go back to
    the backup whether the restore was part of the first launch (an optimizer that steps on
    the parameters) or left for the no-commit branch (the fused SGD)."""
    torch.manual_seed(0)
    model = SimpleModel()

    class Failing(_DoublingPG):
        def allreduce(self, tensors, opts):
            self.calls.append([t.numel() for t in tensors])
            raise RuntimeError("injected collective failure")

    pg = Failing()
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = (optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True) if outer_kind == "sgd"
             else optim.Adam(model.parameters(), lr=1e-3))
    backup = [p.data.clone() for p in model.parameters()]
    with DiLoCo(manager, model, inner, outer, sync_every=1) as diloco:
        with torch.no_grad():
            for p in model.parameters():
                p.add_(1e-3 * torch.randn_like(p))
                p.grad = torch.zeros_like(p)
        inner.step()
        assert len(pg.calls) == 1 and manager.errored() is not None
        for p, b, w in zip(model.parameters(), diloco._backup_parameters.values(), backup):
            assert_bits_equal(p.data, w)
            assert_bits_equal(b, w)
        assert outer.state_dict()["state"] == {}
        assert all(p.grad is None for p in model.parameters())
        assert "mt_outer_sgd" not in cpu_ops.calls
    manager.shutdown(wait=False)


@pytest.mark.parametrize("outer_kind", ["sgd_nesterov", "adam"])
def test_diloco_bucketized_matches_the_reference_loop(cpu_ops, outer_kind):
    """Through an ordinary process group whose peer contributes what this replica does (SUM
    doubles, the average is the replica's own pseudo-gradient again): the wrapper leaves the
    model where the reference's loop over one replica would, with the outer SGD that divides
    the sum on the way in and with an optimizer that steps on the averaged ``p.grad``."""
    torch.manual_seed(3)
    model = SimpleModel()
    twin = SimpleModel()
    twin.load_state_dict(model.state_dict())

    def make_outer(m):
        if outer_kind == "adam":
            return optim.Adam(m.parameters(), lr=1e-2)
        return optim.SGD(m.parameters(), lr=0.7, momentum=0.9, nesterov=True)

    pg = _DoublingPG()
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    inner, outer = optim.SGD(model.parameters(), lr=0.1), make_outer(model)
    twin_inner, twin_outer = optim.SGD(twin.parameters(), lr=0.1), make_outer(twin)
    twin_backup = [p.data.clone() for p in twin.parameters()]
    gloo = O.make_gloo_world1()
    with DiLoCo(manager, model, inner, outer, sync_every=2):
        for step in range(6):
            x = torch.rand(2, 3)
            for m, o in ((model, inner), (twin, twin_inner)):
                o.zero_grad()
                m(x).mean().backward()
                o.step()
            if step % 2 == 1:
                O.diloco_reference_loop_(gloo, list(twin.parameters()), twin_backup, [], twin_outer, 1)
            for a, b in zip(model.parameters(), twin.parameters()):
                assert_bits_equal(a.data, b.data, f"step {step}")
    assert len(pg.calls) == 3  # one collective per sync
    assert (cpu_ops.calls.count("mt_outer_sgd") == 3) == (outer_kind == "sgd_nesterov")
    manager.shutdown(wait=False)


def test_local_sgd_bucketized_one_collective_per_sync(cpu_ops):
    torch.manual_seed(0)
    model = SimpleModel()
    pg = _DoublingPG()
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2, use_async_quorum=False,
                      quorum_client=StaticQuorum(0, 2))
    optimizer = optim.SGD(model.parameters(), lr=0.1)
    n_total = sum(p.numel() for p in model.parameters())
    with LocalSGD(manager, model, optimizer, sync_every=1) as lsgd:
        with torch.no_grad():
            for p in model.parameters():
                p.add_(1e-3 * torch.randn_like(p))
                p.grad = torch.zeros_like(p)
        local = [p.data.clone() for p in model.parameters()]
        optimizer.step()
        assert pg.calls == [[n_total]]
        for p, w in zip(model.parameters(), local):
            assert_bits_equal(p.data, w)  # (x + x) / 2 == x exactly
        torch.testing.assert_close(lsgd._backup_parameters, _params_dict(model))
    manager.shutdown(wait=False)


def test_manager_client_adapter(cpu_ops):
    """A client with the reference's ManagerClient signatures (torchft/torchft.pyi:4-23),
    mocked the way torchft/manager_test.py patches it, drives this package's Manager."""
    from torchft_amd import ManagerClientAdapter

    client = MagicMock()
    client.quorum.return_value = QuorumResult(quorum_id=123, replica_rank=1, replica_world_size=2,
                                              max_step=1, max_rank=1, max_world_size=2)
    client.should_commit.side_effect = lambda rank, step, should_commit, timeout: should_commit
    peer = MagicMock()
    peer.checkpoint_metadata.return_value = "http://peer/checkpoint/"
    adapter = ManagerClientAdapter(client, connect=lambda address: peer)
    m = Manager(pg=create_autospec(ProcessGroup), load_state_dict=None, state_dict=None, min_replica_size=2, quorum_client=adapter,
                timeout=timedelta(seconds=7))
    m._pg.allreduce.return_value = _DummyWork(None)
    m.start_quorum(timeout=timedelta(seconds=12))
    m.wait_quorum()
    assert client.quorum.call_args.kwargs["timeout"] == timedelta(seconds=12)  # manager_test.py:560-563
    assert client.quorum.call_args.kwargs["rank"] == 0 and client.quorum.call_args.kwargs["step"] == 0
    t = torch.tensor([2.0])
    m.allreduce(t).wait()
    torch.testing.assert_close(t, torch.tensor([1.0]))
    assert m.should_commit(timeout=timedelta(seconds=23))
    assert client.should_commit.call_args.kwargs["timeout"] == timedelta(seconds=23)
    assert adapter.checkpoint_metadata("addr", 3, timedelta(seconds=1)) == "http://peer/checkpoint/"
    peer.checkpoint_metadata.assert_called_once_with(3, timeout=timedelta(seconds=1))
    m.shutdown(wait=False)


# ---------------------------------------------------------------------------
# Manager constructor: the reference's signature (torchft/manager.py:87-108)
# ---------------------------------------------------------------------------

REFERENCE_MANAGER_PARAMETERS = [
    # (name, has a default) in the reference's positional order
    ("pg", False), ("load_state_dict", False), ("state_dict", False), ("min_replica_size", False),
    ("use_async_quorum", True), ("timeout", True), ("quorum_timeout", True),
    ("connect_timeout", True), ("rank", True), ("world_size", True), ("world_size_mode", True),
    ("store_addr", True), ("store_port", True), ("lighthouse_addr", True), ("replica_id", True),
    ("port", True), ("hostname", True), ("heartbeat_interval", True),
    ("checkpoint_transport", True),
]


def test_manager_signature_is_the_reference_one():
    import inspect

    params = list(inspect.signature(Manager.__init__).parameters.values())[1:]
    positional = [p for p in params if p.kind is p.POSITIONAL_OR_KEYWORD]
    assert [(p.name, p.default is not p.empty) for p in positional] == REFERENCE_MANAGER_PARAMETERS
    extra = [p for p in params if p.kind is not p.POSITIONAL_OR_KEYWORD]
    assert [(p.name, p.kind) for p in extra] == [("quorum_client", inspect.Parameter.KEYWORD_ONLY)]
    assert inspect.signature(Manager.__init__).parameters["use_async_quorum"].default is True
    assert inspect.signature(Manager.__init__).parameters["timeout"].default == timedelta(seconds=60)


def test_manager_constructed_like_the_reference_integration_test(monkeypatch):
    """The call of torchft/manager_integ_test.py:148-161 binds; without a quorum client it is
    refused with one clear error (the control plane is not part of this package), with one
    it builds a manager that carries the reference's default checkpoint transport."""
    monkeypatch.delenv("TORCHFT_LIGHTHOUSE", raising=False)
    pg = create_autospec(ProcessGroup)
    kwargs = dict(
        pg=pg, min_replica_size=2, load_state_dict=lambda sd: None, state_dict=lambda: {},
        replica_id="0", store_addr="localhost", store_port=29500, rank=0, world_size=1,
        lighthouse_addr="http://localhost:29510", port=19530,
    )
    with pytest.raises(NotImplementedError, match="control plane not built; pass quorum_client="):
        Manager(**kwargs)
    quorum = ScriptedQuorum(QuorumResult(quorum_id=1, replica_rank=0, replica_world_size=2,
                                         max_step=0, max_rank=0, max_world_size=2))
    m = Manager(**kwargs, quorum_client=quorum, use_async_quorum=False)
    try:
        assert isinstance(m._checkpoint_transport, CheckpointServer)
        m.start_quorum()
        assert m.num_participants() == 2 and m.is_participating()
        assert quorum.quorum_calls[0]["checkpoint_metadata"].startswith("http://")
    finally:
        m.shutdown(wait=False)


def test_manager_constructed_like_train_ddp(monkeypatch):
    """The call of train_ddp.py:82-89 (everything else from the environment)."""
    monkeypatch.delenv("TORCHFT_LIGHTHOUSE", raising=False)
    monkeypatch.setenv("RANK", "0")
    pg = create_autospec(ProcessGroup)
    pg.size.return_value = 1
    kwargs = dict(pg=pg, min_replica_size=1, load_state_dict=lambda sd: None, state_dict=lambda: {},
                  replica_id="train_ddp_0", timeout=timedelta(seconds=10))
    m = Manager(**kwargs)
    m.start_quorum()
    m.wait_quorum()
    assert m.num_participants() == 1 and m._rank == 0 and m._timeout == timedelta(seconds=10)
    m.shutdown(wait=False)
    monkeypatch.setenv("TORCHFT_LIGHTHOUSE", "http://lighthouse:29510")
    with pytest.raises(NotImplementedError, match="control plane not built"):
        Manager(**kwargs)
    # positional, in the reference's order
    m = Manager(pg, None, None, 1, False, timedelta(seconds=5), timedelta(seconds=6),
                timedelta(seconds=7), 3, 4, WorldSizeMode.FIXED_WITH_SPARES, None, None, None, "r",
                None, "host", timedelta(milliseconds=50), None, quorum_client=StaticQuorum(0, 1))
    assert (m._rank, m._use_async_quorum, m._world_size_mode) == (3, False, WorldSizeMode.FIXED_WITH_SPARES)
    assert (m._timeout, m._quorum_timeout, m._connect_timeout) == (
        timedelta(seconds=5), timedelta(seconds=6), timedelta(seconds=7))
    m.shutdown(wait=False)


def test_local_sgd_fused_waits_for_an_asynchronous_quorum(cpu_ops):
    """LocalSGD allows ``use_async_quorum=True`` (the Manager's default).  The single-launch
    sync decides before it reduces, so it must join the quorum thread first: otherwise the
    vote reads the previous quorum's participant count (0 before the first one, so no
    commit) and a recovered state is not applied (torchft/manager.py:265 reaches
    ``wait_quorum`` through ``allreduce`` before ``should_commit``)."""
    import time

    torch.manual_seed(3)
    model = SimpleModel()
    peers, lookup = _replica_world(model, 2)
    for peer in peers:
        for q in peer.parameters():
            q.data.add_(0.01)

    class SlowQuorum(StaticQuorum):
        def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
            time.sleep(0.3)
            return super().quorum(rank, step, checkpoint_metadata, shrink_only, timeout)

    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    client = SlowQuorum(0, 2)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                      use_async_quorum=True, quorum_client=client)
    optimizer = optim.SGD(model.parameters(), lr=0.1)
    with LocalSGD(manager, model, optimizer, sync_every=1) as local_sgd:
        with torch.no_grad():
            for p in model.parameters():
                p.grad = torch.zeros_like(p)
        local = [p.data.clone() for p in model.parameters()]
        want = O.localsgd_perform_sync(
            [local, [q.data.clone() for q in peers[0].parameters()]],
            [b.clone() for b in local_sgd._backup_parameters.values()], [True, True], 2, True)
        optimizer.step()  # first sync: quorum still running when the sync starts
        assert client.commit_votes == [True]
        assert manager.current_step() == 1 and manager.batches_committed() == 2
        for p, w in zip(model.parameters(), want["params"]):
            assert_bits_equal(p.data, w)
        assert cpu_ops.calls.count("mt_reduce_avg") == 1
    manager.shutdown(wait=False)


def test_local_sgd_fused_applies_recovered_state_with_asynchronous_quorum(cpu_ops):
    """A healing replica under an asynchronous quorum: the pending state dict is loaded by
    the vote (torchft/manager.py:572-575), the replica does not participate, and its
    parameters end as the average of the others."""
    import time

    torch.manual_seed(4)
    model = SimpleModel()
    peers, lookup = _replica_world(model, 2)
    loaded = []

    class HealingQuorum(QuorumClient):
        def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
            time.sleep(0.2)
            return QuorumResult(quorum_id=7, replica_rank=0, replica_world_size=2,
                                recover_src_manager_address="peer", recover_src_rank=1,
                                max_step=5, max_rank=None, max_world_size=1, heal=True)

        def should_commit(self, rank, step, should_commit, timeout):
            return should_commit

        def checkpoint_metadata(self, address, rank, timeout):
            return "meta"

    transport = MagicMock()
    transport.metadata.return_value = ""
    transport.recv_checkpoint.return_value = {"user": {"tag": 1}, "torchft": {"step": 5, "batches_committed": 10}}
    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup)
    manager = Manager(pg=pg, load_state_dict=loaded.append, state_dict=lambda: {}, min_replica_size=1,
                      use_async_quorum=True, quorum_client=HealingQuorum(), checkpoint_transport=transport)
    optimizer = optim.SGD(model.parameters(), lr=0.1)
    with LocalSGD(manager, model, optimizer, sync_every=1):
        with torch.no_grad():
            for p in model.parameters():
                p.grad = torch.zeros_like(p)
        optimizer.step()
        assert loaded == [{"tag": 1}]
        assert manager.current_step() == 6
        # not participating: contributes zeros, one participant -> the peer's values
        for p, q in zip(model.parameters(), peers[0].parameters()):
            assert_bits_equal(p.data, q.data)
    manager.shutdown(wait=False)


@pytest.mark.parametrize("group", ["local_replicas", "ordinary"])
def test_local_sgd_ends_with_the_recovered_state_when_the_vote_loads_it(cpu_ops, group):
    """A healing replica under an asynchronous quorum whose ``load_state_dict`` really loads the
    model: the reference averages first and the vote then loads the recovered state over it
    (torchft/local_sgd.py:151-158, torchft/manager.py:572-575), so the sync ends with the
    recovered parameters, and the backup equals them."""
    import time

    torch.manual_seed(4)
    model = SimpleModel()
    peers, lookup = _replica_world(model, 2)
    recovered = {k: torch.full_like(v, 0.125) for k, v in model.state_dict().items()}

    class HealingQuorum(QuorumClient):
        def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
            time.sleep(0.1)
            return QuorumResult(quorum_id=7, replica_rank=0, replica_world_size=2,
                                recover_src_manager_address="peer", recover_src_rank=1,
                                max_step=5, max_rank=None, max_world_size=1, heal=True)

        def should_commit(self, rank, step, should_commit, timeout):
            return should_commit

        def checkpoint_metadata(self, address, rank, timeout):
            return "meta"

    transport = MagicMock()
    transport.metadata.return_value = ""
    transport.recv_checkpoint.return_value = {"user": recovered, "torchft": {"step": 5, "batches_committed": 10}}
    pg = (ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=lookup) if group == "local_replicas"
          else _DoublingPG())
    manager = Manager(pg=pg, load_state_dict=model.load_state_dict, state_dict=model.state_dict, min_replica_size=1,
                      use_async_quorum=True, quorum_client=HealingQuorum(), checkpoint_transport=transport)
    optimizer = optim.SGD(model.parameters(), lr=0.1)
    with LocalSGD(manager, model, optimizer, sync_every=1) as lsgd:
        with torch.no_grad():
            for p in model.parameters():
                p.grad = torch.zeros_like(p)
        optimizer.step()
        assert manager.current_step() == 6
        for (name, p), b in zip(model.named_parameters(), lsgd._backup_parameters.values()):
            assert_bits_equal(p.data, recovered[name], name)
            assert_bits_equal(b, recovered[name], f"backup {name}")
    manager.shutdown(wait=False)


# ---------------------------------------------------------------------------
# What a wrapper keeps between syncs, and what makes it look again
# ---------------------------------------------------------------------------

def _stable_world(model: nn.Module, n: int):
    """Peer models whose buffers never move, a lookup that counts its calls, and a process
    group that has been told so (``peers_are_stable``)."""
    import copy

    peers = [copy.deepcopy(model) for _ in range(n - 1)]
    calls = []

    def lookup(t):
        calls.append(t.data_ptr())
        for k, p in enumerate(model.parameters()):
            if p.data.data_ptr() == t.data_ptr():
                return [list(peer.parameters())[k].data for peer in peers]
        raise KeyError("unknown tensor")

    pg = ProcessGroupLocalReplicas(rank=0, world_size=n, peer_lookup=lookup, peers_are_stable=True)
    return peers, pg, calls


def _checked_diloco_sync(diloco, model, peers, outer, state, lr=0.7):
    """One sync, compared with the checker; ``state`` carries (backup, momentum) along."""
    with torch.no_grad():
        for p in model.parameters():
            p.add_(1e-3 * torch.randn_like(p))
    local = [p.data.clone() for p in model.parameters()]
    want = O.diloco_perform_sync(
        [local] + [[q.data.clone() for q in peer.parameters()] for peer in peers],
        state["backup"], state["bufs"], [True] * (len(peers) + 1), len(peers) + 1, True,
        lr=lr, momentum=0.9, nesterov=True)
    diloco.sync()
    for p, w in zip(model.parameters(), want["params"]):
        assert_bits_equal(p.data, w)
    for b_, w in zip(diloco._backup_parameters.values(), want["backup"]):
        assert_bits_equal(b_, w)
    for p, w in zip(model.parameters(), want["momentum"]):
        assert_bits_equal(outer.state[p]["momentum_buffer"], w)
    state["backup"], state["bufs"] = want["backup"], want["momentum"]


def test_diloco_keeps_its_prepared_sync_and_notices_every_change(cpu_ops):
    """Steady state: no peer lookups, no new tensor lists, the same prepared launch.  Each thing a
    user may change between syncs - ``p.data``, ``_backup_parameters``, the learning rate, the
    optimizer's state, the peers - is noticed, and the results stay the checker's."""
    torch.manual_seed(0)
    model = SimpleModel()
    peers, pg, lookups = _stable_world(model, 2)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1,
                      use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    n = len(list(model.parameters()))
    state = {"backup": [p.data.clone() for p in model.parameters()], "bufs": None}
    with DiLoCo(manager, model, inner, outer, sync_every=10 ** 9) as diloco:
        _checked_diloco_sync(diloco, model, peers, outer, state)      # first step: creates momentum
        _checked_diloco_sync(diloco, model, peers, outer, state)      # steady state: prepared anew once
        assert len(lookups) == n                                      # asked once per tensor, ever
        kept, bound, plan = diloco._launches["fused"], diloco._bound, diloco._plan
        for _ in range(2):
            _checked_diloco_sync(diloco, model, peers, outer, state)
        assert len(lookups) == n
        assert diloco._launches["fused"] is kept and diloco._bound is bound and diloco._plan is plan

        # the learning rate moves (a scheduler): new plan, same tensors
        outer.param_groups[0]["lr"] = 0.35
        _checked_diloco_sync(diloco, model, peers, outer, state, lr=0.35)
        assert diloco._plan is not plan and diloco._bound is bound and len(lookups) == n
        outer.param_groups[0]["lr"] = 0.7

        # a parameter's storage is replaced (model.to(), a load that rebinds .data)
        first = next(model.parameters())
        first.data = first.data.clone()
        _checked_diloco_sync(diloco, model, peers, outer, state)
        assert diloco._bound is not bound and len(lookups) == 2 * n   # peers looked up again
        bound = diloco._bound

        # the user's load_state_dict assigns a new backup dict (torchft/manager_integ_test.py:279)
        diloco._backup_parameters = {k: v.clone() for k, v in diloco._backup_parameters.items()}
        _checked_diloco_sync(diloco, model, peers, outer, state)
        assert diloco._bound is not bound
        bound = diloco._bound

        # the outer optimizer's state is replaced (load_state_dict after healing)
        copy_state = outer.state_dict()
        outer.load_state_dict(copy_state)
        state["bufs"] = [outer.state[p]["momentum_buffer"].clone() for p in model.parameters()]
        plan = diloco._plan
        _checked_diloco_sync(diloco, model, peers, outer, state)
        assert diloco._plan is not plan

        # a momentum buffer is swapped inside the state
        p0 = next(model.parameters())
        outer.state[p0]["momentum_buffer"] = outer.state[p0]["momentum_buffer"].clone()
        plan = diloco._plan
        _checked_diloco_sync(diloco, model, peers, outer, state)
        assert diloco._plan is not plan

        # the peers move and say so
        for q in peers[0].parameters():
            q.data = q.data.clone()
        pg.invalidate_peers()
        before = len(lookups)
        _checked_diloco_sync(diloco, model, peers, outer, state)
        assert len(lookups) == before + n
    manager.shutdown(wait=False)


def test_peer_lookups_are_repeated_unless_declared_stable(cpu_ops):
    torch.manual_seed(0)
    model = SimpleModel()
    peers, lookup = _replica_world(model, 2)
    seen = []

    def counting(t):
        seen.append(1)
        return lookup(t)

    pg = ProcessGroupLocalReplicas(rank=0, world_size=2, peer_lookup=counting)
    assert pg.peers_generation() is None          # a callback may answer differently next time
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1,
                      use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    n = len(list(model.parameters()))
    with LocalSGD(manager, model, inner, sync_every=10 ** 9) as lsgd:
        for k in range(3):
            lsgd.sync()
            assert len(seen) == (k + 1) * n
    # registered peers only change through the group: a generation, and no repeated look-ups
    pg2 = ProcessGroupLocalReplicas(rank=0, world_size=2)
    t, peer = torch.zeros(4), torch.ones(4)
    g0 = pg2.peers_generation()
    pg2.register_peers(t, [peer])
    assert pg2.peers_generation() == g0 + 1
    pg2.set_peer_participating([False])
    assert pg2.peers_generation() == g0 + 2
    manager.shutdown(wait=False)


def test_diloco_mirrors_a_backup_kept_elsewhere(cpu_ops, monkeypatch):
    """Backup tensors that do not live with the parameters (host memory, a user's own tensors)
    are copied into device buffers for the sync and written back after a committed step; a
    step that is not committed leaves them alone and restores the parameters from them."""
    from torchft_amd import local_sgd

    torch.manual_seed(0)
    model = SimpleModel()
    peers, pg, _ = _stable_world(model, 2)
    flag = [True]

    class Vote(StaticQuorum):
        def should_commit(self, rank, step, should_commit, timeout):
            return should_commit and flag[0]

    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1,
                      use_async_quorum=False, quorum_client=Vote(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
    elsewhere = set()
    monkeypatch.setattr(local_sgd.LocalSGD, "_on_device", staticmethod(
        lambda params, backups: bool(params) and not any(b.data_ptr() in elsewhere for b in backups)))
    monkeypatch.setattr(local_sgd.LocalSGD, "_on_one_gpu", staticmethod(lambda params: bool(params)))
    monkeypatch.setattr(torch.cuda, "current_stream", lambda device=None: MagicMock())
    state = {"backup": [p.data.clone() for p in model.parameters()], "bufs": None}
    with DiLoCo(manager, model, inner, outer, sync_every=10 ** 9) as diloco:
        _checked_diloco_sync(diloco, model, peers, outer, state)
        mine = {k: v.clone() for k, v in diloco._backup_parameters.items()}
        elsewhere.update(v.data_ptr() for v in mine.values())
        diloco._backup_parameters = mine
        for _ in range(2):
            _checked_diloco_sync(diloco, model, peers, outer, state)   # compares ``mine`` with the checker
            assert diloco._backup_parameters is mine
        mirror = diloco._flat["backup_mirror"][2]
        assert all(m.data_ptr() != b.data_ptr() for m, b in zip(mirror, mine.values()))
        # not committed: parameters back to the backup, backup and momentum untouched
        flag[0] = False
        before = [v.clone() for v in mine.values()]
        momentum = [outer.state[p]["momentum_buffer"].clone() for p in model.parameters()]
        with torch.no_grad():
            for p in model.parameters():
                p.add_(1e-3 * torch.randn_like(p))
        diloco.sync()
        for p, b, w, m in zip(model.parameters(), mine.values(), before, momentum):
            assert_bits_equal(b, w)
            assert_bits_equal(p.data, w)
            assert_bits_equal(outer.state[p]["momentum_buffer"], m)
        flag[0] = True
        _checked_diloco_sync(diloco, model, peers, outer, state)
    manager.shutdown(wait=False)


def test_local_sgd_keeps_its_prepared_average(cpu_ops):
    torch.manual_seed(0)
    model = SimpleModel()
    peers, pg, lookups = _stable_world(model, 3)
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=1,
                      use_async_quorum=False, quorum_client=StaticQuorum(0, 3))
    inner = optim.SGD(model.parameters(), lr=0.1)
    n = len(list(model.parameters()))
    with LocalSGD(manager, model, inner, sync_every=10 ** 9) as lsgd:
        backup = [b.clone() for b in lsgd._backup_parameters.values()]
        for k in range(3):
            with torch.no_grad():
                for p in model.parameters():
                    p.add_(1e-3 * torch.randn_like(p))
            reps = [[p.data.clone() for p in model.parameters()]] + [
                [q.data.clone() for q in peer.parameters()] for peer in peers]
            want = O.localsgd_perform_sync(reps, backup, [True] * 3, 3, True)
            lsgd.sync()
            for p, w in zip(model.parameters(), want["params"]):
                assert_bits_equal(p.data, w)
            backup = want["backup"]
            if k == 0:
                kept = lsgd._launches["average"]
        assert lsgd._launches["average"] is kept and len(lookups) == n
    manager.shutdown(wait=False)
