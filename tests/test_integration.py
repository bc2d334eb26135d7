"""End-to-end: replica groups as threads, quorum, all-reduce among them, failure and live
recovery over the checkpoint transport - the scenarios of the reference's integration tests
(torchft/manager_integ_test.py: test_ddp_healthy / test_ddp_recovery / test_local_sgd_recovery
/ test_diloco_healthy / test_diloco_recovery).  Their assertions are kept: final models equal
across replicas; for LocalSGD / DiLoCo the backup parameters and the outer optimizer state
equal across replicas at every manager step.

The GPU variants run the real kernels; the CPU variants run the same control flow over the
CPU stand-in for the kernels (tests/fake_backend.py)."""

import pytest
import torch

import integ_harness as H
from helpers import assert_bits_equal


def _devices():
    return [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]


@pytest.fixture
def dev(request, cpu_ops_if_cpu):
    return cpu_ops_if_cpu


@pytest.fixture
def cpu_ops_if_cpu(request):
    kind = request.param
    if kind == "cpu":
        request.getfixturevalue("cpu_ops")
        return torch.device("cpu")
    return torch.device("cuda", 0)


def _assert_models_equal(results):
    (state0, step0), *rest = results
    for state, step in rest:
        assert step == step0
        for k in state0:
            assert_bits_equal(state[k], state0[k], k)


def _assert_syncs_match_the_checker(results, kind):
    """Every synchronisation the cluster ran, held to the CPU checker: the recorded inputs of
    all replicas of a quorum (parameters after the inner steps, shared backup, outer momentum)
    go through ``O.diloco_perform_sync`` / ``O.localsgd_perform_sync`` and every participating
    replica's recorded outputs must equal the result bit for bit
    (torchft/manager_integ_test.py:553-562 asserts only that replicas agree with each other)."""
    from oracle import replica_sync as O

    by_step = {}
    for _, _, records in results:
        for rec in records:
            by_step.setdefault(rec["step"], {})[rec["rank"]] = rec
    checked = 0
    for step, ranks in sorted(by_step.items()):
        world = next(iter(ranks.values()))["world"]
        if sorted(ranks) != list(range(world)) or any(r["world"] != world for r in ranks.values()):
            continue  # a replica died before this sync: the others latched an error or re-formed
        recs = [ranks[r] for r in range(world)]
        flags = [r["participating"] for r in recs]
        if not any(flags):
            continue
        src = recs[flags.index(True)]
        nump = src["num_participants"]
        assert all(r["num_participants"] == nump for r in recs)
        commit = src["committed"]
        assert all(r["committed"] == commit for r in recs)
        reps = [r["params"] for r in recs]
        if kind == "diloco":
            want = O.diloco_perform_sync(reps, src["backup"], src["momentum"], flags, nump, commit,
                                         lr=0.7, momentum=0.9, nesterov=True)
        else:
            want = O.localsgd_perform_sync(reps, src["backup"], flags, nump, commit)
        for rec, part in zip(recs, flags):
            if not part:
                continue  # a healing replica ends with the recovered state, checked elsewhere
            for t in range(len(want["params"])):
                assert_bits_equal(rec["post_params"][t], want["params"][t], f"step {step} params[{t}]")
                assert_bits_equal(rec["post_backup"][t], want["backup"][t], f"step {step} backup[{t}]")
                if kind == "diloco" and commit:
                    assert_bits_equal(rec["post_momentum"][t], want["momentum"][t],
                                      f"step {step} momentum[{t}]")
            checked += 1
    assert checked >= 4, f"only {checked} replica-syncs could be held to the checker"


def _assert_histories_equal(results, check_momentum):
    results = [(r[0], r[1]) for r in results]
    (hist0, step0), *rest = results
    assert step0 >= 4
    for hist, step in rest:
        assert step == step0
        common = sorted(set(hist) & set(hist0))
        assert common, "no common manager steps"
        for s in common:
            for k, v in hist0[s]["backup_params"].items():
                assert_bits_equal(hist[s]["backup_params"][k], v, f"step {s} backup {k}")
            if check_momentum:
                assert len(hist[s]["outer_momentum"]) == len(hist0[s]["outer_momentum"])
                for a, b in zip(hist[s]["outer_momentum"], hist0[s]["outer_momentum"]):
                    assert_bits_equal(a, b, f"step {s} outer momentum")


@pytest.mark.parametrize("cpu_ops_if_cpu", _devices(), indirect=True)
def test_ddp_healthy(dev):
    results = H.run_cluster(H.ddp_train_loop, dev, [H.FailureInjector(), H.FailureInjector()])
    _assert_models_equal(results)


@pytest.mark.parametrize("cpu_ops_if_cpu", _devices(), indirect=True)
def test_ddp_recovery(dev):
    injectors = [H.FailureInjector(), H.FailureInjector().fail_at(1, 2)]
    results = H.run_cluster(H.ddp_train_loop, dev, injectors)
    _assert_models_equal(results)
    assert injectors[1].count == 1


@pytest.mark.parametrize("cpu_ops_if_cpu", _devices(), indirect=True)
def test_local_sgd_recovery(dev):
    injectors = [H.FailureInjector(), H.FailureInjector().fail_at(1, 2)]
    results = H.run_cluster(H.local_sgd_train_loop, dev, injectors)
    _assert_histories_equal(results, check_momentum=False)
    _assert_syncs_match_the_checker(results, "local_sgd")
    assert injectors[1].count == 1


@pytest.mark.parametrize("cpu_ops_if_cpu", _devices(), indirect=True)
def test_diloco_healthy(dev):
    results = H.run_cluster(H.diloco_train_loop, dev, [H.FailureInjector(), H.FailureInjector()],
                            use_async_quorum=False)
    _assert_histories_equal(results, check_momentum=True)
    _assert_syncs_match_the_checker(results, "diloco")


@pytest.mark.parametrize("cpu_ops_if_cpu", _devices(), indirect=True)
def test_diloco_recovery(dev):
    injectors = [H.FailureInjector(), H.FailureInjector().fail_at(1, 2)]
    results = H.run_cluster(H.diloco_train_loop, dev, injectors, use_async_quorum=False)
    _assert_histories_equal(results, check_momentum=True)
    _assert_syncs_match_the_checker(results, "diloco")
    assert injectors[1].count == 1


def test_quorum_results_follow_the_reference_rules():
    """compute_quorum_result against hand-built quorums (src/manager.rs:357-480 and its
    tests at :482-851): ranks by sorted id, max-step cohort, recovery assignment."""
    from torchft_amd.local_cluster import _Member, _Quorum, compute_quorum_result

    q = _Quorum(7, [_Member("b", 10, "mb"), _Member("a", 10, "ma"), _Member("c", 3, "mc")])
    ra = compute_quorum_result("a", 0, q)
    assert (ra.quorum_id, ra.replica_rank, ra.replica_world_size) == (7, 0, 3)
    assert (ra.max_step, ra.max_rank, ra.max_world_size, ra.heal) == (10, 0, 2, False)
    assert ra.recover_dst_ranks == [2] and ra.recover_src_rank is None
    rb = compute_quorum_result("b", 0, q)
    assert (rb.replica_rank, rb.max_rank, rb.heal, rb.recover_dst_ranks) == (1, 1, False, [])
    rc = compute_quorum_result("c", 0, q)
    assert (rc.replica_rank, rc.max_rank, rc.max_world_size, rc.heal) == (2, None, 2, True)
    assert rc.recover_src_rank == 0 and rc.recover_src_manager_address == "a"
    # before the first step everybody but the primary syncs from the primary
    q0 = _Quorum(1, [_Member("a", 0, ""), _Member("b", 0, "")])
    assert compute_quorum_result("a", 0, q0).recover_dst_ranks == [1]
    rb0 = compute_quorum_result("b", 0, q0)
    assert rb0.heal and rb0.recover_src_rank == 0 and rb0.max_rank == 1 and rb0.max_world_size == 2
    with pytest.raises(KeyError):
        compute_quorum_result("z", 0, q)


def test_thread_process_group_masks_and_missing_peer(cpu_ops):
    """Three thread-replicas, one of them a spare (contributes zeros); then a round in which
    one replica never shows up: the others' futures stay pending and the Manager's timeout
    latches an error instead of hanging."""
    import threading
    from datetime import timedelta

    from torchft_amd import Manager, ProcessGroupThreads, QuorumResult, ThreadWorld
    from torchft_amd.manager import QuorumClient

    world = ThreadWorld()

    class Fixed(QuorumClient):
        def __init__(self, rank, quorum_id):
            self.rank, self.quorum_id = rank, quorum_id

        def quorum(self, rank, step, checkpoint_metadata, shrink_only, timeout):
            # replica 2 is behind (not in the max-step cohort): it contributes zeros
            return QuorumResult(quorum_id=self.quorum_id, replica_rank=self.rank, replica_world_size=3,
                                max_step=5, max_rank=self.rank if self.rank < 2 else None,
                                max_world_size=2)

        def should_commit(self, rank, step, should_commit, timeout):
            return should_commit

    values = [torch.tensor([1.0, 2.0]), torch.tensor([3.0, 6.0]), torch.tensor([100.0, 100.0])]
    out = [None] * 3
    commits = [None] * 3

    def replica(r, quorum_id, show_up=True, timeout=5.0):
        m = Manager(pg=ProcessGroupThreads(world), load_state_dict=None, state_dict=None, min_replica_size=2,
                    timeout=timedelta(seconds=timeout), quorum_client=Fixed(r, quorum_id))
        m.start_quorum(allow_heal=False)
        if show_up:
            t = values[r].clone()
            m.allreduce(t).wait()
            out[r] = t
            commits[r] = m.should_commit()
        m.shutdown(wait=False)

    threads = [threading.Thread(target=replica, args=(r, 1)) for r in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=30)
    for r in range(3):
        torch.testing.assert_close(out[r], torch.tensor([2.0, 4.0]))  # (1+3+0)/2, (2+6+0)/2
    assert commits == [True, True, True]

    out[:] = [None] * 3
    commits[:] = [None] * 3
    threads = [threading.Thread(target=replica, args=(r, 2, r != 1, 0.3)) for r in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=30)
    assert commits[0] is False and commits[2] is False  # timed out, error latched, no commit
    torch.testing.assert_close(out[0], values[0])  # the tensor was left as it was
