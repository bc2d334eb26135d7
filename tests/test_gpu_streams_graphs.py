"""The launches are plain stream work: they can be captured into a HIP graph and replayed,
and issued concurrently from several threads on their own streams."""

import threading

import pytest
import torch

from helpers import assert_bits_equal
from oracle import replica_sync as O
from torchft_amd import ops, workloads

pytestmark = pytest.mark.gpu

SHAPES = workloads.mlp_shapes() + [("odd", (77, 3))]


def test_fused_step_in_a_hip_graph(device):
    """Capture two fused outer steps (steady state) in one graph; replay it several times with
    eager work and synchronisations in between; every replay must equal the eager result."""
    wl = workloads.make_diloco_workload(SHAPES, 2, torch.device("cpu"))
    sgd = ops.OuterSGD(lr=0.7, momentum=0.9, nesterov=True)
    bufs0 = workloads.normal_tensors(SHAPES, 1e-3, 5, torch.device("cpu"))
    b = [t.to(device) for t in wl.backup]
    m = [t.to(device) for t in bufs0]
    p = [torch.empty_like(t) for t in b]
    reps = [[t.to(device) for t in rep] for rep in wl.replicas]
    table = ops.mt_diloco_outer(p, b, m, reps, sgd, False)  # warm-up builds the table eagerly
    torch.cuda.synchronize()
    # expected trajectory from the same start: warm-up step + 2 steps per replay
    backup, bufs = wl.backup, bufs0
    expected = []
    for step in range(1 + 2 * 3):
        res = O.diloco_perform_sync(wl.replicas, backup, bufs, [True, True], 2, True,
                                    lr=0.7, momentum=0.9, nesterov=True)
        backup, bufs = res["backup"], res["momentum"]
        expected.append(res)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.mt_diloco_outer(p, b, m, reps, sgd, False, table=table)
            ops.mt_diloco_outer(p, b, m, reps, sgd, False, table=table)
    # capture does not execute: state is still the one after the warm-up step
    for i in range(len(SHAPES)):
        assert_bits_equal(b[i], expected[0]["backup"][i])
    scratch = torch.zeros(1 << 20, device=device)
    for replay in range(3):
        graph.replay()
        scratch.add_(1.0)  # eager work between replays
        torch.cuda.synchronize()
        want = expected[2 * (replay + 1)]
        for i, (name, _) in enumerate(SHAPES):
            assert_bits_equal(p[i], want["params"][i], f"replay {replay} {name}")
            assert_bits_equal(b[i], want["backup"][i], f"replay {replay} backup {name}")
            assert_bits_equal(m[i], want["momentum"][i], f"replay {replay} momentum {name}")


def test_concurrent_launches_from_threads(device):
    """Training thread, autograd thread and checkpoint thread may all call the library: four
    threads, each on its own stream with its own tensors, many launches each."""
    n_threads, rounds = 4, 25
    g = torch.Generator().manual_seed(0)
    inputs = [[torch.randn(300_007, generator=g) for _ in range(3)] for _ in range(n_threads)]
    wants = [O.manager_allreduce_(xs, [True, False, True], 2) for xs in inputs]
    errors = []

    def worker(k):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                dev = [x.to(device) for x in inputs[k]]
                out = torch.empty_like(dev[0])
                copy = torch.empty_like(dev[0])
                for _ in range(rounds):
                    ops.reduce_avg_(out, dev, 0b101, 2)
                    ops.mt_copy([copy], [out])
                stream.synchronize()
                assert_bits_equal(out, wants[k], f"thread {k}")
                assert_bits_equal(copy, wants[k], f"thread {k} copy")
        except BaseException as e:  # surfaced in the main thread
            errors.append((k, e))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not errors, errors


def test_launch_variant_is_thread_local(device, launch_variant):
    """The tuning build's launch-shape override must not leak across threads."""
    seen = {}

    def other():
        launch_variant(4 | 16)
        seen["set"] = True

    t = threading.Thread(target=other)
    t.start()
    t.join()
    # this thread still uses the defaults: results unaffected either way, but the call must
    # not leak state across threads (checked through a launch that succeeds with defaults)
    x = torch.ones(10_000, device=device)
    ops.reduce_avg_(x, [x, x], 0b11, 2)
    assert_bits_equal(x, torch.ones(10_000))
    assert seen["set"]
