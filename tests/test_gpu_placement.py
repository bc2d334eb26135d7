"""HBM bank-group placement of the library's own buffers (MI355X): mechanics and, above
all, that it changes nothing but addresses."""

import pytest
import torch
from torch import nn, optim

from helpers import assert_bits_equal
from oracle import replica_sync as O
from torchft_amd import (
    DiLoCo,
    LocalSGD,
    Manager,
    ProcessGroupLocalReplicas,
    StaticQuorum,
    hbm_placement as H,
)

pytestmark = pytest.mark.gpu


class Wide(nn.Module):
    """1.25 GiB of fp32 parameters in tensors large enough to probe, plus small ones."""

    def __init__(self) -> None:
        super().__init__()
        self.a = nn.Parameter(torch.empty(160 << 20).normal_(0, 0.02))   # 640 MiB
        self.b = nn.Parameter(torch.empty(128 << 20).normal_(0, 0.02))   # 512 MiB
        self.c = nn.Parameter(torch.empty(32 << 20).normal_(0, 0.02))    # 128 MiB
        self.small = nn.Parameter(torch.empty(1000, 7).normal_(0, 0.02))
        self.one = nn.Parameter(torch.zeros(1))


def test_probe_leaves_the_buffer_unchanged(device):
    g = torch.Generator(device).manual_seed(0)
    a = torch.randint(0, 256, (64 << 20,), dtype=torch.uint8, device=device, generator=g)
    a[:4].copy_(torch.tensor([0xFF, 0xFF, 0xBF, 0x7F], dtype=torch.uint8))  # a signalling NaN pattern
    keep = a.clone()
    scratch = torch.zeros_like(a)
    ms = H.probe_ms(a, scratch)
    assert ms > 0
    assert torch.equal(a, keep)
    assert torch.equal(scratch, keep)  # the copy is exact as well


def test_allocate_apart_places_copies_outside_the_models_group(device):
    torch.manual_seed(0)
    model = Wide().to(device)
    like = [p.data for p in model.parameters()]
    copies = None
    for _ in range(3):  # the groups are found by timing: a disturbed measurement makes it give up
        copies = H.allocate_apart(like, 2)
        if copies is not None:
            break
    assert copies is not None, "no bank-group structure found: is this an MI355X?"
    seen = set()
    for col in copies:
        assert len(col) == len(like)
        for t, ref in zip(col, like):
            assert t.shape == ref.shape and t.dtype == ref.dtype and t.device == ref.device
            assert t.is_contiguous() and t.data_ptr() % 256 == 0
            span = (t.data_ptr(), t.data_ptr() + t.numel() * t.element_size())
            assert all(span[1] <= lo or span[0] >= hi for lo, hi in seen), "buffers overlap"
            seen.add(span)
    # the probe agrees: a large model tensor and its copies do not share a group, the two
    # copies of one tensor do (they are kept together)
    big, copy0, copy1 = like[0], copies[0][0], copies[1][0]
    half = copy0.numel() // 2

    def ratios():
        same = H.probe_ms(copy0[:half], copy0[half:], 256 << 20, repeats=6)  # halves of one buffer
        return (H.probe_ms(big, copy0, 256 << 20, repeats=6) / same,
                H.probe_ms(big, copy1, 256 << 20, repeats=6) / same,
                H.probe_ms(copy0, copy1, 256 << 20, repeats=6) / same)

    for attempt in range(3):
        r_big0, r_big1, r_01 = ratios()
        if r_big0 < 0.92 and r_big1 < 0.92 and r_01 > 0.92:
            break
    assert r_big0 < 0.92 and r_big1 < 0.92 and r_01 > 0.92, (r_big0, r_big1, r_01)
    assert_bits_equal(big, model.a.data.cpu())  # probing left the parameters alone


@pytest.mark.parametrize("kind", ["diloco", "local_sgd"])
def test_sync_with_placed_buffers_matches_the_checker(device, kind, monkeypatch):
    """A model large enough for placement to engage: two syncs through the API, results
    against the checker bit for bit, and the same again with placement switched off."""
    results = {}
    for placement in ("1", "0"):
        monkeypatch.setenv("TORCHFT_AMD_HBM_PLACEMENT", placement)
        torch.manual_seed(0)
        model = Wide().to(device)
        peer = [p.data + 1e-3 for p in model.parameters()]
        index = {p.data_ptr(): i for i, p in enumerate(model.parameters())}
        pg = ProcessGroupLocalReplicas(0, 2, peer_lookup=lambda t: [peer[index[t.data_ptr()]]])
        manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                          use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
        inner = optim.SGD(model.parameters(), lr=0.1)
        outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
        ctx = (DiLoCo(manager, model, inner, outer, sync_every=10 ** 9) if kind == "diloco"
               else LocalSGD(manager, model, inner, sync_every=10 ** 9))
        if kind == "diloco" and placement == "0":
            assert ctx._placed_momentum is None  # switched off: the default allocation
        backup = [b.cpu() for b in ctx._backup_parameters.values()]
        bufs = None
        with ctx:
            for step in range(2):
                with torch.no_grad():
                    for p in model.parameters():
                        p.add_(1e-3 * (step + 1))
                reps = [[p.data.cpu() for p in model.parameters()], [t.cpu() for t in peer]]
                if kind == "diloco":
                    want = O.diloco_perform_sync(reps, backup, bufs, [True, True], 2, True, lr=0.7,
                                                 momentum=0.9, nesterov=True)
                else:
                    want = O.localsgd_perform_sync(reps, backup, [True, True], 2, True)
                ctx.sync()
                torch.cuda.synchronize()
                for i, p in enumerate(model.parameters()):
                    assert_bits_equal(p.data, want["params"][i], f"params[{i}] step {step}")
                for i, b in enumerate(ctx._backup_parameters.values()):
                    assert_bits_equal(b, want["backup"][i], f"backup[{i}] step {step}")
                if kind == "diloco":
                    for i, p in enumerate(model.parameters()):
                        assert_bits_equal(outer.state[p]["momentum_buffer"], want["momentum"][i])
                    bufs = want["momentum"]
                backup = want["backup"]
        results[placement] = [p.data.cpu() for p in model.parameters()]
        manager.shutdown(wait=False)
        del model, peer, ctx, outer, inner
        torch.cuda.empty_cache()
    for x, y in zip(results["1"], results["0"]):
        assert_bits_equal(x, y)


def _construct(model, device, kind="diloco", peer=None):
    if peer is None:
        peer = [p.data + 1e-3 for p in model.parameters()]
    index = {p.data_ptr(): i for i, p in enumerate(model.parameters())}
    pg = ProcessGroupLocalReplicas(0, 2, peer_lookup=lambda t: [peer[index[t.data_ptr()]]])
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                      use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    if kind == "diloco":
        outer = optim.SGD(model.parameters(), lr=0.7, momentum=0.9, nesterov=True)
        return DiLoCo(manager, model, inner, outer, sync_every=10 ** 9), manager, peer
    return LocalSGD(manager, model, inner, sync_every=10 ** 9), manager, peer


def test_a_second_construction_finds_the_groups_already_known(device):
    """What the first search learnt about the device stays: the anchors are kept, and the blocks
    of a dropped wrapper come back from torch's cache at addresses whose group is known.  The
    second construction measures the model's own tensors and nothing else."""
    import gc

    H.forget_devices()
    gc.collect()
    torch.cuda.empty_cache()
    torch.manual_seed(0)
    model = Wide().to(device)
    start = H.launch_count
    ctx, manager, peer = _construct(model, device)
    first = H.launch_count - start
    state = H.device_state(device)
    if ctx._placed_momentum is None:
        pytest.skip("no bank-group structure found: is this an MI355X?")
    assert state.searches == 1 and len(state.map.anchors) >= 2
    assert state.last_search["blocks_probed"] >= 2 and state.last_search["probe_launches"] == first
    first_search = dict(state.last_search)
    anchors = [a.data_ptr() for a in state.map.anchors]
    # Which blocks torch's cache hands back, and in which order, depends on what the process
    # has allocated before; a construction that meets a block it has not seen measures it and
    # knows it from then on.  So: drop and construct again until nothing new turns up (once is
    # the rule, three times the limit), then hold that construction to "measured nothing".
    history = []
    for attempt in range(3):
        manager.shutdown(wait=False)
        del ctx, manager
        gc.collect()  # the wrapper's buffers go back to torch's cache, not to the driver
        start = H.launch_count
        ctx, manager, peer = _construct(model, device, peer=peer)  # nothing else is allocated in between
        second = H.launch_count - start
        assert state.searches == 2 + attempt
        assert [a.data_ptr() for a in state.map.anchors][:len(anchors)] == anchors  # the anchors are kept
        assert ctx._placed_momentum is not None
        assert state.last_search["blocks_known_by_address"] >= 1
        history.append((second, {k: v for k, v in state.last_search.items() if k != "blocks"}))
        if state.last_search["blocks_probed"] == 0:
            break
    # nothing had to be measured again: the model's tensors and the blocks are known by address
    assert state.last_search["blocks_probed"] == 0, (first_search, history)
    assert second < 0.1 * first, (first, history)
    # and the buffers still lie outside the model's group
    big, copy0 = model.a.data, ctx._backup_parameters["a"]
    half = copy0.numel() // 2
    for attempt in range(3):
        same = H.probe_ms(copy0[:half], copy0[half:], 256 << 20, repeats=6)
        ratio = H.probe_ms(big, copy0, 256 << 20, repeats=6) / same
        if ratio < 0.92:
            break
    assert ratio < 0.92, ratio
    manager.shutdown(wait=False)


def test_two_replicas_constructing_at_once_take_turns(device):
    """Two thread-replicas on one GPU build their wrappers at the same time: the searches run
    one after the other under the device's lock, both get placed buffers that do not overlap,
    and a sync of each equals the checker."""
    import threading

    torch.manual_seed(0)
    models = [Wide().to(device) for _ in range(2)]
    built = [None, None]
    errors = []

    def build(k):
        try:
            with torch.cuda.device(device):
                built[k] = _construct(models[k], device, "local_sgd")
        except Exception as e:  # surfaced below
            errors.append(e)

    threads = [threading.Thread(target=build, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    spans = []
    for ctx, _, _ in built:
        for b in ctx._backup_parameters.values():
            spans.append((b.data_ptr(), b.data_ptr() + b.numel() * b.element_size()))
    spans.sort()
    assert all(a_end <= b_start for (_, a_end), (b_start, _) in zip(spans, spans[1:])), "buffers overlap"
    for k, (ctx, manager, peer) in enumerate(built):
        backup = [b.cpu() for b in ctx._backup_parameters.values()]
        reps = [[p.data.cpu() for p in models[k].parameters()], [t.cpu() for t in peer]]
        want = O.localsgd_perform_sync(reps, backup, [True, True], 2, True)
        ctx.sync()
        torch.cuda.synchronize()
        for i, p in enumerate(models[k].parameters()):
            assert_bits_equal(p.data, want["params"][i], f"replica {k} params[{i}]")
        manager.shutdown(wait=False)


def test_momentum_set_aside_for_a_fused_step_is_released_when_the_step_is_not_fused(device):
    """The outer momentum is allocated with the backup when the outer optimizer looks like a
    fusable SGD.  If it then is not (here: a tensor learning rate), the optimizer's own step()
    runs and creates its own state: the buffers set aside must not stay allocated."""
    torch.manual_seed(0)
    model = Wide().to(device)
    peer = [p.data + 1e-3 for p in model.parameters()]
    index = {p.data_ptr(): i for i, p in enumerate(model.parameters())}
    pg = ProcessGroupLocalReplicas(0, 2, peer_lookup=lambda t: [peer[index[t.data_ptr()]]])
    manager = Manager(pg=pg, load_state_dict=None, state_dict=None, min_replica_size=2,
                      use_async_quorum=False, quorum_client=StaticQuorum(0, 2))
    inner = optim.SGD(model.parameters(), lr=0.1)
    outer = optim.SGD(model.parameters(), lr=torch.tensor(0.7), momentum=0.9, nesterov=True)
    ctx = DiLoCo(manager, model, inner, outer, sync_every=10 ** 9)
    if ctx._placed_momentum is None:
        pytest.skip("no bank-group structure found: is this an MI355X?")
    set_aside = ctx._placed_momentum[0].data_ptr()
    with ctx:
        with torch.no_grad():
            for p in model.parameters():
                p.add_(1e-3)
        ctx.sync()
    torch.cuda.synchronize()
    assert ctx._placed_momentum is None
    # the optimizer made its own buffers; ours are not among them
    assert all(outer.state[p]["momentum_buffer"].data_ptr() != set_aside for p in model.parameters())
    for p, b in zip(model.parameters(), ctx._backup_parameters.values()):
        assert_bits_equal(p.data, b)
    manager.shutdown(wait=False)
