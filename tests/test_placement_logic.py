"""The bank-group search of torchft_amd.hbm_placement as host logic, without a GPU: device
memory is one host arena whose byte ranges are assigned to three fake bank groups, and the
probe is a function of the two buffers' groups (plus noise), as the real timings are."""

import random

import pytest
import torch

from torchft_amd import hbm_placement as H

MiB = 1 << 20


class FakeDevice:
    """A bump allocator over one arena.  Like the GPU driver it hands memory out in address
    order; every ``group_bytes`` the next bank group starts."""

    def __init__(self, total=96 * MiB, group_bytes=24 * MiB, n_groups=3, noise=0.0, seed=0):
        self.arena = torch.zeros(total, dtype=torch.uint8)
        self.base = self.arena.data_ptr()
        self.total, self.group_bytes, self.n_groups = total, group_bytes, n_groups
        self.cursor = 0
        self.noise, self.rng = noise, random.Random(seed)
        self.released = 0
        self.probes = 0

    def allocate(self, nbytes: int) -> torch.Tensor:
        start = -(-self.cursor // 256) * 256
        if start + nbytes > self.total:
            raise RuntimeError("fake device out of memory")
        self.cursor = start + nbytes
        return self.arena[start:start + nbytes]

    def free_memory(self) -> int:
        return self.total - self.cursor

    def release(self) -> None:
        self.released += 1

    def group_at(self, t: torch.Tensor, last: bool = False) -> int:
        off = t.data_ptr() - self.base + (t.numel() * t.element_size() - 1 if last else 0)
        return (off // self.group_bytes) % self.n_groups

    def probe_ms(self, a, b, nbytes=None, repeats=3):
        self.probes += 1
        n = min(a.numel() * a.element_size(), b.numel() * b.element_size(), nbytes or H.PROBE_BYTES)
        same = self.group_at(a) == self.group_at(b)
        ms = (1.0 if same else 0.83) * n / MiB
        return ms * (1.0 + self.rng.uniform(-self.noise, self.noise)) + 0.0


@pytest.fixture
def small_constants(monkeypatch):
    monkeypatch.setattr(H, "PROBE_BYTES", 256 << 10)
    monkeypatch.setattr(H, "MIN_PROBE_BYTES", 64 << 10)
    monkeypatch.setattr(H, "BLOCK_BYTES", 1 * MiB)
    monkeypatch.setattr(H, "BLOCK_GRANULE", 1 * MiB)
    monkeypatch.setattr(H, "NO_STRUCTURE_BYTES", 40 * MiB)


def make_pool(dev: FakeDevice, monkeypatch, state=None) -> H.GroupedPool:
    monkeypatch.setattr(H, "probe_ms", dev.probe_ms)
    pool = H.GroupedPool(torch.device("cpu"), allocate=dev.allocate, free_memory=dev.free_memory,
                         release=dev.release, state=state, epoch=lambda: dev.released)
    pool.keep_free = 2 * MiB
    pool.limit = dev.total  # the allowance has a test of its own
    return pool


def model_on(dev: FakeDevice, sizes):
    return [dev.allocate(n * 4).view(torch.float32) for n in sizes]


@pytest.mark.parametrize("noise", [0.0, 0.015])
def test_blocks_are_classified_and_buffers_land_in_the_next_group(small_constants, monkeypatch, noise):
    dev = FakeDevice(noise=noise, seed=3)
    # a model of 6 MiB at the start of group 0: two probe-sized tensors and small ones
    like = model_on(dev, [MiB // 2, 1000, MiB // 2, 10, 300_000])
    pool = make_pool(dev, monkeypatch)
    sizes = [t.numel() * 4 for t in like]
    copies = H._allocate_apart(like, sizes, 2, torch.device("cpu"), pool=pool)
    assert copies is not None and len(copies) == 2
    # the search stops as soon as the group after the model's holds what is needed: the third
    # group is never visited
    assert len(pool.map.anchors) == 2
    seen = []
    for copy in copies:
        for t, ref in zip(copy, like):
            assert t.shape == ref.shape and t.dtype == ref.dtype
            assert (t.data_ptr() - dev.base) % 256 == 0
            # entirely inside the group after the model's
            assert dev.group_at(t) == dev.group_at(t, last=True) == (dev.group_at(ref) + 1) % 3
            seen.append((t.data_ptr(), t.data_ptr() + t.numel() * 4))
    seen.sort()
    assert all(a_end <= b_start for (_, a_end), (b_start, _) in zip(seen, seen[1:])), "buffers overlap"
    assert dev.released >= 1  # what the search held and did not use went back
    # what is left holds tensors; the two anchors are allocations of their own, outside any block
    assert all(b.used > 0 for b in pool.blocks)
    assert pool.state.anchor_blocks == []
    for a in pool.map.anchors:
        lo = a.data_ptr()
        assert all(not (b.storage.data_ptr() <= lo < b.storage.data_ptr() + b.storage.numel())
                   for b in pool.blocks)


def test_a_model_across_two_groups_gets_each_tensor_its_own_neighbour(small_constants, monkeypatch):
    dev = FakeDevice(group_bytes=8 * MiB, total=64 * MiB)
    like = model_on(dev, [MiB] * 3)  # 4 MiB each: tensors 0, 1 in group 0, tensor 2 in group 1
    assert [dev.group_at(t) for t in like] == [0, 0, 1]
    pool = make_pool(dev, monkeypatch)
    copies = H._allocate_apart(like, [t.numel() * 4 for t in like], 1, torch.device("cpu"), pool=pool)
    got = [dev.group_at(t) for t in copies[0]]
    # every copy outside its own tensor's group, each in one group; the two tensors that share a
    # group get the same other group
    assert all(g != own for g, own in zip(got, [0, 0, 1]))
    assert got[0] == got[1]
    assert all(dev.group_at(t) == dev.group_at(t, last=True) for t in copies[0])


def test_a_block_across_a_boundary_is_held_but_never_used(small_constants, monkeypatch):
    dev = FakeDevice(group_bytes=8 * MiB + 512 * 1024, total=64 * MiB)  # boundaries inside blocks
    like = model_on(dev, [MiB // 2])
    pool = make_pool(dev, monkeypatch)
    copies = H._allocate_apart(like, [like[0].numel() * 4], 2, torch.device("cpu"), pool=pool)
    assert copies is not None
    for copy in copies:
        t = copy[0]
        assert dev.group_at(t) == dev.group_at(t, last=True) != dev.group_at(like[0])
    for b in pool.blocks:
        assert dev.group_at(b.storage) == dev.group_at(b.storage, last=True)


def test_a_device_without_groups_is_left_alone(small_constants, monkeypatch):
    dev = FakeDevice(n_groups=1, total=64 * MiB)
    like = model_on(dev, [MiB // 2])
    pool = make_pool(dev, monkeypatch)
    assert H._allocate_apart(like, [like[0].numel() * 4], 1, torch.device("cpu"), pool=pool) is None
    # nothing is kept on such a device, not even the one reference buffer
    assert not pool.structured and pool.map.anchors == [] and pool.state.anchor_blocks == []
    assert pool.blocks == [] and dev.released >= 1


def test_running_out_of_memory_falls_back_to_the_other_groups(small_constants, monkeypatch):
    # the device ends inside group 1 (there is no group 2 to be found): what does not fit there
    # goes to whatever other block the search holds, and what fits nowhere in the pool is
    # allocated plainly once the pool has given its unused blocks back
    class Spilling(FakeDevice):
        """A bump allocator cannot take memory back; what a real device would serve from the
        returned blocks comes from outside the arena here."""

        def allocate(self, nbytes):
            try:
                return super().allocate(nbytes)
            except RuntimeError:
                if not self.released:
                    raise
                self.spilled = getattr(self, "spilled", 0) + 1
                return torch.zeros(nbytes, dtype=torch.uint8)

    dev = Spilling(group_bytes=8 * MiB, total=15 * MiB)
    like = model_on(dev, [MiB * 3 // 8] * 4)  # 4 x 1.5 MiB = 6 MiB in group 0
    pool = make_pool(dev, monkeypatch)
    pool.keep_free = 0
    sizes = [t.numel() * 4 for t in like]
    copies = H._allocate_apart(like, sizes, 1, torch.device("cpu"), pool=pool)
    assert copies is not None and len(pool.map.anchors) == 2
    inside = [t for t in copies[0] if dev.base <= t.data_ptr() < dev.base + dev.total]
    assert sum(dev.group_at(t) == 1 for t in inside) >= 2  # group 1 first, for as long as it has room
    assert len(inside) + getattr(dev, "spilled", 0) == len(like)
    for t, ref in zip(copies[0], like):
        assert t.shape == ref.shape
    for t in inside:
        assert dev.group_at(t) == dev.group_at(t, last=True)


def test_small_tensors_take_the_group_of_their_nearest_probed_neighbour(small_constants, monkeypatch):
    dev = FakeDevice(group_bytes=8 * MiB, total=64 * MiB)
    a = dev.allocate(512 << 10).view(torch.float32)       # group 0, probed
    small0 = dev.allocate(1000).view(torch.uint8)           # next to it
    dev.cursor = 9 * MiB
    b = dev.allocate(512 << 10).view(torch.float32)       # group 1, probed
    small1 = dev.allocate(1000).view(torch.uint8)
    pool = make_pool(dev, monkeypatch)
    pool.grow_until(lambda pl: len(pl.map.anchors) >= 3)
    groups = H.groups_of_tensors(pool, [a, small0, b, small1])
    assert groups[0] == groups[1] and groups[2] == groups[3] and groups[0] != groups[2]


def test_allocate_apart_declines_what_it_cannot_help(monkeypatch):
    cpu = [torch.zeros(10)]
    assert H.allocate_apart(cpu, 1) is None            # not on a GPU
    assert H.allocate_apart([], 1) is None
    assert H.allocate_apart(cpu, 3) is None            # one or two copies only
    monkeypatch.setenv("TORCHFT_AMD_HBM_PLACEMENT", "0")
    assert not H.enabled()
    copies = H.model_copies(cpu, 2)                    # plain allocations instead
    assert len(copies) == 2 and copies[0][0].shape == cpu[0].shape


# ---------------------------------------------------------------------------
# What a device's state keeps between searches
# ---------------------------------------------------------------------------

def search(dev, state, like, n_copies, monkeypatch, limit=None):
    def factory(st):
        pool = make_pool(dev, monkeypatch, state=st)
        if limit is not None:
            pool.limit = limit
        factory.pools.append(pool)
        return pool

    factory.pools = []
    sizes = [t.numel() * 4 for t in like]
    copies = H._locked_search(state, like, sizes, n_copies, torch.device("cpu"), make_pool=factory)
    return copies, factory.pools[-1] if factory.pools else None


def test_a_second_search_reuses_the_anchors_of_the_first(small_constants, monkeypatch):
    dev = FakeDevice(total=160 * MiB, group_bytes=32 * MiB)
    like = model_on(dev, [MiB // 2, MiB // 2, 1000])
    state = H.DeviceState(torch.device("cpu"))
    first, pool1 = search(dev, state, like, 2, monkeypatch)
    probes_first = dev.probes
    anchors = [a.data_ptr() for a in state.map.anchors]
    assert first is not None and len(anchors) == 2 and state.searches == 1
    second, pool2 = search(dev, state, like, 1, monkeypatch)
    assert second is not None and state.searches == 2
    assert [a.data_ptr() for a in state.map.anchors][:2] == anchors  # nothing was rediscovered
    # the second search never measured a same-group reference pair again, and it found the
    # groups' reference buffers in place: it only classified blocks and the model sample
    assert pool2.map is pool1.map
    for t, ref in zip(second[0], like):
        assert dev.group_at(t) == dev.group_at(t, last=True) != dev.group_at(ref)
    spans = sorted((t.data_ptr(), t.data_ptr() + t.numel() * 4) for col in (*first, *second) for t in col)
    assert all(a_end <= b_start for (_, a_end), (b_start, _) in zip(spans, spans[1:])), "buffers overlap"
    assert dev.probes - probes_first < probes_first


def test_blocks_known_by_address_are_not_probed_again(small_constants, monkeypatch):
    """Blocks a dropped wrapper returns to torch's cache come back at the same addresses: as long
    as the allocator has given nothing back to the driver they are known without a probe."""

    class Recycling(FakeDevice):
        """Hands previously returned blocks out again first, like torch's caching allocator."""

        def __init__(self, *a, **k):
            super().__init__(*a, **k)
            self.cache = []

        def allocate(self, nbytes):
            for i, t in enumerate(self.cache):
                if t.numel() == nbytes:
                    return self.cache.pop(i)
            return super().allocate(nbytes)

    dev = Recycling(total=160 * MiB, group_bytes=32 * MiB)
    like = model_on(dev, [MiB // 2, MiB // 2])
    state = H.DeviceState(torch.device("cpu"))
    first, pool1 = search(dev, state, like, 2, monkeypatch)
    probes_first = dev.probes
    blocks = [b.storage for b in pool1.blocks if b.used > 0 and b not in state.anchor_blocks]
    assert blocks
    del first
    dev.cache = list(blocks)  # the wrapper died: its blocks are cached, nothing went to the driver
    second, pool2 = search(dev, state, like, 2, monkeypatch)
    assert second is not None and pool2.cache_hits >= 1
    # only the model sample was measured
    assert dev.probes - probes_first <= 0.25 * probes_first
    # ... but once memory has gone back to the driver the addresses are forgotten
    dev.released += 1
    pool3 = make_pool(dev, monkeypatch, state=state)
    assert state.known == {} and pool3.cache_hits == 0


def test_two_threads_search_one_at_a_time(small_constants, monkeypatch):
    import threading

    dev = FakeDevice(total=256 * MiB, group_bytes=48 * MiB)
    busy = threading.Lock()
    overlaps = []
    plain = dev.probe_ms

    def exclusive_probe(a, b, nbytes=None, repeats=3):
        if not busy.acquire(blocking=False):
            overlaps.append(1)
            return plain(a, b, nbytes, repeats)
        try:
            return plain(a, b, nbytes, repeats)
        finally:
            busy.release()

    dev.probe_ms = exclusive_probe
    models = [model_on(dev, [MiB // 2, MiB // 2, 100]) for _ in range(2)]
    state = H.DeviceState(torch.device("cpu"))
    results = [None, None]

    def construct(k):
        results[k] = search(dev, state, models[k], 2, monkeypatch)[0]

    threads = [threading.Thread(target=construct, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not overlaps, "two searches probed at the same time"
    assert all(r is not None for r in results) and state.searches == 2
    spans = sorted((t.data_ptr(), t.data_ptr() + t.numel() * 4) for r in results for col in r for t in col)
    assert all(a_end <= b_start for (_, a_end), (b_start, _) in zip(spans, spans[1:])), "buffers overlap"
    for r, like in zip(results, models):
        for col in r:
            for t, ref in zip(col, like):
                assert dev.group_at(t) != dev.group_at(ref)


def test_the_search_never_holds_more_than_its_allowance(small_constants, monkeypatch):
    dev = FakeDevice(total=160 * MiB, group_bytes=32 * MiB)
    like = model_on(dev, [MiB // 2, MiB // 2])   # 4 MiB at the start of group 0: 28 MiB to walk
    held = []
    plain = dev.allocate

    def counting(nbytes):
        t = plain(nbytes)
        held.append(nbytes)
        return t

    dev.allocate = counting
    state = H.DeviceState(torch.device("cpu"))
    copies, pool = search(dev, state, like, 2, monkeypatch, limit=10 * MiB)
    # ten blocks of 1 MiB do not reach the next group: no placement, and no more was taken
    assert copies is None
    assert sum(held) <= 10 * MiB + H.PROBE_BYTES  # the allowance, and the first anchor (which stays)
    assert state.structured  # not a verdict on the device: a later search may get further
    # with room to walk the same state carries on from its first anchor
    copies, pool = search(dev, state, like, 2, monkeypatch, limit=64 * MiB)
    assert copies is not None and len(state.map.anchors) == 2


def test_the_allowance_follows_the_environment(monkeypatch):
    assert H.search_limit_bytes(100 << 30) == 75 << 30
    monkeypatch.setenv("TORCHFT_AMD_HBM_PLACEMENT_MAX_GIB", "16")
    assert H.search_limit_bytes(100 << 30) == 16 << 30
    monkeypatch.setenv("TORCHFT_AMD_HBM_PLACEMENT_MAX_GIB", "1000")
    assert H.search_limit_bytes(100 << 30) == 75 << 30   # never more than the default share
    monkeypatch.setenv("TORCHFT_AMD_HBM_PLACEMENT_MAX_GIB", "lots")
    assert H.search_limit_bytes(100 << 30) == 75 << 30


def test_a_model_of_many_tensors_is_classified_from_a_sample(small_constants, monkeypatch):
    dev = FakeDevice(total=400 * MiB, group_bytes=100 * MiB)
    # 60 probe-able tensors of 2 MiB: 0-49 in group 0, 50-59 in group 1
    like = model_on(dev, [MiB // 2] * 60)
    truth = [dev.group_at(t) for t in like]
    assert truth.count(0) == 50 and truth.count(1) == 10
    pool = make_pool(dev, monkeypatch)
    pool.grow_until(lambda pl: len(pl.map.anchors) >= 3)
    before = dev.probes
    groups = H.groups_of_tensors(pool, like)
    measured = (dev.probes - before) / len(pool.map.anchors)
    assert measured <= 5 + 8 + 8, "a sample, one bisection and the checks, not one probe per tensor"
    names = {truth[0]: groups[0], truth[-1]: groups[-1]}
    assert [names[g] for g in truth] == groups


def test_a_model_scattered_over_the_groups_is_measured_tensor_by_tensor(small_constants, monkeypatch):
    """Parameters allocated into memory that others had used and freed can alternate between
    groups from one tensor to the next; a sample with bisection cannot see that, the checks
    in between do, and then every probe-able tensor is measured."""
    dev = FakeDevice(total=900 * MiB, group_bytes=100 * MiB)
    flat = model_on(dev, [MiB // 2] * 80)            # 0-49 in group 0, 50-79 in group 1
    like = [t for pair in zip(flat[:30], flat[50:80]) for t in pair] + flat[30:50]
    truth = [dev.group_at(t) for t in like]
    assert truth[:6] == [0, 1, 0, 1, 0, 1] and truth[-20:] == [0] * 20
    pool = make_pool(dev, monkeypatch)
    pool.grow_until(lambda pl: len(pl.map.anchors) >= 3)
    before = dev.probes
    groups = H.groups_of_tensors(pool, like)
    names = {}
    for t, g in zip(truth, groups):
        assert names.setdefault(t, g) == g, "one name per true group"
    assert len(set(names.values())) == 2
    assert (dev.probes - before) / len(pool.map.anchors) >= len(like)  # everything was measured
    # and the placement follows: every copy outside its own tensor's group
    state = pool.state
    copies = H._allocate_apart(like, [t.numel() * 4 for t in like], 1, torch.device("cpu"), pool=pool, state=state)
    assert copies is not None
    for t, c in zip(like, copies[0]):
        assert dev.group_at(c) != dev.group_at(t)


def test_a_model_without_a_tensor_long_enough_to_time_is_left_alone(monkeypatch):
    """300 MiB of parameters in tensors of 1 MiB: nothing can tell which group they lie in, so
    no search is started (and no device memory is taken for one)."""
    monkeypatch.setattr(H, "enabled", lambda: True)
    started = []
    monkeypatch.setattr(H, "_locked_search", lambda *a, **k: started.append(1))

    class OnGpu:  # what allocate_apart reads of a tensor
        device = torch.device("cuda", 0)

        def __init__(self, n):
            self.n = n

        def numel(self):
            return self.n

        def element_size(self):
            return 4

    assert H.allocate_apart([OnGpu(MiB // 4)] * 300, 2) is None and not started
    H.allocate_apart([OnGpu(MiB // 4)] * 300 + [OnGpu(64 * MiB)], 2)
    assert started == [1]
