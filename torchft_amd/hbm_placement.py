"""Placement of the library's own buffers in HBM, by bank group.

MI355X's HBM3E is addressed as three groups of banks of 96 GiB each; every
group is a contiguous range of physical memory.  Streams that are WRITTEN
concurrently slow each other down when they lie in the same group: a pair of
in-place (read + write) streams runs at 5.6 TB/s inside one group against
6.4 TB/s across two, two pure write streams at 5.8 against 7.1 TB/s, and a
LocalSGD average whose parameters and backup share a group at 0.79 of the
8 TB/s peak against 0.85 when they do not.  Read-only streams do not care.

The replica-sync kernels write the live parameters, the backup and the outer
momentum at the same element offsets at the same time.  Measured over the
assignments of the streams to groups (fused DiLoCo step, parameters updated in
place): everything in one group 0.77 of peak - which is exactly what a model of
up to 32 GB gets when its backup and momentum are allocated right behind it -
against 0.80 as soon as backup and momentum lie outside the parameters' group;
keeping them TOGETHER in one other group is as good as or better than splitting
them over the two remaining groups.  For the LocalSGD average the same move is
worth 0.79 -> 0.85.  The parameters are the user's; the backup and momentum
buffers are allocated here, so this module

* finds out which group a piece of device memory lies in.  Virtual addresses
  say nothing about it, and there is no query for it; what tells is time: the
  probe kernel (``tft_probe_rw_pair``) rewrites a buffer in place, unchanged,
  while copying it into a scratch buffer, and runs 18-20 % longer when both lie
  in one group;
* hands out per-tensor buffers from blocks of device memory whose group is
  known (:class:`GroupedPool`): every tensor's backup and momentum in the group
  after its parameter's.

Nothing here affects results: a wrong or impossible placement only costs
bandwidth.  ``TORCHFT_AMD_HBM_PLACEMENT=0`` switches the probing off, and it is
skipped by itself for models too small to matter or when the timings show no
group structure (other GPUs).
"""

from __future__ import annotations

import ctypes
import logging
import os
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from . import _native
from .multi_tensor import current_stream_handle

logger: logging.Logger = logging.getLogger(__name__)

N_GROUPS = 3
PROBE_BYTES = 512 << 20      # per buffer and probe: long enough to time reliably (0.3 ms), short enough to be free
MIN_PROBE_BYTES = 128 << 20  # tensors below this are not probed (they take their neighbour's group)
BLOCK_BYTES = 2 << 30        # device memory is taken from torch in blocks of this size
BLOCK_GRANULE = 1 << 30      # ... or of the largest tensor's size rounded up to this, if that is more
# probe time / time of a same-group pair: 0.97-1.05 measured inside one group, 0.83-0.85
# across two (probes of 128 MiB and more)
SAME_GROUP_RATIO = 0.92
AMBIGUOUS_BAND = 0.03        # a ratio this close to the threshold is measured again
RELATIVE_CONTRAST = 1.06     # own-group probe time / next longest, with all three anchors known
NO_STRUCTURE_BYTES = 110 << 30  # this much memory in ONE group: the device has no such groups
MIN_MODEL_BYTES = 256 << 20  # smaller models are left alone (a GPT-2-small of 0.5 GB still gains 1-2 %)
ALIGN = 256


def enabled() -> bool:
    return os.environ.get("TORCHFT_AMD_HBM_PLACEMENT", "1") not in ("0", "false", "off")


def _as_bytes(t: torch.Tensor) -> torch.Tensor:
    return t.detach().reshape(-1).view(torch.uint8)


def probe_ms(a: torch.Tensor, b: torch.Tensor, nbytes: Optional[int] = None, repeats: int = 3) -> float:
    """Shortest of ``repeats`` timings of the pair probe over the first ``nbytes`` bytes of
    ``a`` and ``b`` (default: as much as both hold, at most PROBE_BYTES).  ``a`` keeps its
    contents (nothing else may touch it meanwhile); ``b`` is scratch and is overwritten."""
    a8, b8 = _as_bytes(a), _as_bytes(b)
    n = min(a8.numel(), b8.numel(), PROBE_BYTES if nbytes is None else nbytes)
    # 16-byte alignment of both ends
    a_off = (-a8.data_ptr()) % 16
    b_off = (-b8.data_ptr()) % 16
    n = (n - max(a_off, b_off)) // 16 * 16
    if n <= 0:
        raise ValueError("buffers too small to probe")
    lib = _native.lib()
    stream = current_stream_handle(a.device)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    with torch.cuda.device(a.device):
        for _ in range(repeats + 1):  # the first one warms up
            start.record()
            rc = lib.tft_probe_rw_pair(a8.data_ptr() + a_off, b8.data_ptr() + b_off, n, stream)
            _native.check(rc, "tft_probe_rw_pair")
            stop.record()
            stop.synchronize()
            best = min(best, start.elapsed_time(stop))
    return best


@dataclass
class _Block:
    storage: torch.Tensor  # uint8, BLOCK_BYTES (or larger for a tensor that needs it)
    group: int
    used: int = 0

    def free(self) -> int:
        return self.storage.numel() - self.used


@dataclass
class GroupMap:
    """One anchor buffer per bank group found so far, and the time a same-group pair takes."""

    device: torch.device
    anchors: List[torch.Tensor] = field(default_factory=list)
    same_ms: Dict[int, float] = field(default_factory=dict)   # probe size -> same-group time

    def _same_ms(self, nbytes: int) -> float:
        """Time of a pair that certainly shares a group: the two halves of anchor 0."""
        key = nbytes
        if key not in self.same_ms:
            a = self.anchors[0]
            half = a.numel() // 2 // 16 * 16
            n = min(nbytes, half)
            t = min(probe_ms(a[:half], a[half:], n, repeats=5) for _ in range(2))
            # scale to the requested size if the anchor is shorter than the probe
            self.same_ms[key] = t * (nbytes / n)
        return self.same_ms[key]

    def group_of(self, t: torch.Tensor, nbytes: Optional[int] = None) -> Optional[int]:
        """Index of the anchor whose group ``t`` shares, or None if it shares none of the known
        ones (an unseen group) - or if ``t`` is too small to tell.

        Once an anchor of every group is known the decision is relative: the probe against
        the anchor of ``t``'s own group takes clearly longer than against the other two,
        whatever constant a profiler or a busy host adds to every launch.  Before that, the
        probe times are compared with the time of a pair that certainly shares a group.
        An unclear measurement is repeated with more launches."""
        size = _as_bytes(t).numel()
        n = min(size, PROBE_BYTES if nbytes is None else nbytes) // 16 * 16
        if n < MIN_PROBE_BYTES or not self.anchors:
            return None
        for repeats in (3, 6, 9):
            times = [probe_ms(t, anchor, n, repeats) for anchor in self.anchors]
            best = max(range(len(times)), key=lambda k: times[k])
            if len(self.anchors) >= N_GROUPS:
                second = max(x for k, x in enumerate(times) if k != best)
                contrast = times[best] / second
                if contrast > RELATIVE_CONTRAST:
                    return best
                continue  # no anchor stands out: measure again
            ratio = times[best] / self._same_ms(n)
            if abs(ratio - SAME_GROUP_RATIO) > AMBIGUOUS_BAND:
                return best if ratio > SAME_GROUP_RATIO else None
        if len(self.anchors) >= N_GROUPS:
            return None
        return best if ratio > SAME_GROUP_RATIO else None


class GroupedPool:
    """Device memory in blocks of known bank group, handed out tensor by tensor.

    Blocks come from torch's allocator (so they are accounted for and returned like any
    other tensor): ``grow_until`` takes them, ``take`` carves tensors out of them,
    ``release_unused`` returns the untouched ones.
    """

    def __init__(
        self,
        device: torch.device,
        allocate: Optional[Callable[[int], torch.Tensor]] = None,
        free_memory: Optional[Callable[[], int]] = None,
        release: Optional[Callable[[], None]] = None,
    ) -> None:
        self.device = device
        self.map = GroupMap(device)
        self.blocks: List[_Block] = []
        self._straddling: List[torch.Tensor] = []  # blocks across a group boundary: held, unused
        self.structured = True  # False once the timings show no group structure
        # where blocks come from and go back to (replaceable: the search logic is host code
        # and is tested without a GPU)
        self._allocate = allocate or (lambda n: torch.empty(n, dtype=torch.uint8, device=device))
        self._free_memory = free_memory or (lambda: torch.cuda.mem_get_info(device)[0])
        self._release = release or torch.cuda.empty_cache
        self.keep_free = 6 << 30  # device memory the search never touches

    # -- discovery ---------------------------------------------------------------
    def _classify_block(self, storage: torch.Tensor) -> Optional[int]:
        """Group of a fresh block (a new anchor is made of it if its group is new); None if
        the block straddles two groups."""
        m = self.map
        if not m.anchors:
            m.anchors.append(storage[:PROBE_BYTES])
            return 0
        n = storage.numel()
        ends = []
        for piece in (storage[:PROBE_BYTES], storage[n - PROBE_BYTES:]):
            g = m.group_of(piece)
            if g is None:
                if len(m.anchors) >= N_GROUPS or not self._clearly_new(storage):
                    return None  # matches no group clearly: leave it alone
                m.anchors.append(piece)
                g = len(m.anchors) - 1
            ends.append(g)
        return ends[0] if ends[0] == ends[1] else None

    def _clearly_new(self, storage: torch.Tensor) -> bool:
        """A second, longer measurement before a block founds a new group: an anchor that in
        truth lies in a known group would make every later block of that group unclassifiable."""
        m = self.map
        n = min(storage.numel(), 2 * PROBE_BYTES) // 16 * 16
        same = m._same_ms(n)
        return all(probe_ms(storage, anchor, n, repeats=9) / same < SAME_GROUP_RATIO - AMBIGUOUS_BAND
                   for anchor in m.anchors)

    def free_bytes(self, group: int) -> int:
        return sum(b.free() for b in self.blocks if b.group == group)

    def grow_until(self, satisfied, keep_free: Optional[int] = None, block_bytes: Optional[int] = None) -> bool:
        """Takes blocks from the device, one at a time, until ``satisfied(self)`` holds; False if
        the device ran out first.  Every block that lies in one group is kept as a candidate
        (the driver hands physical memory out in address order, so the way to the next group
        leads through the rest of the current one: what is not wanted must be held, not
        returned, until the search is over - ``release_unused`` gives it back)."""
        keep_free = self.keep_free if keep_free is None else keep_free
        block_bytes = BLOCK_BYTES if block_bytes is None else block_bytes
        while not satisfied(self):
            if self._free_memory() < keep_free + block_bytes:
                logger.info("hbm placement: device memory ran out before the search was satisfied")
                return False
            storage = self._allocate(block_bytes)
            g = self._classify_block(storage)
            if g is None:
                self._straddling.append(storage)
            else:
                self.blocks.append(_Block(storage, g))
            if len(self.map.anchors) == 1 and len(self.blocks) * block_bytes > NO_STRUCTURE_BYTES:
                # more than a whole group's worth of memory and still one group: this
                # device shows no group structure
                self.structured = False
                return False
        return True

    # -- hand-out ------------------------------------------------------------------
    def take(self, nbytes: int, groups: Sequence[int]) -> Optional[torch.Tensor]:
        """``nbytes`` bytes (256-byte aligned) from the first group of ``groups`` that has
        room; None if none has."""
        for g in groups:
            for b in self.blocks:
                if b.group != g:
                    continue
                start = -(-b.used // ALIGN) * ALIGN
                if start + nbytes <= b.storage.numel():
                    b.used = start + nbytes
                    return b.storage[start:start + nbytes]
        return None

    def reset(self) -> None:
        """Forgets everything handed out (the caller has dropped those tensors)."""
        for b in self.blocks:
            b.used = 0

    def release_unused(self) -> None:
        """Gives every block nothing was taken from back to the device."""
        self.blocks = [b for b in self.blocks if b.used > 0]
        self._straddling = []
        self._release()


def groups_of_tensors(pool: GroupedPool, tensors: Sequence[torch.Tensor]) -> List[Optional[int]]:
    """Bank group of every tensor (against the pool's anchors); tensors too small to probe
    take the group of the nearest probed tensor by address."""
    out: List[Optional[int]] = [None] * len(tensors)
    probed: List[Tuple[int, int]] = []  # (address, group)
    for i, t in enumerate(tensors):
        if _as_bytes(t).numel() >= MIN_PROBE_BYTES:
            g = pool.map.group_of(t)
            out[i] = g
            if g is not None:
                probed.append((t.data_ptr(), g))
    if probed:
        for i, t in enumerate(tensors):
            if out[i] is None and _as_bytes(t).numel() < MIN_PROBE_BYTES:
                addr = t.data_ptr()
                out[i] = min(probed, key=lambda ag: abs(ag[0] - addr))[1]
    return out


def allocate_apart(
    like: Sequence[torch.Tensor], n_copies: int
) -> Optional[List[List[torch.Tensor]]]:
    """``n_copies`` (1 or 2) sets of uninitialised tensors shaped like ``like``, every tensor
    of every copy in the bank group after its model tensor's: group (g + 1) mod 3, where g
    is the group of the corresponding tensor of ``like``; what does not fit there goes to
    group (g + 2) mod 3, and only then to g itself.  Returns None when placement does not
    apply (switched off, not on a GPU, model too small, no group structure found); the
    caller then allocates as it always did."""
    if not enabled() or not like or n_copies not in (1, 2):
        return None
    device = like[0].device
    if device.type != "cuda" or any(t.device != device for t in like):
        return None
    sizes = [t.numel() * t.element_size() for t in like]
    if sum(sizes) < MIN_MODEL_BYTES:
        return None
    try:
        return _allocate_apart(like, sizes, n_copies, device)
    except Exception as e:  # placement is an optimisation: never let it fail an allocation
        logger.warning("hbm placement gave up (%s); default allocation", e)
        torch.cuda.empty_cache()
        return None


def _allocate_apart(
    like: Sequence[torch.Tensor], sizes: List[int], n_copies: int, device: torch.device,
    pool: Optional[GroupedPool] = None,
) -> Optional[List[List[torch.Tensor]]]:
    if pool is None:
        torch.cuda.synchronize(device)
        pool = GroupedPool(device)
    largest = max(sizes)
    block = max(BLOCK_BYTES, -(-largest // BLOCK_GRANULE) * BLOCK_GRANULE)
    # first: reach all groups, so that there is an anchor to compare the model with in each
    pool.grow_until(lambda pl: len(pl.map.anchors) >= N_GROUPS, block_bytes=block)
    if not pool.structured or len(pool.map.anchors) < 2:
        logger.info("hbm placement: no bank-group structure found on %s; default allocation", device)
        pool.release_unused()
        return None
    n_groups = len(pool.map.anchors)
    groups = groups_of_tensors(pool, like)
    need: Dict[int, int] = {g: 0 for g in range(n_groups)}
    wanted: List[List[int]] = []
    for size, g in zip(sizes, groups):
        g0 = 0 if g is None else g
        row = [(g0 + 1) % n_groups] * n_copies
        wanted.append(row)
        for w in row:
            need[w] += -(-size // ALIGN) * ALIGN
    # head room for blocks that cannot be filled to the last byte
    need = {g: n + block for g, n in need.items() if n > 0}
    pool.grow_until(lambda pl: all(pl.free_bytes(g) >= n for g, n in need.items()), block_bytes=block)
    copies: List[List[torch.Tensor]] = [[] for _ in range(n_copies)]
    order = sorted(range(len(like)), key=lambda i: -sizes[i])  # large tensors first: they pack better
    placed: Dict[Tuple[int, int], Optional[torch.Tensor]] = {}
    misplaced = 0
    for i in order:
        for k in range(n_copies):
            prefer = wanted[i][k]
            others = [(prefer + 1) % n_groups, (prefer + 2) % n_groups][: n_groups - 1]
            raw = pool.take(sizes[i], [prefer]) if sizes[i] else None
            if raw is None and sizes[i]:
                raw = pool.take(sizes[i], others)
                misplaced += 1
            placed[(i, k)] = raw
    # everything the search held but did not use goes back BEFORE anything else is allocated:
    # what found no room in the pool must not fail for memory the pool itself is sitting on
    pool.release_unused()
    for (i, k), raw in list(placed.items()):
        if raw is None:
            raw = pool._allocate(max(sizes[i], 1))[: sizes[i]]
        placed[(i, k)] = raw.view(like[i].dtype).view(like[i].shape)
    for k in range(n_copies):
        copies[k] = [placed[(i, k)] for i in range(len(like))]
    logger.info(
        "hbm placement: %d tensors x %d copies over %d bank groups (%d not in their preferred group)",
        len(like), n_copies, n_groups, misplaced,
    )
    return copies


def model_copies(like: Sequence[torch.Tensor], n_copies: int) -> List[List[torch.Tensor]]:
    """``n_copies`` sets of uninitialised tensors shaped like ``like``: placed by bank group
    where that applies (:func:`allocate_apart`), otherwise one plain allocation per tensor."""
    placed = allocate_apart(like, n_copies) if n_copies in (1, 2) else None
    if placed is not None:
        return placed
    return [[torch.empty_like(t) for t in like] for _ in range(n_copies)]
