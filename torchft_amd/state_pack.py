"""Device-side pack / unpack of a training state dict.

The reference serialises a recovering replica's state with ``torch.save`` into
the HTTP response and ``torch.load`` on the other side
(torchft/checkpointing.py:164, 197-203): every device storage is copied to
pageable host memory one by one and framed in a zip/pickle stream.  Here all
device tensors of the (nested) state dict are gathered by ONE kernel launch into
one contiguous staging buffer in HBM, described by a small header; the staging
buffer then moves as a few large DMA transfers, and the receiver scatters it
back with one launch.  The round trip is bit-exact.

Wire layout of a packed state::

    b"TFTPACK1" | u64 header_len | header | payload (header.total_bytes)

``header`` is UTF-8 JSON ``{"skeleton", "entries", "total_bytes"}``: the state
dict with every device tensor replaced by a slot number; per slot the byte
offset (256-byte aligned), dtype and shape.  The skeleton carries dicts (any
key type), lists, tuples, strings, numbers, booleans, None and CPU tensors
(raw bytes, base64) as tagged JSON nodes, so an ordinary training state -
model, optimizer state, param_groups, step counters - is rebuilt without
unpickling anything.  A leaf JSON cannot express (an lr_scheduler object, say)
is embedded as a pickle; the receiver only unpickles such leaves when called
with ``allow_pickle=True``, which is the transport's default because the
reference's receive path is ``torch.load(weights_only=False)``
(torchft/checkpointing.py:201-203) and must keep working for such states.
"""

from __future__ import annotations

import base64
import io
import json
import pickle
import struct
import threading
from collections import OrderedDict
from dataclasses import dataclass
from typing import Any, BinaryIO, Dict, List, Optional, Sequence, Tuple

import torch

from . import ops
from .multi_tensor import TensorTable

MAGIC = b"TFTPACK1"
ALIGN = 256
_DTYPES = {
    str(d): d
    for d in (
        torch.float32, torch.float64, torch.float16, torch.bfloat16, torch.int8, torch.uint8,
        torch.int16, torch.int32, torch.int64, torch.bool,
        torch.float8_e4m3fn, torch.float8_e5m2, torch.float8_e4m3fnuz, torch.float8_e5m2fnuz,
    )
}


@dataclass(frozen=True)
class TensorSlot:
    """Placeholder for a device tensor inside the skeleton."""

    index: int


@dataclass(frozen=True)
class TensorEntry:
    offset: int
    nbytes: int
    dtype: str
    shape: Tuple[int, ...]
    requires_grad: bool
    is_parameter: bool


def _walk(obj: Any, tensors: List[Tuple[torch.Tensor, bool, bool]], seen: Dict[Tuple, int]) -> Any:
    if isinstance(obj, torch.Tensor) and obj.is_cuda:
        if str(obj.dtype) not in _DTYPES:
            raise TypeError(f"cannot pack tensors of {obj.dtype}")
        t = obj.detach()
        if not t.is_contiguous():
            t = t.contiguous()
        is_param = isinstance(obj, torch.nn.Parameter)
        key = (t.data_ptr(), t.dtype, tuple(t.shape), is_param)
        if t.numel() and key in seen:  # the same tensor reachable twice stays one tensor
            return TensorSlot(seen[key])
        seen[key] = len(tensors)
        tensors.append((t, bool(obj.requires_grad), is_param))
        return TensorSlot(len(tensors) - 1)
    if isinstance(obj, (dict, OrderedDict)):
        out = type(obj)()
        for k, v in obj.items():
            out[k] = _walk(v, tensors, seen)
        return out
    if isinstance(obj, list):
        return [_walk(v, tensors, seen) for v in obj]
    if isinstance(obj, tuple):
        items = [_walk(v, tensors, seen) for v in obj]
        return type(obj)(*items) if hasattr(obj, "_fields") else tuple(items)
    return obj


def _fill(obj: Any, tensors: Sequence[torch.Tensor]) -> Any:
    if isinstance(obj, TensorSlot):
        return tensors[obj.index]
    if isinstance(obj, (dict, OrderedDict)):
        out = type(obj)()
        for k, v in obj.items():
            out[k] = _fill(v, tensors)
        return out
    if isinstance(obj, list):
        return [_fill(v, tensors) for v in obj]
    if isinstance(obj, tuple):
        items = [_fill(v, tensors) for v in obj]
        return type(obj)(*items) if hasattr(obj, "_fields") else tuple(items)
    return obj


@dataclass
class PackPlan:
    skeleton: Any
    tensors: List[torch.Tensor]
    entries: List[TensorEntry]
    total_bytes: int

    def header(self) -> bytes:
        doc = {
            "skeleton": _encode(self.skeleton),
            "entries": [
                [e.offset, e.nbytes, e.dtype, list(e.shape), e.requires_grad, e.is_parameter]
                for e in self.entries
            ],
            "total_bytes": self.total_bytes,
        }
        return json.dumps(doc, separators=(",", ":")).encode("utf-8")


def plan_pack(state_dict: Any) -> PackPlan:
    """Walks the state dict and lays its device tensors out back to back
    (each at a 256-byte aligned offset)."""
    found: List[Tuple[torch.Tensor, bool, bool]] = []
    skeleton = _walk(state_dict, found, {})
    entries = []
    offset = 0
    for t, requires_grad, is_param in found:
        nbytes = t.numel() * t.element_size()
        entries.append(
            TensorEntry(offset, nbytes, str(t.dtype), tuple(t.shape), requires_grad, is_param)
        )
        offset += -(-nbytes // ALIGN) * ALIGN
    return PackPlan(skeleton, [t for t, _, _ in found], entries, offset)


def _views(staging: torch.Tensor, entries: Sequence[TensorEntry]) -> List[torch.Tensor]:
    return [staging[e.offset : e.offset + e.nbytes] for e in entries]


class PackedState:
    """A packed state: ``header`` bytes and the ``staging`` buffer (uint8, on the device)."""

    def __init__(self, plan: PackPlan, staging: Optional[torch.Tensor]) -> None:
        self.plan = plan
        self.header = plan.header()
        self.staging = staging

    @property
    def total_bytes(self) -> int:
        return self.plan.total_bytes


def pack(
    state_dict: Any,
    staging: Optional[torch.Tensor] = None,
    table_cache: Optional[Dict[str, TensorTable]] = None,
) -> PackedState:
    """Gathers every device tensor of ``state_dict`` into one staging buffer with one
    kernel launch on the current stream.  ``staging`` (uint8, >= total bytes) is reused
    if given, else allocated.  Padding bytes between tensors are left as they are."""
    plan = plan_pack(state_dict)
    if not plan.tensors:
        return PackedState(plan, None)
    device = plan.tensors[0].device
    if staging is None:
        staging = torch.empty(plan.total_bytes, dtype=torch.uint8, device=device)
    if staging.dtype != torch.uint8 or staging.numel() < plan.total_bytes or staging.device != device:
        raise ValueError(
            f"staging must be uint8[>= {plan.total_bytes}] on {device}, got "
            f"{staging.dtype}[{staging.numel()}] on {staging.device}"
        )
    dsts = _views(staging, plan.entries)
    srcs = plan.tensors
    cached = table_cache.get("pack") if table_cache is not None else None
    table = ops.mt_copy(dsts, srcs, table=cached)
    if table_cache is not None:
        table_cache["pack"] = table
    return PackedState(plan, staging)


_TAG = "__tft__"


def _encode(obj: Any) -> Any:
    """Skeleton -> JSON-able tree.  Plain JSON values stay as they are; everything else
    becomes a ``{"__tft__": kind, ...}`` node."""
    if obj is None or isinstance(obj, (bool, str)):
        return obj
    if isinstance(obj, int):
        return obj if -(2 ** 53) < obj < 2 ** 53 else {_TAG: "int", "v": str(obj)}
    if isinstance(obj, float):
        return obj if obj == obj and obj not in (float("inf"), float("-inf")) else {
            _TAG: "float", "v": repr(obj)}
    if isinstance(obj, TensorSlot):
        return {_TAG: "slot", "i": obj.index}
    if isinstance(obj, torch.Tensor) and not isinstance(obj, torch.nn.Parameter) \
            and obj.device.type == "cpu" and str(obj.dtype) in _DTYPES and not obj.is_sparse:
        raw = obj.detach().contiguous().reshape(-1).view(torch.uint8).numpy().tobytes()
        return {_TAG: "cpu_tensor", "dtype": str(obj.dtype), "shape": list(obj.shape),
                "requires_grad": bool(obj.requires_grad),
                "data": base64.b64encode(raw).decode("ascii")}
    if type(obj) is dict and all(isinstance(k, str) and k != _TAG for k in obj):
        return {k: _encode(v) for k, v in obj.items()}
    if type(obj) in (dict, OrderedDict):  # keys of any hashable kind, order kept
        return {_TAG: "odict" if type(obj) is OrderedDict else "dict",
                "items": [[_encode(k), _encode(v)] for k, v in obj.items()]}
    if type(obj) is list:
        return [_encode(v) for v in obj]
    if type(obj) is tuple:
        return {_TAG: "tuple", "v": [_encode(v) for v in obj]}
    blob = pickle.dumps(obj, protocol=pickle.HIGHEST_PROTOCOL)
    return {_TAG: "pickle", "type": type(obj).__name__, "data": base64.b64encode(blob).decode("ascii")}


def _decode(node: Any, allow_pickle: bool) -> Any:
    if isinstance(node, list):
        return [_decode(v, allow_pickle) for v in node]
    if not isinstance(node, dict):
        return node
    kind = node.get(_TAG)
    if kind is None:
        return {k: _decode(v, allow_pickle) for k, v in node.items()}
    if kind == "slot":
        return TensorSlot(int(node["i"]))
    if kind == "int":
        return int(node["v"])
    if kind == "float":
        return float(node["v"])
    if kind == "tuple":
        return tuple(_decode(v, allow_pickle) for v in node["v"])
    if kind in ("dict", "odict"):
        out = OrderedDict() if kind == "odict" else {}
        for k, v in node["items"]:
            key = _decode(k, allow_pickle)
            out[tuple(key) if isinstance(key, list) else key] = _decode(v, allow_pickle)
        return out
    if kind == "cpu_tensor":
        dtype = _DTYPES[node["dtype"]]
        raw = bytearray(base64.b64decode(node["data"]))
        t = torch.frombuffer(raw, dtype=torch.uint8).clone() if raw else torch.empty(0, dtype=torch.uint8)
        t = t.view(dtype).view(node["shape"])
        return t.requires_grad_(True) if node.get("requires_grad") else t
    if kind == "pickle":
        if not allow_pickle:
            raise ValueError(
                f"the packed state holds a pickled {node.get('type', 'object')}; "
                "pass allow_pickle=True to accept it (trusted peers only)"
            )
        return pickle.loads(base64.b64decode(node["data"]))
    raise ValueError(f"unknown node kind {kind!r} in packed-state header")


def header_total_bytes(header: bytes) -> int:
    """Payload size announced by a header; decodes nothing else."""
    try:
        doc = json.loads(header.decode("utf-8"))
        total = int(doc["total_bytes"])
    except (UnicodeDecodeError, ValueError, KeyError, TypeError) as e:
        raise ValueError(f"not a packed-state header: {e}") from None
    if total < 0:
        raise ValueError("not a packed-state header: negative payload size")
    return total


def parse_header(header: bytes, allow_pickle: bool = True, decode_skeleton: bool = True) -> Dict[str, Any]:
    """Decodes a header into ``{"skeleton", "entries", "total_bytes"}``.  Nothing is
    unpickled unless the sender embedded a leaf JSON cannot express and
    ``allow_pickle`` is true.  ``decode_skeleton=False`` only validates the entries
    (every tensor inside the payload, shapes and byte counts consistent)."""
    try:
        doc = json.loads(header.decode("utf-8"))
    except (UnicodeDecodeError, ValueError) as e:
        raise ValueError(f"not a packed-state header: {e}") from None
    if not isinstance(doc, dict) or set(doc) != {"skeleton", "entries", "total_bytes"}:
        raise ValueError("not a packed-state header")
    entries = [
        TensorEntry(int(o), int(n), str(d), tuple(int(x) for x in sh), bool(rg), bool(ip))
        for o, n, d, sh, rg, ip in doc["entries"]
    ]
    total = int(doc["total_bytes"])
    for e in entries:
        if e.dtype not in _DTYPES or e.offset < 0 or e.nbytes < 0 or e.offset + e.nbytes > total:
            raise ValueError("packed-state header describes a tensor outside the payload")
        numel = 1
        for x in e.shape:
            numel *= x
        if numel * _DTYPES[e.dtype].itemsize != e.nbytes:
            raise ValueError("packed-state header: shape and byte count disagree")
    if total < 0:
        raise ValueError("packed-state header: negative payload size")
    skeleton = _decode(doc["skeleton"], allow_pickle) if decode_skeleton else None
    return {"skeleton": skeleton, "entries": entries, "total_bytes": total}


def unpack(
    header: bytes,
    staging: Optional[torch.Tensor],
    copy: bool = True,
    allow_pickle: bool = True,
) -> Any:
    """Rebuilds the state dict from ``header`` and the device-resident ``staging``.

    ``copy=True`` scatters into freshly allocated tensors with one kernel launch;
    ``copy=False`` returns views into ``staging`` (no traffic at all; the tensors
    then live as long as the staging buffer does)."""
    meta = parse_header(header, allow_pickle)
    entries: List[TensorEntry] = meta["entries"]
    if not entries:
        return _fill(meta["skeleton"], [])
    if staging is None or staging.dtype != torch.uint8 or staging.numel() < meta["total_bytes"]:
        raise ValueError(f"staging must be uint8[>= {meta['total_bytes']}]")
    srcs = _views(staging, entries)
    typed = [
        s.view(_DTYPES[e.dtype]).view(e.shape) if e.nbytes else
        torch.empty(e.shape, dtype=_DTYPES[e.dtype], device=staging.device)
        for s, e in zip(srcs, entries)
    ]
    if copy:
        outs = [torch.empty_like(t) for t in typed]
        ops.mt_copy(outs, typed)
    else:
        outs = typed
    final = []
    for t, e in zip(outs, entries):
        if e.is_parameter:
            t = torch.nn.Parameter(t, requires_grad=e.requires_grad)
        elif e.requires_grad:
            t.requires_grad_(True)
        final.append(t)
    return _fill(meta["skeleton"], final)


# ---------------------------------------------------------------------------
# Moving a packed state over PCIe and over a byte stream
# ---------------------------------------------------------------------------

DEFAULT_CHUNK_BYTES = 64 << 20
MAX_HEADER_BYTES = 256 << 20  # a header is a few hundred bytes per tensor


class _PinnedPool:
    """Pinned host buffers, kept between transfers (pinning a fresh 64 MiB costs tens of
    milliseconds; a recovery moves tens of gigabytes through a handful of them)."""

    def __init__(self, keep_bytes: int = 2 << 30) -> None:
        self._lock = threading.Lock()
        self._free: List[torch.Tensor] = []
        self._keep_bytes = keep_bytes

    def acquire(self, nbytes: int) -> torch.Tensor:
        with self._lock:
            for i, t in enumerate(self._free):
                if t.numel() >= nbytes:
                    return self._free.pop(i)
        return torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)

    def release(self, t: torch.Tensor) -> None:
        with self._lock:
            if sum(x.numel() for x in self._free) + t.numel() <= self._keep_bytes:
                self._free.append(t)


PINNED = _PinnedPool()


class _RingPool:
    """Device rings of the serving pipeline with the two streams that work on them, kept
    between requests: a recovery fetches one payload as several ranges, again and again over
    a job's life, and each request would otherwise allocate 3 x chunk_bytes of device memory
    and two streams of its own.  A ring is allocated under its own gather stream, so taking
    one never touches the training thread's stream."""

    def __init__(self, keep: int = 8) -> None:
        self._lock = threading.Lock()
        self._free: List[Tuple[torch.Tensor, "torch.cuda.Stream", "torch.cuda.Stream"]] = []
        self._keep = keep

    def acquire(self, device: torch.device, nbytes: int):
        with self._lock:
            for i, (ring, _, _) in enumerate(self._free):
                if ring.device == device and ring.numel() >= nbytes:
                    return self._free.pop(i)
        pack_stream, copy_stream = torch.cuda.Stream(device=device), torch.cuda.Stream(device=device)
        with torch.cuda.stream(pack_stream):
            # every byte that is sent is gathered into the ring first: no need to clear it
            ring = torch.empty(nbytes, dtype=torch.uint8, device=device)
        return ring, pack_stream, copy_stream

    def release(self, item) -> None:
        with self._lock:
            if len(self._free) < self._keep:
                self._free.append(item)


RINGS = _RingPool()


def split_range(total: int, part: int, parts: int) -> Tuple[int, int]:
    """Byte range [lo, hi) of ``part`` when a payload of ``total`` bytes is cut into
    ``parts`` ranges of (almost) equal size on 256-byte boundaries."""
    if not 0 <= part < parts:
        raise ValueError(f"part {part} of {parts}")
    per_part = -(-total // parts)
    step = -(-per_part // ALIGN) * ALIGN
    return min(part * step, total), min((part + 1) * step, total)


def _pieces(plan: PackPlan, lo: int, hi: int) -> Tuple[List[int], List[torch.Tensor]]:
    """The tensors' bytes that fall into payload range [lo, hi): (offsets inside the range,
    byte views of the sources)."""
    offs: List[int] = []
    srcs: List[torch.Tensor] = []
    for e, t in zip(plan.entries, plan.tensors):
        a, b = max(lo, e.offset), min(hi, e.offset + e.nbytes)
        if a < b:
            raw = t.reshape(-1).view(torch.uint8)
            offs.append(a - lo)
            srcs.append(raw[a - e.offset : b - e.offset])
    return offs, srcs


def stream_packed(
    plan: PackPlan,
    out: BinaryIO,
    lo: int = 0,
    hi: Optional[int] = None,
    chunk_bytes: int = DEFAULT_CHUNK_BYTES,
    after: Optional["torch.cuda.Event"] = None,
) -> None:
    """Writes MAGIC | header length | header | payload bytes [lo, hi) to ``out`` without ever
    holding more than a few chunks: chunk k+2 is gathered on the device (one launch into a
    slot of a three-slot ring) while chunk k+1 crosses PCIe into pinned memory and chunk k is
    written to ``out``.  Device memory: 3 x chunk_bytes; pinned memory: 3 x chunk_bytes (both
    pooled between calls).  The gather and the device-to-host copies run on two streams of
    their own, ordered after ``after`` (an event recorded by whoever last wrote the state)
    and after nothing else: the calling thread's current stream is not involved."""
    header = plan.header()
    out.write(MAGIC)
    out.write(struct.pack("<Q", len(header)))
    out.write(header)
    total = plan.total_bytes
    hi = total if hi is None else hi
    if not 0 <= lo <= hi <= total:
        raise ValueError(f"range [{lo}, {hi}) outside a payload of {total} bytes")
    if hi == lo or not plan.tensors:
        return
    device = plan.tensors[0].device
    n_slots = 3
    chunk_bytes = max(ALIGN, min(chunk_bytes, -(-(hi - lo) // ALIGN) * ALIGN))
    starts = list(range(lo, hi, chunk_bytes))
    leased = RINGS.acquire(device, n_slots * chunk_bytes)
    ring, pack_stream, copy_stream = leased
    slots = [ring[j * chunk_bytes : (j + 1) * chunk_bytes] for j in range(n_slots)]
    pinned = [PINNED.acquire(chunk_bytes) for _ in range(n_slots)]
    if after is not None:
        pack_stream.wait_event(after)
    packed = [torch.cuda.Event() for _ in starts]
    landed = [torch.cuda.Event() for _ in starts]

    def size(k: int) -> int:
        return min(chunk_bytes, hi - starts[k])

    try:
        for k in range(len(starts) + 2):
            if k < len(starts):  # gather chunk k into its ring slot
                if k >= n_slots:
                    pack_stream.wait_event(landed[k - n_slots])  # the slot's last copy left it
                offs, srcs = _pieces(plan, starts[k], starts[k] + size(k))
                if srcs:
                    dsts = [slots[k % n_slots][o : o + s.numel()] for o, s in zip(offs, srcs)]
                    with torch.cuda.stream(pack_stream):
                        ops.mt_copy(dsts, srcs)
                packed[k].record(pack_stream)
            j = k - 1
            if 0 <= j < len(starts):  # chunk j crosses PCIe (its pinned slot was written out)
                copy_stream.wait_event(packed[j])
                with torch.cuda.stream(copy_stream):
                    pinned[j % n_slots][: size(j)].copy_(slots[j % n_slots][: size(j)], non_blocking=True)
                landed[j].record(copy_stream)
            j = k - 2
            if 0 <= j < len(starts):  # chunk j goes out
                landed[j].synchronize()
                out.write(memoryview(pinned[j % n_slots][: size(j)].numpy()))
    finally:
        copy_stream.synchronize()
        pack_stream.synchronize()
        for t in pinned:
            PINNED.release(t)
        RINGS.release(leased)


def write_packed(packed: PackedState, out: BinaryIO, chunk_bytes: int = DEFAULT_CHUNK_BYTES) -> None:
    """Writes the wire layout of an already packed state (a full staging buffer on the
    device) to ``out``; the payload goes through two pinned bounce buffers so that the copy
    of chunk k+1 overlaps the write of chunk k."""
    out.write(MAGIC)
    out.write(struct.pack("<Q", len(packed.header)))
    out.write(packed.header)
    total = packed.total_bytes
    if total == 0:
        return
    staging = packed.staging
    assert staging is not None
    stream = torch.cuda.current_stream(staging.device)
    chunk_bytes = min(chunk_bytes, total)
    bounce = [PINNED.acquire(chunk_bytes), PINNED.acquire(chunk_bytes)]
    events = [torch.cuda.Event(), torch.cuda.Event()]
    offsets = list(range(0, total, chunk_bytes))

    def start(i: int) -> None:
        lo = offsets[i]
        n = min(chunk_bytes, total - lo)
        bounce[i % 2][:n].copy_(staging[lo : lo + n], non_blocking=True)
        events[i % 2].record(stream)

    try:
        start(0)
        for i, lo in enumerate(offsets):
            n = min(chunk_bytes, total - lo)
            events[i % 2].synchronize()
            if i + 1 < len(offsets):
                start(i + 1)
            out.write(memoryview(bounce[i % 2][:n].numpy()))
    finally:
        stream.synchronize()
        for t in bounce:
            PINNED.release(t)


def _read_exact(src: BinaryIO, view: memoryview) -> None:
    got = 0
    while got < len(view):
        n = src.readinto(view[got:])  # type: ignore[attr-defined]
        if not n:
            raise EOFError(f"stream ended after {got} of {len(view)} bytes")
        got += n


def read_header(src: BinaryIO) -> bytes:
    """Reads MAGIC | header length | header and returns the header bytes.  The length field
    comes from the peer: it is bounded before anything of that size is read."""
    magic = src.read(len(MAGIC))
    if magic != MAGIC:
        raise ValueError(f"bad magic {magic!r}: not a packed state")
    raw = src.read(8)
    if len(raw) != 8:
        raise EOFError("stream ended inside the header")
    (hlen,) = struct.unpack("<Q", raw)
    if hlen > MAX_HEADER_BYTES:
        raise ValueError(f"packed-state header of {hlen} bytes: refused (limit {MAX_HEADER_BYTES})")
    header = src.read(hlen)
    if len(header) != hlen:
        raise EOFError("stream ended inside the header")
    return header


def check_payload_fits(header: bytes, device: torch.device) -> int:
    """Validates the header's entries against its announced payload size, and that size
    against the device's free memory, BEFORE a staging buffer of that size is allocated;
    returns the payload size."""
    total = header_total_bytes(header)
    parse_header(header, allow_pickle=False, decode_skeleton=False)
    if total:
        free, _ = torch.cuda.mem_get_info(device)
        reusable = torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
        if total > free + reusable:
            raise ValueError(
                f"packed state announces {total} payload bytes, the device has {free + reusable} free"
            )
    return total


def read_payload(
    src: BinaryIO,
    staging: torch.Tensor,
    lo: int,
    hi: int,
    chunk_bytes: int = DEFAULT_CHUNK_BYTES,
) -> None:
    """Receives payload bytes [lo, hi) from ``src`` into ``staging[lo:hi]`` (on the device):
    chunk by chunk into pinned memory and up to the device as it arrives, on a stream of its
    own, so host memory use is bounded by two chunks."""
    if hi <= lo:
        return
    device = staging.device
    stream = torch.cuda.Stream(device=device)
    chunk_bytes = min(chunk_bytes, hi - lo)
    bounce = [PINNED.acquire(chunk_bytes), PINNED.acquire(chunk_bytes)]
    events: List[Optional[torch.cuda.Event]] = [None, None]
    try:
        for i, a in enumerate(range(lo, hi, chunk_bytes)):
            n = min(chunk_bytes, hi - a)
            ev = events[i % 2]
            if ev is not None:
                ev.synchronize()  # the previous upload from this bounce buffer is done
            _read_exact(src, memoryview(bounce[i % 2][:n].numpy()))
            with torch.cuda.stream(stream):
                staging[a : a + n].copy_(bounce[i % 2][:n], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record(stream)
            events[i % 2] = ev
    finally:
        stream.synchronize()
        for t in bounce:
            PINNED.release(t)


def read_packed(
    src: BinaryIO,
    device: Optional[torch.device],
    chunk_bytes: int = DEFAULT_CHUNK_BYTES,
) -> Tuple[bytes, Optional[torch.Tensor]]:
    """Reads the wire layout (whole payload); returns ``(header, staging on device)``."""
    header = read_header(src)
    if device is None and torch.cuda.is_available():
        device = torch.device("cuda", torch.cuda.current_device())
    total = header_total_bytes(header)
    parse_header(header, allow_pickle=False, decode_skeleton=False)  # before any allocation
    if total == 0:
        return header, None
    if device is None:
        raise RuntimeError("the packed state holds device tensors and no GPU is visible")
    check_payload_fits(header, device)
    staging = torch.empty(total, dtype=torch.uint8, device=device)
    # the allocation is ordered on the current stream; the upload runs on another
    torch.cuda.current_stream(device).synchronize()
    read_payload(src, staging, 0, total, chunk_bytes)
    return header, staging


def dumps(state_dict: Any) -> bytes:
    """pack + write_packed into bytes (small states, tests)."""
    buf = io.BytesIO()
    write_packed(pack(state_dict), buf)
    return buf.getvalue()


def loads(data: bytes, device: Optional[torch.device] = None, allow_pickle: bool = True) -> Any:
    header, staging = read_packed(io.BytesIO(data), device)
    return unpack(header, staging, copy=False, allow_pickle=allow_pickle)
