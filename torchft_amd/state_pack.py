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


def parse_header(header: bytes, allow_pickle: bool = True) -> Dict[str, Any]:
    """Decodes a header into ``{"skeleton", "entries", "total_bytes"}``.  Nothing is
    unpickled unless the sender embedded a leaf JSON cannot express and
    ``allow_pickle`` is true."""
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
    return {"skeleton": _decode(doc["skeleton"], allow_pickle), "entries": entries,
            "total_bytes": total}


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
# Moving a staging buffer over PCIe and over a byte stream
# ---------------------------------------------------------------------------

DEFAULT_CHUNK_BYTES = 256 << 20


def _pinned(nbytes: int) -> torch.Tensor:
    return torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)


def write_packed(packed: PackedState, out: BinaryIO, chunk_bytes: int = DEFAULT_CHUNK_BYTES) -> None:
    """Writes the wire layout to ``out``; the payload goes through two pinned bounce
    buffers so that the copy of chunk k+1 overlaps the write of chunk k."""
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
    bounce = [_pinned(chunk_bytes), _pinned(chunk_bytes)]
    events = [torch.cuda.Event(), torch.cuda.Event()]
    offsets = list(range(0, total, chunk_bytes))

    def start(i: int) -> None:
        lo = offsets[i]
        n = min(chunk_bytes, total - lo)
        bounce[i % 2][:n].copy_(staging[lo : lo + n], non_blocking=True)
        events[i % 2].record(stream)

    start(0)
    for i, lo in enumerate(offsets):
        n = min(chunk_bytes, total - lo)
        events[i % 2].synchronize()
        if i + 1 < len(offsets):
            start(i + 1)
        out.write(memoryview(bounce[i % 2][:n].numpy()))


def _read_exact(src: BinaryIO, view: memoryview) -> None:
    got = 0
    while got < len(view):
        n = src.readinto(view[got:])  # type: ignore[attr-defined]
        if not n:
            raise EOFError(f"stream ended after {got} of {len(view)} bytes")
        got += n


def read_packed(
    src: BinaryIO,
    device: Optional[torch.device],
    chunk_bytes: int = DEFAULT_CHUNK_BYTES,
) -> Tuple[bytes, Optional[torch.Tensor]]:
    """Reads the wire layout; returns ``(header, staging on device)``.  The payload is
    received chunk by chunk into pinned memory and copied to the device as it arrives,
    so host memory use is bounded by two chunks."""
    magic = src.read(len(MAGIC))
    if magic != MAGIC:
        raise ValueError(f"bad magic {magic!r}: not a packed state")
    (hlen,) = struct.unpack("<Q", src.read(8))
    header = src.read(hlen)
    if len(header) != hlen:
        raise EOFError("stream ended inside the header")
    total = header_total_bytes(header)
    if total == 0:
        return header, None
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    staging = torch.empty(total, dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream(device)
    chunk_bytes = min(chunk_bytes, total)
    bounce = [_pinned(chunk_bytes), _pinned(chunk_bytes)]
    events: List[Optional[torch.cuda.Event]] = [None, None]
    for i, lo in enumerate(range(0, total, chunk_bytes)):
        n = min(chunk_bytes, total - lo)
        ev = events[i % 2]
        if ev is not None:
            ev.synchronize()  # the previous upload from this bounce buffer is done
        _read_exact(src, memoryview(bounce[i % 2][:n].numpy()))
        staging[lo : lo + n].copy_(bounce[i % 2][:n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record(stream)
        events[i % 2] = ev
    stream.synchronize()
    return header, staging


def dumps(state_dict: Any) -> bytes:
    """pack + write_packed into bytes (small states, tests)."""
    buf = io.BytesIO()
    write_packed(pack(state_dict), buf)
    return buf.getvalue()


def loads(data: bytes, device: Optional[torch.device] = None, allow_pickle: bool = True) -> Any:
    header, staging = read_packed(io.BytesIO(data), device)
    return unpack(header, staging, copy=False, allow_pickle=allow_pickle)
