"""Device-resident tensor tables for the multi-tensor kernels.

A table describes T tensors by C pointer columns (for example, for the fused
DiLoCo step: live parameter, backup, momentum buffer, replica 0, replica 1 ...).
It is uploaded once and reused for every sync as long as the tensors keep
their storage, so a sync over 291 parameter tensors is one kernel launch and no
host-to-device traffic.
"""

from __future__ import annotations

import ctypes
import itertools
import operator
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _native

_DTYPE_CODES = {
    torch.float32: _native.TFT_F32,
    torch.bfloat16: _native.TFT_BF16,
    torch.float16: _native.TFT_F16,
    torch.float64: _native.TFT_F64,  # the replica average only
}


_DATA_PTR = torch.Tensor.data_ptr
_NUMEL = torch.Tensor.numel
_DTYPE = operator.attrgetter("dtype")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise TypeError(
            f"torchft_amd kernels support float32, bfloat16, float16 and (replica average only) "
            f"float64, got {dtype}"
        ) from None


def require_device_tensor(t: torch.Tensor, what: str) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise RuntimeError(
            f"{what}: tensor is on {t.device}; the torchft_amd kernels only run on GPU "
            "tensors (there is no CPU path)"
        )
    if not t.is_contiguous():
        raise ValueError(f"{what}: tensor of shape {tuple(t.shape)} is not contiguous")


def plan_chunks(numel: Sequence[int], chunk_elems: int) -> Tuple[np.ndarray, np.ndarray]:
    """(chunk_start[0..T], chunk_tensor[0..K)) for the given sizes.

    Host-only; both arrays are computed by the C library (tft_mt_plan)."""
    n = len(numel)
    arr = np.asarray(numel, dtype=np.uint64)
    start = np.zeros(n + 1, dtype=np.uint32)
    u64p, u32p = ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint32)
    plan = _native.lib().tft_mt_plan
    total = plan(arr.ctypes.data_as(u64p), n, chunk_elems, start.ctypes.data_as(u32p), None)
    _native.check(int(total), "tft_mt_plan")
    owner = np.zeros(max(int(total), 1), dtype=np.uint32)
    total = plan(
        arr.ctypes.data_as(u64p), n, chunk_elems, start.ctypes.data_as(u32p),
        owner.ctypes.data_as(u32p),
    )
    _native.check(int(total), "tft_mt_plan")
    return start, owner[: int(total)]


def pick_chunk_elems(sizes: Sequence[int], default: int, minimum: int) -> int:
    """Largest power-of-two chunk <= default whose last-chunk padding wastes < 1.5 % of the
    workgroups (models made of many small tensors want small chunks: GPT-2-small's 98 tensors
    of under 8 Ki elements measure 1-2 % faster with 16 Ki chunks than with 32 Ki)."""
    total = sum(sizes)
    chunk = default
    while chunk > minimum:
        launched = sum(-(-s // chunk) for s in sizes) * chunk
        if launched - total <= 0.015 * total:
            break
        chunk //= 2
    return chunk


class TensorTable:
    """T tensors x C columns, uploaded to the device of the tensors.

    ``columns[c][t]`` is the tensor of column c, row t.  All columns of a row
    must have the same number of elements; with ``as_bytes`` sizes are counted
    in bytes and dtypes may differ between rows (but not within a row).
    Rows with zero elements are dropped.
    """

    def __init__(
        self,
        columns: Sequence[Sequence[torch.Tensor]],
        *,
        as_bytes: bool = False,
        chunk_elems: Optional[int] = None,
        what: str = "TensorTable",
    ) -> None:
        if not columns or not all(len(col) == len(columns[0]) for col in columns):
            raise ValueError(f"{what}: columns must be non-empty and of equal length")
        n_cols = len(columns)
        n_rows_in = len(columns[0])
        self.dtype: Optional[torch.dtype] = None
        device: Optional[torch.device] = None
        rows: List[int] = []
        for t in range(n_rows_in):
            first = columns[0][t]
            for c in range(n_cols):
                x = columns[c][t]
                require_device_tensor(x, f"{what}[col {c}, row {t}]")
                if device is None:
                    device = x.device
                elif x.device != device:
                    raise ValueError(f"{what}: tensors on {device} and {x.device} in one table")
                if as_bytes:
                    if x.numel() * x.element_size() != first.numel() * first.element_size():
                        raise ValueError(
                            f"{what}: row {t} pairs {first.numel() * first.element_size()} bytes "
                            f"with {x.numel() * x.element_size()} bytes (col {c})"
                        )
                elif x.dtype != first.dtype or x.numel() != first.numel():
                    raise ValueError(
                        f"{what}: row {t} mixes {first.dtype}[{first.numel()}] "
                        f"with {x.dtype}[{x.numel()}] (col {c})"
                    )
            if not as_bytes:
                if self.dtype is None:
                    self.dtype = first.dtype
                elif first.dtype != self.dtype:
                    raise ValueError(f"{what}: rows of {self.dtype} and {first.dtype} in one table")
            if first.numel() > 0:
                rows.append(t)
        if device is None:
            raise ValueError(f"{what}: empty table")
        self.device = device
        self.as_bytes = as_bytes
        self.n_cols = n_cols
        self.n_tensors = len(rows)
        if as_bytes:
            code = -1
        else:
            assert self.dtype is not None
            code = dtype_code(self.dtype)
        self.dtype_code = code
        sizes = [
            columns[0][t].numel() * (columns[0][t].element_size() if as_bytes else 1) for t in rows
        ]
        self.chunk_elems = int(
            chunk_elems
            or pick_chunk_elems(
                sizes,
                _native.lib().tft_default_chunk_elems(code),
                _native.MIN_CHUNK_BYTES if as_bytes else _native.MIN_CHUNK_ELEMS,
            )
        )
        self.numel_total = int(sum(sizes))
        # keep the tensors alive and remember their identity for cache checks
        self._keepalive = [[columns[c][t] for t in rows] for c in range(n_cols)]
        self.key = self.make_key(columns)
        if self.n_tensors == 0:
            self.total_chunks = 0
            self._blob = None
            self.struct = _native.MtTable(None, None, None, None, 0, n_cols, self.chunk_elems, 0)
            return
        chunk_start, chunk_tensor = plan_chunks(sizes, self.chunk_elems)
        self.total_chunks = int(chunk_start[-1])
        ptrs = np.empty((n_cols, self.n_tensors), dtype=np.uint64)
        for c in range(n_cols):
            for i, t in enumerate(rows):
                ptrs[c, i] = columns[c][t].data_ptr()
        numel = np.asarray(sizes, dtype=np.uint64)
        ptr_bytes = ptrs.tobytes()
        numel_bytes = numel.tobytes()
        start_bytes = chunk_start.tobytes()
        owner_bytes = chunk_tensor.tobytes()
        blob = np.frombuffer(
            ptr_bytes + numel_bytes + start_bytes + owner_bytes, dtype=np.uint8
        ).copy()
        self._blob = torch.from_numpy(blob).to(self.device)
        base = self._blob.data_ptr()
        self.struct = _native.MtTable(
            base,
            base + len(ptr_bytes),
            base + len(ptr_bytes) + len(numel_bytes),
            base + len(ptr_bytes) + len(numel_bytes) + len(start_bytes),
            self.n_tensors,
            n_cols,
            self.chunk_elems,
            self.total_chunks,
        )

    @staticmethod
    def make_key(columns: Sequence[Sequence[torch.Tensor]]) -> Tuple:
        """Identity of the tensors a table describes: address, size and dtype of every one
        (checked on every launch, so built with C-level maps rather than a Python loop)."""
        flat = list(itertools.chain.from_iterable(columns))
        return (
            tuple(map(_DATA_PTR, flat)),
            tuple(map(_NUMEL, flat)),
            tuple(map(_DTYPE, flat)),
            tuple(map(len, columns)),
        )

    def matches(self, columns: Sequence[Sequence[torch.Tensor]]) -> bool:
        return self.key == self.make_key(columns)

    def ref(self):
        return ctypes.byref(self.struct)


def current_stream_handle(device: torch.device) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
