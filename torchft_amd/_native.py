"""ctypes binding of libtorchft_amd.so (declared in include/torchft_amd.h).

There is no fallback: if the library is missing or fails to load, every call
raises.  torch is imported first so that the HIP runtime torch already mapped
is the one the library binds to (streams and device pointers are only valid
inside one runtime instance).
"""

from __future__ import annotations

import ctypes
import threading
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_uint32, c_uint64, c_void_p
from pathlib import Path
from typing import Optional

import torch  # noqa: F401  (must precede loading the library, see module docstring)

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libtorchft_amd.so"

ABI_VERSION = 6
MAX_REPLICAS = 8
MIN_CHUNK_ELEMS = 8192
MIN_CHUNK_BYTES = 16384  # tft_mt_copy_bytes counts bytes
NOALLOC_MAX_TENSORS = 4096

TFT_F32 = 0
TFT_BF16 = 1
TFT_F16 = 2
TFT_F64 = 3  # replica average only


class MtTable(Structure):
    _fields_ = [
        ("ptrs", c_void_p),
        ("numel", c_void_p),
        ("chunk_start", c_void_p),
        ("chunk_tensor", c_void_p),
        ("n_tensors", c_uint32),
        ("n_cols", c_uint32),
        ("chunk_elems", c_uint32),
        ("total_chunks", c_uint32),
    ]


class SgdParams(Structure):
    _fields_ = [
        ("lr", c_float),
        ("momentum", c_float),
        ("dampening", c_float),
        ("weight_decay", c_float),
        ("nesterov", c_int32),
        ("first_step", c_int32),
    ]


# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "tft_abi_version": (c_int, []),
    "tft_last_error": (c_char_p, []),
    "tft_mt_plan": (
        c_int64,
        [POINTER(c_uint64), c_uint32, c_uint32, POINTER(c_uint32), POINTER(c_uint32)],
    ),
    "tft_default_chunk_elems": (c_uint32, [c_int]),
    "tft_reduce_avg": (
        c_int,
        [c_void_p, POINTER(c_void_p), c_uint32, c_uint32, c_uint32, c_uint64, c_int, c_void_p],
    ),
    "tft_mt_reduce_avg": (
        c_int,
        [POINTER(MtTable), c_uint32, c_uint32, c_uint32, c_uint32, c_int, c_void_p],
    ),
    "tft_mt_diloco_outer": (
        c_int,
        [POINTER(MtTable), c_uint32, c_uint32, c_uint32, c_int, POINTER(SgdParams), c_void_p],
    ),
    "tft_mt_diloco_outer_noalloc": (
        c_int,
        [POINTER(c_void_p), POINTER(c_uint64), c_uint32, c_uint32, c_uint32, c_uint32, c_int,
         POINTER(SgdParams), c_void_p],
    ),
    "tft_mt_pseudograd_avg": (
        c_int,
        [POINTER(MtTable), c_uint32, c_uint32, c_uint32, c_int, c_int, c_void_p],
    ),
    "tft_mt_outer_sgd": (c_int, [POINTER(MtTable), c_int, POINTER(SgdParams), c_void_p]),
    "tft_mt_outer_sgd_of_sum": (c_int, [POINTER(MtTable), c_uint32, c_int, POINTER(SgdParams), c_void_p]),
    "tft_mt_copy_bytes": (c_int, [POINTER(MtTable), c_void_p]),
    "tft_probe_rw_pair": (c_int, [c_void_p, c_void_p, c_uint64, c_void_p]),
}


class NativeLibraryError(RuntimeError):
    pass


_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


def _check_single_hip_runtime() -> None:
    seen = set()
    try:
        with open("/proc/self/maps") as f:
            for line in f:
                if "libamdhip64" in line:
                    seen.add(line.split()[-1])
    except OSError:
        return
    if len(seen) > 1:
        raise NativeLibraryError(
            "two HIP runtimes are mapped in this process (" + ", ".join(sorted(seen)) + "); "
            "libtorchft_amd.so must share torch's runtime"
        )


def load(path: Path, extra_signatures: Optional[dict] = None) -> ctypes.CDLL:
    """Loads a build of the library from ``path`` and binds every declared symbol."""
    if not path.exists():
        raise NativeLibraryError(
            f"{path} is not built; run `python -m torchft_amd._build` "
            "(needs hipcc, cross-compiles for gfx950 without a GPU)"
        )
    try:
        handle = ctypes.CDLL(str(path), mode=ctypes.RTLD_LOCAL)
    except OSError as e:
        raise NativeLibraryError(f"cannot load {path}: {e}") from e
    for name, (restype, argtypes) in {**SIGNATURES, **(extra_signatures or {})}.items():
        try:
            fn = getattr(handle, name)
        except AttributeError as e:
            raise NativeLibraryError(f"{path} does not export {name}") from e
        fn.restype = restype
        fn.argtypes = argtypes
    version = handle.tft_abi_version()
    if version != ABI_VERSION:
        raise NativeLibraryError(f"ABI version {version}, this package expects {ABI_VERSION}")
    _check_single_hip_runtime()
    return handle


def lib() -> ctypes.CDLL:
    """Returns the loaded library; raises NativeLibraryError if it cannot be loaded."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            _lib = load(LIB_PATH)
        return _lib


def check(rc: int, what: str) -> None:
    if rc < 0:
        msg = lib().tft_last_error()
        raise RuntimeError(f"{what} failed ({rc}): {msg.decode() if msg else 'unknown error'}")


def is_available() -> bool:
    try:
        lib()
        return True
    except NativeLibraryError:
        return False
