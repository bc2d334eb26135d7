"""The C-ABI library loads and exports exactly what include/torchft_amd.h declares.
No kernel is launched here (no GPU needed): only host-side entry points are called."""

import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from torchft_amd import _native, multi_tensor

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "torchft_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tft_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert names, "no declarations found"
    assert sorted(_native.SIGNATURES) == names


def test_library_exports_every_declared_symbol():
    lib = _native.lib()
    out = subprocess.run(["nm", "-D", "--defined-only", str(_native.LIB_PATH)],
                         check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    for name in declared_functions():
        assert name in exported, f"{name} is declared but not exported"
        assert getattr(lib, name) is not None
    # nothing else leaks out of the library under the tft_ prefix
    assert {n for n in exported if n.startswith("tft_")} == set(declared_functions())


def test_tuning_build_adds_only_the_launch_shape_override():
    from torchft_amd import _build

    out = subprocess.run(["nm", "-D", "--defined-only", str(_build.TUNING_LIB_PATH)],
                         check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    assert {n for n in exported if n.startswith("tft_")} == \
        set(declared_functions()) | {"tft_set_launch_variant"}


def test_abi_version_and_constants():
    lib = _native.lib()
    text = open(HEADER).read()
    assert lib.tft_abi_version() == int(re.search(r"#define TFT_ABI_VERSION (\d+)", text).group(1))
    assert _native.ABI_VERSION == lib.tft_abi_version()
    assert _native.MAX_REPLICAS == int(re.search(r"#define TFT_MAX_REPLICAS (\d+)", text).group(1))
    assert _native.MIN_CHUNK_ELEMS == int(re.search(r"#define TFT_MIN_CHUNK_ELEMS (\d+)u", text).group(1))
    dtypes = re.search(r"typedef enum tft_dtype \{([^}]*)\}", text).group(1)
    declared = {k.strip(): int(v) for k, v in (item.split("=") for item in dtypes.split(","))}
    assert declared == {"TFT_F32": _native.TFT_F32, "TFT_BF16": _native.TFT_BF16,
                        "TFT_F16": _native.TFT_F16, "TFT_F64": _native.TFT_F64}
    for code in (_native.TFT_F32, _native.TFT_BF16, _native.TFT_F64, -1):
        chunk = lib.tft_default_chunk_elems(code)
        assert chunk >= _native.MIN_CHUNK_ELEMS and chunk & (chunk - 1) == 0


def test_struct_layouts_match_the_header():
    # field order and sizes as declared: 4 pointers + 4 u32 / 4 floats + 2 i32
    assert ctypes.sizeof(_native.MtTable) == 4 * 8 + 4 * 4
    assert [f[0] for f in _native.MtTable._fields_] == [
        "ptrs", "numel", "chunk_start", "chunk_tensor", "n_tensors", "n_cols", "chunk_elems",
        "total_chunks"]
    assert ctypes.sizeof(_native.SgdParams) == 6 * 4
    assert [f[0] for f in _native.SgdParams._fields_] == [
        "lr", "momentum", "dampening", "weight_decay", "nesterov", "first_step"]


def test_plan_chunks_brute_force():
    sizes = [0, 1, 8191, 8192, 8193, 100_000, 0, 3 * 8192]
    start, owner = multi_tensor.plan_chunks(sizes, 8192)
    want_counts = [-(-s // 8192) for s in sizes]
    assert list(np.diff(start)) == want_counts
    assert start[0] == 0 and start[-1] == sum(want_counts) == len(owner)
    # every chunk names the tensor it belongs to; empty tensors own no chunk
    want_owner = [t for t, c in enumerate(want_counts) for _ in range(c)]
    assert list(owner) == want_owner


def test_plan_rejects_bad_chunk_sizes():
    for bad in (0, 1000, 4096, 8192 + 1024, 3 * 8192):
        with pytest.raises(RuntimeError, match="power of two"):
            multi_tensor.plan_chunks([10], bad)
    with pytest.raises(RuntimeError, match="too many chunks"):
        multi_tensor.plan_chunks([2 ** 44], 8192)


def test_pick_chunk_elems_prefers_small_chunks_for_small_tensors():
    big = [525_336_576, 16_777_216, 4096]
    assert multi_tensor.pick_chunk_elems(big, 65536, 8192) == 65536
    small = [768] * 100 + [2_359_296] * 12
    assert multi_tensor.pick_chunk_elems(small, 65536, 8192) < 65536
    assert multi_tensor.pick_chunk_elems([10], 65536, 8192) == 8192


def test_argument_errors_are_reported_without_a_gpu():
    lib = _native.lib()
    # NULL table / bad replica counts fail validation before anything touches the device
    assert lib.tft_mt_copy_bytes(None, None) == -1
    assert b"table is NULL" in lib.tft_last_error()
    assert lib.tft_reduce_avg(None, None, 9, 0, 1, 16, 0, None) == -2
    assert b"at most 8" in lib.tft_last_error()
    assert lib.tft_reduce_avg(None, None, 1, 0b10, 1, 16, 0, None) == -1
    assert lib.tft_reduce_avg(None, None, 1, 1, 0, 16, 0, None) == -1
    assert lib.tft_reduce_avg(None, None, 1, 1, 1, 16, 7, None) == -2  # unknown dtype
    assert lib.tft_reduce_avg(None, None, 1, 1, 1, 0, 0, None) == 0  # nothing to do
    table = _native.MtTable(None, None, None, None, 0, 5, 65536, 0)
    sgd = _native.SgdParams(0.7, 0.0, 0.0, 0.0, 1, 0)  # nesterov without momentum
    assert lib.tft_mt_diloco_outer(ctypes.byref(table), 2, 3, 2, 0, ctypes.byref(sgd), None) == -1
    assert b"nesterov" in lib.tft_last_error()
    sgd = _native.SgdParams(0.7, 0.9, 0.0, 0.0, 1, 0)
    assert lib.tft_mt_diloco_outer(ctypes.byref(table), 3, 7, 3, 0, ctypes.byref(sgd), None) == -1
    assert b"columns" in lib.tft_last_error()
    assert lib.tft_mt_diloco_outer(ctypes.byref(table), 2, 3, 2, 9, ctypes.byref(sgd), None) == -2  # dtype
    # fp64 is the replica average's alone
    assert lib.tft_mt_diloco_outer(ctypes.byref(table), 2, 3, 2, _native.TFT_F64, ctypes.byref(sgd), None) == -2
    assert b"replica average only" in lib.tft_last_error()
    assert lib.tft_reduce_avg(None, None, 1, 1, 1, 0, _native.TFT_F64, None) == 0
    # an empty table is a successful no-op
    assert lib.tft_mt_diloco_outer(ctypes.byref(table), 2, 3, 2, 0, ctypes.byref(sgd), None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No fallback: without the built library every entry into the native layer raises."""
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", tmp_path / "libtorchft_amd.so")
    assert not _native.is_available()
    with pytest.raises(_native.NativeLibraryError, match="is not built"):
        _native.lib()
    with pytest.raises(_native.NativeLibraryError):
        multi_tensor.plan_chunks([10], 8192)
    (tmp_path / "libtorchft_amd.so").write_bytes(b"not an ELF file")
    with pytest.raises(_native.NativeLibraryError, match="cannot load"):
        _native.lib()
