"""Builds libtorchft_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Run as ``python -m torchft_amd._build`` or call :func:`build`.  The library has
no dependency on torch: it is a plain C-ABI shared object that ctypes loads.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_ROOT = PKG_DIR.parent
SRC = PKG_DIR / "csrc" / "replica_sync.hip"
INCLUDE_DIR = REPO_ROOT / "include"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libtorchft_amd.so"
# same source compiled with -DTFT_TUNING: additionally exports tft_set_launch_variant and
# instantiates every launch shape; loaded only by the test-suite and by tuning sweeps
TUNING_LIB_PATH = LIB_DIR / "libtorchft_amd_tuning.so"

# -packed-fp32-ops: keep hipcc from forming packed fp32 instructions out of the
# scalar float code (they have produced wrong results on this hardware pool).
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; torchft_amd needs the ROCm toolchain to build")
    return exe


def _compile(out_path: Path, defines, verbose: bool) -> subprocess.Popen:
    tmp = out_path.with_suffix(".so.tmp")
    cmd = [hipcc_path(), *HIPCC_FLAGS, *defines, f"-I{INCLUDE_DIR}", str(SRC), "-o", str(tmp)]
    if verbose:
        print("[torchft_amd] " + " ".join(cmd), flush=True)
    return subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def _finish(proc: subprocess.Popen, out_path: Path, verbose: bool) -> None:
    stdout, _ = proc.communicate()
    # the host pass does not know the device-only feature flag; that warning is noise
    out = "\n".join(line for line in stdout.splitlines() if "packed-fp32-ops" not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{out}")
    if verbose and out.strip():
        print(out, flush=True)
    os.replace(out_path.with_suffix(".so.tmp"), out_path)


def build(verbose: bool = True, tuning: bool = True) -> Path:
    """Compiles the library (and its tuning twin) unconditionally; returns the library's path."""
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    jobs = [(_compile(LIB_PATH, [], verbose), LIB_PATH)]
    if tuning:
        jobs.append((_compile(TUNING_LIB_PATH, ["-DTFT_TUNING"], verbose), TUNING_LIB_PATH))
    for proc, path in jobs:
        _finish(proc, path, verbose)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
