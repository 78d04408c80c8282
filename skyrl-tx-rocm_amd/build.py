"""Builds the gfx950 shared library of the W8A8 LoRA linear path with hipcc.

``python build.py`` compiles ``csrc/w8a8_api.hip`` into ``lib/libmi355_w8a8.so``.
hipcc cross-compiles without a GPU.  Flags: ``-ffp-contract=off -fno-fast-math`` keep
the quantizer and the float32 epilogue bit-exact (no fused multiply-add, IEEE
division and square root); packed FP32 instructions are disabled.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB_DIR = HERE / "lib"
LIB_PATH = LIB_DIR / "libmi355_w8a8.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-inline-asm", "-Wl,-z,defs", "-Wl,-z,relro", "-Wl,-z,now",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found; a ROCm toolchain is required to build the gfx950 library")


def jaxlib_include_dir() -> Path | None:
    """Directory holding xla/ffi/api/ffi.h (ships inside jaxlib), or None."""
    env = os.environ.get("JAXLIB_INCLUDE_DIR")
    if env and (Path(env) / "xla" / "ffi" / "api" / "ffi.h").exists():
        return Path(env)
    try:
        import importlib.util

        spec = importlib.util.find_spec("jaxlib")
    except (ImportError, ValueError):
        spec = None
    if spec and spec.submodule_search_locations:
        cand = Path(list(spec.submodule_search_locations)[0]) / "include"
        if (cand / "xla" / "ffi" / "api" / "ffi.h").exists():
            return cand
    return None


def build_ffi(verbose: bool = False) -> Path | None:
    """Build the XLA typed-FFI shim next to the C ABI library where jaxlib's headers exist."""
    inc = jaxlib_include_dir()
    if inc is None:
        return None
    out = LIB_DIR / "libmi355_w8a8_ffi.so"
    cmd = [find_hipcc(), "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared",
           "-isystem", str(inc), str(CSRC / "w8a8_xla_ffi.cc"), f"-L{LIB_DIR}", "-lmi355_w8a8",
           "-Wl,-rpath,$ORIGIN", "-Wl,-z,defs", "-o", str(out)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on the FFI shim ({proc.returncode}):\n{proc.stderr}")
    if verbose and proc.stderr.strip():
        print(proc.stderr, file=sys.stderr)
    return out


def build(verbose: bool = False) -> Path:
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    tmp = LIB_DIR / "libmi355_w8a8.so.tmp"
    cmd = [find_hipcc(), *HIPCC_FLAGS, str(CSRC / "w8a8_api.hip"), "-o", str(tmp)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(tmp, LIB_PATH)
    build_ffi(verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
