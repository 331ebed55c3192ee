"""Builds libringattn_hip.so (gfx950) from csrc/ with hipcc, in-tree.

Usage: python build.py [--force]
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "ring_attention", "libringattn_hip.so")
SOURCES = ["ra_fwd.hip", "ra_bwd.hip", "ra_api.hip"]
# the matrix-rate probe that bench.py reports next to the roofline: a library of its own, so that
# the block-step library exports nothing but the block-step ABI
PROBE_LIB_PATH = os.path.join(HERE, "ring_attention", "libringattn_probe.so")
PROBE_SOURCES = ["ra_probe.hip"]
# the XLA FFI handlers over the C ABI (what a JAX host binds): built only where jaxlib's headers are
FFI_LIB_PATH = os.path.join(HERE, "ring_attention", "libringattn_xla_ffi.so")
FFI_SOURCE = "ra_xla_ffi.cc"
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build the kernels")
    return exe


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stderr}")
    return obj


def xla_ffi_include_dir() -> str | None:
    """Directory that holds xla/ffi/api/ffi.h: $XLA_FFI_INCLUDE_DIR, or the one jaxlib ships
    (jax.ffi.include_dir()); None where neither exists."""
    cands = [os.environ.get("XLA_FFI_INCLUDE_DIR")]
    try:
        import jax  # noqa: F401  (absent from this image: the adapter is then skipped)
        try:
            from jax import ffi as jffi
        except ImportError:
            from jax.extend import ffi as jffi
        cands.append(jffi.include_dir())
    except Exception:
        pass
    for c in cands:
        if c and os.path.exists(os.path.join(c, "xla", "ffi", "api", "ffi.h")):
            return c
    return None


def build_xla_ffi(verbose: bool = False) -> str | None:
    """libringattn_xla_ffi.so from csrc/ra_xla_ffi.cc, linked against the block-step library; skipped
    (None) without the XLA FFI headers."""
    inc = xla_ffi_include_dir()
    if inc is None:
        if verbose:
            print(f"{FFI_SOURCE} skipped: no jaxlib headers (xla/ffi/api/ffi.h not found; set XLA_FFI_INCLUDE_DIR "
                  "or install jaxlib)")
        return None
    cmd = [_hipcc(), "-O2", "-std=c++17", "-fPIC", "-shared", f"-I{inc}",
           os.path.join(CSRC, FFI_SOURCE), "-o", FFI_LIB_PATH, f"-L{os.path.dirname(LIB_PATH)}", "-lringattn_hip",
           "-Wl,-rpath,$ORIGIN"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {FFI_SOURCE}:\n{res.stderr}")
    if verbose:
        print(f"built {FFI_LIB_PATH}")
    return FFI_LIB_PATH


def build(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    """Compile every kernel translation unit and link the shared library. Always rebuilds."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    extra = list(extra_flags or [])
    every = SOURCES + PROBE_SOURCES
    with ThreadPoolExecutor(max_workers=len(every)) as pool:
        objs = dict(zip(every, pool.map(lambda s: _compile(s, extra), every)))
    for lib, srcs in ((LIB_PATH, SOURCES), (PROBE_LIB_PATH, PROBE_SOURCES)):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *(objs[s] for s in srcs), "-o", lib]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stderr}")
        if verbose:
            print(f"built {lib}")
    build_xla_ffi(verbose)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True, extra_flags=[a for a in sys.argv[1:] if a != "--force"])
