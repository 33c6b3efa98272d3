"""Builds libmi355_sdpa.so (hand-written gfx950 HIP kernels + C ABI) with hipcc, in-tree."""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(os.path.dirname(PKG_DIR), "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmi355_sdpa.so")
OBJ_DIR = os.path.join(LIB_DIR, "obj")

SOURCES = ["api", "fwd_generic", "fwd_mfma", "fwd_mfma_w32", "bwd_generic", "bwd_mfma", "bwd_dkdv_w32", "bwd_dq_w32", "decode_fp8kv"]

# packed-fp32 VALU ops are switched off for all device code in this library
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP extension cannot be built")
    return exe


def _run(cmd, verbose):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"build step failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, jobs: int = 6) -> str:
    """Compile every HIP source for gfx950 and link the shared library.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = _hipcc()

    def compile_one(name):
        src = os.path.join(CSRC_DIR, name + ".hip")
        obj = os.path.join(OBJ_DIR, name + ".o")
        _run([hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj], verbose)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
