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

SOURCES = ["api", "fwd_generic", "fwd_mfma", "fwd_mfma_w32", "bwd_generic", "bwd_mfma", "bwd_dkdv_w32", "bwd_dq_w32", "bwd_wide", "decode_fp8kv", "mask_rows", "f32_mfma"]

# packed-fp32 VALU ops are switched off for all device code in this library
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # per-kernel register / scratch / LDS figures, kept next to the library (RESOURCE_PATH)
    "-Rpass-analysis=kernel-resource-usage",
]
RESOURCE_PATH = os.path.join(LIB_DIR, "resource_usage.txt")


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP extension cannot be built")
    return exe


def _resource_lines(stderr: str):
    """'<mangled kernel name> <key>=<value> ...' per kernel, from the compiler's resource remarks."""
    out, cur = [], None
    for line in stderr.splitlines():
        if "[-Rpass-analysis=kernel-resource-usage]" not in line or "remark:" not in line:
            continue
        body = line.split("remark:", 1)[1].rsplit("[-Rpass", 1)[0].strip()
        key, _, val = body.partition(":")
        if key.strip() == "Function Name":
            cur = [val.strip()]
            out.append(cur)
        elif cur is not None:
            cur.append(f"{key.strip().replace(' ', '_')}={val.strip()}")
    return [" ".join(c) for c in out]


def _noise(lines):
    """Compiler output minus what every build prints: the host pass does not know the packed-fp32
    feature, the resource remarks (collected separately), and the note that m0, which the LDS-direct
    loads clobber on purpose, is a reserved register."""
    keep, skip = [], 0
    for l in lines:
        if skip:
            skip -= 1
            continue
        if "packed-fp32-ops" in l:
            continue
        if "-Rpass-analysis=kernel-resource-usage" in l:
            skip = 2 if "Function Name" in l else 0  # the source line and the caret under it
            continue
        if "clobber list contains reserved registers: m0" in l:
            skip = 2
            continue
        if "Reserved registers on the clobber list" in l:
            continue
        if l.strip() in ("", "^") or l.strip().endswith("warnings generated when compiling for gfx950."):
            continue
        keep.append(l)
    return keep


def _run(cmd, verbose):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(_noise(proc.stderr.splitlines()))
    if proc.returncode != 0:
        raise RuntimeError(f"build step failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return _resource_lines(proc.stderr)


def build(verbose: bool = False, jobs: int = 6) -> str:
    """Compile every HIP source for gfx950 and link the shared library.  Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = _hipcc()

    def compile_one(name):
        src = os.path.join(CSRC_DIR, name + ".hip")
        obj = os.path.join(OBJ_DIR, name + ".o")
        return obj, _run([hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj], verbose)

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(compile_one, SOURCES))
    objs = [o for o, _ in results]
    with open(RESOURCE_PATH + ".tmp", "w") as f:
        for name, (_, lines) in zip(SOURCES, results):
            for l in lines:
                f.write(f"{name}.hip {l}\n")
    os.replace(RESOURCE_PATH + ".tmp", RESOURCE_PATH)
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
