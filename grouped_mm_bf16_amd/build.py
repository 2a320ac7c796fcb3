"""Builds libgrouped_mm_hip.so for gfx950 with hipcc, in-tree.

    python -m grouped_mm_bf16_amd.build [--force]

Each .hip source under csrc/ is compiled to an object (in parallel) and the
objects are linked into grouped_mm_bf16_amd/libgrouped_mm_hip.so; csrc/diag/
becomes libgmm_diag.so, which only bench.py loads.  hipcc cross-compiles, so no
GPU is needed to build.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "csrc", "build")
LIB_PATH = os.path.join(HERE, "libgrouped_mm_hip.so")
# bench-only diagnostics (the register-only MFMA rate loop): a library of its own, loaded by bench.py alone
DIAG_SRC = os.path.join(CSRC, "diag", "gmm_diag.hip")
DIAG_LIB_PATH = os.path.join(HERE, "libgmm_diag.so")

ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def sources() -> list:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> list:
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".h", ".inc"))]
    hs.append(os.path.join(HERE, "..", "include", "grouped_mm_hip.h"))
    return hs


def _stale(target: str, deps: list) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    if force or _stale(obj, [src] + _headers()):
        cmd = [_hipcc(), *FLAGS, "-c", src, "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    return obj


def generate(force: bool = False) -> str:
    """Run gen_tile_asm.py -> csrc/gmm_tile_asm.inc (the hand-scheduled tile assembly)."""
    gen = os.path.join(CSRC, "gen_tile_asm.py")
    inc = os.path.join(CSRC, "gmm_tile_asm.inc")
    if force or _stale(inc, [gen]):
        res = subprocess.run([sys.executable, gen], capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"gen_tile_asm.py failed:\n{res.stderr}")
        with open(inc, "w") as f:
            f.write(res.stdout)
    return inc


def build(force: bool = False, verbose: bool = False) -> str:
    """Generate, compile (when stale or forced) and link; returns the library path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    generate(force)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or _stale(LIB_PATH, objs):
        cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if force or _stale(DIAG_LIB_PATH, [DIAG_SRC]):
        cmd = [_hipcc(), *FLAGS, "-shared", "-o", DIAG_LIB_PATH, DIAG_SRC]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {DIAG_SRC}:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH} and {DIAG_LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
