"""Builds pat_amd/libpat_amd.so in-tree with hipcc for gfx950 (MI355X).

    python -m pat_amd.build            # compile every source, link the library
    python -m pat_amd.build --jobs 4   # parallel compile

hipcc cross-compiles gfx950 code objects without a GPU, so this runs on any ROCm
host. The scheduler sources are plain C++17 and are compiled by the same driver so
that one shared object carries the whole C ABI of include/pat_amd.h.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from typing import List

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build", "obj")
OUT = os.path.join(HERE, "libpat_amd.so")

SOURCES = [
    "capi_sched.cc",
    "sched/radix_plan.cc",
    "capi_fwd.hip",
    "hip/pat_split.hip",
    "hip/pat_merge.hip",
    "hip/selftest.hip",
]

COMMON = ["-std=c++17", "-O3", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter",
          f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}"]
# Packed-FP32 VALU forms are switched off for all device code.
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-ffp-contract=off"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: a ROCm toolchain is required to build pat_amd")
    return exe


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, src.replace("/", "_") + ".o")
    path = os.path.join(CSRC, src)
    if src.endswith(".hip"):
        cmd = [hipcc(), *COMMON, *DEVICE, "-c", path, "-o", obj]
    else:
        cmd = [hipcc(), *COMMON, "-x", "c++", "-ffp-contract=off", "-c", path, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"compiling {src} failed:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    return obj


def build(jobs: int = 4, verbose: bool = False) -> str:
    """Compiles all sources and links libpat_amd.so; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs: List[str] = list(pool.map(lambda s: _compile(s, verbose), SOURCES))
    tmp = OUT + ".tmp"
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", tmp, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"linking libpat_amd.so failed:\n{res.stderr}")
    os.replace(tmp, OUT)
    return OUT


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args()
    print(build(a.jobs, a.verbose))


if __name__ == "__main__":
    main()
