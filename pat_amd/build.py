"""Builds pat_amd/libpat_amd.so and the PyTorch-ROCm extension pat_amd/_prefix_attn.so in-tree.

    python -m pat_amd.build            # compile every source, link both
    python -m pat_amd.build --jobs 4   # parallel compile

libpat_amd.so: hipcc, gfx950 (MI355X). hipcc cross-compiles gfx950 code objects without a GPU,
so this runs on any ROCm host. The scheduler sources are plain C++17 and are compiled by the same
driver so that one shared object carries the whole C ABI of include/pat_amd.h.

_prefix_attn.so: the pybind11 / libtorch binding over that C ABI (host code only, g++), linked
against libpat_amd.so (found through its own directory at run time) and the installed torch.
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
# Packed-FP32 VALU forms are switched off for all device code. Kernel arguments: the leading scalar
# arguments of a kernel (up to 16 dwords) arrive in SGPRs with the wave instead of through a first
# load from the argument buffer - the split and merge kernels put what their first memory reads
# need there (-0.2 .. -0.5 us per launch).
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-ffp-contract=off", "-mllvm", "-amdgpu-kernarg-preload-count=16"]


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
    # No RUNPATH to the ROCm the library was built with: a process has ONE HIP runtime. Where torch is
    # loaded, its own libamdhip64 (same SONAME) serves this library too; elsewhere the loader's
    # configured search path (ld.so.conf / LD_LIBRARY_PATH) finds the system's.
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-rtlib-add-rpath", "-o", tmp, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"linking libpat_amd.so failed:\n{res.stderr}")
    os.replace(tmp, OUT)
    return OUT


EXT_SRC = os.path.join(CSRC, "torch_ext", "prefix_attn_ext.cc")
EXT_OUT = os.path.join(HERE, "_prefix_attn.so")


def build_extension(verbose: bool = False) -> str:
    """Compiles the torch binding (one translation unit, about a minute) and links it."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce

    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        raise RuntimeError("g++ not found: needed for the torch extension")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    includes = [os.path.join(ROOT, "include"), *ce.include_paths(), os.path.join(rocm, "include"),
                sysconfig.get_paths()["include"]]
    abi = int(bool(torch._C._GLIBCXX_USE_CXX11_ABI))
    tmp = EXT_OUT + ".tmp"
    cmd = [cxx, "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wno-unused-parameter", "-Wno-sign-compare",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
           "-DTORCH_EXTENSION_NAME=_prefix_attn", "-DTORCH_API_INCLUDE_EXTENSION_H",
           *[f"-isystem{p}" if "torch" in p or "rocm" in p else f"-I{p}" for p in includes],
           EXT_SRC, "-o", tmp,
           # torch's libraries come before libpat_amd in the dependency list: the loader then maps
           # torch's HIP runtime first and resolves libpat_amd's libamdhip64.so.7 to that same object
           f"-L{torch_lib}", "-ltorch_python", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
           f"-L{HERE}", "-lpat_amd", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"building the torch extension failed:\n{res.stderr[-4000:]}")
    os.replace(tmp, EXT_OUT)
    return EXT_OUT


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("-v", "--verbose", action="store_true")
    ap.add_argument("--no-extension", action="store_true", help="only libpat_amd.so (seconds), not the torch binding")
    a = ap.parse_args()
    ap_ext = not a.no_extension
    print(build(a.jobs, a.verbose))
    if ap_ext:
        print(build_extension(a.verbose))


if __name__ == "__main__":
    main()
