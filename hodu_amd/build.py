"""Builds hodu_amd/lib/libhodu_rocm_kernels.so from hodu_amd/csrc with hipcc for gfx950.

hipcc cross-compiles without a GPU, so this runs in the build container; the resulting library is
kept in-tree (git-ignored) and loaded by hodu_amd.ffi.  `python -m hodu_amd.build` rebuilds it.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_build")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libhodu_rocm_kernels.so")
DEBUG_SRC = os.path.join(HERE, "csrc_debug")
DEBUG_LIB = os.path.join(LIB_DIR, "libhodu_rocm_debug.so")
HOST_DIR = os.path.join(HERE, "host")
HOST_LIB = os.path.join(LIB_DIR, "libhodu_rocm_host.so")

ARCH = "gfx950"
# -packed-fp32-ops off: keep hipcc from forming v_pk_{add,mul,fma}_f32 out of scalar float code
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the K loops are written as fully unrolled compile-time schedules; the default pragma-unroll size limit
    # would quietly leave the largest tile rolled (accumulators indexed at run time, i.e. in scratch memory)
    "-mllvm", "-pragma-unroll-threshold=200000",
    f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
]


def hipcc() -> str:
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        raise RuntimeError("hipcc not found: the HIP extension cannot be built on this machine")
    return path


_ONLY_CHANGED = False  # `python -m hodu_amd.build --changed`: keep objects newer than their source and every header


def _deps_mtime(src: str, dep: str) -> float:
    """newest of the source and the project headers the last compile of it read (the compiler's own -MD list)"""
    newest = os.path.getmtime(src)
    try:
        words = open(dep).read().replace("\\\n", " ").split()
    except OSError:
        return float("inf")
    for w in words[1:]:
        if w.startswith(ROOT) and os.path.exists(w):
            newest = max(newest, os.path.getmtime(w))
    return newest


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.basename(os.path.dirname(src)) + "_" + os.path.basename(src) + ".o")
    dep = obj + ".d"
    if _ONLY_CHANGED and os.path.exists(obj) and os.path.getmtime(obj) > _deps_mtime(src, dep):
        return obj
    cmd = [hipcc(), *FLAGS, "-MD", "-MF", dep, "-c", src, "-o", obj]
    if src.endswith(".cpp"):
        cmd[1:1] = ["-x", "hip"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-6000:]}")
    return obj


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def build(verbose: bool = True, jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = LIB + ".tmp"
    r = subprocess.run([hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, LIB)
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources", file=sys.stderr)
    build_debug(verbose, jobs)
    build_host(verbose)
    return LIB


def build_debug(verbose: bool = True, jobs: int = 8) -> str:
    """The test and measurement hooks (include/hodu_rocm_debug.h): a library of their own on top of the kernel
    library, so that the kernel library exports the boundary and nothing else."""
    srcs = sorted(os.path.join(DEBUG_SRC, f) for f in os.listdir(DEBUG_SRC) if f.endswith((".hip", ".cpp")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = DEBUG_LIB + ".tmp"
    r = subprocess.run([hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs, f"-L{LIB_DIR}",
                        "-lhodu_rocm_kernels", "-Wl,-rpath,$ORIGIN"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link of the hooks library failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, DEBUG_LIB)
    if verbose:
        print(f"built {DEBUG_LIB} from {len(srcs)} sources", file=sys.stderr)
    return DEBUG_LIB


def build_host(verbose: bool = True) -> str:
    """The host-side Tensor/Layout/storage mirror: plain C++ over the C ABI, linked against the kernel library."""
    tmp = HOST_LIB + ".tmp"
    cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wextra", f"-I{os.path.join(ROOT, 'include')}",
           f"-I{HOST_DIR}", os.path.join(HOST_DIR, "capi.cpp"), "-o", tmp, f"-L{LIB_DIR}", "-lhodu_rocm_kernels",
           "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"host library build failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, HOST_LIB)
    if verbose:
        print(f"built {HOST_LIB}", file=sys.stderr)
    return HOST_LIB


if __name__ == "__main__":
    _ONLY_CHANGED = "--changed" in sys.argv
    build()
