"""Builds and loads the CPU build of the library's plain kernels (tests/emu): the unmodified sources of api.cpp,
metadata.cpp, softmax.hip, cast.hip, reduce.hip and gemm_generic.hip compiled for the host against a stand-in for
<hip/hip_runtime.h> that runs a workgroup as host threads.  Test infrastructure: what it proves is indexing, masking,
reduction structure and the entry points' argument handling -- arithmetic is the host's, so results are compared at the
parity tolerances, bit for bit only where the kernel's arithmetic is integer or pure bit manipulation.  The matrix-core
and LDS-DMA kernels have no CPU build; their launchers answer UNSUPPORTED here, which routes every product to the
generic kernel."""
import ctypes
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU = os.path.join(ROOT, "tests", "emu")
OUT = os.path.join(EMU, "_build")
CSRC = os.path.join(ROOT, "hodu_amd", "csrc")
SOURCES = [os.path.join(CSRC, f) for f in ("api.cpp", "metadata.cpp", "softmax.hip", "cast.hip", "reduce.hip", "gemm_generic.hip")] + \
          [os.path.join(EMU, "emu_runtime.cpp")]
LIB = os.path.join(OUT, "libhodu_emu.so")


def compiler():
    for c in ("/opt/rocm/llvm/bin/clang++", shutil.which("amdclang++"), shutil.which("clang++")):
        if c and os.path.exists(c):
            return c
    return None


def _newest_input():
    paths = list(SOURCES) + [os.path.join(EMU, "hip", "hip_runtime.h"), os.path.join(ROOT, "include", "hodu_rocm_kernels.h")]
    paths += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    return max(os.path.getmtime(p) for p in paths)


def build():
    """compiles the CPU build unless it is newer than every input; returns the library's path (None: no host clang)"""
    cxx = compiler()
    if cxx is None:
        return None
    if os.path.exists(LIB) and os.path.getmtime(LIB) > _newest_input():
        return LIB
    os.makedirs(OUT, exist_ok=True)
    flags = ["-std=c++17", "-O1", "-fPIC", "-x", "c++", f"-I{EMU}", f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
             "-Wno-unused-function", "-Wno-unknown-attributes"]

    def one(src):
        obj = os.path.join(OUT, os.path.basename(src) + ".o")
        r = subprocess.run([cxx, *flags, "-c", src, "-o", obj], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"CPU build of {src} failed:\n{r.stderr[-4000:]}")
        return obj
    with ThreadPoolExecutor(max_workers=7) as ex:
        objs = list(ex.map(one, SOURCES))
    tmp = LIB + ".tmp"
    r = subprocess.run([cxx, "-shared", "-o", tmp, *objs, "-lpthread"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link of the CPU build failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, LIB)
    return LIB


DTYPE_ID = {"bool": 0, "f8e4m3": 1, "f8e5m2": 2, "bf16": 3, "f16": 4, "f32": 5, "f64": 6, "u8": 7, "u16": 8, "u32": 9,
            "u64": 10, "i8": 11, "i16": 12, "i32": 13, "i64": 14}


class Emu:
    """the entry points of api.cpp as compiled for the host; every pointer argument is a numpy array"""

    def __init__(self):
        path = build()
        if path is None:
            raise RuntimeError("no host clang++ to build tests/emu with")
        self.lib = lib = ctypes.CDLL(path)
        vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
        szp = ctypes.POINTER(sz)
        lib.emu_ctx_create.restype = vp
        lib.emu_ctx_destroy.argtypes = [vp]
        lib.emu_last_kernel.restype = ctypes.c_char_p
        lib.emu_last_kernel.argtypes = [vp]
        lib.emu_last_error.restype = ctypes.c_char_p
        lib.hodu_rocm_softmax.argtypes = [vp, ci, vp, vp, szp, sz, ci]
        lib.hodu_rocm_softmax_masked.argtypes = [vp, ci, vp, vp, szp, sz, ci, vp, ci, szp, sz]
        lib.hodu_rocm_cast.argtypes = [vp, ci, ci, vp, vp, szp, sz]
        lib.hodu_rocm_contiguous.argtypes = [vp, ci, vp, vp, szp, sz]
        lib.hodu_rocm_sum.argtypes = [vp, ci, vp, vp, szp, sz]
        self.ctx = lib.emu_ctx_create()

    def close(self):
        if self.ctx:
            self.lib.emu_ctx_destroy(self.ctx)
            self.ctx = None

    @staticmethod
    def _md(md):
        return (ctypes.c_size_t * len(md))(*[int(v) for v in md]), len(md)

    def _check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what}: status {rc}: {self.lib.emu_last_error().decode()}")
        assert self.lib.emu_unsupported_hits() == 0, f"{what} reached an instruction without a CPU stand-in"

    def last_kernel(self):
        return self.lib.emu_last_kernel(self.ctx).decode()

    def softmax(self, dt, x, out, md, causal=False):
        a, n = self._md(md)
        self._check(self.lib.hodu_rocm_softmax(self.ctx, DTYPE_ID[dt], x.ctypes.data, out.ctypes.data, a, n, int(causal)), "softmax")

    def softmax_masked(self, dt, x, out, md, mask, mask_strides, mask_offset=0, causal=False, mask_dt="u8"):
        a, n = self._md(md)
        la, ln = self._md([len(mask_strides)] + list(mask_strides) + [mask_offset])
        self._check(self.lib.hodu_rocm_softmax_masked(self.ctx, DTYPE_ID[dt], x.ctypes.data, out.ctypes.data, a, n, int(causal),
                                                      mask.ctypes.data, DTYPE_ID[mask_dt], la, ln), "softmax_masked")

    def cast(self, src, dst, x, out, md):
        a, n = self._md(md)
        self._check(self.lib.hodu_rocm_cast(self.ctx, DTYPE_ID[src], DTYPE_ID[dst], x.ctypes.data, out.ctypes.data, a, n), "cast")

    def contiguous(self, dt, x, out, md):
        a, n = self._md(md)
        self._check(self.lib.hodu_rocm_contiguous(self.ctx, DTYPE_ID[dt], x.ctypes.data, out.ctypes.data, a, n), "contiguous")

    def sum(self, dt, x, out, md):
        a, n = self._md(md)
        self._check(self.lib.hodu_rocm_sum(self.ctx, DTYPE_ID[dt], x.ctypes.data, out.ctypes.data, a, n), "sum")

    def product(self, op, name, a, b, out, md):
        fn = getattr(self.lib, f"hodu_rocm_{op}_{name}")
        fn.argtypes = [ctypes.c_void_p] * 4 + [ctypes.POINTER(ctypes.c_size_t), ctypes.c_size_t]
        arr, n = self._md(md)
        self._check(fn(self.ctx, a.ctypes.data, b.ctypes.data, out.ctypes.data, arr, n), f"{op}_{name}")
