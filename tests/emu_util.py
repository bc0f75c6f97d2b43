"""Builds and loads the CPU build of the library's kernels (tests/emu): their unmodified sources compiled for the host
against a stand-in for <hip/hip_runtime.h> that runs a wavefront as a host thread and its lanes as contexts on it, and
against CPU models of the gfx950 instructions they use (tests/emu/gfx950_insn_emu.hpp).  Test infrastructure.

Two libraries.  build() / Emu: api.cpp, metadata.cpp, softmax.hip, cast.hip, reduce.hip, gemm_generic.hip and
gemm_refsum.hip -- the kernels without matrix-core or LDS-DMA instructions; every other launcher answers UNSUPPORTED,
which routes every product to the generic kernel.  Emu takes numpy arrays as operands.  build(mfma=True) / EmuContext:
all kernel families, with the real variant selection; EmuContext is hodu_amd.ffi.Context over that library, so the
GPU tests' helpers and test functions run against it unchanged.

Arithmetic is the host's (libm's expf, one summation order inside an MFMA), so float results are compared at the
parity tolerances and bit for bit only where the kernels' arithmetic is integer, pure bit manipulation, or exact by
the choice of operands."""
import ctypes
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import numpy as np

from hodu_amd import ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU = os.path.join(ROOT, "tests", "emu")
# HODU_EMU_SANITIZE=1: an undefined-behaviour-checked build of its own; =thread: a race-checked one, which only a
# program that carries the ThreadSanitizer runtime can load (build_race_driver, build_race_checked_python)
RACE_CHECKED = os.environ.get("HODU_EMU_SANITIZE", "") == "thread"
ADDRESS_CHECKED = os.environ.get("HODU_EMU_SANITIZE", "") == "address"  # likewise, with AddressSanitizer
SANITIZE = os.environ.get("HODU_EMU_SANITIZE", "") not in ("", "0") and not RACE_CHECKED and not ADDRESS_CHECKED
OUT = os.path.join(EMU, "_build_tsan" if RACE_CHECKED else "_build_asan" if ADDRESS_CHECKED else "_build_ubsan" if SANITIZE else "_build")
CSRC = os.path.join(ROOT, "hodu_amd", "csrc")
SOURCES = [os.path.join(CSRC, f) for f in ("api.cpp", "metadata.cpp", "softmax.hip", "cast.hip", "reduce.hip", "gemm_generic.hip", "gemm_refsum.hip")] + \
          [os.path.join(EMU, "emu_runtime.cpp")]
LIB = os.path.join(OUT, "libhodu_emu.so")
MFMA_SOURCES = [os.path.join(CSRC, f) for f in ("gemm_mfma.hip", "gemm_mfma_bf16.hip", "gemm_mfma_mi16_bf16.hip", "gemm_mfma_w8a16.hip",
                                                "gemm_mfma_f16.hip", "gemm_mfma_mi16_f16.hip", "gemm_mfma_f32.hip", "gemm_mfma_i8.hip",
                                                "gemm_mfma_i8_out.hip", "gemm_mfma_u8_out.hip", "gemm_mfma_f8.hip", "skinny.hip",
                                                "gemv.hip", "gemv_rows.hip", "small_f32.hip", "gemm_f64.hip", "attention.hip", "runtime.cpp")] + \
               [os.path.join(ROOT, "hodu_amd", "csrc_debug", "timing.cpp")]
MFMA_LIB = os.path.join(OUT, "libhodu_emu_mfma.so")


def compiler():
    for c in ("/opt/rocm/llvm/bin/clang++", shutil.which("amdclang++"), shutil.which("clang++")):
        if c and os.path.exists(c):
            return c
    return None


def _newest_input():
    paths = list(SOURCES) + list(MFMA_SOURCES) + [os.path.join(EMU, "hip", "hip_runtime.h"), os.path.join(EMU, "gfx950_insn_emu.hpp"), os.path.join(EMU, "emu_models.cpp"),
                                                  os.path.join(ROOT, "include", "hodu_rocm_kernels.h"), os.path.abspath(__file__)]
    paths += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    return max(os.path.getmtime(p) for p in paths)


def build(mfma=False, race_checked=RACE_CHECKED):
    """compiles the CPU build unless it is newer than every input; returns the library's path (None: no host clang).
    race_checked: a build of its own under ThreadSanitizer, for a natively linked program (build_race_driver)"""
    cxx = compiler()
    if cxx is None:
        return None
    OUT = os.path.join(EMU, "_build_tsan") if race_checked else globals()["OUT"]
    lib = os.path.join(OUT, os.path.basename(MFMA_LIB if mfma else LIB))
    if os.path.exists(lib) and os.path.getmtime(lib) > _newest_input():
        return lib
    os.makedirs(OUT, exist_ok=True)
    sanitize = SANITIZE and not race_checked
    flags = ["-std=c++17", "-fPIC", "-x", "c++", f"-I{EMU}", f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}",
             "-Wno-unused-function", "-Wno-unknown-attributes", "-Wno-psabi"]
    if sanitize:
        # undefined behaviour in the kernels' and the host code's own arithmetic (signed overflow in index arithmetic,
        # shifts, out-of-range conversions, indexing past a fixed-size array) aborts with a report.  Not the alignment
        # check: the kernels' 16-byte accesses at element alignment are what the hardware does.
        flags += ["-fsanitize=undefined", "-fno-sanitize=alignment,vptr,function", "-fno-sanitize-recover=all", "-g1"]
    if ADDRESS_CHECKED and not race_checked:
        # every access of host code and kernels against the red zones around heap blocks, globals (the LDS array, the
        # static scratch) and stack frames (the kernels' fixed-size register arrays)
        flags += ["-fsanitize=address", "-fno-omit-frame-pointer", "-g1"]
    if race_checked:
        # every load and store of the kernels' source is recorded per host thread, i.e. per wavefront.  Not function
        # entries and exits: the lanes of a wavefront are contexts that one thread switches between in the middle of
        # functions, which the sanitizer's per-thread call stack cannot follow (reports name the accessing line only).
        flags += ["-fsanitize=thread", "-mllvm", "-tsan-instrument-func-entry-exit=0", "-g1"]
    with_models = ["-DEMU_WITH_RUNTIME", "-include", os.path.join(EMU, "gfx950_insn_emu.hpp")]
    # Without optimisation: a fifth of the compile time (cast.hip alone takes a minute at -O1), and a run spends its
    # time starting threads and in the lanes' barriers, not in the kernels' arithmetic.
    jobs = [(src, "", ["-O0"]) for src in SOURCES]
    if mfma:
        # the plain kernels keep their static __shared__ arrays; only the runtime and the tile kernels see the models
        jobs = [(src, ".mfma" if src.endswith("emu_runtime.cpp") else "", ["-O0"] + (with_models if src.endswith("emu_runtime.cpp") else []))
                for src in SOURCES] + [(src, ".mfma", ["-O0"] + with_models) for src in MFMA_SOURCES] + \
               [(os.path.join(EMU, "emu_models.cpp"), ".mfma", ["-O2", "-ffp-contract=off"])]

    def one(job):
        src, tag, extra = job
        obj = os.path.join(OUT, os.path.basename(src) + tag + ".o")
        if os.path.exists(obj) and os.path.getmtime(obj) > _newest_input():
            return obj
        tmp_obj = obj + f".{os.getpid()}.tmp"
        r = subprocess.run([cxx, *flags, *extra, "-c", src, "-o", tmp_obj], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"CPU build of {src} failed:\n{r.stderr[-4000:]}")
        os.replace(tmp_obj, obj)
        return obj
    with ThreadPoolExecutor(max_workers=7) as ex:
        objs = list(ex.map(one, jobs))
    tmp = lib + f".{os.getpid()}.tmp"
    r = subprocess.run([cxx, "-shared", "-o", tmp, *objs, "-lpthread", *(["-fsanitize=undefined", "-shared-libsan"] if sanitize else [])],
                       capture_output=True, text=True)  # (race_checked: the program that links it brings the runtime)
    if r.returncode != 0:
        raise RuntimeError(f"link of the CPU build failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, lib)
    return lib


def build_race_driver():
    """tests/emu/race_driver.cpp linked with the ThreadSanitizer build of all kernels; returns the program's path"""
    kernels = build(mfma=True, race_checked=True)
    if kernels is None:
        return None
    out_dir = os.path.dirname(kernels)
    exe, src = os.path.join(out_dir, "race_driver"), os.path.join(EMU, "race_driver.cpp")
    if os.path.exists(exe) and os.path.getmtime(exe) > max(os.path.getmtime(kernels), os.path.getmtime(src)):
        return exe
    tmp = exe + f".{os.getpid()}.tmp"
    cmd = [compiler(), "-std=c++17", "-O0", "-g1", "-fsanitize=thread", "-mllvm", "-tsan-instrument-func-entry-exit=0", "-x", "c++",
           f"-I{EMU}", f"-I{os.path.join(ROOT, 'include')}", f"-I{CSRC}", f"-I{os.path.join(ROOT, 'hodu_amd', 'csrc_debug')}",
           "-Wno-unused-function", "-Wno-unknown-attributes", "-Wno-psabi", "-DEMU_WITH_RUNTIME", "-include", os.path.join(EMU, "gfx950_insn_emu.hpp"),
           src, "-o", tmp, f"-L{out_dir}", "-lhodu_emu_mfma", "-lpthread", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"race driver failed to build:\n{r.stderr[-4000:]}")
    os.replace(tmp, exe)
    return exe


def build_race_checked_python(sanitizer="thread"):
    """tests/emu/python_host.cpp: this Python with the ThreadSanitizer (or AddressSanitizer) runtime linked in; returns
    the program's path (None: no host clang, or no Python headers / library to link)"""
    import sysconfig
    cxx, inc, libdir = compiler(), sysconfig.get_paths()["include"], sysconfig.get_config_var("LIBDIR")
    ver = sysconfig.get_config_var("LDVERSION")
    if cxx is None or not os.path.exists(os.path.join(inc, "Python.h")) or not ver:
        return None
    out_dir = os.path.join(EMU, "_build_tsan" if sanitizer == "thread" else "_build_asan")
    os.makedirs(out_dir, exist_ok=True)
    exe, src = os.path.join(out_dir, "python_tsan" if sanitizer == "thread" else "python_asan"), os.path.join(EMU, "python_host.cpp")
    if os.path.exists(exe) and os.path.getmtime(exe) > os.path.getmtime(src):
        return exe
    tmp = exe + f".{os.getpid()}.tmp"
    r = subprocess.run([cxx, "-O1", f"-fsanitize={sanitizer}", f"-I{inc}", src, "-o", tmp, f"-L{libdir}", f"-lpython{ver}", "-ldl", "-lm"],
                       capture_output=True, text=True)
    if r.returncode != 0:
        return None
    os.replace(tmp, exe)
    return exe


HOST_LIB = os.path.join(OUT, "libhodu_emu_host.so")


def build_host():
    """the host mirror's compiled library (hodu_amd/host/capi.cpp, unmodified) linked against the CPU build of all
    kernels instead of the real kernel library; returns its path (None: no host clang)"""
    kernels = build(mfma=True)
    if kernels is None:
        return None
    host_dir = os.path.join(ROOT, "hodu_amd", "host")
    inputs = [os.path.join(host_dir, f) for f in os.listdir(host_dir)] + [kernels]
    if os.path.exists(HOST_LIB) and os.path.getmtime(HOST_LIB) > max(os.path.getmtime(p) for p in inputs):
        return HOST_LIB
    tmp = HOST_LIB + f".{os.getpid()}.tmp"
    cmd = [compiler(), "-std=c++17", "-O1", "-fPIC", "-shared", f"-I{os.path.join(ROOT, 'include')}", f"-I{host_dir}",
           os.path.join(host_dir, "capi.cpp"), "-o", tmp, f"-L{OUT}", "-lhodu_emu_mfma", "-Wl,-rpath,$ORIGIN",
           *(["-fsanitize=address", "-fno-omit-frame-pointer", "-g1"] if ADDRESS_CHECKED else [])]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"host mirror over the CPU build failed to build:\n{r.stderr[-4000:]}")
    os.replace(tmp, HOST_LIB)
    return HOST_LIB


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
        lib.emu_unsupported_first.restype = ctypes.c_char_p
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
        if self.lib.emu_unsupported_hits() != 0:
            first = self.lib.emu_unsupported_first().decode()
            self.lib.emu_unsupported_reset()
            raise AssertionError(f"{what} ({self.last_kernel()}) reached an instruction without a CPU stand-in: {first}")

    def last_kernel(self):
        return self.lib.emu_last_kernel(self.ctx).decode()

    def set_reference_sums(self, on):
        self.lib.hodu_rocm_ctx_set_reference_sums.argtypes = [ctypes.c_void_p, ctypes.c_int]
        assert self.lib.hodu_rocm_ctx_set_reference_sums(self.ctx, int(on)) == 0

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


# ---- hodu_amd.ffi.Context over the CPU build, so that the GPU tests' helpers and test functions run against it unchanged ----
class EmuContext(ffi.Context):
    """hodu_amd.ffi.Context with the CPU build of the whole library (build(mfma=True): every kernel family, api.cpp,
    runtime.cpp, the debug library's timing.cpp) in the place of the HIP libraries: the same Python methods with their
    host-side extent checks, the same entry points and hooks, hodu_rocm_alloc handing out host memory between two
    inaccessible pages.  What it adds are the switches of the instruction models."""

    _emu_lib = None

    @classmethod
    def library(cls):
        if cls._emu_lib is None:
            path = build(mfma=True)
            if path is None:
                raise RuntimeError("no host clang++ to build tests/emu with")
            lib = ctypes.CDLL(path)
            ffi.declare_runtime(lib)
            ffi.declare_compute(lib)
            ffi.declare_debug(lib)
            lib.emu_unsupported_first.restype = ctypes.c_char_p
            lib.emu_lds_fill.argtypes = [ctypes.c_int]
            lib.emu_alloc_tight.argtypes = [ctypes.c_int]
            lib.emu_dma_lazy.argtypes = [ctypes.c_int]
            cls._emu_lib = lib
        return cls._emu_lib

    def __init__(self, device=0, tight="end"):
        self.lib = self.library()
        h = ctypes.c_void_p()
        rc = self.lib.hodu_rocm_ctx_create(int(device), ctypes.byref(h))
        self.handle = h.value if rc == 0 else None
        if rc != 0:
            raise ffi.HoduRocmError(rc, self.lib.hodu_rocm_last_error(None).decode())
        self.device = device
        self.tight = tight

    @property
    def tight(self):
        return self._tight

    @tight.setter
    def tight(self, where):
        """which end of an allocation touches its guard page: "end" (a clamped row or a biased pointer would overrun
        there) or "start"; applies to allocations made from now on, by any context"""
        self._tight = where
        self.lib.emu_alloc_tight(int(where == "end"))

    @property
    def debug(self):
        return self.lib  # the hooks are part of the same library here

    def _check(self, rc):
        super()._check(rc)
        if self.lib.emu_unsupported_hits() != 0:
            first = self.lib.emu_unsupported_first().decode()
            self.lib.emu_unsupported_reset()
            raise AssertionError(f"{self.last_kernel()} reached an instruction without a CPU stand-in: {first}")

    def dma_lazy(self, model):
        """LDS-DMA bytes arrive at issue (0), only when an s_waitcnt vmcnt retires them (1), or one load later than
        that (2: a model under which a correct kernel must FAIL)"""
        self.lib.emu_dma_lazy(int(model))

    def lds_fill(self, byte):
        self.lib.emu_lds_fill(int(byte))
