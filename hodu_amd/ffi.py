"""ctypes binding of include/hodu_rocm_kernels.h -- the same C ABI a Rust `hodu_rocm_kernels`
crate would bind.  Loading fails loudly when the HIP library has not been built: there is no CPU
fallback anywhere in this package.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libhodu_rocm_kernels.so")
# test and measurement hooks (include/hodu_rocm_debug.h): a library of their own, not part of the boundary
DEBUG_LIB_PATH = os.path.join(_HERE, "lib", "libhodu_rocm_debug.so")

OK, INVALID_ARG, UNSUPPORTED, HIP_ERROR, OOM, SCRATCH = 0, 1, 2, 3, 4, 5
_STATUS = {1: "INVALID_ARG", 2: "UNSUPPORTED", 3: "HIP_ERROR", 4: "OOM", 5: "SCRATCH"}

# dtype ids: crates/hodu_core/src/types/dtype.rs:6-28
DTYPE_ID = {
    "bool": 0, "f8e4m3": 1, "f8e5m2": 2, "bf16": 3, "f16": 4, "f32": 5, "f64": 6,
    "u8": 7, "u16": 8, "u32": 9, "u64": 10, "i8": 11, "i16": 12, "i32": 13, "i64": 14,
}
DTYPE_SIZE = {"bool": 1, "f8e4m3": 1, "f8e5m2": 1, "bf16": 2, "f16": 2, "f32": 4, "f64": 8, "u8": 1, "u16": 2,
              "u32": 4, "u64": 8, "i8": 1, "i16": 2, "i32": 4, "i64": 8}
PRODUCT_DTYPES = [d for d in DTYPE_ID if d != "bool"]
FUSED_PRODUCTS = ("bf16_f8e4m3w", "i32_i8i8")


class HoduRocmError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"hodu_rocm {_STATUS.get(status, status)}: {message}")
        self.status = status
        self.message = message


_lib: Optional[ctypes.CDLL] = None
_debug_lib: Optional[ctypes.CDLL] = None


class EpilogueStep(ctypes.Structure):
    """hodu_rocm_epilogue_step of include/hodu_rocm_kernels.h"""
    _fields_ = [("op", ctypes.c_int), ("vector", ctypes.c_void_p), ("stride", ctypes.c_size_t),
                ("offset", ctypes.c_size_t), ("scalar", ctypes.c_ubyte * 8)]


EPI_ADD_ROW, EPI_MUL_SCALAR, EPI_RELU = 1, 2, 3
# dtypes whose products take fused element-wise steps (the 8-bit floats do not)
EPILOGUE_DTYPES = ["bf16", "f16", "f32", "f64", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]


def add_row(vector: "DeviceBuffer", stride: int = 1, offset: int = 0) -> EpilogueStep:
    """out[.., m, n] += vector[offset + n * stride] (a bias along the last axis)"""
    return EpilogueStep(EPI_ADD_ROW, vector.ptr, int(stride), int(offset), (ctypes.c_ubyte * 8)())


def mul_scalar(scalar) -> EpilogueStep:
    """out *= scalar; scalar: a numpy scalar / 1-element array in the output dtype's storage"""
    raw = np.ascontiguousarray(scalar).reshape(1).tobytes()
    buf = (ctypes.c_ubyte * 8)(*raw, *([0] * (8 - len(raw))))
    return EpilogueStep(EPI_MUL_SCALAR, None, 0, 0, buf)


def relu() -> EpilogueStep:
    return EpilogueStep(EPI_RELU, None, 0, 0, (ctypes.c_ubyte * 8)())


def _steps_array(steps):
    steps = list(steps)
    return (EpilogueStep * max(1, len(steps)))(*steps), len(steps)


def declare_runtime(lib: ctypes.CDLL):
    """argument types of the context, memory and timing entry points"""
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    lib.hodu_rocm_device_count.argtypes = [ctypes.POINTER(ci)]
    lib.hodu_rocm_ctx_create.argtypes = [ci, ctypes.POINTER(vp)]
    lib.hodu_rocm_ctx_destroy.argtypes = [vp]
    lib.hodu_rocm_alloc.argtypes = [vp, sz, ctypes.POINTER(vp)]
    lib.hodu_rocm_free.argtypes = [vp, vp]
    lib.hodu_rocm_memcpy_h2d.argtypes = [vp, vp, vp, sz]
    lib.hodu_rocm_memcpy_d2h.argtypes = [vp, vp, vp, sz]
    lib.hodu_rocm_memcpy_d2d.argtypes = [vp, vp, vp, sz]
    lib.hodu_rocm_memset.argtypes = [vp, vp, ci, sz]
    lib.hodu_rocm_sync.argtypes = [vp]
    lib.hodu_rocm_last_error.argtypes = [vp]
    lib.hodu_rocm_last_error.restype = ctypes.c_char_p
    lib.hodu_rocm_last_kernel.argtypes = [vp]
    lib.hodu_rocm_last_kernel.restype = ctypes.c_char_p
    lib.hodu_rocm_device_info.argtypes = [vp, ctypes.c_char_p, sz, ctypes.POINTER(ci), ctypes.POINTER(ci),
                                          ctypes.POINTER(sz)]
    lib.hodu_rocm_timer_create.argtypes = [vp, ctypes.POINTER(vp)]
    lib.hodu_rocm_timer_start.argtypes = [vp, vp]
    lib.hodu_rocm_timer_stop.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_float)]
    lib.hodu_rocm_timer_destroy.argtypes = [vp, vp]


def declare_compute(lib: ctypes.CDLL):
    """argument types of the compute entry points (everything in include/hodu_rocm_kernels.h that launches kernels)"""
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    szp = ctypes.POINTER(ctypes.c_size_t)
    for dt in PRODUCT_DTYPES + list(FUSED_PRODUCTS):
        for op in ("matmul", "dot"):
            getattr(lib, f"hodu_rocm_{op}_{dt}").argtypes = [vp, vp, vp, vp, szp, sz]
    for dt in EPILOGUE_DTYPES + list(FUSED_PRODUCTS):
        for op in ("matmul", "dot"):
            getattr(lib, f"hodu_rocm_{op}_{dt}_ex").argtypes = [vp, vp, vp, vp, szp, sz, ctypes.POINTER(EpilogueStep), sz]
    lib.hodu_rocm_cast.argtypes = [vp, ci, ci, vp, vp, szp, sz]
    lib.hodu_rocm_contiguous.argtypes = [vp, ci, vp, vp, szp, sz]
    lib.hodu_rocm_sum.argtypes = [vp, ci, vp, vp, szp, sz]
    lib.hodu_rocm_softmax.argtypes = [vp, ci, vp, vp, szp, sz, ci]
    lib.hodu_rocm_softmax_masked.argtypes = [vp, ci, vp, vp, szp, sz, ci, vp, ci, szp, sz]
    lib.hodu_rocm_attention.argtypes = [vp, ci, vp, vp, vp, vp, szp, sz, vp, ci]
    lib.hodu_rocm_attention_masked.argtypes = [vp, ci, vp, vp, vp, vp, szp, sz, vp, ci, vp, ci, szp, sz]
    lib.hodu_rocm_dot_bf16_f8e4m3w_noalloc.argtypes = [vp, vp, vp, vp, szp, sz]
    lib.hodu_rocm_ctx_set_reference_sums.argtypes = [vp, ci]


def load() -> ctypes.CDLL:
    """Load the built HIP library; raises if it is missing (build with `python -m hodu_amd.build`)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build the HIP extension first (python -m hodu_amd.build). "
            "hodu_amd has no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    declare_runtime(lib)
    declare_compute(lib)
    _lib = lib
    return lib


def declare_debug(lib: ctypes.CDLL):
    """argument types of the hooks library (include/hodu_rocm_debug.h)"""
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    szp, fp = ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_float)
    vpp = ctypes.POINTER(vp)
    lib.hodu_rocm_debug_force_tile.argtypes = [vp, ci]
    lib.hodu_rocm_debug_force_splitk.argtypes = [vp, ci]
    lib.hodu_rocm_debug_scratch_state.argtypes = [vp, szp, ctypes.POINTER(ci), ctypes.POINTER(ci)]
    lib.hodu_rocm_debug_time_product.argtypes = [vp, ci, ci, ci, vp, vpp, sz, vp, szp, sz, ci, fp]
    lib.hodu_rocm_debug_time_product_graph.argtypes = lib.hodu_rocm_debug_time_product.argtypes
    lib.hodu_rocm_debug_time_product_ex.argtypes = [vp, ci, ci, ci, vp, vpp, sz, vp, szp, sz,
                                                    ctypes.POINTER(EpilogueStep), sz, ci, fp]
    lib.hodu_rocm_debug_time_noalloc.argtypes = [vp, vp, vpp, sz, vp, szp, sz, ci, ci, fp]
    lib.hodu_rocm_debug_time_cast.argtypes = [vp, ci, ci, vpp, vpp, sz, szp, sz, ci, fp]
    lib.hodu_rocm_debug_time_sum.argtypes = [vp, ci, vpp, vpp, sz, szp, sz, ci, fp]
    lib.hodu_rocm_debug_mfma_clock.argtypes = [vp, ci, vp, ci, fp, ctypes.POINTER(ctypes.c_double),
                                               ctypes.POINTER(ctypes.c_double)]
    lib.hodu_rocm_debug_read_floor.argtypes = [vp, vpp, sz, sz, ci, fp, fp]


def load_debug() -> ctypes.CDLL:
    """Load the hooks library (include/hodu_rocm_debug.h); it links against the kernel library."""
    global _debug_lib
    if _debug_lib is not None:
        return _debug_lib
    load()
    if not os.path.exists(DEBUG_LIB_PATH):
        raise ImportError(f"{DEBUG_LIB_PATH} is missing: build it first (python -m hodu_amd.build)")
    lib = ctypes.CDLL(DEBUG_LIB_PATH)
    declare_debug(lib)
    _debug_lib = lib
    return lib


def device_count() -> int:
    n = ctypes.c_int(0)
    load().hodu_rocm_device_count(ctypes.byref(n))
    return n.value


def _view_span(shape, strides, offset) -> int:
    """elements a strided view can touch: highest index + 1 (0 for an empty view)"""
    if any(int(d) == 0 for d in shape):
        return 0
    return int(offset) + sum((int(d) - 1) * int(s) for d, s in zip(shape, strides)) + 1


def product_spans(op: str, md: Sequence[int]):
    """(lhs elements, rhs elements, out elements) a matmul / dot metadata vector addresses.

    The C ABI receives bare pointers, as the reference's kernels do, so the extents of the buffers
    behind them can only be checked by the caller that owns them; this is that check."""
    md = [int(v) for v in md]
    if op == "dot":
        if len(md) != 9:
            return None
        m, k, n, am, ak, bk, bn, ao, bo = md
        return _view_span([m, k], [am, ak], ao), _view_span([k, n], [bk, bn], bo), m * n
    if len(md) < 4:
        return None
    lnd, rnd, bnd = md[1], md[2], md[3]
    if len(md) != 4 + 2 * lnd + 2 * rnd + bnd + 5:
        return None
    ls = md[4:4 + lnd]
    rs = md[4 + lnd:4 + lnd + rnd]
    p = 4 + lnd + rnd + bnd
    lst, rst = md[p:p + lnd], md[p + lnd:p + lnd + rnd]
    lo, ro = md[p + lnd + rnd], md[p + lnd + rnd + 1]
    return _view_span(ls, lst, lo), _view_span(rs, rst, ro), md[0]


def _md_array(md: Sequence[int]):
    arr = (ctypes.c_size_t * len(md))(*[int(v) for v in md])
    return arr, len(md)


class DeviceBuffer:
    """A device allocation owned by a Context (what CudaSlice is to the CUDA sibling)."""

    def __init__(self, ctx: "Context", nbytes: int):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        ctx._check(ctx.lib.hodu_rocm_alloc(ctx.handle, self.nbytes, ctypes.byref(p)))
        self.ptr = p.value

    def free(self):
        if self.ptr is not None and self.ctx.handle is not None:
            self.ctx.lib.hodu_rocm_free(self.ctx.handle, self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context:
    """One device context: stream, allocations, kernel launches (hodu_rocm_ctx)."""

    def __init__(self, device: int = 0):
        self.lib = load()
        h = ctypes.c_void_p()
        rc = self.lib.hodu_rocm_ctx_create(int(device), ctypes.byref(h))
        self.handle = h.value if rc == 0 else None
        if rc != 0:
            raise HoduRocmError(rc, self.lib.hodu_rocm_last_error(None).decode())
        self.device = device

    @property
    def debug(self) -> ctypes.CDLL:
        """the hooks library, loaded on first use (tests and bench.py only)"""
        return load_debug()

    def close(self):
        if self.handle is not None:
            self.lib.hodu_rocm_ctx_destroy(self.handle)
            self.handle = None

    def _check(self, rc: int):
        if rc != 0:
            raise HoduRocmError(rc, self.lib.hodu_rocm_last_error(self.handle).decode())

    # memory ---------------------------------------------------------------------------------
    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def upload_into(self, buf: DeviceBuffer, host: np.ndarray, first_byte: int = 0):
        """copy a host array into an existing buffer at a byte offset (large operands are filled piece by piece)"""
        host = np.ascontiguousarray(host)
        if first_byte < 0 or first_byte + host.nbytes > buf.nbytes:
            raise HoduRocmError(INVALID_ARG, "upload_into: the range lies outside the buffer")
        self._check(self.lib.hodu_rocm_memcpy_h2d(self.handle, buf.ptr + int(first_byte), host.ctypes.data, host.nbytes))

    def upload(self, host: np.ndarray) -> DeviceBuffer:
        host = np.ascontiguousarray(host)
        buf = DeviceBuffer(self, host.nbytes)
        self._check(self.lib.hodu_rocm_memcpy_h2d(self.handle, buf.ptr, host.ctypes.data, host.nbytes))
        return buf

    def download(self, buf: DeviceBuffer, dtype, count: Optional[int] = None, first: int = 0) -> np.ndarray:
        """`count` elements of `dtype` starting at element `first` of the buffer (default: all of it)"""
        dtype = np.dtype(dtype)
        first = int(first)
        n = buf.nbytes // dtype.itemsize - first if count is None else int(count)
        if first < 0 or n < 0 or (first + n) * dtype.itemsize > buf.nbytes:
            raise HoduRocmError(INVALID_ARG, "download: the range lies outside the buffer")
        out = np.empty(n, dtype=dtype)
        self._check(self.lib.hodu_rocm_memcpy_d2h(self.handle, out.ctypes.data, buf.ptr + first * dtype.itemsize, out.nbytes))
        return out

    def fill(self, buf: DeviceBuffer, byte: int):
        self._check(self.lib.hodu_rocm_memset(self.handle, buf.ptr, int(byte), buf.nbytes))

    def sync(self):
        self._check(self.lib.hodu_rocm_sync(self.handle))

    # compute --------------------------------------------------------------------------------
    def product(self, op: str, name: str, lhs: DeviceBuffer, rhs: DeviceBuffer, out: DeviceBuffer, md):
        """op in {'matmul','dot'}; name a dtype ('bf16') or a fused kind ('bf16_f8e4m3w')."""
        self._check_extents(op, name, lhs, [rhs], out, md)
        arr, n = _md_array(md)
        fn = getattr(self.lib, f"hodu_rocm_{op}_{name}")
        self._check(fn(self.handle, lhs.ptr, rhs.ptr, out.ptr, arr, n))

    def dot_noalloc(self, lhs: DeviceBuffer, rhs: DeviceBuffer, out: DeviceBuffer, md):
        """hodu_rocm_dot_bf16_f8e4m3w_noalloc: the fused f8e4m3-weight dot with its scratch in the library's static
        device array (no device allocation inside the call)"""
        self._check_extents("dot", "bf16_f8e4m3w", lhs, [rhs], out, md)
        arr, n = _md_array(md)
        self._check(self.lib.hodu_rocm_dot_bf16_f8e4m3w_noalloc(self.handle, lhs.ptr, rhs.ptr, out.ptr, arr, n))

    def time_noalloc(self, lhs: DeviceBuffer, rhs_list, out: DeviceBuffer, md, iters: int, graph: bool = False) -> float:
        """back-to-back calls of the entry point that allocates nothing, HIP-event timed; total ms"""
        self._check_extents("dot", "bf16_f8e4m3w", lhs, rhs_list, out, md)
        arr, n = _md_array(md)
        ptrs = (ctypes.c_void_p * len(rhs_list))(*[b.ptr for b in rhs_list])
        ms = ctypes.c_float()
        self._check(self.debug.hodu_rocm_debug_time_noalloc(self.handle, lhs.ptr, ptrs, len(rhs_list), out.ptr, arr, n,
                                                            int(iters), int(bool(graph)), ctypes.byref(ms)))
        return float(ms.value)

    def set_reference_sums(self, on: bool):
        """hodu_rocm_ctx_set_reference_sums: narrow-float products in the reference's own arithmetic (the running sum
        re-rounded to the dtype after every multiply and add), byte for byte hodu's CPU result; slow"""
        self._check(self.lib.hodu_rocm_ctx_set_reference_sums(self.handle, int(bool(on))))

    def product_ex(self, op: str, name: str, lhs: DeviceBuffer, rhs: DeviceBuffer, out: DeviceBuffer, md, steps):
        """hodu_rocm_<op>_<name>_ex: the product with element-wise steps (add_row / mul_scalar / relu) fused into
        its store"""
        self._check_extents(op, name, lhs, [rhs], out, md)
        arr, n = _md_array(md)
        sarr, ns = _steps_array(steps)
        fn = getattr(self.lib, f"hodu_rocm_{op}_{name}_ex")
        self._check(fn(self.handle, lhs.ptr, rhs.ptr, out.ptr, arr, n, sarr, ns))

    @staticmethod
    def _check_extents(op, name, lhs, rhs_list, out, md):
        """refuse a launch whose metadata reaches past one of the device buffers"""
        spans = product_spans(op, md)
        if spans is None:
            return  # malformed metadata: the library reports it
        l_sz, r_sz, o_sz = {"bf16_f8e4m3w": (2, 1, 2), "i32_i8i8": (1, 1, 4)}.get(name) or (DTYPE_SIZE[name],) * 3
        need = [("lhs", lhs, spans[0] * l_sz), ("out", out, spans[2] * o_sz)] + \
               [("rhs", r, spans[1] * r_sz) for r in rhs_list]
        for what, buf, nbytes in need:
            if nbytes > buf.nbytes:
                raise HoduRocmError(INVALID_ARG, f"{op}_{name}: metadata addresses {nbytes} bytes of {what} "
                                                 f"but the buffer holds {buf.nbytes}")

    @staticmethod
    def _check_strided(what, src_size, dst_size, x, out, md):
        md = [int(v) for v in md]
        if len(md) < 2 or len(md) != 2 + 2 * md[1] + 1:
            return
        nd = md[1]
        span = _view_span(md[2:2 + nd], md[2 + nd:2 + 2 * nd], md[2 + 2 * nd])
        if span * src_size > x.nbytes or md[0] * dst_size > out.nbytes:
            raise HoduRocmError(INVALID_ARG, f"{what}: metadata reaches past a device buffer")

    def cast(self, src: str, dst: str, x: DeviceBuffer, out: DeviceBuffer, md):
        self._check_strided(f"cast_{src}_to_{dst}", DTYPE_SIZE[src], DTYPE_SIZE[dst], x, out, md)
        arr, n = _md_array(md)
        self._check(self.lib.hodu_rocm_cast(self.handle, DTYPE_ID[src], DTYPE_ID[dst], x.ptr, out.ptr, arr, n))

    def contiguous(self, dt: str, x: DeviceBuffer, out: DeviceBuffer, md):
        self._check_strided(f"contiguous_{dt}", DTYPE_SIZE[dt], DTYPE_SIZE[dt], x, out, md)
        arr, n = _md_array(md)
        self._check(self.lib.hodu_rocm_contiguous(self.handle, DTYPE_ID[dt], x.ptr, out.ptr, arr, n))

    def sum(self, dt: str, x: DeviceBuffer, out: DeviceBuffer, md):
        """hodu_rocm_sum: md is reduce_metadata [nd, shape.., strides.., offset, out_nd, out_shape.., n_reduce,
        reduce_dims.., keep_dim, reduce_size]"""
        m = [int(v) for v in md]
        if m and len(m) >= 3 + 2 * m[0]:
            nd = m[0]
            span = _view_span(m[1:1 + nd], m[1 + nd:1 + 2 * nd], m[1 + 2 * nd])
            out_nd = m[2 + 2 * nd]
            n_out = int(np.prod(m[3 + 2 * nd:3 + 2 * nd + out_nd], dtype=np.int64)) if len(m) >= 3 + 2 * nd + out_nd else 0
            if span * DTYPE_SIZE[dt] > x.nbytes or n_out * DTYPE_SIZE[dt] > out.nbytes:
                raise HoduRocmError(INVALID_ARG, f"sum_{dt}: metadata reaches past a device buffer")
        arr, n = _md_array(md)
        self._check(self.lib.hodu_rocm_sum(self.handle, DTYPE_ID[dt], x.ptr, out.ptr, arr, n))

    def softmax(self, dt: str, x: DeviceBuffer, out: DeviceBuffer, md, causal: bool = False):
        """hodu_rocm_softmax: md is reduce_metadata of the input layout with the softmax dim reduced; the output is
        contiguous in the input's shape"""
        m = [int(v) for v in md]
        if m and len(m) >= 2 + 2 * m[0]:
            nd = m[0]
            span = _view_span(m[1:1 + nd], m[1 + nd:1 + 2 * nd], m[1 + 2 * nd])
            n = int(np.prod(m[1:1 + nd], dtype=np.int64)) if nd else 1
            if span * DTYPE_SIZE[dt] > x.nbytes or n * DTYPE_SIZE[dt] > out.nbytes:
                raise HoduRocmError(INVALID_ARG, f"softmax_{dt}: metadata reaches past a device buffer")
        arr, n_md = _md_array(md)
        self._check(self.lib.hodu_rocm_softmax(self.handle, DTYPE_ID[dt], x.ptr, out.ptr, arr, n_md, int(bool(causal))))

    def softmax_masked(self, dt: str, x: DeviceBuffer, out: DeviceBuffer, md, mask: DeviceBuffer, mask_strides,
                       mask_offset: int = 0, causal: bool = False, mask_dt: str = "u8"):
        """hodu_rocm_softmax_masked: softmax along the last dim with attention's attn_mask (one byte per element, 0 =
        masked; mask_strides in elements over the input's shape, 0 where the mask is broadcast) and optionally the
        causal mask folded in"""
        m = [int(v) for v in md]
        nd = m[0] if m else 0
        strides = [int(v) for v in mask_strides]
        if len(m) < 2 + 2 * nd or len(strides) != nd:
            raise HoduRocmError(INVALID_ARG, f"softmax_masked_{dt}: the mask layout needs one stride per input dim")
        span = _view_span(m[1:1 + nd], m[1 + nd:1 + 2 * nd], m[1 + 2 * nd])
        n = int(np.prod(m[1:1 + nd], dtype=np.int64)) if nd else 1
        mask_span = _view_span(m[1:1 + nd], strides, int(mask_offset))
        if span * DTYPE_SIZE[dt] > x.nbytes or n * DTYPE_SIZE[dt] > out.nbytes or mask_span > mask.nbytes:
            raise HoduRocmError(INVALID_ARG, f"softmax_masked_{dt}: a layout reaches past a device buffer")
        arr, n_md = _md_array(md)
        larr, n_l = _md_array([nd] + strides + [int(mask_offset)])
        self._check(self.lib.hodu_rocm_softmax_masked(self.handle, DTYPE_ID[dt], x.ptr, out.ptr, arr, n_md, int(bool(causal)),
                                                      mask.ptr, DTYPE_ID[mask_dt], larr, n_l))

    def attention(self, dt: str, q: DeviceBuffer, k: DeviceBuffer, v: DeviceBuffer, out: DeviceBuffer, md, scale, causal=False,
                  mask: DeviceBuffer = None, mask_strides=None, mask_offset: int = 0, mask_dt: str = "u8"):
        """hodu_rocm_attention; md = [nb, batch_shape.., Sq, Sk, D, q_strides.., k_strides.., v_strides.., q_off, k_off,
        v_off]; scale: 1-element array in dt's storage.  With mask (one byte per element, 0 = masked; mask_strides in
        elements over [batch_shape.., Sq, Sk], 0 where the mask is broadcast): hodu_rocm_attention_masked"""
        m = [int(x) for x in md]
        nb = m[0] if m else 0
        if len(m) == 1 + nb + 3 + 3 * (nb + 2) + 3:
            bshape, (sq, sk, d) = m[1:1 + nb], m[1 + nb:4 + nb]
            base = 4 + nb
            for name, buf, rows, st, off in (("q", q, sq, m[base:base + nb + 2], m[-3]),
                                             ("k", k, sk, m[base + nb + 2:base + 2 * (nb + 2)], m[-2]),
                                             ("v", v, sk, m[base + 2 * (nb + 2):base + 3 * (nb + 2)], m[-1])):
                if _view_span(bshape + [rows, d], st, off) * DTYPE_SIZE[dt] > buf.nbytes:
                    raise HoduRocmError(INVALID_ARG, f"attention: metadata reaches past the {name} buffer")
            n_out = int(np.prod(bshape + [sq, d], dtype=np.int64))
            if n_out * DTYPE_SIZE[dt] > out.nbytes:
                raise HoduRocmError(INVALID_ARG, "attention: the output buffer is too small")
        arr, n = _md_array(md)
        sc = np.ascontiguousarray(scale).reshape(1)
        if mask is not None:
            strides = [int(x) for x in mask_strides]
            if len(m) != 1 + nb + 3 + 3 * (nb + 2) + 3 or len(strides) != nb + 2:
                raise HoduRocmError(INVALID_ARG, "attention: the mask layout needs one stride per dim of the scores")
            if _view_span(m[1:1 + nb] + [m[1 + nb], m[2 + nb]], strides, int(mask_offset)) > mask.nbytes:
                raise HoduRocmError(INVALID_ARG, "attention: the mask layout reaches past the mask buffer")
            larr, n_l = _md_array([nb + 2] + strides + [int(mask_offset)])
            self._check(self.lib.hodu_rocm_attention_masked(self.handle, DTYPE_ID[dt], q.ptr, k.ptr, v.ptr, out.ptr, arr, n,
                                                            sc.ctypes.data, int(bool(causal)), mask.ptr, DTYPE_ID[mask_dt], larr, n_l))
            return
        self._check(self.lib.hodu_rocm_attention(self.handle, DTYPE_ID[dt], q.ptr, k.ptr, v.ptr, out.ptr, arr, n,
                                                 sc.ctypes.data, int(bool(causal))))

    def time_product(self, op: str, name: str, lhs: DeviceBuffer, rhs_list, out: DeviceBuffer, md, iters: int,
                     graph: bool = False, steps=None) -> float:
        """back-to-back launches issued from C (graph=True: recorded once into a HIP graph and replayed as
        one graph launch), HIP-event timed on the context's stream; total ms"""
        self._check_extents(op, name, lhs, rhs_list, out, md)
        kind = {"bf16_f8e4m3w": 1, "i32_i8i8": 2}.get(name, 0)
        dtype = DTYPE_ID["bf16"] if kind == 1 else DTYPE_ID["i32"] if kind == 2 else DTYPE_ID[name]
        arr, n = _md_array(md)
        ptrs = (ctypes.c_void_p * len(rhs_list))(*[b.ptr for b in rhs_list])
        ms = ctypes.c_float()
        if steps:
            sarr, ns = _steps_array(steps)
            self._check(self.debug.hodu_rocm_debug_time_product_ex(
                self.handle, 1 if op == "matmul" else 0, kind, dtype, lhs.ptr, ptrs, len(rhs_list), out.ptr, arr, n,
                sarr, ns, int(iters), ctypes.byref(ms)))
            return float(ms.value)
        fn = self.debug.hodu_rocm_debug_time_product_graph if graph else self.debug.hodu_rocm_debug_time_product
        self._check(fn(self.handle, 1 if op == "matmul" else 0, kind, dtype, lhs.ptr, ptrs, len(rhs_list), out.ptr, arr,
                       n, int(iters), ctypes.byref(ms)))
        return float(ms.value)

    def time_cast(self, src: str, dst: str, ins, outs, md, iters: int) -> float:
        """back-to-back cast (src != dst) or contiguous (src == dst) launches issued from C over the buffer pairs in
        turn, HIP-event timed on the context's stream; total ms"""
        if len(ins) != len(outs) or not ins:
            raise HoduRocmError(INVALID_ARG, "time_cast: need as many outputs as inputs, at least one")
        for x, out in zip(ins, outs):
            self._check_strided(f"time_cast_{src}_to_{dst}", DTYPE_SIZE[src], DTYPE_SIZE[dst], x, out, md)
        arr, n = _md_array(md)
        pin = (ctypes.c_void_p * len(ins))(*[b.ptr for b in ins])
        pout = (ctypes.c_void_p * len(outs))(*[b.ptr for b in outs])
        ms = ctypes.c_float()
        self._check(self.debug.hodu_rocm_debug_time_cast(self.handle, DTYPE_ID[src], DTYPE_ID[dst], pin, pout, len(ins), arr, n,
                                                       int(iters), ctypes.byref(ms)))
        return float(ms.value)

    def time_sum(self, dt: str, ins, outs, md, iters: int) -> float:
        """back-to-back hodu_rocm_sum launches issued from C over the buffer pairs in turn; total ms (the caller sizes
        the buffers for the metadata, as for Context.sum)"""
        if len(ins) != len(outs) or not ins:
            raise HoduRocmError(INVALID_ARG, "time_sum: need as many outputs as inputs, at least one")
        arr, n = _md_array(md)
        pin = (ctypes.c_void_p * len(ins))(*[b.ptr for b in ins])
        pout = (ctypes.c_void_p * len(outs))(*[b.ptr for b in outs])
        ms = ctypes.c_float()
        self._check(self.debug.hodu_rocm_debug_time_sum(self.handle, DTYPE_ID[dt], pin, pout, len(ins), arr, n, int(iters),
                                                      ctypes.byref(ms)))
        return float(ms.value)

    def mfma_clock(self, kind: int, operands: DeviceBuffer, iters: int = 20000) -> dict:
        """register-only MFMA loop on the given operand bits (16 KB): sustained TFLOP/s and shader clock"""
        if operands.nbytes < 16384:
            raise HoduRocmError(INVALID_ARG, "mfma_clock: operands must hold 16 KB")
        ms, tf, mhz = ctypes.c_float(), ctypes.c_double(), ctypes.c_double()
        self._check(self.debug.hodu_rocm_debug_mfma_clock(self.handle, int(kind), operands.ptr, int(iters), ctypes.byref(ms),
                                                        ctypes.byref(tf), ctypes.byref(mhz)))
        return {"ms": ms.value, "tflops": tf.value, "shader_mhz": mhz.value}

    def read_floor(self, buffers, nbytes: int, iters: int = 200) -> dict:
        """flat streaming read of nbytes from each buffer in turn, and an empty kernel: microseconds per launch"""
        if any(b.nbytes < nbytes for b in buffers):
            raise HoduRocmError(INVALID_ARG, "read_floor: a buffer is smaller than nbytes")
        ptrs = (ctypes.c_void_p * len(buffers))(*[b.ptr for b in buffers])
        r, e = ctypes.c_float(), ctypes.c_float()
        self._check(self.debug.hodu_rocm_debug_read_floor(self.handle, ptrs, len(buffers), int(nbytes), int(iters),
                                                        ctypes.byref(r), ctypes.byref(e)))
        return {"read_us": r.value, "empty_us": e.value}

    def force_tile(self, tile: int):
        """testing hook: 0 = 256x256 / 8 wavefronts, 1 = 256x256 / 4, 2 = 128x128, 3 = 64x64, 10..16 the pipelined
        kernel's tiles (15: the 16x16x32 instruction, 16: its respaced-issue form), 30..34 the GEMV kernel's shapes, 35..39 the M <= 16 kernel's, -1 = automatic"""
        self._check(self.debug.hodu_rocm_debug_force_tile(self.handle, int(tile)))

    def force_splitk(self, splits: int):
        """testing hook: K ranges of the pipelined kernels (-1 automatic, 1 never, n forced)"""
        self._check(self.debug.hodu_rocm_debug_force_splitk(self.handle, int(splits)))

    def scratch_state(self) -> dict:
        """testing hook: what this context has allocated for its kernels' scratch, and whether it is pointed at the
        static scratch of the entry point that allocates nothing (never, between calls)"""
        ws, arr, fixed = ctypes.c_size_t(), ctypes.c_int(), ctypes.c_int()
        self._check(self.debug.hodu_rocm_debug_scratch_state(self.handle, ctypes.byref(ws), ctypes.byref(arr), ctypes.byref(fixed)))
        return {"workspace_bytes": ws.value, "arrival_allocated": bool(arr.value), "fixed": bool(fixed.value)}

    def last_kernel(self) -> str:
        return self.lib.hodu_rocm_last_kernel(self.handle).decode()

    def device_info(self) -> dict:
        name = ctypes.create_string_buffer(256)
        cus, khz, mem = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
        self._check(self.lib.hodu_rocm_device_info(self.handle, name, 256, ctypes.byref(cus), ctypes.byref(khz),
                                                   ctypes.byref(mem)))
        return {"name": name.value.decode(), "compute_units": cus.value, "clock_khz": khz.value,
                "total_mem": mem.value}

    # timing ---------------------------------------------------------------------------------
    def timer(self) -> "Timer":
        return Timer(self)


class Timer:
    """HIP-event stopwatch on the context's stream."""

    def __init__(self, ctx: Context):
        self.ctx = ctx
        h = ctypes.c_void_p()
        ctx._check(ctx.lib.hodu_rocm_timer_create(ctx.handle, ctypes.byref(h)))
        self.handle = h.value

    def start(self):
        self.ctx._check(self.ctx.lib.hodu_rocm_timer_start(self.ctx.handle, self.handle))

    def stop_ms(self) -> float:
        ms = ctypes.c_float()
        self.ctx._check(self.ctx.lib.hodu_rocm_timer_stop(self.ctx.handle, self.handle, ctypes.byref(ms)))
        return float(ms.value)

    def close(self):
        if self.handle is not None:
            self.ctx.lib.hodu_rocm_timer_destroy(self.ctx.handle, self.handle)
            self.handle = None
