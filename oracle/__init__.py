"""ctypes front-end of the CPU oracle (oracle/liboracle.so) and of the compiled reference
kernels (oracle/_ref/libhodu_cpu_ref.so, when built).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py as the checker.  The product (hodu_amd and the C-ABI library) never imports it.

Narrow types travel as raw bit patterns: bf16 / f16 in uint16 arrays, f8e4m3 / f8e5m2 / bool in
uint8 arrays -- the little-endian element encodings of crates/hodu_core/src/tensor/bytes.rs:90-180.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

# dtype ids: crates/hodu_core/src/types/dtype.rs:6-28
DTYPE_ID = {
    "bool": 0, "f8e4m3": 1, "f8e5m2": 2, "bf16": 3, "f16": 4, "f32": 5, "f64": 6,
    "u8": 7, "u16": 8, "u32": 9, "u64": 10, "i8": 11, "i16": 12, "i32": 13, "i64": 14,
}
# numpy container for each dtype's storage
STORAGE = {
    "bool": np.uint8, "f8e4m3": np.uint8, "f8e5m2": np.uint8, "bf16": np.uint16, "f16": np.uint16,
    "f32": np.float32, "f64": np.float64, "u8": np.uint8, "u16": np.uint16, "u32": np.uint32,
    "u64": np.uint64, "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
}
MATMUL_DTYPES = [d for d in DTYPE_ID if d != "bool"]
F8_HODU, F8_OCP = 0, 1


def build(force: bool = False) -> None:
    """Compile liboracle.so (and _ref when the reference tree is present) with oracle/Makefile."""
    if force or not os.path.exists(os.path.join(_HERE, "liboracle.so")):
        subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


def _md(md) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(md, dtype=np.uint64))


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        # HODU_ORACLE_LIB: another build of hodu_oracle.c to check the checker with (`make -C oracle ubsan` writes one
        # compiled with the undefined-behaviour sanitizer)
        other = os.environ.get("HODU_ORACLE_LIB")
        if not other:
            build()
        _lib = ctypes.CDLL(os.path.abspath(other) if other else os.path.join(_HERE, "liboracle.so"))
        _lib.oracle_f8e4m3_to_f32.restype = ctypes.c_float
        _lib.oracle_f8e4m3_to_f32.argtypes = [ctypes.c_uint8, ctypes.c_int]
        _lib.oracle_f32_to_f8e4m3.restype = ctypes.c_uint8
        _lib.oracle_f32_to_f8e4m3.argtypes = [ctypes.c_float]
        _lib.oracle_f32_to_f16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.oracle_f16_to_f32.restype = ctypes.c_float
        _lib.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.oracle_reference_threads.restype = ctypes.c_size_t
        _lib.oracle_reference_threads.argtypes = [ctypes.c_size_t] * 3
    return _lib


def set_threads(n: int) -> None:
    lib().oracle_set_threads(int(n))


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"oracle: {what} failed (rc={rc})")


def matmul_out_elems(md) -> int:
    return int(md[0])


def dot_out_elems(md) -> int:
    return int(md[0]) * int(md[2])


def matmul_asis(dt: str, lhs: np.ndarray, rhs: np.ndarray, md) -> np.ndarray:
    """hodu_cpu_matmul_<dt>, bit-faithful."""
    md = _md(md)
    out = np.empty(matmul_out_elems(md), dtype=STORAGE[dt])
    _check(lib().oracle_matmul_asis(DTYPE_ID[dt], _ptr(lhs), _ptr(rhs), _ptr(out), _ptr(md)), "matmul_asis")
    return out


def dot_asis(dt: str, lhs: np.ndarray, rhs: np.ndarray, md) -> np.ndarray:
    """hodu_cpu_dot_<dt>, bit-faithful."""
    md = _md(md)
    out = np.empty(dot_out_elems(md), dtype=STORAGE[dt])
    _check(lib().oracle_dot_asis(DTYPE_ID[dt], _ptr(lhs), _ptr(rhs), _ptr(out), _ptr(md)), "dot_asis")
    return out


def _spec(fn, n, l_dt, r_dt, lhs, rhs, md, decode, want64):
    out32 = np.empty(n, dtype=np.float32)
    out64 = np.empty(n, dtype=np.float64) if want64 else None
    outabs = np.empty(n, dtype=np.float64) if want64 else None
    rc = fn(DTYPE_ID[l_dt], DTYPE_ID[r_dt], decode, _ptr(lhs), _ptr(rhs), _ptr(out32),
            _ptr(out64) if want64 else None, _ptr(outabs) if want64 else None, _ptr(md))
    _check(rc, "spec")
    return out32, out64, outabs


def matmul_spec(l_dt, r_dt, lhs, rhs, md, decode=F8_OCP, want64=True):
    """f32-accumulated comparator (matmul metadata).  Returns (f32 sums, f64 sums, f64 sum|a*b|)."""
    md = _md(md)
    return _spec(lib().oracle_matmul_spec, matmul_out_elems(md), l_dt, r_dt, lhs, rhs, md, decode, want64)


def dot_spec(l_dt, r_dt, lhs, rhs, md, decode=F8_OCP, want64=True):
    """f32-accumulated comparator (dot metadata)."""
    md = _md(md)
    return _spec(lib().oracle_dot_spec, dot_out_elems(md), l_dt, r_dt, lhs, rhs, md, decode, want64)


def cast(src: str, dst: str, x: np.ndarray, md, decode=F8_HODU) -> np.ndarray:
    """hodu_cpu_cast_<src>_to_<dst>; decode picks the f8e4m3 table (hodu CPU or OCP)."""
    md = _md(md)
    out = np.empty(int(md[0]), dtype=STORAGE[dst])
    _check(lib().oracle_cast(DTYPE_ID[src], DTYPE_ID[dst], decode, _ptr(x), _ptr(out), _ptr(md)), "cast")
    return out


def contiguous(dt: str, x: np.ndarray, md) -> np.ndarray:
    """hodu_cpu_contiguous_<dt>"""
    md = _md(md)
    out = np.empty(int(md[0]), dtype=STORAGE[dt])
    _check(lib().oracle_contiguous(DTYPE_ID[dt], _ptr(x), _ptr(out), _ptr(md)), "contiguous")
    return out


def add(dt: str, lhs: np.ndarray, rhs: np.ndarray, md) -> np.ndarray:
    """hodu_cpu_add_<dt>; md in the binary-op format [n, nd, lhs_shape, rhs_shape, lhs_strides, rhs_strides, lo, ro]"""
    md = _md(md)
    out = np.empty(int(md[0]), dtype=STORAGE[dt])
    _check(lib().oracle_add(DTYPE_ID[dt], _ptr(lhs), _ptr(rhs), _ptr(out), _ptr(md)), "add")
    return out


def mul_scalar(dt: str, x: np.ndarray, md, scalar: np.ndarray) -> np.ndarray:
    """hodu_cpu_mul_scalar_<dt>; scalar: one element in dt's storage; md in the unary format"""
    md = _md(md)
    scalar = np.ascontiguousarray(scalar, dtype=STORAGE[dt]).reshape(1)
    out = np.empty(int(md[0]), dtype=STORAGE[dt])
    _check(lib().oracle_mul_scalar(DTYPE_ID[dt], _ptr(x), _ptr(out), _ptr(md), _ptr(scalar)), "mul_scalar")
    return out


def relu(dt: str, x: np.ndarray, md) -> np.ndarray:
    """hodu_cpu_relu_<dt>"""
    md = _md(md)
    out = np.empty(int(md[0]), dtype=STORAGE[dt])
    _check(lib().oracle_relu(DTYPE_ID[dt], _ptr(x), _ptr(out), _ptr(md)), "relu")
    return out


def reduce_out_elems(md) -> int:
    nd = int(md[0])
    out_nd = int(md[2 + 2 * nd])
    return int(np.prod([int(v) for v in md[3 + 2 * nd:3 + 2 * nd + out_nd]], dtype=np.int64))


def sum_asis(dt: str, x: np.ndarray, md) -> np.ndarray:
    """hodu_cpu_sum_<dt>: accumulator in the storage type; md is reduce_metadata"""
    md = _md(md)
    out = np.empty(reduce_out_elems(md), dtype=STORAGE[dt])
    _check(lib().oracle_sum_asis(DTYPE_ID[dt], _ptr(x), _ptr(out), _ptr(md)), "sum")
    return out


def sum_spec(dt: str, x: np.ndarray, md, decode=F8_OCP):
    """(f32-accumulated sums, f64 sums, sums of magnitudes)"""
    md = _md(md)
    n = reduce_out_elems(md)
    o32, o64, oabs = np.empty(n, np.float32), np.empty(n, np.float64), np.empty(n, np.float64)
    _check(lib().oracle_sum_spec(DTYPE_ID[dt], decode, _ptr(x), _ptr(md), _ptr(o32), _ptr(o64), _ptr(oabs)), "sum_spec")
    return o32, o64, oabs


def softmax_spec(dt: str, x: np.ndarray, md, causal: bool = False):
    """(f32, f64) softmax along the single reduced dim of md, contiguous in the input's shape"""
    md = _md(md)
    nd = int(md[0])
    n = int(np.prod([int(v) for v in md[1:1 + nd]], dtype=np.int64)) if nd else 1
    o32, o64 = np.empty(n, np.float32), np.empty(n, np.float64)
    _check(lib().oracle_softmax_spec(DTYPE_ID[dt], _ptr(x), _ptr(md), int(causal), _ptr(o32), _ptr(o64)), "softmax_spec")
    return o32, o64


def softmax_masked_spec(dt: str, x: np.ndarray, md, mask: np.ndarray, mask_strides, mask_offset: int = 0, causal: bool = False):
    """(f32, f64) softmax along the last dim with attention's masks applied as the reference applies them (masked_fill
    with the dtype's stand-in for -inf, then the softmax over every entry).  mask: one byte per element, 0 = masked;
    mask_strides: element strides of the mask over the input's shape (0 where it is broadcast)."""
    md = _md(md)
    nd = int(md[0])
    n = int(np.prod([int(v) for v in md[1:1 + nd]], dtype=np.int64)) if nd else 1
    o32, o64 = np.empty(n, np.float32), np.empty(n, np.float64)
    ms = _md(mask_strides)
    assert len(ms) == nd
    mask = np.ascontiguousarray(mask).view(np.uint8)
    _check(lib().oracle_softmax_masked_spec(DTYPE_ID[dt], _ptr(x), _ptr(md), int(causal), _ptr(mask), _ptr(ms),
                                            ctypes.c_size_t(int(mask_offset)), _ptr(o32), _ptr(o64)), "softmax_masked_spec")
    return o32, o64


def f8e4m3_table(decode: int) -> np.ndarray:
    """All 256 decoded values as f32."""
    return np.array([lib().oracle_f8e4m3_to_f32(b, decode) for b in range(256)], dtype=np.float32)


def reference_threads(work: int, min_per_thread: int, online: int) -> int:
    return int(lib().oracle_reference_threads(work, min_per_thread, online))


# ---------------------------------------------------------------------------------------------
# the compiled reference (only where oracle/_ref was built; never present in git history)
# ---------------------------------------------------------------------------------------------
class RefLib:
    """hodu_cpu_* symbols of the reference's own C kernels compiled by oracle/Makefile."""

    PATH = os.path.join(_HERE, "_ref", "libhodu_cpu_ref.so")

    @classmethod
    def available(cls) -> bool:
        return os.path.exists(cls.PATH)

    def __init__(self):
        self.lib = ctypes.CDLL(self.PATH)

    @staticmethod
    def _sfx(dt: str) -> str:
        # on Linux the plain f32/f64 product symbols exist only with the openblas feature
        # (build.rs:137-159); the C file defines *_fallback
        return dt + "_fallback" if dt in ("f32", "f64") else dt

    def matmul(self, dt, lhs, rhs, md):
        md = _md(md)
        out = np.empty(matmul_out_elems(md), dtype=STORAGE[dt])
        fn = getattr(self.lib, f"hodu_cpu_matmul_{self._sfx(dt)}")
        fn.restype = None
        fn(_ptr(lhs), _ptr(rhs), _ptr(out), _ptr(md))
        return out

    def dot(self, dt, lhs, rhs, md):
        md = _md(md)
        out = np.empty(dot_out_elems(md), dtype=STORAGE[dt])
        fn = getattr(self.lib, f"hodu_cpu_dot_{self._sfx(dt)}")
        fn.restype = None
        fn(_ptr(lhs), _ptr(rhs), _ptr(out), _ptr(md))
        return out

    def cast(self, src, dst, x, md):
        md = _md(md)
        out = np.empty(int(md[0]), dtype=STORAGE[dst])
        fn = getattr(self.lib, f"hodu_cpu_cast_{src}_to_{dst}")
        fn.restype = None
        fn(_ptr(x), _ptr(out), _ptr(md))
        return out

    def contiguous(self, dt, x, md):
        md = _md(md)
        out = np.empty(int(md[0]), dtype=STORAGE[dt])
        fn = getattr(self.lib, f"hodu_cpu_contiguous_{dt}")
        fn.restype = None
        fn(_ptr(x), _ptr(out), _ptr(md))
        return out

    def add(self, dt, lhs, rhs, md):
        md = _md(md)
        out = np.empty(int(md[0]), dtype=STORAGE[dt])
        fn = getattr(self.lib, f"hodu_cpu_add_{dt}")
        fn.restype = None
        fn(_ptr(lhs), _ptr(rhs), _ptr(out), _ptr(md))
        return out

    def mul_scalar(self, dt, x, md, scalar):
        md = _md(md)
        scalar = np.ascontiguousarray(scalar, dtype=STORAGE[dt]).reshape(1)
        out = np.empty(int(md[0]), dtype=STORAGE[dt])
        fn = getattr(self.lib, f"hodu_cpu_mul_scalar_{dt}")
        fn.restype = None
        fn(_ptr(x), _ptr(out), _ptr(md), _ptr(scalar))
        return out

    def relu(self, dt, x, md):
        md = _md(md)
        out = np.empty(int(md[0]), dtype=STORAGE[dt])
        fn = getattr(self.lib, f"hodu_cpu_relu_{dt}")
        fn.restype = None
        fn(_ptr(x), _ptr(out), _ptr(md))
        return out

    def sum(self, dt, x, md):
        md = _md(md)
        out = np.empty(reduce_out_elems(md), dtype=STORAGE[dt])
        fn = getattr(self.lib, f"hodu_cpu_sum_{dt}")
        fn.restype = None
        fn(_ptr(x), _ptr(out), _ptr(md))
        return out

    def softmax_chain_f32(self, x, shape):
        """Tensor::softmax(-1) on a contiguous f32 tensor as the reference runs it: hodu_cpu_max_f32 (keep_dim),
        sub_f32, exp_f32, sum_f32 (keep_dim), div_f32 (normalization.rs:14-20)"""
        shape = [int(v) for v in shape]
        nd, n = len(shape), int(np.prod(shape))
        strides = [int(np.prod(shape[i + 1:])) for i in range(nd)]
        red = _md([nd] + shape + strides + [0, nd] + shape[:-1] + [1] + [1, nd - 1, 1, shape[-1]])
        kept = shape[:-1] + [1]
        kstr = [int(np.prod(kept[i + 1:])) for i in range(nd)]
        bstr = kstr[:-1] + [0]
        binary = _md([n, nd] + shape + shape + strides + bstr + [0, 0])
        unary = _md([n, nd] + shape + strides + [0])

        def call(name, *args):
            fn = getattr(self.lib, name)
            fn.restype = None
            fn(*[_ptr(a) for a in args])

        x = np.ascontiguousarray(x, dtype=np.float32)
        mx = np.empty(n // shape[-1], np.float32)
        call("hodu_cpu_max_f32", x, mx, red)
        shifted, e, sm, out = np.empty(n, np.float32), np.empty(n, np.float32), np.empty(n // shape[-1], np.float32), np.empty(n, np.float32)
        call("hodu_cpu_sub_f32", x, mx, shifted, binary)
        call("hodu_cpu_exp_f32", shifted, e, unary)
        call("hodu_cpu_sum_f32", e, sm, red)
        call("hodu_cpu_div_f32", e, sm, out, binary)
        return out
