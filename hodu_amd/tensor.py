"""Python face of the host-side Tensor mirror (hodu_amd/host/*.hpp, built into lib/libhodu_rocm_host.so).

The method names and argument meanings are those of hodu's Tensor on this path
(crates/hodu_core/src/tensor/ops/matrix.rs, cast_memory.rs, shape.rs): matmul, dot, to_dtype,
contiguous, transpose, t, broadcast, reshape, squeeze, unsqueeze, slice.  Data enters and leaves as raw
bit patterns (numpy arrays of the storage width), the way Tensor::from_bytes does.  Loading fails
loudly when the library has not been built; nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence

import numpy as np

from .ffi import DTYPE_ID, DTYPE_SIZE, load as _load_kernels

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "lib", "libhodu_rocm_host.so")
DTYPE_NAME = {v: k for k, v in DTYPE_ID.items()}
_BITS = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}

ERROR_KINDS = ["IncompatibleShapes", "InvalidLayout", "InvalidArgument", "InvalidAxis", "DTypeMismatch",
               "UnsupportedDTypeForOp", "DeviceMismatch", "InternalError", "RocmKernelError"]


class HoduError(RuntimeError):
    def __init__(self, code: int, message: str):
        self.kind = ERROR_KINDS[code - 1] if 1 <= code <= len(ERROR_KINDS) else f"code {code}"
        super().__init__(f"{self.kind}: {message}")


class _Then(ctypes.Structure):
    _fields_ = [("op", ctypes.c_int), ("operand", ctypes.c_void_p), ("scalar", ctypes.c_ubyte * 8)]


_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    _load_kernels()  # raises when the HIP library is missing
    if not os.path.exists(HOST_LIB_PATH):
        raise ImportError(f"{HOST_LIB_PATH} is missing: build it first (python -m hodu_amd.build)")
    lib = ctypes.CDLL(HOST_LIB_PATH)
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    szp, vpp = ctypes.POINTER(sz), ctypes.POINTER(vp)
    lib.hodu_host_last_error.restype = ctypes.c_char_p
    lib.hodu_host_tensor_from_bytes.argtypes = [ci, ci, szp, sz, vp, sz, vpp]
    lib.hodu_host_tensor_free.argtypes = [vp]
    lib.hodu_host_tensor_free.restype = None
    for name in ("ndim", "dtype", "physical_dtype"):
        getattr(lib, f"hodu_host_tensor_{name}").argtypes = [vp]
    lib.hodu_host_tensor_shares_storage.argtypes = [vp, vp]
    lib.hodu_host_tensor_layout.argtypes = [vp, szp, szp, szp]
    lib.hodu_host_tensor_layout.restype = None
    lib.hodu_host_tensor_to_bytes.argtypes = [vp, vp, sz]
    lib.hodu_host_matmul.argtypes = [vp, vp, vpp]
    lib.hodu_host_dot.argtypes = [vp, vp, vpp]
    lib.hodu_host_matmul_then.argtypes = [vp, vp, ctypes.POINTER(_Then), sz, vpp]
    lib.hodu_host_linear.argtypes = [vp, vp, vp, ci, vpp]
    lib.hodu_host_stats_fused_steps.restype = ctypes.c_long
    lib.hodu_host_stats_sum_kernels.restype = ctypes.c_long
    lib.hodu_host_stats_softmax_kernels.restype = ctypes.c_long
    lib.hodu_host_stats_attention_kernels.restype = ctypes.c_long
    lib.hodu_host_softmax.argtypes = [vp, ci, ci, vpp]
    lib.hodu_host_attention.argtypes = [vp, vp, vp, ci, vpp]
    lib.hodu_host_softmax_masked.argtypes = [vp, vp, ci, vpp]
    lib.hodu_host_attention_masked.argtypes = [vp, vp, vp, vp, ci, vpp]
    lib.hodu_host_scalar_bits.argtypes = [ci, ctypes.c_double, ctypes.POINTER(ctypes.c_ubyte), szp]
    lib.hodu_host_sum.argtypes = [vp, ctypes.POINTER(ci), sz, ci, vpp]
    lib.hodu_host_sum_to_shape.argtypes = [vp, szp, sz, vpp]
    lib.hodu_host_matmul_vjp.argtypes = [vp, vp, vp, vpp, vpp]
    lib.hodu_host_dot_vjp.argtypes = [vp, vp, vp, vpp, vpp]
    lib.hodu_host_to_dtype.argtypes = [vp, ci, vpp]
    lib.hodu_host_contiguous.argtypes = [vp, vpp]
    lib.hodu_host_transpose.argtypes = [vp, ci, ci, vpp]
    lib.hodu_host_broadcast.argtypes = [vp, szp, sz, vpp]
    lib.hodu_host_reshape.argtypes = [vp, szp, sz, vpp]
    lib.hodu_host_squeeze.argtypes = [vp, ctypes.POINTER(ci), sz, vpp]
    lib.hodu_host_unsqueeze.argtypes = [vp, ci, vpp]
    lib.hodu_host_slice.argtypes = [vp, ci, ci, ci, ci, ci, vpp]
    lib.hodu_host_view.argtypes = [vp, szp, szp, sz, sz, vpp]
    lib.hodu_host_set_matmul_mode.argtypes = [ci]
    lib.hodu_host_set_matmul_mode.restype = None
    lib.hodu_host_set_reference_sums.argtypes = [ci, ci]
    lib.hodu_host_stats.argtypes = [ctypes.POINTER(ctypes.c_long)] * 4 + [ctypes.POINTER(ctypes.c_longlong)]
    lib.hodu_host_stats.restype = None
    lib.hodu_host_stats_reset.restype = None
    _lib = lib
    return lib


def _sizes(values: Sequence[int]):
    return (ctypes.c_size_t * max(1, len(values)))(*[int(v) for v in values])


def set_matmul_mode(mode: str):
    """'reference': copy non-contiguous operands before broadcasting like hodu does today;
    'nocopy': hand strided / broadcast views to the kernel unchanged (the default)."""
    load().hodu_host_set_matmul_mode({"reference": 0, "nocopy": 1}[mode])


def set_reference_sums(on: bool, device: int = 0):
    """products of f8e4m3 / f8e5m2 / bf16 / f16 on the device in the CPU backend's arithmetic (the running sum re-rounded
    to the dtype after every multiply and add): hodu's CPU bytes, at a scalar loop's speed; off by default"""
    lib = load()
    rc = lib.hodu_host_set_reference_sums(int(device), int(bool(on)))
    if rc != 0:
        raise HoduError(rc, lib.hodu_host_last_error().decode())


def stats(reset: bool = False) -> dict:
    lib = load()
    a, b, c, d, e = (ctypes.c_long(), ctypes.c_long(), ctypes.c_long(), ctypes.c_long(), ctypes.c_longlong())
    lib.hodu_host_stats(a, b, c, d, e)
    fused_steps, sum_kernels = int(lib.hodu_host_stats_fused_steps()), int(lib.hodu_host_stats_sum_kernels())
    if reset:
        lib.hodu_host_stats_reset()
    return {"cast_kernels": a.value, "contiguous_kernels": b.value, "product_kernels": c.value,
            "fused_products": d.value, "bytes_copied": e.value, "fused_steps": fused_steps, "sum_kernels": sum_kernels,
            "softmax_kernels": int(lib.hodu_host_stats_softmax_kernels()),
            "attention_kernels": int(lib.hodu_host_stats_attention_kernels())}


class Tensor:
    def __init__(self, handle: int):
        self._h = handle

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.hodu_host_tensor_free(self._h)
            self._h = None

    @staticmethod
    def _wrap(rc: int, out: ctypes.c_void_p) -> "Tensor":
        if rc != 0:
            raise HoduError(rc, load().hodu_host_last_error().decode())
        return Tensor(out.value)

    @classmethod
    def from_bits(cls, bits: np.ndarray, dtype: str, shape: Sequence[int], device: int = 0) -> "Tensor":
        """bits: the elements' bit patterns, row-major, as an unsigned array of the storage width"""
        bits = np.ascontiguousarray(bits)
        if bits.dtype.itemsize != DTYPE_SIZE[dtype]:
            raise ValueError(f"{dtype} needs {DTYPE_SIZE[dtype]}-byte elements, got {bits.dtype}")
        out = ctypes.c_void_p()
        rc = load().hodu_host_tensor_from_bytes(device, DTYPE_ID[dtype], _sizes(shape), len(shape),
                                                bits.ctypes.data, bits.nbytes, ctypes.byref(out))
        return cls._wrap(rc, out)

    # ---- facts ------------------------------------------------------------------------------------
    @property
    def dtype(self) -> str:
        return DTYPE_NAME[load().hodu_host_tensor_dtype(self._h)]

    @property
    def physical_dtype(self) -> str:
        """differs from dtype while a to_dtype is deferred into the next matmul"""
        return DTYPE_NAME[load().hodu_host_tensor_physical_dtype(self._h)]

    def layout(self):
        nd = load().hodu_host_tensor_ndim(self._h)
        sh, st, off = _sizes([0] * nd), _sizes([0] * nd), ctypes.c_size_t()
        load().hodu_host_tensor_layout(self._h, sh, st, ctypes.byref(off))
        return list(sh[:nd]), list(st[:nd]), off.value

    @property
    def shape(self):
        return self.layout()[0]

    def shares_storage_with(self, other: "Tensor") -> bool:
        return bool(load().hodu_host_tensor_shares_storage(self._h, other._h))

    def to_bits(self) -> np.ndarray:
        """row-major elements of the view, as bit patterns of the logical dtype"""
        n = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        out = np.empty(n, dtype=_BITS[DTYPE_SIZE[self.dtype]])
        rc = load().hodu_host_tensor_to_bytes(self._h, out.ctypes.data, out.nbytes)
        if rc != 0:
            raise HoduError(rc, load().hodu_host_last_error().decode())
        return out

    # ---- the path -----------------------------------------------------------------------------------
    def _unary(self, fn, *args) -> "Tensor":
        out = ctypes.c_void_p()
        return self._wrap(fn(self._h, *args, ctypes.byref(out)), out)

    def matmul(self, other: "Tensor") -> "Tensor":
        return self._unary(load().hodu_host_matmul, other._h)

    def matmul_then(self, other: "Tensor", steps) -> "Tensor":
        """matmul with the caller's next element-wise kernels applied inside its store.  steps: a list of
        ("add", tensor) -- a bias along the last axis, as Linear::forward adds it --, ("mul_scalar", bits) -- the
        scalar as a 1-element array in the tensor dtype's storage -- and ("relu",)."""
        arr = (_Then * max(1, len(steps)))()
        for i, step in enumerate(steps):
            if step[0] == "add":
                arr[i].op, arr[i].operand = 1, step[1]._h
            elif step[0] == "mul_scalar":
                raw = np.ascontiguousarray(step[1]).reshape(1).tobytes()
                arr[i].op = 2
                arr[i].scalar = (ctypes.c_ubyte * 8)(*raw, *([0] * (8 - len(raw))))
            elif step[0] == "relu":
                arr[i].op = 3
            else:
                raise ValueError(f"unknown fused step {step[0]!r}")
        out = ctypes.c_void_p()
        return self._wrap(load().hodu_host_matmul_then(self._h, other._h, arr, len(steps), ctypes.byref(out)), out)

    def softmax(self, dim: int = -1, causal: bool = False) -> "Tensor":
        """Tensor::softmax (tensor/ops/normalization.rs:4-21) as one launch.  causal (last dim only): entries j > i of
        every [.., Sq, Sk] matrix are masked first (attention.rs:40-48)"""
        return self._unary(load().hodu_host_softmax, int(dim), int(causal))

    def softmax_masked(self, mask: "Tensor", causal: bool = False) -> "Tensor":
        """softmax(-1) of masked_fill(mask == 0, the dtype's -inf stand-in) (attention.rs:50-56) as one launch; the mask
        (bool / u8 / i8) broadcasts against the scores and is read in place"""
        return self._unary(load().hodu_host_softmax_masked, mask._h, int(causal))

    def sum(self, dims: Sequence[int] = (), keep_dim: bool = False) -> "Tensor":
        """Tensor::sum (tensor/ops/reduce.rs:11-13): no dims = all of them"""
        arr = (ctypes.c_int * max(1, len(dims)))(*dims)
        return self._unary(load().hodu_host_sum, arr, len(dims), int(keep_dim))

    def sum_to_shape(self, shape: Sequence[int]) -> "Tensor":
        return self._unary(load().hodu_host_sum_to_shape, _sizes(shape), len(shape))

    def dot(self, other: "Tensor") -> "Tensor":
        return self._unary(load().hodu_host_dot, other._h)

    def to_dtype(self, dtype: str) -> "Tensor":
        return self._unary(load().hodu_host_to_dtype, DTYPE_ID[dtype])

    def contiguous(self) -> "Tensor":
        return self._unary(load().hodu_host_contiguous)

    def transpose(self, d1: int, d2: int) -> "Tensor":
        return self._unary(load().hodu_host_transpose, d1, d2)

    def t(self) -> "Tensor":
        return self.transpose(-2, -1)

    def broadcast(self, shape: Sequence[int]) -> "Tensor":
        return self._unary(load().hodu_host_broadcast, _sizes(shape), len(shape))

    def reshape(self, shape: Sequence[int]) -> "Tensor":
        return self._unary(load().hodu_host_reshape, _sizes(shape), len(shape))

    def squeeze(self, dims: Sequence[int] = ()) -> "Tensor":
        arr = (ctypes.c_int * max(1, len(dims)))(*dims)
        return self._unary(load().hodu_host_squeeze, arr, len(dims))

    def unsqueeze(self, dim: int) -> "Tensor":
        return self._unary(load().hodu_host_unsqueeze, dim)

    def slice(self, dim: int, start: int, end: Optional[int] = None, step: int = 1) -> "Tensor":
        return self._unary(load().hodu_host_slice, dim, start, 0 if end is None else 1, 0 if end is None else end, step)

    def view(self, shape: Sequence[int], strides: Sequence[int], offset: int = 0) -> "Tensor":
        """an arbitrary strided view over the same storage (what chained view ops produce)"""
        return self._unary(load().hodu_host_view, _sizes(shape), _sizes(strides), len(shape), offset)


def _vjp(fn, a: Tensor, b: Tensor, grad: Tensor):
    da, db = ctypes.c_void_p(), ctypes.c_void_p()
    rc = fn(a._h, b._h, grad._h, ctypes.byref(da), ctypes.byref(db))
    if rc != 0:
        raise HoduError(rc, load().hodu_host_last_error().decode())
    return Tensor(da.value), Tensor(db.value)


def matmul_vjp(a: Tensor, b: Tensor, grad: Tensor):
    """(dA, dB) of matmul(a, b) for the output gradient `grad` (tensor/gradient/vjp_matrix.rs:17-45)"""
    return _vjp(load().hodu_host_matmul_vjp, a, b, grad)


def dot_vjp(a: Tensor, b: Tensor, grad: Tensor):
    """(dA, dB) of dot(a, b) (tensor/gradient/vjp_matrix.rs:46-67)"""
    return _vjp(load().hodu_host_dot_vjp, a, b, grad)


def scalar_bits(dtype: str, value: float) -> np.ndarray:
    """`value` as a 1-element array in dtype's storage, rounded to nearest even (Scalar::to_dtype)"""
    buf, n = (ctypes.c_ubyte * 8)(), ctypes.c_size_t()
    rc = load().hodu_host_scalar_bits(DTYPE_ID[dtype], float(value), buf, ctypes.byref(n))
    if rc != 0:
        raise HoduError(rc, load().hodu_host_last_error().decode())
    return np.frombuffer(bytes(buf[:n.value]), dtype=_BITS[n.value]).copy()


def scaled_dot_product_attention(q: Tensor, k: Tensor, v: Tensor, is_causal: bool = False,
                                 attn_mask: Optional[Tensor] = None) -> Tensor:
    """hodu_nn's scaled_dot_product_attention (crates/hodu_nn/src/modules/attention.rs:25-70) without dropout: one launch
    where the fused kernel applies (bf16 / f16, head dim 64 or 128, dense aligned rows; with or without attn_mask),
    otherwise three (product with the scale in its store, masked softmax, product).  attn_mask: a bool / u8 / i8 tensor,
    1 = attend, 0 = mask out, broadcast against the scores and read in place."""
    out = ctypes.c_void_p()
    if attn_mask is not None:
        rc = load().hodu_host_attention_masked(q._h, k._h, v._h, attn_mask._h, int(is_causal), ctypes.byref(out))
        return Tensor._wrap(rc, out)
    rc = load().hodu_host_attention(q._h, k._h, v._h, int(is_causal), ctypes.byref(out))
    return Tensor._wrap(rc, out)


class Linear:
    """hodu_nn's Linear (crates/hodu_nn/src/modules/linear.rs:4-57): weight [out_features, in_features], optional
    bias [out_features]; forward(input) = input @ weight.T + bias, as ONE launch (the bias add -- and a ReLU that
    follows, if asked for -- run inside the product's store)."""

    def __init__(self, weight: Tensor, bias: Optional[Tensor] = None):
        self.weight, self.bias = weight, bias

    def forward(self, x: Tensor, relu: bool = False) -> Tensor:
        out = ctypes.c_void_p()
        rc = load().hodu_host_linear(x._h, self.weight._h, self.bias._h if self.bias is not None else None, int(relu),
                                     ctypes.byref(out))
        return Tensor._wrap(rc, out)

    def parameters(self):
        return [self.weight] + ([self.bias] if self.bias is not None else [])
