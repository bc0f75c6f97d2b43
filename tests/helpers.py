"""Shared test utilities: a minimal strided-view description, the three metadata encoders written
independently of the product's host layer (so each can check the other), seeded input generators
and numpy encoders for the narrow float formats.

Metadata formats follow crates/hodu_core/src/op_metadatas.rs:192-291 (matmul), :464-506 (dot),
:1615-1656 (cast / contiguous).
"""
from __future__ import annotations

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


class View:
    """shape / strides / offset in ELEMENTS (crates/hodu_core/src/types/layout.rs:15-19)."""

    def __init__(self, shape, strides=None, offset=0):
        self.shape = [int(s) for s in shape]
        if strides is None:
            strides, acc = [], 1
            for s in reversed(self.shape):
                strides.append(acc)
                acc *= s
            strides.reverse()
        self.strides = [int(s) for s in strides]
        self.offset = int(offset)

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        n = 1
        for s in self.shape:
            n *= s
        return n

    def t(self, d1=-2, d2=-1):
        sh, st = list(self.shape), list(self.strides)
        sh[d1], sh[d2] = sh[d2], sh[d1]
        st[d1], st[d2] = st[d2], st[d1]
        return View(sh, st, self.offset)

    def broadcast_to(self, shape):
        shape = list(shape)
        pad = len(shape) - self.ndim
        st = []
        for i, tgt in enumerate(shape):
            if i < pad:
                st.append(0)
            else:
                src = self.shape[i - pad]
                if src == tgt:
                    st.append(self.strides[i - pad])
                elif src == 1:
                    st.append(0)
                else:
                    raise ValueError("not broadcastable")
        return View(shape, st, self.offset)

    def slice(self, dim, start, stop, step=1):
        sh, st = list(self.shape), list(self.strides)
        n = (stop - start + step - 1) // step
        off = self.offset + start * st[dim]
        sh[dim] = n
        st[dim] = st[dim] * step
        return View(sh, st, off)

    def span(self):
        """number of buffer elements the view can touch (max index + 1)"""
        if self.size == 0:
            return self.offset
        return self.offset + sum((s - 1) * t for s, t in zip(self.shape, self.strides)) + 1

    def take(self, buf: np.ndarray) -> np.ndarray:
        """materialise the logical array from a flat buffer"""
        idx = np.full(self.shape, self.offset, dtype=np.int64)
        for d, (s, t) in enumerate(zip(self.shape, self.strides)):
            ix = np.arange(s, dtype=np.int64) * t
            idx += ix.reshape([-1 if i == d else 1 for i in range(self.ndim)])
        return buf[idx]


def dot_md(lv: View, rv: View):
    assert lv.ndim == 2 and rv.ndim == 2 and lv.shape[1] == rv.shape[0]
    return [lv.shape[0], lv.shape[1], rv.shape[1], lv.strides[0], lv.strides[1], rv.strides[0], rv.strides[1],
            lv.offset, rv.offset]


def matmul_md(lv: View, rv: View):
    lb, rb = lv.shape[:-2], rv.shape[:-2]
    nb = max(len(lb), len(rb))
    batch = []
    for i in range(nb):
        li, ri = len(lb) - nb + i, len(rb) - nb + i
        ld = lb[li] if li >= 0 else 1
        rd = rb[ri] if ri >= 0 else 1
        assert ld == rd or ld == 1 or rd == 1
        batch.append(max(ld, rd))
    m, k, n = lv.shape[-2], lv.shape[-1], rv.shape[-1]
    assert rv.shape[-2] == k
    num = m * n
    for b in batch:
        num *= b
    return ([num, lv.ndim, rv.ndim, nb] + lv.shape + rv.shape + batch + lv.strides + rv.strides
            + [lv.offset, rv.offset, m, k, n])


def cast_md(v: View):
    return [v.size, v.ndim] + v.shape + v.strides + [v.offset]


def reduce_md(v: View, dims, keep_dim: bool):
    """reduce_metadata of crates/hodu_core/src/op_metadatas.rs:525-586"""
    dims = [d % v.ndim for d in dims]
    out_shape = []
    for i, s in enumerate(v.shape):
        if i in dims:
            if keep_dim:
                out_shape.append(1)
        else:
            out_shape.append(s)
    if not out_shape:
        out_shape = [1]
    rs = 1
    for d in dims:
        rs *= v.shape[d]
    return [v.ndim] + v.shape + v.strides + [v.offset, len(out_shape)] + out_shape + [len(dims)] + dims + [int(keep_dim), rs]


def binary_md(lv: View, rv: View):
    """binary_metadata of crates/hodu_core/src/op_metadatas.rs:36-73 (both operands already broadcast to one shape)"""
    assert lv.shape == rv.shape
    return [lv.size, lv.ndim] + lv.shape + rv.shape + lv.strides + rv.strides + [lv.offset, rv.offset]


# ---------------------------------------------------------------------------------------------
# narrow-float encoders used to GENERATE inputs (independent of the oracle's C code)
# ---------------------------------------------------------------------------------------------
def f32_to_bf16_rne(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return rounded.astype(np.uint16)


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def f16_bits(x: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.float16).view(np.uint16)


def _ocp_e4m3_positive():
    vals = []
    for code in range(0x7F):  # 0x7F is NaN
        e, m = code >> 3, code & 7
        vals.append((m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7))
    return np.array(vals, dtype=np.float64)


_E4M3_POS = _ocp_e4m3_positive()


def ocp_e4m3_decode(b: np.ndarray) -> np.ndarray:
    b = np.asarray(b, dtype=np.uint8)
    mag = np.where((b & 0x7F) == 0x7F, np.nan, _E4M3_POS[np.minimum(b & 0x7F, 0x7E)])
    return np.where(b & 0x80, -mag, mag).astype(np.float32)


def f32_to_ocp_e4m3_rne(x: np.ndarray) -> np.ndarray:
    """round-to-nearest-even, saturating to +-448 (OCP E4M3FN)"""
    x = np.asarray(x, dtype=np.float64)
    a = np.minimum(np.abs(x), 448.0)
    hi = np.searchsorted(_E4M3_POS, a, side="left").clip(0, 0x7E)
    lo = (hi - 1).clip(0, 0x7E)
    dlo, dhi = a - _E4M3_POS[lo], _E4M3_POS[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    return (code | np.where(np.signbit(x), 0x80, 0).astype(np.uint8)).astype(np.uint8)


def rng(seed):
    return np.random.default_rng(seed)


def random_storage(dt: str, n: int, seed: int, scale: float = 1.0) -> np.ndarray:
    """n elements of dtype dt as a storage array (bit patterns for narrow floats)"""
    g = rng(seed)
    if dt == "bf16":
        return f32_to_bf16_rne((g.standard_normal(n) * scale).astype(np.float32))
    if dt == "f16":
        return f16_bits((g.standard_normal(n) * scale).astype(np.float32))
    if dt == "f8e4m3":
        return f32_to_ocp_e4m3_rne(g.standard_normal(n) * scale)
    if dt == "f8e5m2":
        return (f16_bits((g.standard_normal(n) * scale).astype(np.float32)) >> 8).astype(np.uint8)
    if dt == "f32":
        return (g.standard_normal(n) * scale).astype(np.float32)
    if dt == "f64":
        return g.standard_normal(n) * scale
    if dt == "bool":
        return g.integers(0, 2, n).astype(np.uint8)
    info = np.iinfo({"u8": np.uint8, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64, "i8": np.int8,
                     "i16": np.int16, "i32": np.int32, "i64": np.int64}[dt])
    lo, hi = max(info.min, -100), min(info.max, 100)
    return g.integers(lo, hi + 1, n).astype(info.dtype)


def widen(dt: str, x: np.ndarray, ocp=True) -> np.ndarray:
    """storage array -> float64 values (independent of the oracle)"""
    if dt == "bf16":
        return bf16_to_f32(x).astype(np.float64)
    if dt == "f16":
        return x.view(np.float16).astype(np.float64)
    if dt == "f8e4m3":
        assert ocp
        return ocp_e4m3_decode(x).astype(np.float64)
    if dt == "f8e5m2":
        return (x.astype(np.uint16) << 8).view(np.float16).astype(np.float64)
    return x.astype(np.float64)


# unit round-off of the accumulator a product is summed in
EPS_F32, EPS_F64 = 2.0 ** -24, 2.0 ** -53
# Constant of the rounding-model floor.  A sum of K products accumulated in a type of unit round-off eps, in any
# order, is off by a random walk of about 0.5 * eps * sum|a b| (standard deviation: each partial sum of zero-mean
# terms is ~ sqrt(k) terms large and is rounded once); the largest of 10^7 such errors is ~ 3 * eps * sum|a b|, and
# the comparator's own f32 sum carries the same.  8 leaves a factor of two above that.
FLOOR_C = 8.0


def rel_floor(sumabs, k: int, tol: float, eps_acc: float = EPS_F32) -> np.ndarray:
    """The least denominator an element is judged against: the smaller of
      * sum|a b| / sqrt(K): the magnitude a random-sign sum of the element's own products would have (no element is
        ever judged against something larger than an ordinary output), and
      * FLOOR_C * eps_acc * sum|a b| / tol: the accumulation error of a correct kernel expressed in units of `tol`,
        so that an element which cancelled to (almost) zero is allowed exactly that absolute error and no more.
    For bf16 / f16 / fp8 outputs at tol = 2e-2 the second is the smaller by two to three orders of magnitude
    (2.4e-5 * sum|a b| against 1.6e-2 * sum|a b| at K = 4096); for f32 outputs at 1e-5 the two are comparable."""
    sumabs = np.asarray(sumabs, dtype=np.float64)
    return np.minimum(sumabs / np.sqrt(max(int(k), 1)), FLOOR_C * eps_acc * sumabs / tol)


def rel_err(got: np.ndarray, want: np.ndarray, sumabs: np.ndarray, k: int, tol: float,
            eps_acc: float = EPS_F32) -> np.ndarray:
    """Per-element relative error |got - want| / max(|want|, rel_floor).

    Dividing by |want| alone reports arbitrarily large 'relative' errors for a correct kernel on the few of 10^7
    zero-mean sums that cancel to ~0; the floor (rel_floor) is what the accumulator's rounding alone can contribute
    there, expressed in units of the tolerance the caller is about to apply.  An element of ordinary size is judged
    against |want| alone: at bf16 tolerances and K = 4096 that is every element above ~0.1 % of the typical output
    magnitude."""
    den = np.maximum(np.abs(want), rel_floor(sumabs, k, tol, eps_acc))
    den = np.where(den == 0, 1.0, den)
    return np.abs(np.asarray(got, dtype=np.float64) - want) / den


def floor_fraction(want, sumabs, k: int, tol: float, eps_acc: float = EPS_F32) -> float:
    """fraction of elements whose denominator is the floor rather than |want|"""
    want = np.asarray(want, dtype=np.float64)
    return float(np.mean(np.abs(want) < rel_floor(sumabs, k, tol, eps_acc))) if want.size else 0.0


def assert_close(got, want, sumabs, k: int, tol: float, what: str = "", eps_acc: float = EPS_F32):
    """asserts rel_err <= tol for every element; the message names the worst element and how many elements were
    judged on the floor"""
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    sumabs = np.asarray(sumabs, dtype=np.float64).ravel()
    if got.size == 0:
        return
    rel = rel_err(got, want, sumabs, k, tol, eps_acc)
    worst = int(np.argmax(rel))
    assert rel[worst] <= tol, (
        f"{what}: max rel err {rel[worst]:.3e} > {tol:g} at element {worst} (got {got[worst]!r}, want {want[worst]!r}, "
        f"sum|ab| {sumabs[worst]!r}); {int((rel > tol).sum())} of {rel.size} elements fail; "
        f"{100 * floor_fraction(want, sumabs, k, tol, eps_acc):.2f} % of elements are judged on the floor")
