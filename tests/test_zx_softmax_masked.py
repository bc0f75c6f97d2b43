"""GPU parity of hodu_rocm_softmax_masked and of the attn_mask path of scaled_dot_product_attention
(crates/hodu_nn/src/modules/attention.rs:40-56).  (The file name sorts it behind the tests of the kernels that have a
longer history on the hardware; these cases also run against the CPU build of the same kernel source,
tests/test_emu_gpu_suites_cpu.py and tests/test_emu_host_mirror_cpu.py.)

The comparator is oracle.softmax_masked_spec, pinned on the CPU by tests/test_oracle_softmax_masked_cpu.py.
Tolerances as in test_gpu_softmax.py: f32 1e-5, bf16 / f16 2e-2, f64 1e-12 relative; a masked entry of a row that
has an open one must be an exact zero; a row masked entirely is uniform (16-bit types) or NaN (f32 / f64)."""
import numpy as np
import pytest

import helpers as H
import oracle
from hodu_amd import ffi
from hodu_amd import tensor as T

pytestmark = pytest.mark.gpu
V = H.View
TOL = {"f32": 1e-5, "bf16": 2e-2, "f16": 2e-2, "f64": 1e-12}
FLOOR = {"f32": 1e-30, "bf16": 1e-30, "f16": 2.0 ** -24, "f64": 1e-30}


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def mask_strides(mask_shape, full_shape):
    ms = [1] * (len(full_shape) - len(mask_shape)) + list(mask_shape)
    strides, acc = [0] * len(ms), 1
    for d in range(len(ms) - 1, -1, -1):
        strides[d] = 0 if ms[d] == 1 and full_shape[d] != 1 else acc
        acc *= ms[d]
    return strides


def check(ctx, dt, v, mask_shape, causal=False, seed=0, closed_rows=(), mask_dt="u8"):
    full = v.shape
    g = np.random.default_rng(1234 + seed)
    x = H.random_storage(dt, v.span(), 900 + seed, 3.0)
    mask = (g.random(mask_shape) > 0.4).astype(np.uint8)
    mask[..., 0] = 1
    for r in closed_rows:   # rows of the flattened mask closed entirely
        mask.reshape(-1, mask_shape[-1])[r, :] = 0
    strides = mask_strides(mask_shape, full)
    md = H.reduce_md(v, [len(full) - 1], True)
    n = v.size
    dx, dm, dout = ctx.upload(x), ctx.upload(mask.ravel()), ctx.alloc(n * ffi.DTYPE_SIZE[dt])
    ctx.fill(dout, 0xFF)
    ctx.softmax_masked(dt, dx, dout, md, dm, strides, 0, causal, mask_dt)
    assert ctx.last_kernel() == "softmax_masked"
    got = H.widen(dt, ctx.download(dout, oracle.STORAGE[dt], n))
    for b in (dx, dm, dout):
        b.free()
    _, want = oracle.softmax_masked_spec(dt, x, md, mask.ravel(), strides, 0, causal)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.all(got[~nan][want[~nan] == 0.0] == 0.0)
    err = np.abs(got[~nan] - want[~nan])
    assert np.all(err <= TOL[dt] * np.abs(want[~nan]) + FLOOR[dt]), f"{dt}: max rel err {(err / np.maximum(np.abs(want[~nan]), FLOOR[dt])).max():.3e}"


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_masks_of_every_broadcast_shape(ctx, dt):
    full = [2, 3, 50, 70]
    for n, ms in enumerate(([2, 3, 50, 70], [1, 1, 50, 70], [2, 1, 1, 70], [50, 70], [70])):
        check(ctx, dt, V(full), ms, seed=n)
        check(ctx, dt, V(full), ms, causal=True, seed=10 + n)
    check(ctx, dt, V([5, 1]), [5, 1], seed=20)          # rows of one entry
    check(ctx, dt, V([3, 4100]), [3, 4100], seed=21)    # longer than one pass of a wavefront many times over
    check(ctx, dt, V([70, 50]).t(), [50, 70], seed=22)  # scores as a transposed view


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_rows_masked_entirely(ctx, dt):
    check(ctx, dt, V([4, 6, 33]), [4, 6, 33], seed=30, closed_rows=(0, 7, 23))
    check(ctx, dt, V([4, 6, 33]), [4, 1, 33], seed=31, closed_rows=(2,))


def test_bool_and_i8_masks(ctx):
    check(ctx, "bf16", V([3, 9, 40]), [9, 40], seed=40, mask_dt="bool")
    check(ctx, "f32", V([3, 9, 40]), [9, 40], seed=41, mask_dt="i8")


@pytest.mark.parametrize("D, launches", [(64, 1), (32, 3)])
def test_attention_with_a_padding_mask_against_float64(ctx, D, launches):
    """scaled_dot_product_attention(q, k, v, attn_mask) through the host mirror: a [B, 1, 1, Sk] padding mask.  Head dim
    64: the one kernel (hodu_rocm_attention_masked); head dim 32, which that kernel does not take: three launches, the
    middle one hodu_rocm_softmax_masked.  Held to the float64 function at the products' 2e-2 of the sum's size"""
    B, Hh, S = 2, 4, 96
    g = np.random.default_rng(77)
    q, k, v = (g.standard_normal((B, Hh, S, D)).astype(np.float32) for _ in range(3))
    keep = np.ones((B, 1, 1, S), np.uint8)
    keep[0, ..., 70:] = 0
    keep[1, ..., 33:] = 0
    qb, kb, vb = (H.f32_to_bf16_rne(a.ravel()) for a in (q, k, v))
    tq, tk, tv = (T.Tensor.from_bits(b, "bf16", [B, Hh, S, D]) for b in (qb, kb, vb))
    tm = T.Tensor.from_bits(keep.ravel(), "u8", [B, 1, 1, S])
    T.stats(reset=True)
    out = T.scaled_dot_product_attention(tq, tk, tv, False, tm)
    st = T.stats()
    if launches == 1:
        assert st["attention_kernels"] == 1 and st["product_kernels"] == 0 and st["softmax_kernels"] == 0 and st["contiguous_kernels"] == 0
    else:
        assert st["product_kernels"] == 2 and st["softmax_kernels"] == 1 and st["attention_kernels"] == 0 and st["contiguous_kernels"] == 0
    got = H.bf16_to_f32(out.to_bits()).astype(np.float64).reshape(B, Hh, S, D)
    q64, k64, v64 = (H.bf16_to_f32(b).astype(np.float64).reshape(B, Hh, S, D) for b in (qb, kb, vb))
    scale = float(H.bf16_to_f32(T.scalar_bits("bf16", 1.0 / np.sqrt(float(D))))[0])
    s = q64 @ k64.transpose(0, 1, 3, 2) * scale
    s = np.where(keep.astype(bool), s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p = p / p.sum(-1, keepdims=True)
    want = p @ v64
    # the three-launch path rounds the scores to bf16 twice (product, scale) and the probabilities once: relative errors
    # of every p_j of up to 2^-8 |s|, i.e. an error of the output that scales with sum_j p_j |v_j| -- the size of the sum,
    # not of its (possibly cancelling) value; with as few as 33 unmasked keys that floor matters
    assert np.all(np.abs(got - want) <= 2e-2 * np.maximum(np.abs(want), p @ np.abs(v64)))


@pytest.mark.parametrize("D", [64, 32])
def test_a_mask_of_another_dtype_is_its_nonzero_pattern(ctx, D):
    """`mask.eq_scalar(0)` (attention.rs:52) takes any dtype: an f32 mask holding -0.0 (masks), 0.5 and a NaN (attend)
    gives the bytes of the u8 mask with the same nonzero pattern, through the one kernel (D = 64) and the three launches"""
    B, Hh, S = 2, 2, 40
    g = np.random.default_rng(1)
    q, k, v = (H.f32_to_bf16_rne(g.standard_normal(B * Hh * S * D).astype(np.float32)) for _ in range(3))
    tq, tk, tv = (T.Tensor.from_bits(b, "bf16", [B, Hh, S, D]) for b in (q, k, v))
    keep = np.ones((B, 1, 1, S), np.float32)
    keep[0, ..., 30:] = 0.0
    keep[1, ..., 5:9] = -0.0
    keep[1, ..., 20] = 0.5
    keep[1, ..., 21] = np.nan
    pattern = np.ones((B, 1, 1, S), np.uint8)
    pattern[0, ..., 30:] = 0
    pattern[1, ..., 5:9] = 0
    as_f32 = T.Tensor.from_bits(keep.ravel().view(np.uint32), "f32", [B, 1, 1, S])
    as_u8 = T.Tensor.from_bits(pattern.ravel(), "u8", [B, 1, 1, S])
    for causal in (False, True):
        T.stats(reset=True)
        got = T.scaled_dot_product_attention(tq, tk, tv, causal, as_f32).to_bits()
        assert T.stats()["cast_kernels"] == 1
        assert np.array_equal(got, T.scaled_dot_product_attention(tq, tk, tv, causal, as_u8).to_bits())
