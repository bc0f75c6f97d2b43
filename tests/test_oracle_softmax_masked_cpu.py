"""The masked-softmax comparator (attention's attn_mask, crates/hodu_nn/src/modules/attention.rs:40-56), pinned without
a GPU: against the softmax of each row's unmasked entries, against the unmasked comparator for a mask of ones, against an
explicit masked_fill + softmax in numpy float64, for rows masked entirely (uniform in the 16-bit types, NaN in f32 /
f64, as the reference's fill values make them), with broadcast masks, and -- f32, where the compiled reference is
present -- against the reference's own five softmax kernels run on the filled scores."""
import numpy as np
import pytest

import helpers as H
import oracle

V = H.View


def _mask_strides(mask_shape, full_shape):
    """element strides of a dense mask of `mask_shape` (right-aligned, extent 1 = broadcast) over `full_shape`"""
    ms = [1] * (len(full_shape) - len(mask_shape)) + list(mask_shape)
    strides, acc = [0] * len(ms), 1
    for d in range(len(ms) - 1, -1, -1):
        strides[d] = 0 if ms[d] == 1 and full_shape[d] != 1 else acc
        acc *= ms[d]
    return strides, np.broadcast_to(np.zeros(ms, np.uint8), full_shape).shape


def _numpy_masked_softmax(x64, open_mask, fill):
    filled = np.where(open_mask, x64, fill)
    with np.errstate(invalid="ignore"):
        e = np.exp(filled - filled.max(axis=-1, keepdims=True))
        return e / e.sum(axis=-1, keepdims=True)


@pytest.mark.parametrize("mask_shape", [(2, 3, 7, 12), (1, 1, 7, 12), (2, 1, 1, 12), (7, 12), (12,)])
@pytest.mark.parametrize("causal", [False, True])
def test_against_numpy_fill_then_softmax_and_the_unmasked_subset(mask_shape, causal):
    full = (2, 3, 7, 12)
    g = np.random.default_rng(hash((mask_shape, causal)) % 2 ** 32)
    x = (g.standard_normal(full) * 3).astype(np.float32)
    mask = (g.random(mask_shape) > 0.35).astype(np.uint8)
    mask.reshape(-1)[0] = 1
    # every row keeps at least its first entry open (also under the causal mask): rows masked entirely are their own test
    mask[..., 0] = 1
    strides, _ = _mask_strides(mask_shape, full)
    md = H.reduce_md(V(list(full)), [3], True)
    o32, o64 = oracle.softmax_masked_spec("f32", x.ravel(), md, mask.ravel(), strides, 0, causal)
    open_mask = np.broadcast_to(mask.reshape((1,) * (4 - len(mask_shape)) + mask_shape), full).astype(bool)
    if causal:
        open_mask = open_mask & (np.arange(12)[None, :] <= np.arange(7)[:, None])
    want = _numpy_masked_softmax(x.astype(np.float64), open_mask, -np.inf)
    assert np.allclose(o64.reshape(full), want, rtol=1e-12, atol=0)
    assert np.allclose(o32.reshape(full), want, rtol=2e-6, atol=1e-9)
    # a masked entry is an exact zero, and each row is the softmax of its open entries alone
    assert np.all(o64.reshape(full)[~open_mask] == 0.0)
    for idx in [(0, 0, 0), (1, 2, 6), (0, 1, 3)]:
        row, keep = x[idx].astype(np.float64), open_mask[idx]
        e = np.exp(row[keep] - row[keep].max())
        assert np.allclose(o64.reshape(full)[idx][keep], e / e.sum(), rtol=1e-12)


def test_mask_of_ones_is_the_unmasked_comparator():
    full = (3, 5, 33)
    x = H.random_storage("bf16", 3 * 5 * 33, 7, 2.0)
    md = H.reduce_md(V(list(full)), [2], True)
    ones = np.ones(33, np.uint8)
    for causal in (False, True):
        a32, a64 = oracle.softmax_masked_spec("bf16", x, md, ones, [0, 0, 1], 0, causal)
        b32, b64 = oracle.softmax_spec("bf16", x, md, causal)
        assert np.array_equal(a64, b64) and np.array_equal(a32, b32)


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_rows_masked_entirely(dt):
    """get_neg_inf (attention.rs:88-96) is finite for the 16-bit types: a row without an open entry is a softmax of
    equal values, 1 / len; in f32 / f64 the fill is -inf and the row is NaN"""
    full = (4, 10)
    x = H.random_storage(dt, 40, 11, 2.0)
    mask = np.ones(full, np.uint8)
    mask[1, :] = 0
    mask[3, 5:] = 0
    md = H.reduce_md(V(list(full)), [1], True)
    o32, o64 = oracle.softmax_masked_spec(dt, x, md, mask.ravel(), [10, 1])
    o64, o32 = o64.reshape(full), o32.reshape(full)
    if dt in ("bf16", "f16"):
        assert np.allclose(o64[1], 0.1, rtol=1e-12) and np.allclose(o32[1], 0.1, rtol=1e-6)
    else:
        assert np.all(np.isnan(o64[1])) and np.all(np.isnan(o32[1]))
    assert np.all(np.isfinite(o64[[0, 2, 3]])) and np.all(o64[3, 5:] == 0.0)
    assert np.allclose(o64[[0, 2, 3]].sum(axis=1), 1.0, rtol=1e-12)


def test_strided_input_and_mask_offset():
    # scores as a transposed view, the mask a window of a larger buffer
    x = (H.rng(5).standard_normal(6 * 9) * 2).astype(np.float32)
    xv = V([9, 6]).t()                       # logical [6, 9]
    big = (H.rng(6).random(4 + 6 * 9) > 0.4).astype(np.uint8)
    big[4::9] = 1                            # first entry of every row open
    md = H.reduce_md(xv, [1], True)
    _, o64 = oracle.softmax_masked_spec("f32", x, md, big, [9, 1], 4)
    open_mask = big[4:].reshape(6, 9).astype(bool)
    want = _numpy_masked_softmax(x.reshape(9, 6).T.astype(np.float64), open_mask, -np.inf)
    assert np.allclose(o64.reshape(6, 9), want, rtol=1e-12, atol=0)


def test_f32_against_the_reference_five_kernel_chain():
    """masked_fill is a select; the softmax that follows it is the reference's own five kernels
    (hodu_cpu_max / sub / exp / sum / div through oracle/_ref) run on the filled scores"""
    if not oracle.RefLib.available():
        pytest.skip("oracle/_ref is not built here")
    ref = oracle.RefLib()
    full = [4, 9, 33]
    g = H.rng(43)
    x = (g.standard_normal(4 * 9 * 33) * 4).astype(np.float32)
    mask = (g.random((4, 1, 33)) > 0.3).astype(np.uint8)
    mask[..., 0] = 1
    filled = np.where(np.broadcast_to(mask, full).astype(bool), x.reshape(full), np.float32(-np.inf)).astype(np.float32)
    chain = ref.softmax_chain_f32(filled.ravel(), full)
    o32, o64 = oracle.softmax_masked_spec("f32", x, H.reduce_md(V(full), [2], True), mask.ravel(), [33, 0, 1])
    assert np.allclose(chain, o64, rtol=3e-6, atol=1e-12) and np.allclose(chain, o32, rtol=3e-6, atol=1e-12)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("causal", [False, True])
def test_the_masked_attention_tests_float64_function_is_this_softmax_between_two_products(dt, causal):
    """tests/test_zx_attention_masked.py compares the one-kernel attention with a float64 function of its own; that
    function's probabilities are the oracle's masked softmax of the (unrounded) scaled scores -- fill value, causal mask
    and rows masked entirely included"""
    import test_zx_attention_masked as A
    g = np.random.default_rng(5)
    b, sq, sk, d = 2, 9, 13, 8
    q, k, v = (g.standard_normal((b, n, d)) for n in (sq, sk, sk))
    keep = (g.random((b, 1, sk)) < 0.6).astype(np.uint8)
    keep[1, 0, :] = 0  # a batch whose every row is masked entirely
    scale = 0.35
    want, _, p, _ = A.reference(q, k, v, scale, causal, keep, A.FILL[dt])
    # the oracle takes the scores in a storage type: f64 holds them exactly
    scores = q @ np.swapaxes(k, -1, -2) * scale
    md = H.reduce_md(H.View([b, sq, sk]), [2], True)
    _, o64 = oracle.softmax_masked_spec("f64", scores.ravel(), md, keep.ravel(), [sk, 0, 1], 0, causal)
    # f64's fill is -inf: identical wherever a row has an open key; rows masked entirely are uniform in the 16-bit types
    o64 = o64.reshape(b, sq, sk)
    open_rows = ~np.isnan(o64).any(-1)
    assert open_rows[0].all() and not open_rows[1].any()
    assert np.allclose(p[open_rows], o64[open_rows], rtol=1e-12, atol=1e-300)
    assert np.allclose(p[~open_rows], 1.0 / sk)
    assert np.allclose(want, p @ v)
