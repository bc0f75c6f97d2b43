"""Where oracle/_ref was built (the build container), the oracle is compared bit for bit with the
reference's own compiled C kernels on fresh seeded cases beyond the committed fixtures."""
import numpy as np
import pytest

import helpers as H
import oracle

pytestmark = pytest.mark.skipif(not oracle.RefLib.available(), reason="oracle/_ref not built on this machine")


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


@pytest.fixture(scope="module")
def ref():
    return oracle.RefLib()


CASES = [
    ("dot", H.View([64, 130]), H.View([130, 70])),
    ("dot", H.View([530, 33]), H.View([33, 9])),
    ("dot", H.View([12, 300]), H.View([16, 300]).t()),
    ("dot", H.View([50, 12], offset=9).t(), H.View([50, 12], offset=1)),
    ("matmul", H.View([5, 8, 33]), H.View([5, 33, 6])),
    ("matmul", H.View([300, 20]), H.View([20, 8])),
    ("matmul", H.View([2, 3, 4, 20]), H.View([7, 20]).t().broadcast_to([2, 3, 20, 7])),
    ("matmul", H.View([1, 6, 20]), H.View([4, 20, 5])),
]


@pytest.mark.parametrize("dt", oracle.MATMUL_DTYPES)
def test_products_match_compiled_reference(ref, dt):
    for n, (op, lv, rv) in enumerate(CASES):
        a = H.random_storage(dt, lv.span(), 1000 + n, 2.0)
        b = H.random_storage(dt, rv.span(), 2000 + n, 2.0)
        md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
        want = ref.dot(dt, a, b, md) if op == "dot" else ref.matmul(dt, a, b, md)
        got = oracle.dot_asis(dt, a, b, md) if op == "dot" else oracle.matmul_asis(dt, a, b, md)
        assert np.array_equal(_bits(got), _bits(want)), (dt, n)


def test_every_cast_pair_matches_compiled_reference(ref):
    v = H.View([7, 9, 5], offset=3).t(0, 2)
    md = H.cast_md(v)
    for src in oracle.DTYPE_ID:
        for dst in oracle.DTYPE_ID:
            x = H.random_storage(src, v.span(), 77, 3.0)
            if src in ("f32", "f64") and dst.startswith("u") or dst == "bool" and src in ("f32", "f64"):
                x = np.abs(x)
            if src in ("bf16", "f16") and dst.startswith("u"):
                x = x & 0x7FFF
            if src in ("f8e4m3", "f8e5m2") and dst.startswith("u"):
                x = x & 0x7F
            want, got = ref.cast(src, dst, x, md), oracle.cast(src, dst, x, md)
            if dst in ("f32", "f64"):
                gf, wf = got, want
                assert np.array_equal(np.isnan(gf), np.isnan(wf)), (src, dst)
                assert np.array_equal(gf[~np.isnan(gf)], wf[~np.isnan(wf)]), (src, dst)
            else:
                assert np.array_equal(_bits(got), _bits(want)), (src, dst)


def test_contiguous_matches_compiled_reference(ref):
    for v in (H.View([300]), H.View([13, 21]).t(), H.View([4, 5, 6], offset=2).slice(1, 1, 5, 2)):
        for dt in oracle.DTYPE_ID:
            x = H.random_storage(dt, v.span(), 5)
            assert np.array_equal(_bits(ref.contiguous(dt, x, H.cast_md(v))), _bits(oracle.contiguous(dt, x, H.cast_md(v))))


ELEMENTWISE_DTYPES = [d for d in oracle.DTYPE_ID if d != "bool"]


@pytest.mark.parametrize("dt", ELEMENTWISE_DTYPES)
def test_elementwise_match_compiled_reference(ref, dt):
    """add over every layout branch of the reference (both contiguous, one strided, both strided), mul_scalar and
    relu, on fresh seeded values"""
    V = H.View
    full = V([5, 6, 33])
    layouts = [(full, V([33], offset=1).broadcast_to([5, 6, 33])), (V([33]).broadcast_to([5, 6, 33]), full),
               (full, V([5, 6, 33], offset=7)), (V([33, 6, 5]).t(0, 2), V([5, 1, 33], offset=2).broadcast_to([5, 6, 33]))]
    floating = dt in ("f8e4m3", "f8e5m2", "bf16", "f16", "f32", "f64")
    for n, (lv, rv) in enumerate(layouts):
        a = H.random_storage(dt, lv.span(), 300 + n, 3.0)
        b = H.random_storage(dt, rv.span(), 400 + n, 3.0)
        md = H.binary_md(lv, rv)
        assert np.array_equal(_bits(oracle.add(dt, a, b, md)), _bits(ref.add(dt, a, b, md))), (dt, n)
    x = H.random_storage(dt, 200_000, 9, 3.0)  # above the reference's threading threshold (ops_unary.c:164)
    md = H.cast_md(V([200_000]))
    c = H.random_storage(dt, 8, 10, 3.0)[3:4]
    assert np.array_equal(_bits(oracle.mul_scalar(dt, x, md, c)), _bits(ref.mul_scalar(dt, x, md, c))), dt
    v = V([40, 50], offset=3).t()
    assert np.array_equal(_bits(oracle.mul_scalar(dt, x, H.cast_md(v), c)), _bits(ref.mul_scalar(dt, x, H.cast_md(v), c))), dt
    if floating:
        assert np.array_equal(_bits(oracle.relu(dt, x, md)), _bits(ref.relu(dt, x, md))), dt
        assert np.array_equal(_bits(oracle.relu(dt, x, H.cast_md(v))), _bits(ref.relu(dt, x, H.cast_md(v)))), dt


@pytest.mark.parametrize("dt", ELEMENTWISE_DTYPES)
def test_sums_match_compiled_reference(ref, dt):
    V = H.View
    cases = [(V([4, 9, 20]), [0], False), (V([4, 9, 20]), [0], True), (V([2, 3, 5, 8]), [1], True),
             (V([2, 3, 5, 8]), [0, 2], False), (V([7, 30], offset=2).t(), [1], False), (V([5, 6]), [0, 1], False)]
    for n, (v, dims, keep) in enumerate(cases):
        x = H.random_storage(dt, v.span(), 500 + n, 2.0)
        md = H.reduce_md(v, dims, keep)
        assert np.array_equal(_bits(oracle.sum_asis(dt, x, md)), _bits(ref.sum(dt, x, md))), (dt, n)


def test_softmax_comparator_matches_the_reference_five_kernel_chain(ref):
    """Tensor::softmax(-1) as hodu runs it on f32 (max, sub, exp, sum, div through the compiled reference kernels)
    against the one-pass comparator: the same function to rounding"""
    V = H.View
    x = (H.rng(42).standard_normal(4 * 9 * 33) * 4).astype(np.float32)
    chain = ref.softmax_chain_f32(x, [4, 9, 33])
    o32, o64 = oracle.softmax_spec("f32", x, H.reduce_md(V([4, 9, 33]), [2], True))
    assert np.allclose(chain, o64, rtol=3e-6, atol=1e-12) and np.allclose(chain, o32, rtol=3e-6, atol=1e-12)
