"""GPU checks of the Tensor-level path (hodu_amd.tensor over the C++ host mirror over the C ABI):
routing, broadcast, deferred casts and the copy/no-copy equivalence, against the oracle and against the
known-answer vectors of the reference's own kernel tests."""
import numpy as np
import pytest

import helpers as H
import oracle
from hodu_amd import tensor as T

pytestmark = pytest.mark.gpu


def f32_bits(values):
    return np.asarray(values, dtype=np.float32).view(np.uint32)


def f32_of(t):
    return t.to_bits().view(np.float32)


def from_f32(values, shape):
    return T.Tensor.from_bits(f32_bits(values), "f32", shape)


# ---- the reference's known-answer tests, through the Tensor API ------------------------------------
def test_reference_known_answers():
    a = from_f32([1, 2, 3, 4, 5, 6], [2, 3])
    b = from_f32([7, 8, 9, 10, 11, 12], [3, 2])
    # crates/hodu_cpu_kernels/tests/ops_matrix.rs:8-61 and :119-147
    assert f32_of(a.matmul(b)).tolist() == [58, 64, 139, 154]
    assert f32_of(a.dot(b)).tolist() == [58, 64, 139, 154]
    # :63-117
    l = from_f32([1, 2, 3, 4, 2, 3, 4, 5], [2, 2, 2])
    r = from_f32([5, 6, 7, 8, 6, 7, 8, 9], [2, 2, 2])
    out = l.matmul(r)
    assert out.shape == [2, 2, 2] and f32_of(out).tolist() == [19, 22, 43, 50, 36, 41, 64, 73]
    # crates/hodu_cuda_kernels/tests/ops_matrix.rs:188-262: shared weight without a batch dim
    l = from_f32(np.arange(1, 13), [2, 2, 3])
    w = from_f32([1, 0, 0, 1, 1, 1], [3, 2])
    assert f32_of(l.matmul(w)).tolist() == [4, 5, 10, 11, 16, 17, 22, 23]
    # crates/hodu_metal_kernels/tests/ops_matrix.rs:230-313
    w = from_f32([1, 2, 3, 4, 5, 6], [3, 2])
    assert f32_of(l.matmul(w)).tolist() == [22, 28, 49, 64, 76, 100, 103, 136]
    # crates/hodu_cuda_kernels/tests/ops_matrix.rs:103-151 (3x3 square)
    s = from_f32(np.arange(1, 10), [3, 3])
    r = from_f32([9, 8, 7, 6, 5, 4, 3, 2, 1], [3, 3])
    assert f32_of(s.matmul(r)).tolist() == [30, 24, 18, 84, 69, 54, 138, 114, 90]


def test_cast_known_answers():
    # crates/hodu_cuda_kernels/tests/ops_cast.rs:48-89: float -> int truncates toward zero
    x = from_f32([1.7, -2.3, 3.9, -4.1], [4])
    assert x.to_dtype("i32").to_bits().view(np.int32).tolist() == [1, -2, 3, -4]
    assert from_f32([1.7, 2.3, 3.9, 4.1], [4]).to_dtype("u32").to_bits().tolist() == [1, 2, 3, 4]
    i = T.Tensor.from_bits(np.array([1, -2, 3, -4], np.int32).view(np.uint32), "i32", [4])
    assert f32_of(i.to_dtype("f32")).tolist() == [1, -2, 3, -4]


# ---- rank routing: numpy matmul semantics for 1-D / 2-D / N-D --------------------------------------
@pytest.mark.parametrize("ls,rs", [([7], [7]), ([5, 7], [7]), ([7], [7, 3]), ([5, 7], [7, 3]), ([2, 5, 7], [2, 7, 3]),
                                   ([2, 5, 7], [7, 3]), ([5, 7], [4, 7, 3]), ([3, 1, 5, 7], [2, 7, 3]),
                                   ([1, 5, 7], [4, 1, 7, 3])])
def test_matmul_routing_matches_numpy(ls, rs):
    g = np.random.default_rng(5)
    a = g.integers(-4, 5, ls).astype(np.float32)
    b = g.integers(-4, 5, rs).astype(np.float32)
    out = from_f32(a.ravel(), ls).matmul(from_f32(b.ravel(), rs))
    want = np.matmul(a, b)
    assert out.shape == list(want.shape)
    assert np.array_equal(f32_of(out), want.ravel())  # small integers: exact in f32


def test_dot_rejects_batched_operands_and_mismatches():
    a = from_f32(np.zeros(12), [2, 2, 3])
    b = from_f32(np.zeros(6), [3, 2])
    with pytest.raises(T.HoduError) as e:
        a.dot(b)
    assert e.value.kind == "InternalError"
    with pytest.raises(T.HoduError) as e:
        b.matmul(b)
    assert e.value.kind == "IncompatibleShapes"
    with pytest.raises(T.HoduError) as e:
        a.matmul(from_f32(np.zeros(18), [3, 3, 2]))
    assert e.value.kind == "IncompatibleShapes"
    i = T.Tensor.from_bits(np.zeros(6, np.uint32), "i32", [3, 2])
    with pytest.raises(T.HoduError) as e:
        b.t().matmul(i)
    assert e.value.kind == "DTypeMismatch"
    q = T.Tensor.from_bits(np.zeros(4, np.uint8), "bool", [2, 2])
    with pytest.raises(T.HoduError) as e:
        q.matmul(q)
    assert e.value.kind == "UnsupportedDTypeForOp"


# ---- views -------------------------------------------------------------------------------------------
def test_views_share_storage_and_contiguous_gathers():
    x = np.arange(24, dtype=np.float32)
    t = from_f32(x, [2, 3, 4])
    tt = t.t()
    assert tt.shares_storage_with(t) and tt.layout() == ([2, 4, 3], [12, 1, 4], 0)
    assert np.array_equal(f32_of(tt), x.reshape(2, 3, 4).transpose(0, 2, 1).ravel())
    c = tt.contiguous()
    assert not c.shares_storage_with(t) and c.layout() == ([2, 4, 3], [12, 3, 1], 0)
    assert t.contiguous().shares_storage_with(t)
    # a second view op on a non-contiguous tensor copies first (shape.rs:232-237, :296-299)
    assert not tt.transpose(0, 1).shares_storage_with(t)
    s = t.slice(1, 1, None, 1)
    assert s.layout() == ([2, 2, 4], [12, 4, 1], 4)
    assert np.array_equal(f32_of(s), x.reshape(2, 3, 4)[:, 1:, :].ravel())
    b = from_f32([1, 2, 3], [3]).broadcast([2, 3])
    assert b.layout() == ([2, 3], [0, 1], 0) and f32_of(b).tolist() == [1, 2, 3, 1, 2, 3]
    with pytest.raises(T.HoduError) as e:
        t.view([4, 4, 4], [16, 4, 1]).to_bits()
    assert e.value.kind == "InvalidLayout"


# ---- deferred to_dtype: the cast is fused into the product ------------------------------------------
def test_f8_weight_cast_is_deferred_and_fused():
    m, k, n = 24, 256, 96
    w8 = H.random_storage("f8e4m3", n * k, 11, 40.0)
    xb = H.random_storage("bf16", m * k, 12, 1.0)
    w = T.Tensor.from_bits(w8, "f8e4m3", [n, k])
    x = T.Tensor.from_bits(xb, "bf16", [m, k])
    T.stats(reset=True)
    wb = w.to_dtype("bf16")
    assert wb.dtype == "bf16" and wb.physical_dtype == "f8e4m3" and wb.shares_storage_with(w)
    y = x.matmul(wb.t())
    st = T.stats(reset=True)
    assert st["cast_kernels"] == 0 and st["contiguous_kernels"] == 0 and st["fused_products"] == 1
    lv, rv = H.View([m, k]), H.View([n, k]).t()
    want32, _, sumabs = oracle.dot_spec("bf16", "f8e4m3", xb, w8, H.dot_md(lv, rv), decode=oracle.F8_OCP)
    got = H.bf16_to_f32(y.to_bits())
    assert H.rel_err(got, want32, sumabs, k).max() <= 2e-2  # bf16 output, f32 accumulate
    # reading the deferred tensor materialises the cast: bit-exact with the cast oracle (OCP decode)
    want_bits = oracle.cast("f8e4m3", "bf16", w8, H.cast_md(H.View([n, k])), decode=oracle.F8_OCP)
    assert np.array_equal(wb.to_bits(), want_bits)
    # the unfused route (cast of a strided view runs the kernel) gives the same product to one bf16 step
    wt_dense = w.t().to_dtype("bf16")  # non-dense input: materialised, [k, n] contiguous
    assert wt_dense.physical_dtype == "bf16"
    y2 = x.matmul(wt_dense)
    assert H.rel_err(H.bf16_to_f32(y2.to_bits()), want32, sumabs, k).max() <= 2e-2


def test_i8_casts_are_deferred_and_the_product_is_bit_exact():
    m, k, n = 40, 192, 56
    g = np.random.default_rng(3)
    a8 = g.integers(-127, 128, m * k).astype(np.int8)
    b8 = g.integers(-127, 128, k * n).astype(np.int8)
    a = T.Tensor.from_bits(a8.view(np.uint8), "i8", [m, k])
    b = T.Tensor.from_bits(b8.view(np.uint8), "i8", [k, n])
    T.stats(reset=True)
    out = a.to_dtype("i32").matmul(b.to_dtype("i32"))
    st = T.stats(reset=True)
    assert st["fused_products"] == 1 and st["cast_kernels"] == 0
    want = a8.reshape(m, k).astype(np.int64) @ b8.reshape(k, n).astype(np.int64)
    assert out.dtype == "i32" and np.array_equal(out.to_bits().view(np.int32), want.astype(np.int32).ravel())
    # one deferred operand against a plain i32 operand: the deferred one is materialised, same numbers
    b32 = T.Tensor.from_bits(b8.astype(np.int32).view(np.uint32), "i32", [k, n])
    out2 = a.to_dtype("i32").matmul(b32)
    st = T.stats(reset=True)
    assert st["fused_products"] == 0 and st["cast_kernels"] == 1
    assert np.array_equal(out2.to_bits(), out.to_bits())


# ---- config-5 shape in miniature: reference copies vs the no-copy path ------------------------------
def test_reference_mode_copies_and_nocopy_mode_agree_bit_for_bit():
    b, s, d, f = 3, 16, 64, 96
    xb = H.random_storage("bf16", b * s * f, 21, 0.5)
    wb = H.random_storage("bf16", d * f, 22, 0.05)
    x = T.Tensor.from_bits(xb, "bf16", [b, s, f])
    w_down = T.Tensor.from_bits(wb, "bf16", [d, f]).t()  # logical [f, d], a transposed view
    try:
        T.set_matmul_mode("reference")
        T.stats(reset=True)
        y_ref = x.matmul(w_down)
        st_ref = T.stats(reset=True)
        T.set_matmul_mode("nocopy")
        y_new = x.matmul(w_down)
        st_new = T.stats(reset=True)
    finally:
        T.set_matmul_mode("nocopy")
    assert st_ref["contiguous_kernels"] == 1 and st_ref["bytes_copied"] == d * f * 2  # the hidden weight copy
    assert st_new["contiguous_kernels"] == 0 and st_new["bytes_copied"] == 0
    assert y_ref.shape == [b, s, d] and np.array_equal(y_ref.to_bits(), y_new.to_bits())
    lv, rv = H.View([b, s, f]), H.View([d, f]).t().broadcast_to([b, f, d])
    want32, _, sumabs = oracle.matmul_spec("bf16", "bf16", xb, wb, H.matmul_md(lv, rv))
    assert H.rel_err(H.bf16_to_f32(y_new.to_bits()), want32, sumabs, f).max() <= 2e-2


def test_to_dtype_of_a_view_matches_the_cast_oracle():
    n, m = 48, 20
    xs = H.random_storage("f32", n * m, 31, 3.0)
    t = T.Tensor.from_bits(xs, "f32", [n, m]).t()
    got = t.to_dtype("bf16")
    want = oracle.cast("f32", "bf16", xs, H.cast_md(H.View([n, m]).t()))
    assert got.layout() == ([m, n], [n, 1], 0) and np.array_equal(got.to_bits(), want)  # truncating f32 -> bf16
    same = t.to_dtype("f32")  # same dtype: contiguous()
    assert np.array_equal(same.to_bits().view(np.float32), xs.reshape(n, m).T.ravel())
