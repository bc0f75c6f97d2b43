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
    H.assert_close(got, want32, sumabs, k, 2e-2, "bf16 output, f32 accumulate")
    # reading the deferred tensor materialises the cast: bit-exact with the cast oracle (OCP decode)
    want_bits = oracle.cast("f8e4m3", "bf16", w8, H.cast_md(H.View([n, k])), decode=oracle.F8_OCP)
    assert np.array_equal(wb.to_bits(), want_bits)
    # the unfused route (cast of a strided view runs the kernel) gives the same product to one bf16 step
    wt_dense = w.t().to_dtype("bf16")  # non-dense input: materialised, [k, n] contiguous
    assert wt_dense.physical_dtype == "bf16"
    y2 = x.matmul(wt_dense)
    H.assert_close(H.bf16_to_f32(y2.to_bits()), want32, sumabs, k, 2e-2, "deferred cast")


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
    H.assert_close(H.bf16_to_f32(y_new.to_bits()), want32, sumabs, f, 2e-2, "no-copy mode")


def test_to_dtype_of_a_view_matches_the_cast_oracle():
    n, m = 48, 20
    xs = H.random_storage("f32", n * m, 31, 3.0)
    t = T.Tensor.from_bits(xs, "f32", [n, m]).t()
    got = t.to_dtype("bf16")
    want = oracle.cast("f32", "bf16", xs, H.cast_md(H.View([n, m]).t()))
    assert got.layout() == ([m, n], [n, 1], 0) and np.array_equal(got.to_bits(), want)  # truncating f32 -> bf16
    same = t.to_dtype("f32")  # same dtype: contiguous()
    assert np.array_equal(same.to_bits().view(np.float32), xs.reshape(n, m).T.ravel())


# ---- the product with its caller's next element-wise kernels fused in ------------------------------------
def _oracle_after(dt, plain_bits, out_shape, steps):
    """hodu_cpu_add / mul_scalar / relu (the oracle's restatement) applied to the plain product's output"""
    V = H.View
    x = plain_bits.view(oracle.STORAGE[dt])
    for step in steps:
        if step[0] == "add":
            bias_bits, bias_view = step[1], step[2]
            x = oracle.add(dt, x, bias_bits.view(oracle.STORAGE[dt]), H.binary_md(V(out_shape), bias_view.broadcast_to(out_shape)))
        elif step[0] == "mul_scalar":
            x = oracle.mul_scalar(dt, x, H.cast_md(V(out_shape)), step[1].view(oracle.STORAGE[dt]))
        else:
            x = oracle.relu(dt, x, H.cast_md(V(out_shape)))
    return x.view(plain_bits.dtype)


def test_linear_layer_equals_matmul_then_add():
    """Linear::forward (hodu_nn/src/modules/linear.rs:40-46): 3-D input, [out, in] weight, bias -- one launch, and the
    bits of matmul followed by add"""
    V = H.View
    g = H.rng(11)
    x = H.f32_to_bf16_rne(g.standard_normal(2 * 5 * 64).astype(np.float32))
    w = H.f32_to_bf16_rne((g.standard_normal(24 * 64) / 8).astype(np.float32))
    b = H.f32_to_bf16_rne(g.standard_normal(24).astype(np.float32))
    tx, tw, tb = (T.Tensor.from_bits(x, "bf16", [2, 5, 64]), T.Tensor.from_bits(w, "bf16", [24, 64]),
                  T.Tensor.from_bits(b, "bf16", [24]))
    plain = tx.matmul(tw.t()).to_bits()
    T.stats(reset=True)
    layer = T.Linear(tw, tb)
    got = layer.forward(tx)
    s = T.stats()
    assert got.shape == [2, 5, 24] and s["product_kernels"] == 1 and s["fused_steps"] == 1
    assert np.array_equal(got.to_bits(), _oracle_after("bf16", plain, [2, 5, 24], [("add", b, V([24]))]))
    got = layer.forward(tx, relu=True).to_bits()
    assert np.array_equal(got, _oracle_after("bf16", plain, [2, 5, 24], [("add", b, V([24])), ("relu",)]))
    assert np.array_equal(T.Linear(tw).forward(tx).to_bits(), plain)  # no bias: the plain product
    assert [p.shape for p in layer.parameters()] == [[24, 64], [24]]


def test_linear_layer_with_deferred_f8_weight():
    """x.matmul(w8.to_dtype(bf16).t()) + bias: cast, product and add in one launch (config 3 as a layer)"""
    V = H.View
    g = H.rng(12)
    x = H.f32_to_bf16_rne(g.standard_normal(16 * 512).astype(np.float32))
    w8 = H.f32_to_ocp_e4m3_rne(g.standard_normal(300 * 512) * 4)
    b = H.f32_to_bf16_rne(g.standard_normal(300).astype(np.float32))
    tx, tb = T.Tensor.from_bits(x, "bf16", [16, 512]), T.Tensor.from_bits(b, "bf16", [300])
    tw = T.Tensor.from_bits(w8, "f8e4m3", [300, 512]).to_dtype("bf16")
    assert tw.physical_dtype == "f8e4m3"
    plain = tx.matmul(tw.t()).to_bits()
    T.stats(reset=True)
    got = T.Linear(tw, tb).forward(tx)
    s = T.stats()
    want = {"cast_kernels": 0, "contiguous_kernels": 0, "product_kernels": 1, "fused_products": 1, "bytes_copied": 0,
            "fused_steps": 1}
    assert {key: s[key] for key in want} == want
    assert np.array_equal(got.to_bits(), _oracle_after("bf16", plain, [16, 300], [("add", b, V([300]))]))


def test_matmul_then_scale_and_strided_bias():
    """attention.rs:37 scales the scores; a bias that is a strided slice of a larger tensor, or a [1, N] row, or one
    value, broadcasts the way Tensor::add broadcasts it"""
    V = H.View
    g = H.rng(13)
    q = g.standard_normal(3 * 10 * 32).astype(np.float32)
    k = g.standard_normal(3 * 12 * 32).astype(np.float32)
    tq, tk = from_f32(q, [3, 10, 32]), from_f32(k, [3, 12, 32])
    plain = tq.matmul(tk.t()).to_bits()
    scale = np.array([1.0 / np.sqrt(32.0)], dtype=np.float32)
    got = tq.matmul_then(tk.t(), [("mul_scalar", scale)]).to_bits()
    assert np.array_equal(got, _oracle_after("f32", plain, [3, 10, 12], [("mul_scalar", scale.view(np.uint32))]))
    big = g.standard_normal(40).astype(np.float32)
    tbig = from_f32(big, [40])
    sl = tbig.slice(0, 3, 39, 3)  # 12 entries, stride 3, offset 3
    want = _oracle_after("f32", plain, [3, 10, 12], [("add", big.view(np.uint32), V([12], [3], 3))])
    assert np.array_equal(tq.matmul_then(tk.t(), [("add", sl)]).to_bits(), want)
    row = from_f32(big[:12], [1, 12])
    want = _oracle_after("f32", plain, [3, 10, 12], [("add", big[:12].view(np.uint32), V([1, 12]))])
    assert np.array_equal(tq.matmul_then(tk.t(), [("add", row)]).to_bits(), want)
    one = from_f32(big[5:6], [1])
    want = _oracle_after("f32", plain, [3, 10, 12], [("add", big[5:6].view(np.uint32), V([1]))])
    assert np.array_equal(tq.matmul_then(tk.t(), [("add", one)]).to_bits(), want)


def test_matmul_then_rejects_what_add_would_not_broadcast_along_the_last_axis():
    a, b = from_f32(np.ones(6), [2, 3]), from_f32(np.ones(12), [3, 4])
    with pytest.raises(T.HoduError) as e:
        a.matmul_then(b, [("add", from_f32(np.ones(2), [2, 1]))])  # a column: a real add kernel's job
    assert e.value.kind == "IncompatibleShapes"
    with pytest.raises(T.HoduError) as e:
        a.matmul_then(b, [("add", from_f32(np.ones(5), [5]))])
    assert e.value.kind == "IncompatibleShapes"
    with pytest.raises(T.HoduError) as e:
        a.matmul_then(b, [("add", T.Tensor.from_bits(np.ones(4, np.uint16), "bf16", [4]))])
    assert e.value.kind == "DTypeMismatch"
    with pytest.raises(T.HoduError) as e:
        from_f32(np.ones(3), [3]).matmul_then(b, [("relu",)])
    assert e.value.kind == "InvalidArgument"
    i = T.Tensor.from_bits(np.ones(6, np.uint32), "i32", [2, 3])
    j = T.Tensor.from_bits(np.ones(12, np.uint32), "i32", [3, 4])
    with pytest.raises(T.HoduError) as e:
        i.matmul_then(j, [("relu",)])
    assert e.value.kind == "RocmKernelError"


# ---- backward through the path (tensor/gradient/vjp_matrix.rs) ------------------------------------------
def _i32(values, shape):
    return T.Tensor.from_bits(np.asarray(values, np.int32).view(np.uint32), "i32", shape)


def _i32_of(t):
    return t.to_bits().view(np.int32)


def test_sum_and_sum_to_shape_follow_the_reference_shapes():
    x = np.arange(2 * 3 * 4, dtype=np.int32)
    t = _i32(x, [2, 3, 4])
    a = x.reshape(2, 3, 4)
    assert t.sum([0]).shape == [3, 4] and np.array_equal(_i32_of(t.sum([0])), a.sum(0).ravel())
    assert t.sum([-1], keep_dim=True).shape == [2, 3, 1] and np.array_equal(_i32_of(t.sum([-1], True)), a.sum(2).ravel())
    assert t.sum().shape == [] and _i32_of(t.sum())[0] == a.sum()  # tensor/ops/reduce.rs:154-156: no dims = all
    assert t.sum([0, 2]).shape == [3] and np.array_equal(_i32_of(t.sum([0, 2])), a.sum((0, 2)))
    # sum_to_shape (tensor/ops/reduce.rs:19-50): leading dims go, extent-1 dims of the target are kept
    assert t.sum_to_shape([3, 4]).shape == [3, 4] and np.array_equal(_i32_of(t.sum_to_shape([3, 4])), a.sum(0).ravel())
    assert t.sum_to_shape([1, 4]).shape == [1, 4] and np.array_equal(_i32_of(t.sum_to_shape([1, 4])), a.sum((0, 1)))
    assert t.sum_to_shape([2, 1, 4]).shape == [2, 1, 4]
    assert np.array_equal(_i32_of(t.sum_to_shape([2, 1, 4])), a.sum(1).ravel())
    assert t.sum_to_shape([2, 3, 4]).shares_storage_with(t)
    # a transposed view sums like its contiguous copy
    assert np.array_equal(_i32_of(t.t().sum([1])), a.transpose(0, 2, 1).sum(1).ravel())


def test_matmul_vjp_integers_exact_in_both_modes():
    """dA = grad @ B^T, dB = A^T @ grad summed over the batch the weight was broadcast along: exact in i32, so the
    literal path (batched product, then sum launches) and the folded one (batch inside the contraction) must agree
    with numpy and with each other"""
    g = H.rng(21)
    a = g.integers(-9, 10, (4, 5, 6)).astype(np.int32)
    w = g.integers(-9, 10, (6, 7)).astype(np.int32)
    go = g.integers(-9, 10, (4, 5, 7)).astype(np.int32)
    want_da = (go.astype(np.int64) @ w.T.astype(np.int64)).astype(np.int32)
    want_dw = np.einsum("bmk,bmn->kn", a.astype(np.int64), go.astype(np.int64)).astype(np.int32)
    ta, tw, tg = _i32(a, [4, 5, 6]), _i32(w, [6, 7]), _i32(go, [4, 5, 7])
    for mode, sums in (("reference", 1), ("nocopy", 0)):
        T.set_matmul_mode(mode)
        T.stats(reset=True)
        try:
            da, dw = T.matmul_vjp(ta, tw, tg)
            s = T.stats()
        finally:
            T.set_matmul_mode("nocopy")
        assert da.shape == [4, 5, 6] and dw.shape == [6, 7]
        assert np.array_equal(_i32_of(da), want_da.ravel()) and np.array_equal(_i32_of(dw), want_dw.ravel()), mode
        assert s["sum_kernels"] == sums and s["product_kernels"] == 2, (mode, s)
    # both operands batched, the lhs broadcast along a batch dim of extent 1: dA is summed with keep_dim
    a1 = g.integers(-9, 10, (1, 5, 6)).astype(np.int32)
    wb = g.integers(-9, 10, (4, 6, 7)).astype(np.int32)
    da, dw = T.matmul_vjp(_i32(a1, [1, 5, 6]), _i32(wb, [4, 6, 7]), tg)
    assert da.shape == [1, 5, 6] and dw.shape == [4, 6, 7]
    assert np.array_equal(_i32_of(da), np.einsum("bmn,bkn->mk", go.astype(np.int64), wb.astype(np.int64)).astype(np.int32).ravel())
    assert np.array_equal(_i32_of(dw), np.einsum("mk,bmn->bkn", a1[0].astype(np.int64), go.astype(np.int64)).astype(np.int32).ravel())
    # dot: no broadcasting, no sums (vjp_matrix.rs:46-67)
    da, dw = T.dot_vjp(_i32(a[0], [5, 6]), tw, _i32(go[0], [5, 7]))
    assert np.array_equal(_i32_of(da), (go[0].astype(np.int64) @ w.T).astype(np.int32).ravel())
    assert np.array_equal(_i32_of(dw), (a[0].T.astype(np.int64) @ go[0]).astype(np.int32).ravel())


def test_linear_backward_bf16_against_f32_accumulated_comparator():
    """x[8, 64, 256] @ w[256, 192] in bf16: dW through the folded product (K = 8 * 64 rows, operands row-dense) and
    through the literal batched path both sit within the bf16 bar of the f32-accumulated result"""
    g = H.rng(22)
    x = H.f32_to_bf16_rne(g.standard_normal(8 * 64 * 256).astype(np.float32))
    w = H.f32_to_bf16_rne((g.standard_normal(256 * 192) / 16).astype(np.float32))
    go = H.f32_to_bf16_rne(g.standard_normal(8 * 64 * 192).astype(np.float32))
    tx, tw, tg = (T.Tensor.from_bits(x, "bf16", [8, 64, 256]), T.Tensor.from_bits(w, "bf16", [256, 192]),
                  T.Tensor.from_bits(go, "bf16", [8, 64, 192]))
    xf, wf, gf = (H.bf16_to_f32(x).astype(np.float64).reshape(512, 256), H.bf16_to_f32(w).astype(np.float64).reshape(256, 192),
                  H.bf16_to_f32(go).astype(np.float64).reshape(512, 192))
    want_dw, abs_dw = xf.T @ gf, np.abs(xf).T @ np.abs(gf)
    want_dx, abs_dx = gf @ wf.T, np.abs(gf) @ np.abs(wf).T
    for mode in ("nocopy", "reference"):
        T.set_matmul_mode(mode)
        try:
            dx, dw = T.matmul_vjp(tx, tw, tg)
        finally:
            T.set_matmul_mode("nocopy")
        # the reference sequence rounds every batch's [K, N] product to bf16 before sum_to_shape adds them: its
        # error on an element that cancels is a bf16 rounding of the per-batch parts, not an f32 accumulation error
        H.assert_close(H.bf16_to_f32(dw.to_bits()), want_dw.ravel(), abs_dw.ravel(), 512, 2e-2, f"dW, {mode}",
                       eps_acc=2.0 ** -9 if mode == "reference" else H.EPS_F32)
        H.assert_close(H.bf16_to_f32(dx.to_bits()), want_dx.ravel(), abs_dx.ravel(), 192, 2e-2, f"dX, {mode}")


# ---- attention core (hodu_nn/src/modules/attention.rs:25-70) ----------------------------------------------
def _attention_f64(q, k, v, causal):
    s = q @ np.swapaxes(k, -1, -2) / np.sqrt(q.shape[-1])
    if causal:
        i, j = np.arange(s.shape[-2])[:, None], np.arange(s.shape[-1])[None, :]
        s = np.where(j > i, -np.inf, s)
    e = np.exp(s - s.max(-1, keepdims=True))
    return (e / e.sum(-1, keepdims=True)) @ v


@pytest.mark.parametrize("causal", [False, True])
def test_attention_f32(causal):
    g = H.rng(51)
    q, k, v = (g.standard_normal((2, 3, 40, 32)).astype(np.float32) for _ in range(3))
    tq, tk, tv = (from_f32(x, [2, 3, 40, 32]) for x in (q, k, v))
    T.stats(reset=True)
    out = T.scaled_dot_product_attention(tq, tk, tv, causal)
    s = T.stats()
    assert out.shape == [2, 3, 40, 32]
    assert s["product_kernels"] == 2 and s["softmax_kernels"] == 1 and s["fused_steps"] == 1 and s["contiguous_kernels"] == 0
    want = _attention_f64(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), causal)
    assert np.allclose(f32_of(out).reshape(want.shape), want, rtol=1e-4, atol=1e-5)
    # the same through the separate steps of the Tensor API
    scale = T.scalar_bits("f32", 1.0 / np.sqrt(32.0))
    steps = tq.matmul_then(tk.t(), [("mul_scalar", scale)]).softmax(-1, causal).matmul(tv)
    assert np.array_equal(steps.to_bits(), out.to_bits())


def test_attention_bf16_with_cross_lengths():
    """Sq != Sk, bf16: against the float64 function of the bf16 inputs; every intermediate is rounded to bf16 once
    (scores after the scale step twice: product and mul_scalar, as in the reference), so the bar is the bf16 one"""
    g = H.rng(52)
    q = H.f32_to_bf16_rne(g.standard_normal(4 * 24 * 64).astype(np.float32))
    k = H.f32_to_bf16_rne(g.standard_normal(4 * 56 * 64).astype(np.float32))
    v = H.f32_to_bf16_rne(g.standard_normal(4 * 56 * 64).astype(np.float32))
    tq, tk, tv = (T.Tensor.from_bits(q, "bf16", [4, 24, 64]), T.Tensor.from_bits(k, "bf16", [4, 56, 64]),
                  T.Tensor.from_bits(v, "bf16", [4, 56, 64]))
    out = T.scaled_dot_product_attention(tq, tk, tv, False)
    want = _attention_f64(H.bf16_to_f32(q).astype(np.float64).reshape(4, 24, 64), H.bf16_to_f32(k).astype(np.float64).reshape(4, 56, 64),
                          H.bf16_to_f32(v).astype(np.float64).reshape(4, 56, 64), False)
    got = H.bf16_to_f32(out.to_bits()).astype(np.float64).reshape(want.shape)
    assert np.all(np.abs(got - want) <= 2e-2 * np.maximum(np.abs(want), 0.25))


def test_softmax_of_a_view_and_along_other_dims():
    x = H.rng(53).standard_normal(6 * 10).astype(np.float32)
    t = from_f32(x, [6, 10])
    a = x.astype(np.float64).reshape(6, 10)
    e = np.exp(a.T - a.T.max(-1, keepdims=True))
    assert np.allclose(f32_of(t.t().softmax(-1)).reshape(10, 6), e / e.sum(-1, keepdims=True), rtol=1e-5)
    # along the other dim: columns
    e0 = np.exp(a - a.max(0, keepdims=True))
    assert np.allclose(f32_of(t.softmax(0)).reshape(6, 10), e0 / e0.sum(0, keepdims=True), rtol=1e-5)
    with pytest.raises(T.HoduError) as err:
        t.softmax(0, True)  # the causal mask belongs to the last dim
    assert err.value.kind == "InvalidArgument"


# ---- .hdt files straight onto the device (crates/hodu_core/src/format/hdt.rs:25-52) ------------------------
def test_hdt_round_trip_through_the_device(tmp_path):
    from hodu_amd import hdt
    g = H.rng(61)
    w8 = H.f32_to_ocp_e4m3_rne(g.standard_normal(12 * 64) * 4)
    x = H.f32_to_bf16_rne(g.standard_normal(5 * 64).astype(np.float32))
    tw, tx = T.Tensor.from_bits(w8, "f8e4m3", [12, 64]), T.Tensor.from_bits(x, "bf16", [5, 64])
    hdt.save_many({"linear.weight": tw, "x": tx}, tmp_path / "m.hdt")
    back = hdt.load_many(tmp_path / "m.hdt")
    assert set(back) == {"linear.weight", "x"}
    assert back["linear.weight"].dtype == "f8e4m3" and back["linear.weight"].shape == [12, 64]
    assert np.array_equal(back["linear.weight"].to_bits(), w8) and np.array_equal(back["x"].to_bits(), x)
    # the loaded weight goes down the path like any other: deferred cast, one launch
    y0 = tx.matmul(tw.to_dtype("bf16").t()).to_bits()
    y1 = back["x"].matmul(back["linear.weight"].to_dtype("bf16").t()).to_bits()
    assert np.array_equal(y0, y1)
    # a view is saved as its contiguous elements (Tensor::to_bytes)
    hdt.save(tx.t(), tmp_path / "t.hdt")
    t2 = hdt.load(tmp_path / "t.hdt")
    assert t2.shape == [64, 5] and np.array_equal(t2.to_bits(), x.reshape(5, 64).T.ravel())


@pytest.mark.parametrize("causal", [False, True])
def test_attention_takes_the_fused_kernel_at_head_dim_128(causal):
    """bf16, D = 128: one launch; k and v shared across the heads through broadcasting, as the two matmuls would"""
    g = H.rng(54)
    q = H.f32_to_bf16_rne(g.standard_normal(2 * 3 * 72 * 128).astype(np.float32))
    k = H.f32_to_bf16_rne(g.standard_normal(2 * 1 * 90 * 128).astype(np.float32))
    v = H.f32_to_bf16_rne(g.standard_normal(90 * 128).astype(np.float32))
    tq, tk, tv = (T.Tensor.from_bits(q, "bf16", [2, 3, 72, 128]), T.Tensor.from_bits(k, "bf16", [2, 1, 90, 128]),
                  T.Tensor.from_bits(v, "bf16", [90, 128]))
    T.stats(reset=True)
    out = T.scaled_dot_product_attention(tq, tk, tv, causal)
    s = T.stats()
    assert out.shape == [2, 3, 72, 128]
    assert s["attention_kernels"] == 1 and s["product_kernels"] == 0 and s["softmax_kernels"] == 0 and s["contiguous_kernels"] == 0
    qf = H.bf16_to_f32(q).astype(np.float64).reshape(2, 3, 72, 128)
    kf = np.broadcast_to(H.bf16_to_f32(k).astype(np.float64).reshape(2, 1, 90, 128), (2, 3, 90, 128))
    vf = np.broadcast_to(H.bf16_to_f32(v).astype(np.float64).reshape(90, 128), (2, 3, 90, 128))
    scale = float(H.bf16_to_f32(T.scalar_bits("bf16", 1.0 / np.sqrt(128.0)))[0])
    sc = qf @ np.swapaxes(kf, -1, -2) * scale
    if causal:
        i, j = np.arange(72)[:, None], np.arange(90)[None, :]
        sc = np.where(j > i, -np.inf, sc)
    e = np.exp(sc - sc.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    want = p @ vf
    got = H.bf16_to_f32(out.to_bits()).astype(np.float64).reshape(want.shape)
    # floor of the denominator: the magnitude of an average of n unit-variance rows that may cancel
    floor = np.abs(vf).mean() / np.sqrt((p > 0).sum(-1))[..., None]
    assert np.all(np.abs(got - want) <= 2e-2 * np.maximum(np.abs(want), floor))
    # a head dim the kernel does not take goes down the three-launch path, same function
    T.stats(reset=True)
    q32 = T.Tensor.from_bits(q[:2 * 3 * 72 * 32], "bf16", [2, 3, 72, 32])
    k32 = T.Tensor.from_bits(k[:90 * 32], "bf16", [90, 32])
    T.scaled_dot_product_attention(q32, k32, k32, causal)
    s = T.stats()
    assert s["attention_kernels"] == 0 and s["product_kernels"] == 2 and s["softmax_kernels"] == 1
