"""GPU parity: matmul / dot through the C ABI against the CPU oracle, for every dtype and for the
layouts the reference's kernels accept (contiguous, transposed, sliced with offsets, strided,
batched, batch-broadcast with size-1 dims and with stride 0)."""
import numpy as np
import pytest

import helpers as H
import oracle
from gpu_util import FUSED, check_product, run_product
from hodu_amd import ffi

pytestmark = pytest.mark.gpu

V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


LAYOUTS = [
    ("dot", "contig", V([37, 70]), V([70, 29])),
    ("dot", "rhs_t", V([19, 40]), V([23, 40]).t()),
    ("dot", "lhs_t_off", V([40, 17], offset=5).t(), V([40, 21], offset=3)),
    ("dot", "sliced", V([30, 64]).slice(1, 4, 36), V([32, 50]).slice(1, 1, 49, 2)),
    ("dot", "gemv_row", V([1, 96]), V([96, 33])),
    ("dot", "outer_k1", V([20, 1]), V([1, 31])),
    ("matmul", "2d", V([33, 47]), V([47, 18])),
    ("matmul", "batched", V([3, 9, 20]), V([3, 20, 11])),
    ("matmul", "rhs_2d", V([2, 3, 8, 16]), V([16, 10])),
    ("matmul", "bcast_t", V([4, 6, 24]), V([13, 24]).t().broadcast_to([4, 24, 13])),
    ("matmul", "b1_t", V([1, 5, 7, 12]), V([2, 1, 9, 12]).t()),
    ("matmul", "lhs_bcast", V([7, 12]).broadcast_to([3, 7, 12]), V([3, 12, 5])),
    ("matmul", "six_batch_dims", V([2, 1, 2, 1, 2, 2, 3, 8]), V([1, 2, 1, 2, 1, 2, 8, 4])),
]


@pytest.mark.parametrize("dt", ffi.PRODUCT_DTYPES + list(FUSED))
def test_all_dtypes_all_layouts_small(ctx, dt):
    scale = 2.0 if dt.startswith("f8") else 1.0
    for n, (op, _name, lv, rv) in enumerate(LAYOUTS):
        check_product(ctx, op, dt, lv, rv, seed=n, scale=scale)


def test_reference_known_answers_through_the_abi(ctx):
    f = np.float32
    # crates/hodu_cpu_kernels/tests/ops_matrix.rs:8-61, :63-117, :119-147
    a = np.array([1, 2, 3, 4, 5, 6], f); b = np.array([7, 8, 9, 10, 11, 12], f)
    assert run_product(ctx, "matmul", "f32", a, b, [4, 2, 2, 0, 2, 3, 3, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2]).tolist() == [58, 64, 139, 154]
    assert run_product(ctx, "dot", "f32", a, b, [2, 3, 2, 3, 1, 2, 1, 0, 0]).tolist() == [58, 64, 139, 154]
    a = np.array([1, 2, 3, 4, 2, 3, 4, 5], f); b = np.array([5, 6, 7, 8, 6, 7, 8, 9], f)
    md = [8, 3, 3, 1, 2, 2, 2, 2, 2, 2, 2, 4, 2, 1, 4, 2, 1, 0, 0, 2, 2, 2]
    assert run_product(ctx, "matmul", "f32", a, b, md).tolist() == [19, 22, 43, 50, 36, 41, 64, 73]
    # crates/hodu_cuda_kernels/tests/ops_matrix.rs:103-151, :153-186, :188-262
    a = np.arange(1, 10).astype(f); b = np.arange(9, 0, -1).astype(f)
    md = [9, 2, 2, 0, 3, 3, 3, 3, 3, 1, 3, 1, 0, 0, 3, 3, 3]
    assert run_product(ctx, "matmul", "f32", a, b, md).tolist() == [30, 24, 18, 84, 69, 54, 138, 114, 90]
    eye = np.eye(3, dtype=f).ravel()
    assert run_product(ctx, "dot", "f32", eye, eye.copy(), [3, 3, 3, 3, 1, 3, 1, 0, 0]).tolist() == eye.tolist()
    a = np.arange(1, 13).astype(f); b = np.array([1, 0, 0, 1, 1, 1], f)
    md = [8, 3, 2, 1, 2, 2, 3, 3, 2, 2, 6, 3, 1, 2, 1, 0, 0, 2, 3, 2]
    assert run_product(ctx, "matmul", "f32", a, b, md).tolist() == [4, 5, 10, 11, 16, 17, 22, 23]
    # crates/hodu_metal_kernels/tests/ops_matrix.rs:141-228, :230-313
    a = np.array([1, 2, 3, 4, 5, 6, 13, 14, 15, 16, 17, 18], f)
    b = np.array([7, 8, 9, 10, 11, 12, 19, 20, 21, 22, 23, 24], f)
    md = [8, 3, 3, 1, 2, 2, 3, 2, 3, 2, 2, 6, 3, 1, 6, 2, 1, 0, 0, 2, 3, 2]
    assert run_product(ctx, "matmul", "f32", a, b, md).tolist() == [58, 64, 139, 154, 886, 928, 1075, 1126]
    a = np.arange(1, 13).astype(f); b = np.arange(1, 7).astype(f)
    md = [8, 3, 2, 1, 2, 2, 3, 3, 2, 2, 6, 3, 1, 2, 1, 0, 0, 2, 3, 2]
    assert run_product(ctx, "matmul", "f32", a, b, md).tolist() == [22, 28, 49, 64, 76, 100, 103, 136]


def test_integer_golden_fixtures_bit_exact(ctx):
    """the committed reference outputs (tests/golden/products.npz) for every integer dtype"""
    import os
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "products.npz"))
    n = 0
    for entry in gold["index"]:
        key, op, dt = entry.split("|")
        if dt[0] not in "iu":
            continue
        got = run_product(ctx, op, dt, gold[key + "__lhs"], gold[key + "__rhs"], gold[key + "__md"].tolist())
        assert np.array_equal(got, gold[key + "__out"]), key
        n += 1
    assert n >= 40


@pytest.mark.parametrize("dt", ffi.PRODUCT_DTYPES)
def test_product_of_two_long_vectors(ctx, dt):
    """[1, K] x [K, 1] (what Tensor::matmul makes of two 1-D tensors): K is cut into chunks across workgroups; dense
    and strided vectors, a K that leaves a ragged last chunk"""
    scale = 0.25 if dt in ("f8e4m3", "f8e5m2") else 1.0
    check_product(ctx, "dot", dt, V([1, 1 << 17]), V([1 << 17, 1]), seed=1, scale=scale, expect_kernel="inner_product_vec")
    check_product(ctx, "dot", dt, V([1, 100003]), V([100003, 1]), seed=2, scale=scale, expect_kernel="inner_product")
    check_product(ctx, "dot", dt, V([1, 40000], [0, 2]), V([40000, 1], [3, 0]), seed=3, scale=scale, expect_kernel="inner_product")
    check_product(ctx, "dot", dt, V([1, 9000]), V([9000, 1]), seed=4, scale=scale)  # short: the other kernels
    assert not ctx.last_kernel().startswith("inner_product")


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
def test_matrix_times_vector(ctx, dt):
    """[M, K] x [K, 1] (Tensor::matmul of a 2-D and a 1-D tensor) runs as the transposed one-row product"""
    check_product(ctx, "dot", dt, V([300, 1040]), V([1040, 1]), seed=1)
    assert ctx.last_kernel().startswith(("gemv_", "skinny_")), ctx.last_kernel()
    check_product(ctx, "dot", dt, V([1040, 300]).t(), V([1040, 1]), seed=2)          # the matrix row-dense in K
    assert ctx.last_kernel().startswith(("gemv_rows_", "mfma_")), ctx.last_kernel()
    check_product(ctx, "dot", dt, V([64, 512], offset=8), V([512, 1], [3, 0]), seed=3)  # a strided vector: other kernels
    check_product(ctx, "dot", dt, V([2, 70000]), V([70000, 1]), seed=4)


def test_inputs_may_alias_each_other(ctx):
    # a.matmul(a.t()) : lhs and rhs are views of one buffer
    lv = V([24, 40]); rv = lv.t()
    a = H.random_storage("bf16", lv.span(), 7)
    da = ctx.upload(a)
    out = ctx.alloc(24 * 24 * 2)
    ctx.product("dot", "bf16", da, da, out, H.dot_md(lv, rv))
    got = H.bf16_to_f32(ctx.download(out, np.uint16))
    A = H.bf16_to_f32(a).reshape(24, 40).astype(np.float64)
    assert np.allclose(got.reshape(24, 24), A @ A.T, rtol=2e-2, atol=1e-2)


def test_k_zero_writes_zeros(ctx):
    got = run_product(ctx, "dot", "f32", np.zeros(1, np.float32), np.zeros(1, np.float32), [5, 0, 7, 0, 1, 7, 1, 0, 0])
    assert got.shape == (35,) and np.all(got == 0)
    got = run_product(ctx, "dot", "i32", np.zeros(1, np.int32), np.zeros(1, np.int32), [5, 0, 7, 0, 1, 7, 1, 0, 0])
    assert np.all(got == 0)


def test_empty_outputs_launch_nothing(ctx):
    """M = 0, N = 0 or an empty batch: the call succeeds and the (one-element) output buffer keeps its bytes"""
    a = ctx.upload(np.ones(16, np.float32)); b = ctx.upload(np.ones(16, np.float32)); o = ctx.alloc(4)
    ctx.fill(o, 0x5A)
    for md in ([0, 4, 3, 4, 1, 3, 1, 0, 0], [3, 4, 0, 4, 1, 1, 1, 0, 0]):  # dot: [M, K, N, ls_m, ls_k, rs_k, rs_n, l_off, r_off]
        ctx.product("dot", "f32", a, b, o, md)
    # matmul with batch [0]: [num_els, l_nd, r_nd, b_nd, l_shape, r_shape, batch_shape, l_strides, r_strides, l_off, r_off, M, K, N]
    ctx.product("matmul", "f32", a, b, o, [0, 3, 3, 1, 0, 2, 4, 0, 4, 2, 0, 8, 4, 1, 8, 2, 1, 0, 0, 2, 4, 2])
    ctx.sync()
    assert ctx.download(o, np.uint8, 4).tolist() == [0x5A] * 4
    for d in (a, b, o):
        d.free()


def test_errors_are_status_codes(ctx):
    a = ctx.upload(np.zeros(16, np.float32)); b = ctx.upload(np.zeros(16, np.float32)); o = ctx.alloc(64)
    with pytest.raises(ffi.HoduRocmError) as e:
        ctx.product("dot", "f32", a, b, o, [2, 3, 2, 3, 1, 2, 1, 0])  # 8 words
    assert e.value.status == ffi.INVALID_ARG
    with pytest.raises(ffi.HoduRocmError) as e:  # K mismatch between shapes and tail
        ctx.product("matmul", "f32", a, b, o, [4, 2, 2, 0, 2, 3, 4, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2])
    assert e.value.status == ffi.INVALID_ARG and "mismatch" in e.value.message
    with pytest.raises(ffi.HoduRocmError) as e:  # 1-D operand
        ctx.product("matmul", "f32", a, b, o, [4, 1, 2, 0, 3, 3, 2, 1, 2, 1, 0, 0, 2, 3, 2])
    assert e.value.status == ffi.INVALID_ARG
    with pytest.raises(ffi.HoduRocmError) as e:  # num_els inconsistent
        ctx.product("matmul", "f32", a, b, o, [5, 2, 2, 0, 2, 3, 3, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2])
    assert e.value.status == ffi.INVALID_ARG
    with pytest.raises(ffi.HoduRocmError) as e:  # out aliases an input
        ctx.product("dot", "f32", a, b, a, [2, 3, 2, 3, 1, 2, 1, 0, 0])
    assert e.value.status == ffi.INVALID_ARG
    with pytest.raises(ffi.HoduRocmError) as e:
        ctx.cast("f32", "bf16", a, o, [4, 1, 5, 1, 0])  # num_els != prod(shape)
    assert e.value.status == ffi.INVALID_ARG
    ctx.sync()  # nothing was launched; the context is still usable
    ctx.product("dot", "f32", a, b, o, [2, 3, 2, 3, 1, 2, 1, 0, 0])
    ctx.sync()
