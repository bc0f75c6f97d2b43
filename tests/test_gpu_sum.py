"""GPU parity of hodu_rocm_sum (the reduce that Tensor::sum_to_shape launches on a matmul's gradients): every dtype,
the three kernels (a thread per output with and without 16-byte vectors, a wavefront per output), strided inputs,
keep_dim, empty sums.  Integers: bit-exact against the reference-faithful oracle.  Floats: relative error against the
f32-accumulated comparator (1e-5 for f32, 2e-2 for bf16 / f16, one rounding step for the 8-bit floats), denominator
floored at sum|x| / sqrt(R) as for the products; f64 against the float64 sum at 1e-12."""
import numpy as np
import pytest

import helpers as H
import oracle
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View
INTS = ("u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64")


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def check_sum(ctx, dt, v, dims, keep, seed=0, expect_kernel=None):
    x = H.random_storage(dt, max(v.span(), 1), 700 + seed, 2.0)
    md = H.reduce_md(v, dims, keep)
    n_out = oracle.reduce_out_elems(md)
    dx = ctx.upload(x)
    dout = ctx.alloc(max(n_out, 1) * ffi.DTYPE_SIZE[dt])
    ctx.fill(dout, 0xFF)
    ctx.sum(dt, dx, dout, md)
    if expect_kernel is not None:
        # a trailing * admits the kernel's vector variant (whether it applies depends on the element size)
        ok = ctx.last_kernel().startswith(expect_kernel[:-1]) if expect_kernel.endswith("*") else ctx.last_kernel() == expect_kernel
        assert ok, (ctx.last_kernel(), expect_kernel)
    got = ctx.download(dout, oracle.STORAGE[dt], n_out)
    dx.free(); dout.free()
    r = int(md[-1])
    if dt in INTS:
        assert np.array_equal(got, oracle.sum_asis(dt, x, md)), (dt, v.shape, dims)
        return
    o32, o64, oabs = oracle.sum_spec(dt, x, md)
    gotf = H.widen(dt, got)
    assert np.all(np.isfinite(gotf))
    if dt == "f64":
        H.assert_close(gotf, o64, oabs, max(r, 1), 1e-12, f"sum {dt}", eps_acc=H.EPS_F64)
    elif dt in ("f8e4m3", "f8e5m2"):
        step, lim, tiny = (2.0 ** -3, 448.0, 2.0 ** -9) if dt == "f8e4m3" else (2.0 ** -2, 57344.0, 2.0 ** -16)
        want = np.clip(o64, -lim, lim)
        assert np.all(np.abs(gotf - want) <= step * np.abs(want) + tiny + 1e-3 * oabs / np.sqrt(max(r, 1)))
    else:
        tol = 1e-5 if dt == "f32" else 2e-2
        if dt == "f32":
            # the sequential f32 sum (the reference's own arithmetic) of a few thousand terms is itself off the exact
            # sum by about sqrt(r) * 2^-24 of sum|x| -- by r * 2^-25 where terms repeat (a stride-0 dim) and the roundings
            # stop cancelling -- which is the size of the tolerance's floor; a kernel that adds in chunks and trees lands
            # near the exact sum, one that walks the reduced dims in order near the sequential one: either is right
            try:
                H.assert_close(gotf, o64, oabs, max(r, 1), tol, f"sum {dt}")
                return
            except AssertionError:
                pass
        H.assert_close(gotf, o32.astype(np.float64), oabs, max(r, 1), tol, f"sum {dt}")


@pytest.mark.parametrize("dt", oracle.MATMUL_DTYPES)
def test_leading_dims(ctx, dt):
    """sum_to_shape on a weight gradient: [B, K, N] -> [K, N] (and [1, K, N]); N a multiple of the vector or not"""
    check_sum(ctx, dt, V([8, 24, 64]), [0], False, 1, "sum_by_output_vec")
    check_sum(ctx, dt, V([8, 24, 64]), [0], True, 2, "sum_by_output_vec")
    check_sum(ctx, dt, V([8, 23, 63]), [0], False, 3, "sum_by_output")  # 23 x 63 outputs: no whole vectors
    check_sum(ctx, dt, V([3, 4, 24, 64]), [0, 1], False, 4, "sum_by_output_vec")
    check_sum(ctx, dt, V([3, 4, 24, 64]), [1], True, 5, "sum_by_output_vec")


@pytest.mark.parametrize("dt", oracle.MATMUL_DTYPES)
def test_rows_and_everything(ctx, dt):
    check_sum(ctx, dt, V([37, 300]), [1], False, 6, "sum_by_row*")
    check_sum(ctx, dt, V([5, 6, 200]), [1, 2], True, 7, "sum_by_row*")
    check_sum(ctx, dt, V([4, 5, 160]), [0, 1, 2], False, 8, "sum_by_row*")
    check_sum(ctx, dt, V([9, 1024]), [1], False, 15, "sum_by_row_vec")
    check_sum(ctx, dt, V([9, 1031], offset=16), [1], False, 16, "sum_by_row")  # rows that start off a vector boundary
    check_sum(ctx, dt, V([37, 30]), [1], False, 9, "sum_by_output")  # short rows stay on the thread-per-output kernel


@pytest.mark.parametrize("dt", oracle.MATMUL_DTYPES)
def test_few_outputs_long_reduction(ctx, dt):
    """the gradient of a bias, [rows, features] -> [features]: the reduced index space is cut into chunks whose partial
    sums a second kernel adds"""
    check_sum(ctx, dt, V([4096, 256]), [0], False, 17, "sum_chunks_vec")
    check_sum(ctx, dt, V([8, 125, 96]), [0, 1], False, 18, "sum_chunks_vec")
    check_sum(ctx, dt, V([1000, 100], offset=1), [0], True, 19, "sum_chunks")        # off the vector boundary
    check_sum(ctx, dt, V([1001, 7]), [0], False, 20, "sum_chunks")                    # ragged last chunk, 7 outputs
    check_sum(ctx, dt, V([64, 8, 128]).t(0, 1), [0, 1], False, 21, "sum_chunks*")     # two reduced dims that do not merge
    check_sum(ctx, dt, V([40, 300]), [0], False, 22, "sum_by_output*")                # too short to cut


@pytest.mark.parametrize("dt", oracle.MATMUL_DTYPES)
def test_few_long_rows(ctx, dt):
    """sum_all of a large tensor is ONE row: rows this long are cut into chunks across workgroups"""
    check_sum(ctx, dt, V([1 << 18]), [0], False, 23, "sum_row_chunks_vec")
    check_sum(ctx, dt, V([3, 100003]), [1], False, 24, "sum_row_chunks")          # rows start off vector boundaries
    check_sum(ctx, dt, V([2, 4, 20000]), [1, 2], True, 25, "sum_row_chunks_vec")   # the two reduced dims merge
    check_sum(ctx, dt, V([5, 70000], offset=16).slice(1, 0, 66000), [1], False, 26, "sum_row_chunks*")
    check_sum(ctx, dt, V([3, 9000]), [1], False, 27, "sum_by_row*")                # too short to cut


@pytest.mark.parametrize("dt", ["bf16", "f32", "i32", "u8"])
def test_strided_inputs(ctx, dt):
    check_sum(ctx, dt, V([6, 8, 40], offset=3).t(0, 2), [0], False, 10)       # summed dim is the dense one
    check_sum(ctx, dt, V([9, 80]).slice(1, 1, 80, 3), [0], True, 11)         # column-strided
    check_sum(ctx, dt, V([16], [0]).broadcast_to([7, 16]), [0], False, 12)   # a broadcast (stride 0) dim summed
    check_sum(ctx, dt, V([12, 64], offset=8), [0], False, 13)                # offset that keeps vectors aligned
    check_sum(ctx, dt, V([12, 64], offset=5), [0], False, 14, "sum_by_output")


@pytest.mark.parametrize("dt", ["f32", "bf16", "i32"])
def test_few_outputs_that_are_not_dense_take_the_chunked_kernels_too(ctx, dt):
    """a strided tensor summed to a scalar, and a handful of stepped outputs with a long stepped reduction: cut into
    chunks across workgroups like the dense case, not walked by one lane per output"""
    check_sum(ctx, dt, V([500, 300]).t(), [0, 1], False, 1, "sum_chunks")
    check_sum(ctx, dt, V([4, 3000], [2, 8]), [1], False, 2, "sum_chunks")
    check_sum(ctx, dt, V([4, 3000], [2, 8], offset=3), [1], True, 3, "sum_chunks")


def test_config5_weight_gradient_shape(ctx):
    """[8, 512, 1024] bf16 partial gradients summed over the batch: every input element read once"""
    check_sum(ctx, "bf16", V([8, 512, 1024]), [0], False, 15, "sum_by_output_vec")


def test_empty_and_degenerate(ctx):
    check_sum(ctx, "f32", V([0, 5]), [0], False, 16, "sum_empty")
    md = H.reduce_md(V([4, 0]), [0], False)
    x, out = ctx.upload(np.zeros(4, np.float32)), ctx.alloc(16)
    ctx.sum("f32", x, out, md)  # no outputs: nothing to do
    check_sum(ctx, "i32", V([5, 1, 6]), [1], False, 17)  # summing an extent-1 dim copies


def test_malformed_metadata_is_rejected(ctx):
    x, out = ctx.upload(np.zeros(64, np.float32)), ctx.alloc(256)
    good = H.reduce_md(V([4, 16]), [0], False)
    for bad, what in ((good[:-1], "words"), (good[:-1] + [5], "reduce_size"), ([2, 4, 16, 16, 1, 0, 1, 16, 1, 2, 0, 4], "reduce dim"),
                      ([2, 4, 16, 16, 1, 0, 1, 15, 1, 0, 0, 4], "extent")):
        with pytest.raises(ffi.HoduRocmError, match=what):
            ctx.sum("f32", x, out, bad)
    x.free(); out.free()
