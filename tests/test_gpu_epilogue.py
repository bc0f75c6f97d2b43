"""GPU parity of the fused element-wise steps (hodu_rocm_<op>_<dt>_ex): add(bias), mul_scalar and relu applied inside
the product's store.

What hodu runs is the product, then hodu_cpu_add / hodu_cpu_mul_scalar / hodu_cpu_relu as kernels of their own
(crates/hodu_nn/src/modules/linear.rs:40-46, attention.rs:37, activation.rs:8-17).  The fused launch must therefore
equal, bit for bit, the plain launch's output pushed through the oracle's restatement of those kernels.  The plain
launch itself is what the other GPU test files compare with the product oracle.  Every kernel family that stores
outputs is driven at ragged sizes: the generic kernel, the tile kernels, the pipelined kernels with and without a
cut K, the kernels for M <= 16 and the row-streaming one."""
import numpy as np
import pytest

import helpers as H
import oracle
from gpu_util import OUT_STORAGE, dtypes_of, run_product
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View
FLOATS = ("bf16", "f16", "f32", "f64")


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.force_tile(-1)
    c.force_splitk(-1)
    c.close()


def oracle_chain(out_dt, plain, out_shape, spec, bias, scalar):
    """the reference's kernels, one after the other, on the plain product's output"""
    full = V(out_shape)
    x = plain
    for step in spec:
        if step[0] == "add":
            _, stride, offset = step
            bv = V([out_shape[-1]], [stride], offset).broadcast_to(out_shape)
            x = oracle.add(out_dt, x, bias, H.binary_md(full, bv))
        elif step[0] == "mul":
            x = oracle.mul_scalar(out_dt, x, H.cast_md(full), scalar)
        else:
            x = oracle.relu(out_dt, x, H.cast_md(full))
    return x


def check_fused(ctx, op, name, lv, rv, spec, seed=0, scale=1.0, rscale=None, expect_kernel=None, must_change=True):
    l_dt, r_dt, out_dt = dtypes_of(name)
    a = H.random_storage(l_dt, lv.span(), 1000 + seed, scale)
    b = H.random_storage(r_dt, rv.span(), 2000 + seed, scale if rscale is None else rscale)
    md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
    bshape = list(np.broadcast_shapes(tuple(lv.shape[:-2]), tuple(rv.shape[:-2])))
    out_shape = bshape + [lv.shape[-2], rv.shape[-1]]
    n_out, n_cols = int(np.prod(out_shape)), out_shape[-1]
    bias = H.random_storage(out_dt, 3 * n_cols + 8, 3000 + seed, 4.0)
    scalar = H.random_storage(out_dt, 4, 4000 + seed, 2.0)[1:2]
    plain = run_product(ctx, op, name, a, b, md)
    if expect_kernel is not None:
        assert ctx.last_kernel().startswith(expect_kernel), (ctx.last_kernel(), expect_kernel)
    plain_kernel = ctx.last_kernel()

    da, db, dbias = ctx.upload(a), ctx.upload(b), ctx.upload(bias)
    dout = ctx.alloc(n_out * ffi.DTYPE_SIZE[out_dt])
    ctx.fill(dout, 0xFF)
    steps = []
    for step in spec:
        if step[0] == "add":
            steps.append(ffi.add_row(dbias, step[1], step[2]))
        elif step[0] == "mul":
            steps.append(ffi.mul_scalar(scalar))
        else:
            steps.append(ffi.relu())
    ctx.product_ex(op, name, da, db, dout, md, steps)
    assert ctx.last_kernel() == plain_kernel  # the same kernel, not a slower stand-in
    got = ctx.download(dout, OUT_STORAGE[out_dt], n_out)
    for d in (da, db, dbias, dout):
        d.free()
    want = oracle_chain(out_dt, plain, out_shape, spec, bias, scalar)
    if out_dt in ("f32", "f64"):
        assert np.all(np.isfinite(got)) and np.all(np.isfinite(want))
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (op, name, spec, ctx.last_kernel())
    if spec and must_change:
        assert not np.array_equal(got.view(np.uint8), plain.view(np.uint8))  # the steps did something


LINEAR = [("add", 1, 0)]
SPECS = [LINEAR, [("mul",)], [("relu",)], [("mul",), ("add", 2, 3), ("relu",)], [("add", 0, 5)]]


@pytest.mark.parametrize("dt", ffi.EPILOGUE_DTYPES)
def test_generic_kernel_every_dtype(ctx, dt):
    """column-strided operands: the generic kernel, the tile kernel's scalar-load variant for bf16 / f16 / i8 / u8,
    the small-product kernel for f32, the f64 matrix-core kernel"""
    lv, rv = V([37, 50]).slice(1, 1, 49, 2), V([24, 70]).slice(1, 0, 70, 2)
    family = ("mfma_" if dt in ("bf16", "f16", "i8", "u8") else "small_f32" if dt == "f32" else "mfma_f64" if dt == "f64"
              else "generic")
    for n, spec in enumerate(SPECS):
        if dt not in FLOATS and ("relu",) in spec:
            continue
        check_fused(ctx, "dot", dt, lv, rv, spec, seed=n, expect_kernel=family)
        if dt == "f64":  # (and the generic kernel, which keeps the f64 products thinner than a matrix-core tile)
            ctx.force_tile(3)
            try:
                check_fused(ctx, "dot", dt, lv, rv, spec, seed=n, expect_kernel="generic")
            finally:
                ctx.force_tile(-1)
    check_fused(ctx, "matmul", dt, V([3, 2, 9, 12]), V([12, 7], [1, 12]).broadcast_to([3, 2, 12, 7]), LINEAR, seed=9)


@pytest.mark.parametrize("name", ["bf16", "f16", "f32", "bf16_f8e4m3w", "i32_i8i8"])
@pytest.mark.parametrize("tile", [0, 2, 3])
def test_tile_kernels(ctx, name, tile):
    """general MFMA tile kernel: a row-dense right operand whose K is no multiple of the pipelined kernel's stage"""
    ctx.force_tile(tile)
    try:
        rs = 2.0 if "f8" in name else None
        for n, spec in enumerate(SPECS):
            if name == "i32_i8i8" and ("relu",) in spec:
                continue
            check_fused(ctx, "dot", name, V([150, 80]), V([80, 136]), spec, seed=n, rscale=rs, expect_kernel="mfma_")
        check_fused(ctx, "matmul", name, V([2, 70, 48]), V([2, 48, 40]), LINEAR, seed=7, rscale=rs, expect_kernel="mfma_")
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("name", ["bf16", "f16", "f32", "bf16_f8e4m3w", "i32_i8i8"])
@pytest.mark.parametrize("tile", [10, 12, 13])
def test_pipelined_kernels(ctx, name, tile):
    """pipelined kernels (outputs leave through LDS as whole rows): N ragged against the 16-byte store, batches"""
    if tile == 13 and name == "bf16_f8e4m3w":
        pytest.skip("no 64x64 pipelined kernel for f8e4m3 weights")
    ctx.force_tile(tile)
    try:
        rs = 2.0 if "f8" in name else None
        k = 512 if name != "f32" else 256
        for n, spec in enumerate(SPECS):
            if name == "i32_i8i8" and ("relu",) in spec:
                continue
            check_fused(ctx, "dot", name, V([150, k]), V([133, k]).t(), spec, seed=n, rscale=rs, expect_kernel="mfma_")
            assert "pipe" in ctx.last_kernel()
        check_fused(ctx, "matmul", name, V([3, 70, k]), V([3, 72, k]).t(), [("mul",), ("add", 1, 1)], seed=7, rscale=rs)
        assert "pipe" in ctx.last_kernel()
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("name", ["bf16", "f16", "bf16_f8e4m3w"])
def test_16x16_instruction_tiles(ctx, name):
    """the 256 x 256 tile on the 16 x 16 x 32 instruction (bands of 16 rows leave through LDS; the steps' column data is
    fetched once per tile): every step combination, N ragged against the 16-byte store, row-dense operands, batches"""
    ctx.force_tile(15)
    try:
        rs = 2.0 if "f8" in name else None
        for n, spec in enumerate(SPECS):
            check_fused(ctx, "dot", name, V([150, 512]), V([133, 512]).t(), spec, seed=n, rscale=rs, expect_kernel="mfma_")
            assert "mi16_KK" in ctx.last_kernel(), ctx.last_kernel()
        n_km = 528 if "f8" in name else 520  # (row-dense f8e4m3 weights move in 16-byte chunks: N a multiple of 16)
        check_fused(ctx, "dot", name, V([300, 256]), V([256, n_km]), [("mul",), ("add", 2, 3), ("relu",)], seed=8, rscale=rs)
        assert "mi16_KM" in ctx.last_kernel(), ctx.last_kernel()
        check_fused(ctx, "matmul", name, V([3, 70, 512]), V([3, 72, 512]).t(), [("mul",), ("add", 1, 1)], seed=7, rscale=rs)
        assert "mi16_KK" in ctx.last_kernel(), ctx.last_kernel()
        if name != "bf16_f8e4m3w":
            check_fused(ctx, "dot", name, V([256, 296]).t(), V([256, 264]), [("add", 1, 0), ("relu",)], seed=9)
            assert "mi16_MM" in ctx.last_kernel(), ctx.last_kernel()
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("name", ["bf16", "f32", "bf16_f8e4m3w", "i32_i8i8"])
def test_pipelined_kernels_with_k_cut(ctx, name):
    """partial sums of the K ranges carry no steps; the second pass that adds them applies the steps once"""
    ctx.force_tile(12)
    ctx.force_splitk(4)
    try:
        rs = 2.0 if "f8" in name else None
        for n, spec in enumerate([LINEAR, [("mul",), ("add", 2, 3)]]):
            check_fused(ctx, "dot", name, V([100, 1024]), V([132, 1024]).t(), spec, seed=n, rscale=rs)
            assert "splitk" in ctx.last_kernel()
        check_fused(ctx, "matmul", name, V([2, 66, 1024]), V([2, 70, 1024]).t(), LINEAR, seed=5, rscale=rs)
        assert "splitk" in ctx.last_kernel()
    finally:
        ctx.force_tile(-1)
        ctx.force_splitk(-1)


@pytest.mark.parametrize("name", ["bf16", "f16", "f32", "bf16_f8e4m3w", "i32_i8i8"])
def test_small_m_kernels(ctx, name):
    """M <= 16: one-pass kernel, the variant that cuts K across workgroups, and (bf16 activations, M <= 4) the
    row-streaming kernel"""
    rs = 2.0 if "f8" in name else None
    specs = [s for s in SPECS if not (name == "i32_i8i8" and ("relu",) in s)]
    for n, spec in enumerate(specs):
        check_fused(ctx, "dot", name, V([9, 1040]), V([203, 1040]).t(), spec, seed=n, rscale=rs, expect_kernel="skinny_")
    ctx.force_tile(38)
    try:
        for n, spec in enumerate(specs[:2]):
            check_fused(ctx, "dot", name, V([16, 2064]), V([1100, 2064]).t(), spec, seed=10 + n, rscale=rs)
            assert ctx.last_kernel().endswith("_splitk")
    finally:
        ctx.force_tile(-1)
    if name in ("bf16", "bf16_f8e4m3w"):
        for m in (1, 3):
            for n, spec in enumerate(specs):
                check_fused(ctx, "dot", name, V([m, 1040]), V([203, 1040]).t(), spec, seed=20 + n, rscale=rs,
                            expect_kernel="gemv_")


@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
def test_matrix_times_vector_keeps_the_few_rows_route_with_steps(ctx, name):
    """[M, K] x [K, 1] runs as the transposed one-row product; fused steps go along (a vector added along an output row
    of one element is that element for every output)"""
    for n, spec in enumerate(SPECS):
        check_fused(ctx, "dot", name, V([300, 1040]), V([1040, 1]), spec, seed=n, expect_kernel=("gemv_", "skinny_"))
    check_fused(ctx, "dot", name, V([64, 512], offset=8), V([512, 1], [3, 0]), SPECS[3], seed=9)  # a strided vector


def test_linear_layer_of_config3(ctx):
    """x[16, 4096] (bf16) times the f8e4m3 weight [4096, 4096] passed transposed, plus a bf16 bias: the layer the
    fused entry point exists for, at its real size"""
    check_fused(ctx, "dot", "bf16_f8e4m3w", V([16, 4096]), V([4096, 4096]).t(), LINEAR, seed=1, rscale=2.0)
    check_fused(ctx, "dot", "bf16_f8e4m3w", V([1, 4096]), V([4096, 4096]).t(), LINEAR + [("relu",)], seed=2, rscale=2.0,
                expect_kernel="gemv_")


def test_no_steps_is_the_plain_product(ctx):
    check_fused(ctx, "dot", "bf16", V([40, 64]), V([64, 24]), [], seed=3)


def test_rejected_steps(ctx):
    a, b = ctx.upload(np.zeros(64, np.int32)), ctx.upload(np.zeros(64, np.int32))
    out, vec = ctx.alloc(64 * 4), ctx.upload(np.zeros(8, np.int32))
    md = H.dot_md(V([8, 8]), V([8, 8]))
    with pytest.raises(ffi.HoduRocmError, match="relu"):
        ctx.product_ex("dot", "i32", a, b, out, md, [ffi.relu()])
    with pytest.raises(ffi.HoduRocmError, match="at most"):
        ctx.product_ex("dot", "i32", a, b, out, md, [ffi.add_row(vec)] * 4)
    with pytest.raises(ffi.HoduRocmError, match="null vector"):
        ctx.product_ex("dot", "i32", a, b, out, md, [ffi.EpilogueStep(ffi.EPI_ADD_ROW, None, 1, 0, (ffi.ctypes.c_ubyte * 8)())])
    with pytest.raises(ffi.HoduRocmError, match="unknown op"):
        ctx.product_ex("dot", "i32", a, b, out, md, [ffi.EpilogueStep(9, None, 0, 0, (ffi.ctypes.c_ubyte * 8)())])
    with pytest.raises(ffi.HoduRocmError, match="output buffer"):
        ctx.product_ex("dot", "i32", a, b, out, md, [ffi.add_row(out)])
    for d in (a, b, out, vec):
        d.free()


@pytest.mark.parametrize("tile", [15, 11, 12, 2, -1])
def test_steps_on_zero_nan_and_infinite_sums(ctx, tile):
    """bf16 product whose plain output holds exact +0 (a zero row), NaN (a NaN in the row), +inf and -inf beside
    ordinary small integers: a negative scalar turns +0 into -0 and the infinities round, ReLU turns -0, NaN and
    -inf into +0 -- the reference's `(x > 0) ? x : 0` -- and the fused launch equals the reference's kernels on the
    plain output bit for bit, on the 16 x 16 x 32 tile, the 32 x 32 x 16 ones, the general tile kernel and whatever
    the automatic choice is"""
    m, n, k = 272, 208, 256
    g = H.rng(70 + tile)
    af = g.integers(-3, 4, (m, k)).astype(np.float32)
    bf = g.integers(1, 4, (n, k)).astype(np.float32)  # positive: an infinite operand gives an infinite sum, not NaN
    af[0] = 0.0
    af[17] = 0.0
    af[1, 5] = np.nan
    af[2, 100] = np.inf
    af[3, 200] = -np.inf
    af[4, 7], af[4, 9] = np.inf, -np.inf  # inf - inf
    a, b = H.f32_to_bf16_rne(af.ravel()), H.f32_to_bf16_rne(bf.ravel())
    lv, rv = V([m, k]), V([n, k]).t()
    md = H.dot_md(lv, rv)
    bias = H.f32_to_bf16_rne(g.integers(-4, 5, n).astype(np.float32))
    bias[::7] = 0x8000  # -0
    scalar = H.f32_to_bf16_rne(np.array([-1.5], dtype=np.float32))
    ctx.force_tile(tile)
    try:
        plain = run_product(ctx, "dot", "bf16", a, b, md)
        kernel = ctx.last_kernel()
        p = plain.reshape(m, n)
        assert (p[0] == 0).all() and (p[17] == 0).all() and ((p[1] & 0x7FFF) > 0x7F80).all()
        assert (p[2] == 0x7F80).all() and (p[3] == 0xFF80).all() and ((p[4] & 0x7FFF) > 0x7F80).all()
        for spec in ([("mul",)], [("relu",)], [("mul",), ("relu",)], [("add", 1, 0), ("relu",)],
                     [("mul",), ("add", 1, 0), ("relu",)], [("relu",), ("mul",)]):
            da, db, dbias = ctx.upload(a), ctx.upload(b), ctx.upload(bias)
            dout = ctx.alloc(m * n * 2)
            ctx.fill(dout, 0xFF)
            steps = [ffi.add_row(dbias, s[1], s[2]) if s[0] == "add" else ffi.mul_scalar(scalar) if s[0] == "mul" else ffi.relu()
                     for s in spec]
            ctx.product_ex("dot", "bf16", da, db, dout, md, steps)
            assert ctx.last_kernel() == kernel
            got = ctx.download(dout, np.uint16, m * n)
            for d in (da, db, dbias, dout):
                d.free()
            want = oracle_chain("bf16", plain, [m, n], spec, bias, scalar)
            bad = np.flatnonzero(got != want)
            assert bad.size == 0, (kernel, spec, bad[:5], got[bad[:5]], want[bad[:5]], plain[bad[:5]])
    finally:
        ctx.force_tile(-1)
