"""Exact-valued products, compared bit for bit.

Small-integer operands (bf16 activations in [-4, 4], f8e4m3 / bf16 weights in [-8, 8]) make every product and every
partial sum an integer below 2^24, so an f32 accumulator holds the exact sum whatever the order of addition, and
the one rounding to bf16 is the same on every correct kernel: the float kernels that have no integer twin (the
row-streaming GEMV, the M <= 16 kernel and its split-K form, the f8e4m3-weight pipelined tile kernel, split-K through
the workspace) are held to equality here, where the tolerance tests allow 2e-2.  A dropped or doubled k-term, a
wrong decode of one f8 code or a stale partial sum changes the integer and fails.
"""
import numpy as np
import pytest

import helpers as H
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.force_tile(-1)
    c.force_splitk(-1)
    c.close()


def int_bf16(seed, n, top):
    return H.f32_to_bf16_rne(H.rng(seed).integers(-top, top + 1, n).astype(np.float32))


def int_f8(seed, n, top=8):
    codes = H.f32_to_ocp_e4m3_rne(H.rng(seed).integers(-top, top + 1, n).astype(np.float64))
    assert np.array_equal(H.ocp_e4m3_decode(codes), np.round(H.ocp_e4m3_decode(codes)))  # integers survive the encoding
    return codes


def run_exact(ctx, op, name, lv, rv, seed, expect_kernel):
    l_dt, r_dt = ("bf16", "f8e4m3") if name == "bf16_f8e4m3w" else ("bf16", "bf16")
    a = int_bf16(100 + seed, max(lv.span(), 1), 4)
    b = int_f8(200 + seed, max(rv.span(), 1)) if r_dt == "f8e4m3" else int_bf16(200 + seed, max(rv.span(), 1), 8)
    md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
    n_out = int(md[0]) if op == "matmul" else int(md[0]) * int(md[2])
    da, db, dout = ctx.upload(a), ctx.upload(b), ctx.alloc(2 * n_out)
    ctx.fill(dout, 0xFF)
    ctx.product(op, name, da, db, dout, md)
    got = ctx.download(dout, np.uint16, n_out)
    kernel = ctx.last_kernel()
    for d in (da, db, dout):
        d.free()
    assert kernel.startswith(expect_kernel), (kernel, expect_kernel)
    bshape = list(np.broadcast_shapes(tuple(lv.shape[:-2]), tuple(rv.shape[:-2])))
    A = H.widen(l_dt, lv.broadcast_to(bshape + lv.shape[-2:]).take(a))
    B = H.widen(r_dt, rv.broadcast_to(bshape + rv.shape[-2:]).take(b))
    exact = A @ B  # float64 of integers: exact
    assert np.abs(exact).max() < 2 ** 24
    want = H.f32_to_bf16_rne(exact.astype(np.float32).ravel())
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, f"{kernel}: {bad.size} of {got.size} outputs differ, first at {bad[:5]}"
    return kernel


@pytest.mark.parametrize("name", ["bf16_f8e4m3w", "bf16"])
@pytest.mark.parametrize("m", [1, 2, 4])
def test_row_streaming_gemv(ctx, name, m):
    pre = "gemv_bf16_f8w" if name == "bf16_f8e4m3w" else "gemv_bf16"
    run_exact(ctx, "dot", name, V([m, 4096]), V([1024, 4096]).t(), m, pre)
    run_exact(ctx, "dot", name, V([m, 4112]), V([203, 4112]).t(), 10 + m, pre)
    # from 4096 weight rows on a wavefront walks several row groups; K of one pass and of several
    run_exact(ctx, "dot", name, V([m, 4096]), V([4610, 4096]).t(), 20 + m, pre)
    run_exact(ctx, "dot", name, V([m, 9216]), V([4100, 9216]).t(), 30 + m, pre)


@pytest.mark.parametrize("name", ["bf16_f8e4m3w", "bf16"])
@pytest.mark.parametrize("m", [5, 16])
def test_one_pass_and_split_k_skinny(ctx, name, m):
    pre = "skinny_bf16_f8w" if name == "bf16_f8e4m3w" else "skinny_bf16"
    for shape in (35, 36, 37):
        ctx.force_tile(shape)
        run_exact(ctx, "dot", name, V([m, 4096]), V([1040, 4096]).t(), m, pre)
    ctx.force_tile(38)
    for _ in range(2):
        k = run_exact(ctx, "dot", name, V([m, 4224]), V([1100, 4224]).t(), 20 + m, pre)
        assert k.endswith("_splitk")
    ctx.force_tile(-1)


def test_config3_m16_takes_the_split_k_kernel_exactly(ctx):
    k = run_exact(ctx, "dot", "bf16_f8e4m3w", V([16, 4096]), V([4096, 4096]).t(), 3, "skinny_bf16_f8w")
    assert k.endswith("_splitk")


@pytest.mark.parametrize("tile", [10, 11, 12, 14])
@pytest.mark.parametrize("combo", ["KK", "KM"])
def test_f8_weight_pipelined_tiles(ctx, tile, combo):
    """every tile shape of the pipelined kernel on f8e4m3 weights, k-dense ([N, K]^T view) and row-dense ([K, N])"""
    rv = V([384, 1024]).t() if combo == "KK" else V([1024, 384])
    ctx.force_tile(tile)
    try:
        run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, 1024]), rv, tile, "mfma_bf16_f8w_pipe")
        run_exact(ctx, "dot", "bf16", V([296, 1024]), V([384, 1024]).t() if combo == "KK" else V([1024, 384]), tile,
                  "mfma_bf16_pipe")
    finally:
        ctx.force_tile(-1)


def test_16x16_instruction_tile_is_exact_and_equals_the_32x32_one(ctx):
    """the 256 x 256 bf16 tile on the 16 x 16 x 32 matrix instruction (hook value 15, the default for large products;
    right operand k-dense or row-dense): exact sums on ragged shapes, a batch, and a full-size tile grid"""
    for tile in (15, 11):
        ctx.force_tile(tile)
        try:
            name = "mfma_bf16_pipe256x256mi16_KK" if tile == 15 else "mfma_bf16_pipe256x256_KK"
            run_exact(ctx, "dot", "bf16", V([296, 1024]), V([384, 1024]).t(), 3, name)
            run_exact(ctx, "dot", "bf16", V([520, 64]), V([263, 64]).t(), 4, name)            # one stage, ragged tiles
            run_exact(ctx, "dot", "bf16", V([17, 192]), V([5, 192]).t(), 5, name)             # less than one fragment of rows
            run_exact(ctx, "matmul", "bf16", V([3, 160, 512]), V([3, 136, 512]).t(), 6, name)
            run_exact(ctx, "dot", "bf16", V([1024, 2048 + 64]).slice(1, 64, 2048 + 64), V([768, 2048], offset=128).t(), 7, name)
            # the right operand row-dense ([K, N] row-major)
            km = name.replace("_KK", "_KM")
            run_exact(ctx, "dot", "bf16", V([296, 1024]), V([1024, 384]), 9, km)
            run_exact(ctx, "dot", "bf16", V([520, 64]), V([64, 264]), 10, km)
            run_exact(ctx, "matmul", "bf16", V([2, 160, 512]), V([512, 520]).broadcast_to([2, 512, 520]), 11, km)
            # the left operand row-dense (a transposed view)
            run_exact(ctx, "dot", "bf16", V([1024, 296]).t(), V([384, 1024]).t(), 13, name.replace("_KK", "_MK"))
            run_exact(ctx, "dot", "bf16", V([192, 520]).t(), V([192, 264]), 14, name.replace("_KK", "_MM"))
        finally:
            ctx.force_tile(-1)
    # what the launcher picks by itself for a product that fills the chip with 256 x 256 tiles
    assert run_exact(ctx, "dot", "bf16", V([4096, 256]), V([4096, 256]).t(), 8, "mfma_bf16_pipe256x256mi16_KK")
    assert run_exact(ctx, "dot", "bf16", V([4096, 128]), V([128, 4096]), 12, "mfma_bf16_pipe256x256mi16_KM")


def test_16x16_instruction_tile_with_f8_weights_is_exact(ctx):
    """the same tile with f8e4m3 weights widened in front of the MFMA (pairs of stages per weight buffer): 1 to 9 pairs,
    ragged shapes, a batch sharing the weight, and what the launcher picks for a product that fills the chip"""
    name = "mfma_bf16_f8w_pipe256x256mi16_KK"
    ctx.force_tile(15)
    try:
        for k in (128, 256, 384, 1024, 2304):
            run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, k]), V([384, k]).t(), k, name)
        run_exact(ctx, "dot", "bf16_f8e4m3w", V([17, 256]), V([5, 256]).t(), 5, name)
        run_exact(ctx, "matmul", "bf16_f8e4m3w", V([2, 160, 512]), V([520, 512]).t().broadcast_to([2, 512, 520]), 6, name)
        km = name.replace("_KK", "_KM")  # row-dense weights
        for k in (64, 192, 1024):
            run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, k]), V([k, 384]), k + 1, km)
        run_exact(ctx, "matmul", "bf16_f8e4m3w", V([2, 160, 512]), V([512, 528]).broadcast_to([2, 512, 528]), 7, km)
    finally:
        ctx.force_tile(-1)
    assert run_exact(ctx, "dot", "bf16_f8e4m3w", V([4096, 256]), V([4096, 256]).t(), 8, name)
    assert run_exact(ctx, "dot", "bf16_f8e4m3w", V([4096, 128]), V([128, 4096]), 9, name.replace("_KK", "_KM"))


@pytest.mark.parametrize("splits", [2, 4, 7])
def test_pipelined_split_k_through_the_workspace(ctx, splits):
    ctx.force_splitk(splits)
    try:
        for name in ("bf16_f8e4m3w", "bf16"):
            k = run_exact(ctx, "dot", name, V([256, 4096]), V([512, 4096]).t(), splits, "mfma_bf16")
            assert "splitk" in k, k
    finally:
        ctx.force_splitk(-1)


def test_batched_and_broadcast_exact(ctx):
    run_exact(ctx, "matmul", "bf16", V([3, 160, 512]), V([3, 136, 512]).t(), 1, "mfma_bf16")
    run_exact(ctx, "matmul", "bf16_f8e4m3w", V([4, 128, 512]), V([512, 256]).broadcast_to([4, 512, 256]), 2, "mfma_bf16_f8w")


def narrow_e5m2_rne(x):
    """round-to-nearest-even of values that float16 holds exactly (|x| < 2048 integers) to f8e5m2 codes"""
    h = np.asarray(x, dtype=np.float16)
    assert np.array_equal(h.astype(np.float64), x)
    bits = h.view(np.uint16).astype(np.uint32)
    return ((bits + 0x7F + ((bits >> 8) & 1)) >> 8).astype(np.uint8)


@pytest.mark.parametrize("dt", ["f8e4m3", "f8e5m2"])
@pytest.mark.parametrize("tile", [11, 12, 15])
def test_native_f8_products_narrow_the_exact_sum_once(ctx, dt, tile):
    """f8 x f8 -> f8 on the 8-bit matrix instruction: operands in {-2 .. 2} (exact in both formats), so the f32 sum is
    the exact integer in any order and the stored code must be its round-to-nearest-even, saturating at 448 for
    f8e4m3 -- bit for bit, across the ties (sums like 17, 18, 20 ... fall between f8e4m3 codes) and, uncut and cut
    three ways along K"""
    g = H.rng(300 + tile)
    enc = (lambda v: H.f32_to_ocp_e4m3_rne(v.astype(np.float64))) if dt == "f8e4m3" else narrow_e5m2_rne
    ctx.force_tile(tile)
    try:
        for (m, n, k), splits, top in (((296, 200, 640), -1, 2), ((296, 200, 1280), 3, 2), ((130, 264, 2048), -1, 6 if dt == "f8e4m3" else 3)):
            av = g.integers(-top, top + 1, m * k).astype(np.float64)
            bv = g.integers(-top, top + 1, n * k).astype(np.float64)
            a, b = enc(av), enc(bv)
            assert np.array_equal(H.widen(dt, a), av) and np.array_equal(H.widen(dt, b), bv)
            md = H.dot_md(V([m, k]), V([n, k]).t())
            da, db, dout = ctx.upload(a), ctx.upload(b), ctx.alloc(m * n)
            ctx.fill(dout, 0xFF)
            if tile == 15:
                splits = -1  # (the 16 x 16 x 128 tile is never cut along K)
            ctx.force_splitk(splits)
            ctx.product("dot", dt, da, db, dout, md)
            got = ctx.download(dout, np.uint8, m * n)
            kernel = ctx.last_kernel()
            for d in (da, db, dout):
                d.free()
            assert kernel.startswith(f"mfma_{dt}_pipe") and (splits < 0 or "splitk" in kernel), kernel
            exact = (av.reshape(m, k) @ bv.reshape(n, k).T).ravel()
            if dt == "f8e4m3":
                want = H.f32_to_ocp_e4m3_rne(np.clip(exact, -448.0, 448.0))
                assert np.abs(exact).max() > 448 or top == 2  # the wide-range case saturates in places
            else:
                assert np.abs(exact).max() < 2048
                want = narrow_e5m2_rne(exact)
            # +0 and -0 are one value: an exact zero sum is stored as +0
            bad = np.flatnonzero(got != want)
            assert bad.size == 0, f"{kernel}: {bad.size} of {got.size} codes differ, first at {bad[:5]}: " \
                                  f"{got[bad[:5]]} for sums {exact[bad[:5]]}"
    finally:
        ctx.force_tile(-1)
        ctx.force_splitk(-1)



@pytest.mark.parametrize("dt", ["f8e4m3", "f8e5m2"])
@pytest.mark.parametrize("tile", [11, 12, 15])
def test_native_f8_products_keep_nan_and_saturate_infinity(ctx, dt, tile):
    """what the narrowing does where the f32 sum is not finite: a NaN operand makes its whole output row NaN, an
    infinite f8e5m2 operand makes sums of +-inf, stored as the largest finite code of that sign (the narrowing
    saturates), and inf * 0 is NaN; every other output is the exact small sum"""
    m, n, k = 272, 208, 256
    g = H.rng(900 + tile)
    one = 0x38 if dt == "f8e4m3" else 0x3C
    a = np.where(g.integers(0, 2, m * k) == 1, one, 0).astype(np.uint8).reshape(m, k)
    b = np.full((n, k), one, dtype=np.uint8)
    nan_code = 0x7F if dt == "f8e4m3" else 0x7E
    a[3, 17] = nan_code
    a[200, 255] = nan_code | 0x80
    if dt == "f8e5m2":
        a[5, :] = 0
        a[5, 9] = 0x7C   # +inf
        a[130, :] = 0
        a[130, 77] = 0xFC  # -inf
        b[40, 9] = 0     # inf * 0
    ctx.force_tile(tile)
    try:
        md = H.dot_md(V([m, k]), V([n, k]).t())
        da, db, dout = ctx.upload(a.ravel()), ctx.upload(b.ravel()), ctx.alloc(m * n)
        ctx.fill(dout, 0x11)
        ctx.product("dot", dt, da, db, dout, md)
        got = ctx.download(dout, np.uint8, m * n).reshape(m, n)
        kernel = ctx.last_kernel()
        for d in (da, db, dout):
            d.free()
    finally:
        ctx.force_tile(-1)
    assert kernel.startswith(f"mfma_{dt}_pipe"), kernel
    is_nan = (lambda c: (c & 0x7F) == 0x7F) if dt == "f8e4m3" else (lambda c: ((c & 0x7C) == 0x7C) & ((c & 3) != 0))
    assert is_nan(got[3]).all() and is_nan(got[200]).all()
    plain = np.ones(m, dtype=bool)
    plain[[3, 200]] = False
    if dt == "f8e5m2":
        plain[[5, 130]] = False
        cols = np.arange(n) != 40
        assert (got[5, cols] == 0x7B).all() and (got[130] == 0xFB).all(), (got[5, :4], got[130, :4])
        assert is_nan(got[5, 40])
    # each output of a plain row: the number of ones in the row (column 40 of the f8e5m2 case misses k = 9)
    sums = np.repeat((a[plain] == one).sum(axis=1).astype(np.float64)[:, None], n, axis=1)
    if dt == "f8e5m2":
        sums[:, 40] -= a[plain, 9] == one
    want = H.f32_to_ocp_e4m3_rne(sums.ravel()) if dt == "f8e4m3" else narrow_e5m2_rne(sums.ravel())
    assert np.array_equal(got[plain].ravel(), want)
