"""The five benchmark configurations at FULL size through the C ABI.

The GPU computes the whole product; the oracle, which must finish in seconds, checks either the
whole result (configs 1 and 4) or an evenly spaced subset of output rows (a strided row slice of
the left operand is itself a valid hodu view, so the oracle sees it as an ordinary dot/matmul).
"""
import numpy as np
import pytest

import helpers as H
import oracle
from gpu_util import run_product
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def fp8_weights(n, k, seed, top=448.0):
    """N(0, 0.02) weights scaled so that max|W| maps to `top`, rounded to OCP e4m3 (RNE, clamped)."""
    w = H.rng(seed).standard_normal((n, k)).astype(np.float32) * 0.02
    s = top / np.abs(w).max()
    return H.f32_to_ocp_e4m3_rne(np.clip(w * s, -448, 448)).ravel(), s


def check_rows(got_rows, l_dt, r_dt, a, b, md_rows, k, tol):
    o32, o64, oabs = oracle.dot_spec(l_dt, r_dt, a, b, md_rows)
    gotf = H.bf16_to_f32(got_rows).astype(np.float64) if got_rows.dtype == np.uint16 else got_rows.astype(np.float64)
    assert np.all(np.isfinite(gotf)) and np.all(np.isfinite(o32))
    H.assert_close(gotf, o32.astype(np.float64), oabs, k, tol, f"{l_dt} x {r_dt}, K = {k}")


def test_config1_f32_512(ctx):
    a = H.rng(101).standard_normal(512 * 512).astype(np.float32)
    b = H.rng(102).standard_normal(512 * 512).astype(np.float32)
    md = H.dot_md(V([512, 512]), V([512, 512]))
    got = run_product(ctx, "dot", "f32", a, b, md)
    assert ctx.last_kernel() == "small_f32_KM"
    want = oracle.dot_asis("f32", a, b, md)  # sequential-k f32, the reference's fallback arithmetic
    _, o64, oabs = oracle.dot_spec("f32", "f32", a, b, md)
    H.assert_close(got, want.astype(np.float64), oabs, 512, 1e-5, "config 1 against the sequential-k f32 sum")
    H.assert_close(got, o64, oabs, 512, 1e-5, "config 1 against float64")
    # the OpenBLAS flavour of the reference (cblas_sgemm) through numpy's bundled OpenBLAS
    blas = (a.reshape(512, 512) @ b.reshape(512, 512)).ravel()
    H.assert_close(got, blas.astype(np.float64), oabs, 512, 1e-5, "config 1 against sgemm")


def test_config2_bf16_batched_transposed(ctx):
    B, n = 16, 1024
    a = H.f32_to_bf16_rne((H.rng(201).standard_normal(B * n * n) / 32).astype(np.float32))
    b = H.f32_to_bf16_rne((H.rng(202).standard_normal(B * n * n) / 32).astype(np.float32))
    lv, rv = V([B, n, n]), V([B, n, n]).t()  # rhs: transposed view of contiguous [B, N, K]
    got = run_product(ctx, "matmul", "bf16", a, b, H.matmul_md(lv, rv)).reshape(B, n, n)
    assert ctx.last_kernel().startswith("mfma_bf16_") and "256x256" in ctx.last_kernel() and ctx.last_kernel().endswith("_KK")
    for bi in (0, 7, 15):
        rows = V([n, n], offset=bi * n * n).slice(0, 3, n, 97)
        md = H.dot_md(rows, V([n, n], offset=bi * n * n).t())
        check_rows(got[bi, 3::97].ravel(), "bf16", "bf16", a, b, md, n, 2e-2)


@pytest.mark.parametrize("top", [448.0, 240.0])
@pytest.mark.parametrize("m", [1, 16, 256, 4096])
def test_config3_fp8_weight_linear(ctx, m, top):
    n = k = 4096
    w, _ = fp8_weights(n, k, 301, top)
    x = H.f32_to_bf16_rne(H.rng(302).standard_normal(m * k).astype(np.float32))
    lv, wt = V([m, k]), V([n, k]).t()  # linear idiom: W stored [N, K], passed transposed
    got = run_product(ctx, "dot", "bf16_f8e4m3w", x, w, H.dot_md(lv, wt)).reshape(m, n)
    want = "gemv_bf16_f8w" if m <= 4 else "skinny_bf16_f8w_splitk" if m <= 16 else "mfma_bf16_f8w"
    assert ctx.last_kernel().startswith(want), ctx.last_kernel()
    step = max(1, m // 24)
    rows = lv.slice(0, 0, m, step)
    check_rows(got[::step].ravel(), "bf16", "f8e4m3", x, w, H.dot_md(rows, wt), k, 2e-2)
    if m == 16:
        # second orientation: W stored [K, N] contiguous
        wkn = np.ascontiguousarray(w.reshape(n, k).T).ravel()
        got2 = run_product(ctx, "dot", "bf16_f8e4m3w", x, wkn, H.dot_md(lv, V([k, n]))).reshape(m, n)
        check_rows(got2.ravel(), "bf16", "f8e4m3", x, wkn, H.dot_md(lv, V([k, n])), k, 2e-2)
        # fused vs unfused (to_dtype(bf16) on the device, then the plain bf16 product): the widening is
        # exact, so the two differ only by f32 summation order, i.e. by at most one bf16 rounding step
        dw = ctx.upload(w); wb = ctx.alloc(n * k * 2); dx = ctx.upload(x); out = ctx.alloc(m * n * 2)
        ctx.cast("f8e4m3", "bf16", dw, wb, H.cast_md(V([n, k])))
        ctx.product("dot", "bf16", dx, wb, out, H.dot_md(lv, wt))
        unfused = ctx.download(out, np.uint16).reshape(m, n)
        fu, ff = H.bf16_to_f32(unfused).astype(np.float64), H.bf16_to_f32(got).astype(np.float64)
        assert np.all(np.abs(fu - ff) <= 2.0 ** -7 * np.maximum(np.abs(ff), 1.0))
        check_rows(unfused.ravel(), "bf16", "f8e4m3", x, w, H.dot_md(lv, wt), k, 2e-2)


def test_config4_int8_valued_i32(ctx):
    n = 2048
    a8 = H.rng(401).integers(-127, 128, n * n).astype(np.int8)
    b8 = H.rng(402).integers(-127, 128, n * n).astype(np.int8)
    md = H.dot_md(V([n, n]), V([n, n]))
    # exact: |sum| <= 127^2 * 2048 < 2^25, so float64 BLAS reproduces the integer result
    want = (a8.reshape(n, n).astype(np.float64) @ b8.reshape(n, n).astype(np.float64)).astype(np.int32).ravel()
    fused = run_product(ctx, "dot", "i32_i8i8", a8, b8, md)
    assert ctx.last_kernel().startswith("mfma_i32_i8i8")
    assert np.array_equal(fused, want)
    # unfused path of the API: to_dtype(i32) twice on the device, then the i32 product
    da, db = ctx.upload(a8), ctx.upload(b8)
    a32, b32, out = ctx.alloc(n * n * 4), ctx.alloc(n * n * 4), ctx.alloc(n * n * 4)
    ctx.cast("i8", "i32", da, a32, H.cast_md(V([n, n])))
    ctx.cast("i8", "i32", db, b32, H.cast_md(V([n, n])))
    ctx.product("dot", "i32", a32, b32, out, md)
    assert np.array_equal(ctx.download(out, np.int32), want)
    # and the oracle's reference-faithful i32 arithmetic on a row subset
    rows = V([n, n]).slice(0, 5, n, 211)
    sub = oracle.dot_asis("i32", a8.astype(np.int32), b8.astype(np.int32), H.dot_md(rows, V([n, n])))
    assert np.array_equal(fused.reshape(n, n)[5::211].ravel(), sub)


@pytest.mark.parametrize("wkind", ["bf16", "f8e4m3"])
def test_config5_mlp_broadcast(ctx, wkind):
    b, s, d, f = 8, 512, 4096, 14336
    x = H.f32_to_bf16_rne(H.rng(501).standard_normal(b * s * d).astype(np.float32))
    if wkind == "bf16":
        w_up = H.f32_to_bf16_rne((H.rng(502).standard_normal(d * f) * 0.02).astype(np.float32))
        w_down = H.f32_to_bf16_rne((H.rng(503).standard_normal(d * f) * 0.02).astype(np.float32))
        name, r_dt, prefix = "bf16", "bf16", "mfma_bf16_"
    else:
        w_up, _ = fp8_weights(d, f, 502)
        w_down, _ = fp8_weights(d, f, 503)
        name, r_dt, prefix = "bf16_f8e4m3w", "f8e4m3", "mfma_bf16_f8w_"
    # up: [8,512,4096] x [4096,14336] (weight broadcast over the batch with stride 0)
    xv = V([b, s, d])
    up_v = V([d, f]).broadcast_to([b, d, f])
    y = run_product(ctx, "matmul", name, x, w_up, H.matmul_md(xv, up_v))
    assert ctx.last_kernel().startswith(prefix) and "256x256" in ctx.last_kernel() and ctx.last_kernel().endswith("_KM"), ctx.last_kernel()
    rows = V([b * s, d]).slice(0, 7, b * s, 311)
    check_rows(y.reshape(b * s, f)[7::311].ravel(), "bf16", r_dt, x, w_up, H.dot_md(rows, V([d, f])), d, 2e-2)
    # down: Y [8,512,14336] x W_down, stored [4096,14336] and passed as a transposed, broadcast view
    yv = V([b, s, f])
    down_v = V([d, f]).t().broadcast_to([b, f, d])
    z = run_product(ctx, "matmul", name, y, w_down, H.matmul_md(yv, down_v))
    assert ctx.last_kernel().startswith(prefix) and "256x256" in ctx.last_kernel() and ctx.last_kernel().endswith("_KK"), ctx.last_kernel()
    rows = V([b * s, f]).slice(0, 11, b * s, 409)
    check_rows(z.reshape(b * s, d)[11::409].ravel(), "bf16", r_dt, y, w_down, H.dot_md(rows, V([d, f]).t()), f, 2e-2)
