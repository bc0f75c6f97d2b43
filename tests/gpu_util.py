"""Helpers for the GPU parity tests: everything goes through the C ABI (hodu_amd.ffi)."""
import numpy as np

import helpers as H
import oracle
from hodu_amd import ffi

OUT_STORAGE = dict(oracle.STORAGE)
FUSED = {
    # name -> (lhs storage dtype, rhs storage dtype, out dtype)
    "bf16_f8e4m3w": ("bf16", "f8e4m3", "bf16"),
    "i32_i8i8": ("i8", "i8", "i32"),
}

# unit round-off of the format a result is delivered in
FLOAT_TOL = {"bf16": 2e-2, "f16": 2e-2, "f8e4m3": None, "f8e5m2": None, "f32": 1e-5, "f64": 1e-12}


def dtypes_of(name):
    if name in FUSED:
        return FUSED[name]
    return name, name, name


def run_product(ctx, op, name, a, b, md):
    """Runs hodu_rocm_<op>_<name>; the output buffer is pre-filled with 0xFF bytes (NaN for every
    float format) so an element the kernel failed to write is caught."""
    _, _, out_dt = dtypes_of(name)
    n = int(md[0]) if op == "matmul" else int(md[0]) * int(md[2])
    da, db = ctx.upload(a), ctx.upload(b)
    dout = ctx.alloc(max(n, 1) * ffi.DTYPE_SIZE[out_dt])
    ctx.fill(dout, 0xFF)
    ctx.product(op, name, da, db, dout, md)
    got = ctx.download(dout, OUT_STORAGE[out_dt], n)
    for d in (da, db, dout):
        d.free()
    return got


def check_product(ctx, op, name, lv, rv, seed=0, scale=1.0, rscale=None, expect_kernel=None):
    """One parity case: seeded inputs -> HIP path through the C ABI -> compare with the oracle.
    Integers: bit-exact against the reference-faithful (ASIS) oracle.
    Floats:   per-element relative error against the f32-accumulated (SPEC) oracle, tolerance by
              output format (bf16/f16 2e-2, f32 1e-5), denominator floor as documented in
              helpers.rel_err; no NaN/inf where the oracle has none."""
    l_dt, r_dt, out_dt = dtypes_of(name)
    a = H.random_storage(l_dt, max(lv.span(), 1), 1000 + seed, scale)
    b = H.random_storage(r_dt, max(rv.span(), 1), 2000 + seed, scale if rscale is None else rscale)
    md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
    got = run_product(ctx, op, name, a, b, md)
    if expect_kernel is not None:
        assert ctx.last_kernel().startswith(expect_kernel), (ctx.last_kernel(), expect_kernel)
    k = lv.shape[-1]
    if out_dt in ("i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64"):
        if name == "i32_i8i8":
            want = (oracle.dot_asis if op == "dot" else oracle.matmul_asis)("i32", a.astype(np.int32), b.astype(np.int32), md)
        else:
            want = (oracle.dot_asis if op == "dot" else oracle.matmul_asis)(name, a, b, md)
        assert np.array_equal(got, want), f"{op} {name}: integer result differs"
        return
    if out_dt == "f64":
        # f64 has no narrower comparator: sequential-k f64 (the reference's own arithmetic) and
        # sum|a b| from numpy
        want = (oracle.dot_asis if op == "dot" else oracle.matmul_asis)("f64", a, b, md)
        bshape = list(np.broadcast_shapes(tuple(lv.shape[:-2]), tuple(rv.shape[:-2])))
        A = np.abs(lv.broadcast_to(bshape + lv.shape[-2:]).take(a)); B = np.abs(rv.broadcast_to(bshape + rv.shape[-2:]).take(b))
        oabs = (A @ B).ravel()
        assert np.all(np.isfinite(got))
        H.assert_close(got, want, oabs, k, 1e-12, f"{op} f64", eps_acc=H.EPS_F64)
        return
    fn = oracle.dot_spec if op == "dot" else oracle.matmul_spec
    o32, o64, oabs = fn(l_dt, r_dt, a, b, md)
    gotf = H.widen(out_dt, got)
    assert np.array_equal(np.isfinite(gotf), np.isfinite(o64)), f"{op} {name}: non-finite pattern differs"
    fin = np.isfinite(o64)
    if out_dt in ("f8e4m3", "f8e5m2"):
        # delivered in an 8-bit float: within one rounding step (2^-3 / 2^-2 relative) of the
        # f32-accumulated value, saturating at the largest finite code
        step = 2.0 ** -3 if out_dt == "f8e4m3" else 2.0 ** -2
        lim = 448.0 if out_dt == "f8e4m3" else 57344.0
        want = np.clip(o64, -lim, lim)
        err = np.abs(gotf - want)[fin]
        tiny = 2.0 ** -9 if out_dt == "f8e4m3" else 2.0 ** -16
        assert np.all(err <= step * np.abs(want[fin]) + tiny + 1e-3 * oabs[fin] / np.sqrt(k)), f"{op} {name}"
        return
    tol = FLOAT_TOL[out_dt]
    # (a sequential f32 sum over more than a few thousand k is itself off by about sqrt(k) * 2^-24 relative to the
    # floor: products with a very long K, which the device adds in chunks, are held to the float64 value)
    want = o64 if (out_dt == "f64" or (out_dt == "f32" and k > 16384)) else o32.astype(np.float64)
    if out_dt == "f16":
        # f16 subnormals are 2^-24 apart: an output below 2^-14 that lies within half a step of the value is the
        # correctly rounded one, whatever its relative error
        settled = (np.abs(want) < 2.0 ** -14) & (np.abs(gotf - want) <= 2.0 ** -25)
        gotf = np.where(settled, want, gotf)
    H.assert_close(gotf[fin], want[fin], oabs[fin], k, tol, f"{op} {name}")
