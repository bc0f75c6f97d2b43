"""GPU parity of hodu_rocm_softmax against the one-pass comparator (f32 / f64 softmax of exactly widened inputs, pinned
in tests/test_oracle_golden.py and against the reference's five-kernel chain in tests/test_oracle_ref.py).
Tolerances: f32 outputs 1e-5 relative, bf16 / f16 outputs 2e-2 relative (one RNE rounding of the f32 value is 2^-9 /
2^-11), f64 1e-12; an absolute floor covers outputs below the format's normal range (f16: one subnormal step, 2^-24;
the others 1e-30).  Masked entries must be exact
zeros and every row must sum to one within the output format's rounding."""
import numpy as np
import pytest

import helpers as H
import oracle
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View
TOL = {"f32": 1e-5, "bf16": 2e-2, "f16": 2e-2, "f64": 1e-12}
FLOOR = {"f32": 1e-30, "bf16": 1e-30, "f16": 2.0 ** -24, "f64": 1e-30}


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def check_softmax(ctx, dt, v, dim, causal=False, seed=0, scale=3.0, expect_kernel=None):
    x = H.random_storage(dt, v.span(), 900 + seed, scale)
    md = H.reduce_md(v, [dim], True)
    n = v.size
    dx, dout = ctx.upload(x), ctx.alloc(n * ffi.DTYPE_SIZE[dt])
    ctx.fill(dout, 0xFF)
    ctx.softmax(dt, dx, dout, md, causal)
    if expect_kernel is not None:
        assert ctx.last_kernel().startswith(expect_kernel), (ctx.last_kernel(), expect_kernel)
    got = H.widen(dt, ctx.download(dout, oracle.STORAGE[dt], n))
    dx.free(); dout.free()
    o32, o64 = oracle.softmax_spec(dt, x, md, causal)
    want = o64
    assert np.all(np.isfinite(got))
    assert np.all(got[want == 0.0] == 0.0)  # masked entries
    err = np.abs(got - want)
    assert np.all(err <= TOL[dt] * np.abs(want) + FLOOR[dt]), f"softmax {dt}: max rel err {(err / np.maximum(np.abs(want), FLOOR[dt])).max():.3e}"
    sums = got.reshape(v.shape).sum(axis=dim)
    assert np.allclose(sums, 1.0, atol=4 * TOL[dt])


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_rows_in_registers(ctx, dt):
    for n, length in enumerate((1, 7, 64, 128, 129, 500, 1024, 2047, 4096)):
        check_softmax(ctx, dt, V([3, 5, length]), 2, seed=n, expect_kernel="softmax_row")
    check_softmax(ctx, dt, V([2, 4, 9, 33]), -1 % 4, seed=20, expect_kernel="softmax_row")
    assert ctx.last_kernel() == "softmax_row"       # 33 entries: no whole 16-byte vectors
    check_softmax(ctx, dt, V([7, 512]), 1, seed=21, expect_kernel="softmax_row_vec")
    check_softmax(ctx, dt, V([7, 4096]), 1, seed=22, expect_kernel="softmax_row_vec")
    check_softmax(ctx, dt, V([7, 512], offset=3), 1, seed=23, expect_kernel="softmax_row")
    assert ctx.last_kernel() == "softmax_row"       # misaligned base


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_short_rows_share_a_wavefront(ctx, dt):
    """rows of at most 16 (32) vectors are handled 4 (2) to a wavefront; row counts that leave a wavefront or a
    workgroup partly empty"""
    for n, (rows, length) in enumerate(((1, 8), (37, 64), (101, 128), (9, 256), (1030, 32), (5, 16))):
        check_softmax(ctx, dt, V([rows, length]), 1, seed=60 + n, expect_kernel="softmax_row_vec")
    check_softmax(ctx, dt, V([3, 50, 64]), 2, causal=True, seed=70, expect_kernel="softmax_row_vec")


@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_causal_mask(ctx, dt):
    """attention.rs:40-48 with create_causal_mask (:73-86): row i of each [Sq, Sk] matrix keeps entries j <= i"""
    check_softmax(ctx, dt, V([2, 3, 64, 64]), 3, causal=True, seed=30, expect_kernel="softmax_row")
    check_softmax(ctx, dt, V([4, 37, 200]), 2, causal=True, seed=31)   # Sq < Sk
    check_softmax(ctx, dt, V([4, 200, 37]), 2, causal=True, seed=32)   # Sq > Sk: rows beyond Sk see everything
    check_softmax(ctx, dt, V([16, 1024, 1024]), 2, causal=True, seed=33, scale=1.0)


@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_long_and_strided_rows(ctx, dt):
    check_softmax(ctx, dt, V([3, 5000]), 1, seed=40, expect_kernel="softmax_long_vec")     # a workgroup per row
    check_softmax(ctx, dt, V([2, 4099]), 1, seed=44, expect_kernel="softmax_long")         # no whole vectors
    check_softmax(ctx, dt, V([3, 40000]), 1, seed=45, scale=3.0, expect_kernel="softmax_long_vec")
    check_softmax(ctx, dt, V([2, 3, 5000], offset=8).t(0, 1), 2, seed=46, expect_kernel="softmax_long_vec")
    check_softmax(ctx, dt, V([2, 6000, 6000]), 2, causal=True, seed=47, expect_kernel="softmax_long_vec")
    check_softmax(ctx, dt, V([6, 90]).slice(1, 1, 90, 3), 1, seed=41, expect_kernel="softmax_strided")
    check_softmax(ctx, dt, V([5, 8, 40], offset=3).t(0, 1), 2, seed=42, expect_kernel="softmax_row")  # rows still dense
    check_softmax(ctx, dt, V([6, 50]).slice(1, 0, 50, 2), 1, causal=True, seed=43, expect_kernel="softmax_strided")


def test_large_logits_do_not_overflow(ctx):
    check_softmax(ctx, "f32", V([8, 300]), 1, seed=50, scale=200.0)
    check_softmax(ctx, "bf16", V([8, 300]), 1, seed=51, scale=200.0)


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_other_dims(ctx, dt):
    """softmax along a dim that is not the last one: a thread per position of the other dims"""
    check_softmax(ctx, dt, V([8, 8]), 0, seed=80, expect_kernel="softmax_cols")
    check_softmax(ctx, dt, V([3, 50, 70]), 1, seed=81, expect_kernel="softmax_cols")
    check_softmax(ctx, dt, V([5, 300, 2, 9]), 1, seed=82, expect_kernel="softmax_cols")
    check_softmax(ctx, dt, V([1000, 33]), 0, seed=83, scale=20.0, expect_kernel="softmax_cols")
    check_softmax(ctx, dt, V([4, 6, 40], offset=5).t(0, 2), 1, seed=84, expect_kernel="softmax_cols")   # strided input
    check_softmax(ctx, dt, V([7, 9, 1]), 1, seed=85, expect_kernel="softmax_row")                        # nothing after it


def test_rejected_calls(ctx):
    x, out = ctx.upload(np.zeros(64, np.float32)), ctx.alloc(256)
    with pytest.raises(ffi.HoduRocmError, match="causal"):
        ctx.softmax("f32", x, out, H.reduce_md(V([8, 8]), [0], True), causal=True)
    with pytest.raises(ffi.HoduRocmError, match="exactly one dim"):
        ctx.softmax("f32", x, out, H.reduce_md(V([8, 8]), [0, 1], True))
    with pytest.raises(ffi.HoduRocmError, match="causal"):
        ctx.softmax("f32", x, out, H.reduce_md(V([64]), [0], True), causal=True)
    xi = ctx.upload(np.zeros(64, np.int32))
    with pytest.raises(ffi.HoduRocmError, match="dtype"):
        ctx.softmax("i32", xi, out, H.reduce_md(V([8, 8]), [1], True))
    for d in (x, out, xi):
        d.free()
