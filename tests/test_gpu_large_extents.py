"""Extents past 2^31 elements and 4 GiB: an MI355X holds 288 GB, so a product's output, one of its operands, a cast or a
reduction can be larger than 32-bit element counts and byte offsets reach.  Inputs come from a hash of the element's index
(cheap to make in pieces, and a wrapped address reads different values), results are checked where wrapping would show:
the first rows, the rows either side of the 2^31-element and 2^32-byte marks, the last rows."""
import numpy as np
import pytest

import helpers as H
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View
COLS, Q = 4096, 1027
PERIOD = COLS * Q  # elements after which the inputs repeat: has an odd factor, so an address that wraps at a power
                   # of two lands in a different phase of the pattern


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def hashed(first, count):
    """16 well-mixed bits per index"""
    i = np.arange(first, first + count, dtype=np.uint64)
    return ((i * np.uint64(0x9E3779B97F4A7C15)) >> np.uint64(48)).astype(np.uint16)


def bf16_bits(first, count):
    """bf16 values of either sign with magnitudes in [2^-7, 2)"""
    return np.uint16(0x3C00) | (hashed(first, count) & np.uint16(0x83FF))


def f8_bits(first, count):
    """f8e4m3 bytes of either sign, exponent field 4..7 (no NaN pattern)"""
    return (np.uint8(0x20) | (hashed(first, count) & np.uint16(0x9F)).astype(np.uint8))


def fill_periodic(ctx, buf, period, n):
    """element i of the buffer = period[i % len(period)]"""
    size = period.itemsize
    for first in range(0, n, len(period)):
        count = min(len(period), n - first)
        ctx.upload_into(buf, period[:count], first * size)


def take_periodic(period, first, count):
    return period[(first + np.arange(count, dtype=np.int64)) % len(period)]


def test_output_past_2_31_elements(ctx):
    m = n = 46400  # 2.153e9 outputs, 4.3 GB of bf16
    k = 64
    assert m * n > 2 ** 31
    a, b = bf16_bits(0, m * k), bf16_bits(1 << 40, n * k)
    da, db, out = ctx.upload(a), ctx.upload(b), ctx.alloc(m * n * 2)
    ctx.fill(out, 0xFF)
    ctx.product("dot", "bf16", da, db, out, H.dot_md(V([m, k]), V([n, k]).t()))
    assert ctx.last_kernel().startswith("mfma_bf16")
    af, bf = H.widen("bf16", a).reshape(m, k), H.widen("bf16", b).reshape(n, k)
    rows = [0, 1, 255, 256, 23199, (2 ** 31) // n - 1, (2 ** 31) // n, (2 ** 31) // n + 1, m - 257, m - 2, m - 1]
    for r in rows:
        got = H.widen("bf16", ctx.download(out, np.uint16, n, first=r * n))
        want, sumabs = af[r] @ bf.T, np.abs(af[r]) @ np.abs(bf).T
        H.assert_close(got, want, sumabs, k, 2e-2, f"row {r}")
    for x in (da, db, out):
        x.free()


def test_operand_past_4_gib(ctx):
    m, k, n = 33000, 65600, 64  # 2.165e9 elements, 4.33 GB of bf16 on the left
    assert m * k > 2 ** 31
    period = bf16_bits(0, PERIOD)
    da = ctx.alloc(m * k * 2)
    fill_periodic(ctx, da, period, m * k)
    b = bf16_bits(1 << 41, n * k)
    db, out = ctx.upload(b), ctx.alloc(m * n * 2)
    ctx.fill(out, 0xFF)
    ctx.product("dot", "bf16", da, db, out, H.dot_md(V([m, k]), V([n, k]).t()))
    assert ctx.last_kernel().startswith("mfma_bf16")
    got = H.widen("bf16", ctx.download(out, np.uint16)).reshape(m, n)
    assert np.all(np.isfinite(got))
    bf = H.widen("bf16", b).reshape(n, k)
    r31, r32 = (2 ** 31) // k, (2 ** 32) // (2 * k)  # rows holding element 2^31 and byte 2^32
    for r in [0, 1, r31 - 1, r31, r31 + 1, 16384, 32767, r32 - 1, r32, r32 + 1, m - 2, m - 1]:
        ar = H.widen("bf16", take_periodic(period, r * k, k))
        want, sumabs = bf @ ar, np.abs(bf) @ np.abs(ar)
        H.assert_close(got[r], want, sumabs, k, 2e-2, f"row {r}")
    for x in (da, db, out):
        x.free()


def test_cast_and_sum_past_2_31_elements(ctx):
    n = 2 ** 31 + COLS * 3
    period = f8_bits(0, PERIOD)
    src = ctx.alloc(n)
    fill_periodic(ctx, src, period, n)
    dst = ctx.alloc(n * 2)
    ctx.fill(dst, 0xFF)
    ctx.cast("f8e4m3", "bf16", src, dst, H.cast_md(V([n])))
    for first, count in ((0, 4096), (2 ** 30 - 2048, 4096), (2 ** 31 - 2048, 4096), (n - 4096, 4096)):
        got = ctx.download(dst, np.uint16, count, first=first)
        want = H.f32_to_bf16_rne(H.widen("f8e4m3", take_periodic(period, first, count)).astype(np.float32))
        assert np.array_equal(got, want), f"cast at {first}"
    # the converted tensor as [rows, 4096]: sum over the rows (every output adds 2^19 values from all over the buffer)
    # against float64 sums of the same values -- the pattern repeats every Q rows, so whole periods add up in closed
    # form (f32 accumulation, one rounding: the 2e-2 bar of bf16)
    rows = n // COLS
    out = ctx.alloc(COLS * 2)
    ctx.sum("bf16", dst, out, H.reduce_md(V([rows, COLS]), [0], False))
    got = H.widen("bf16", ctx.download(out, np.uint16))
    v = H.widen("f8e4m3", period).reshape(Q, COLS)
    want = (rows // Q) * v.sum(0) + v[:rows % Q].sum(0)
    sumabs = (rows // Q) * np.abs(v).sum(0) + np.abs(v[:rows % Q]).sum(0)
    H.assert_close(got, want, sumabs, rows, 2e-2, "sum over 2^19 rows")
    for x in (src, dst, out):
        x.free()
