"""GPU parity: to_dtype casts and contiguous through the C ABI, bit-exact against the CPU oracle
and against the fixtures written from the reference's own C kernels."""
import os

import numpy as np
import pytest

import helpers as H
import oracle
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


def gpu_cast(ctx, src, dst, x, md):
    dx = ctx.upload(x)
    n = int(md[0])
    out = ctx.alloc(max(n, 1) * ffi.DTYPE_SIZE[dst])
    ctx.fill(out, 0xA5)
    if src == "contiguous":
        ctx.contiguous(dst, dx, out, md)
    else:
        ctx.cast(src, dst, dx, out, md)
    got = ctx.download(out, oracle.STORAGE[dst], n)
    dx.free(); out.free()
    return got


def same(got, want, dst):
    if dst in ("f32", "f64"):
        nan = np.isnan(want)
        return np.array_equal(np.isnan(got), nan) and np.array_equal(_bits(got[~nan]), _bits(want[~nan]))
    return np.array_equal(_bits(got), _bits(want))


def in_domain(src, dst, x):
    """keeps inputs where the reference's C conversion is defined (see oracle header)"""
    if dst[0] == "u" or dst == "bool":
        if src in ("f32", "f64"):
            return np.abs(x)
        if src in ("bf16", "f16"):
            return x & 0x7FFF
        if src in ("f8e4m3", "f8e5m2"):
            return x & 0x7F
    return x


def test_every_cast_pair_matches_oracle_dense_and_strided(ctx):
    views = [V([1031]), V([7, 9, 5], offset=3).t(0, 2), V([1, 9]).broadcast_to([5, 9]), V([6, 10, 12], offset=7).slice(2, 1, 11, 3)]
    for v in views:
        md = H.cast_md(v)
        for src in oracle.DTYPE_ID:
            for dst in oracle.DTYPE_ID:
                x = in_domain(src, dst, H.random_storage(src, v.span(), 77, 3.0))
                want = oracle.cast(src, dst, x, md, decode=oracle.F8_OCP)
                assert same(gpu_cast(ctx, src, dst, x, md), want, dst), (src, dst, v.shape)


def test_cast_golden_fixtures(ctx):
    gold = np.load(os.path.join(GOLD, "casts.npz"))
    for entry in gold["index"]:
        key, src, dst = entry.split("|")
        x, md, want = gold[key + "__in"], gold[key + "__md"].tolist(), gold[key + "__out"]
        got = gpu_cast(ctx, src, dst, x, md)
        if src == "f8e4m3":
            # the 14 exponent-15 codes decode as OCP on the GPU (finite) and as inf/NaN in the
            # reference's C decoder: compare everywhere else
            pos = H.View(md[2:2 + md[1]], md[2 + md[1]:2 + 2 * md[1]], md[-1]).take(x).ravel()
            keep = (pos & 0x78) != 0x78
            assert same(got[keep], want[keep], dst), key
        else:
            assert same(got, want, dst), key


def test_scalar_tables_match_reference_fixtures(ctx):
    t = np.load(os.path.join(GOLD, "tables.npz"))
    one = lambda n: H.cast_md(V([n]))  # noqa: E731
    h = np.arange(65536, dtype=np.uint16)
    x = t["f32_samples"].view(np.float32)
    for name, src, dst, inp in [("f16_to_f32", "f16", "f32", h), ("bf16_to_f16", "bf16", "f16", h),
                                ("bf16_to_f8e4m3", "bf16", "f8e4m3", h), ("bf16_to_f8e5m2", "bf16", "f8e5m2", h),
                                ("f16_to_f8e4m3", "f16", "f8e4m3", h), ("f32_to_bf16", "f32", "bf16", x),
                                ("f32_to_f16", "f32", "f16", x), ("f32_to_f8e4m3", "f32", "f8e4m3", x),
                                ("f32_to_f8e5m2", "f32", "f8e5m2", x)]:
        want = t[name]
        want = want.view(np.float32) if dst == "f32" else want
        assert same(gpu_cast(ctx, src, dst, inp, one(inp.size)), want, dst), name
    # f8e4m3 decode: OCP on the device
    codes = np.arange(256, dtype=np.uint8)
    got = gpu_cast(ctx, "f8e4m3", "f32", codes, one(256))
    assert same(got, oracle.f8e4m3_table(oracle.F8_OCP), "f32")
    ref = t["f8e4m3_to_f32"].view(np.float32)
    agree = (codes & 0x78) != 0x78
    assert np.array_equal(got[agree].view(np.uint32), ref[agree].view(np.uint32))


def test_reference_known_answers_casts(ctx):
    # crates/hodu_cuda_kernels/tests/ops_cast.rs:48-89
    one = lambda n: [n, 1, n, 1, 0]  # noqa: E731
    assert gpu_cast(ctx, "f32", "i32", np.array([1.5, -2.7, 3.2, -4.9], np.float32), one(4)).tolist() == [1, -2, 3, -4]
    assert gpu_cast(ctx, "i32", "f32", np.array([1, -2, 3, -4], np.int32), one(4)).tolist() == [1.0, -2.0, 3.0, -4.0]
    assert gpu_cast(ctx, "f32", "u32", np.array([1.5, 2.7, 3.2, 4.9], np.float32), one(4)).tolist() == [1, 2, 3, 4]
    assert gpu_cast(ctx, "u32", "f32", np.array([1, 2, 3, 4], np.uint32), one(4)).tolist() == [1.0, 2.0, 3.0, 4.0]
    x64 = np.array([1.5, 2.7, 3.2, 4.9])
    assert np.array_equal(gpu_cast(ctx, "f64", "f32", x64, one(4)), x64.astype(np.float32))


def test_contiguous_all_sizes(ctx):
    for v in (V([4099]), V([130, 70]).t(), V([4, 5, 6], offset=2).slice(1, 1, 5, 2), V([3, 1, 8]).broadcast_to([3, 4, 8])):
        for dt in ("u8", "bf16", "f32", "i64", "f8e4m3", "bool"):
            x = H.random_storage(dt, v.span(), 5)
            assert same(gpu_cast(ctx, "contiguous", dt, x, H.cast_md(v)), oracle.contiguous(dt, x, H.cast_md(v)), dt)


def test_transposed_views_go_through_the_tiled_kernel(ctx):
    """a view whose unit stride is not on the last dim (a transpose, a permutation) is gathered in 64 x 64 tiles
    through LDS: ragged tiles, several outer dims (one of them broadcast), an offset, casts that change the element size"""
    views = [V([130, 70]).t(), V([3, 65, 200], offset=5).t(1, 2), V([33, 4, 129]).t(0, 2),
             V([100, 48]).t().broadcast_to([3, 48, 100]), V([2, 3, 64, 64]).t(2, 3), V([17, 300]).t()]
    for n, v in enumerate(views):
        for dt in ("u8", "bf16", "f32", "i64"):
            x = H.random_storage(dt, v.span(), 40 + n)
            assert same(gpu_cast(ctx, "contiguous", dt, x, H.cast_md(v)), oracle.contiguous(dt, x, H.cast_md(v)), dt), (n, dt)
            assert ctx.last_kernel().startswith("cast_transpose"), (n, dt, ctx.last_kernel())
        for src, dst in (("f8e4m3", "bf16"), ("i8", "i32"), ("f32", "bf16"), ("bf16", "f32"), ("f64", "i16")):
            x = H.random_storage(src, v.span(), 60 + n, 20.0)
            md = H.cast_md(v)
            assert same(gpu_cast(ctx, src, dst, x, md), oracle.cast(src, dst, x, md, decode=oracle.F8_OCP), dst), (n, src, dst)
            assert ctx.last_kernel().startswith("cast_transpose")
    # 8 bytes per lane where every address stays a multiple of the vector, one element per lane otherwise
    for v, dt, name in ((V([2, 3, 64, 64]).t(2, 3), "bf16", "cast_transpose_vec"), (V([256, 512]).t(), "u8", "cast_transpose_vec"),
                        (V([130, 70]).t(), "bf16", "cast_transpose"), (V([64, 64], offset=1).t(), "f32", "cast_transpose"),
                        (V([64, 64]).t(), "i64", "cast_transpose")):
        x = H.random_storage(dt, v.span(), 3)
        assert same(gpu_cast(ctx, "contiguous", dt, x, H.cast_md(v)), oracle.contiguous(dt, x, H.cast_md(v)), dt)
        assert ctx.last_kernel() == name, (dt, ctx.last_kernel(), name)
    # too thin for tiles, or the last dim already dense: the flat-index kernel
    for v in (V([8, 300]).t(), V([300, 8]).t(), V([40, 50]).slice(1, 0, 50, 2)):
        x = H.random_storage("bf16", v.span(), 9)
        assert same(gpu_cast(ctx, "contiguous", "bf16", x, H.cast_md(v)), oracle.contiguous("bf16", x, H.cast_md(v)), "bf16")
        assert ctx.last_kernel() == "cast_strided", ctx.last_kernel()


def test_config_sized_casts(ctx):
    """C3/C4-sized casts (16.8 M f8e4m3 -> bf16, 4.2 M i8 -> i32) against the oracle"""
    w = H.rng(301).integers(0, 256, 4096 * 4096, dtype=np.uint8)
    w[(w & 0x7F) == 0x7F] = 0x7E  # no NaN codes, so that bit patterns compare
    md = H.cast_md(V([4096, 4096]))
    assert np.array_equal(gpu_cast(ctx, "f8e4m3", "bf16", w, md), oracle.cast("f8e4m3", "bf16", w, md, decode=oracle.F8_OCP))
    a = H.rng(401).integers(-127, 128, 2048 * 2048).astype(np.int8)
    md = H.cast_md(V([2048, 2048]))
    assert np.array_equal(gpu_cast(ctx, "i8", "i32", a, md), a.astype(np.int32))
    # transposed view of the weight matrix, as Linear would cast it
    md = H.cast_md(V([2048, 2048]).t())
    assert np.array_equal(gpu_cast(ctx, "i8", "i32", a, md).reshape(2048, 2048), a.reshape(2048, 2048).T.astype(np.int32))
