"""GPU parity of the bandwidth-bound M <= 16 path (decode-shape GEMV) through the C ABI."""
import pytest

import helpers as H
from gpu_util import check_product
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View
KINDS = {"bf16_f8e4m3w": "skinny_bf16_f8w", "bf16": "skinny_bf16", "f16": "skinny_f16", "f32": "skinny_f32",
         "i32_i8i8": "skinny_i32_i8i8"}


GEMV_KINDS = {"bf16_f8e4m3w": "gemv_bf16_f8w", "bf16": "gemv_bf16"}


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


@pytest.fixture()
def no_gemv(ctx):
    """route M <= 4 products past the row-streaming GEMV kernel so that the MFMA skinny kernel is exercised"""
    ctx.force_tile(30)
    yield ctx
    ctx.force_tile(-1)


@pytest.mark.parametrize("kind", list(KINDS))
@pytest.mark.parametrize("m", [1, 3, 16])
def test_linear_idiom_weight_k_dense(no_gemv, kind, m):
    ctx = no_gemv
    rs = 2.0 if "f8" in kind else None
    # ragged N (not a multiple of 16), K leaves an uneven split over the 8 wavefronts
    check_product(ctx, "dot", kind, V([m, 1040]), V([203, 1040]).t(), seed=m, rscale=rs, expect_kernel=KINDS[kind])
    # short K (one load per wavefront at most), tiny N
    check_product(ctx, "dot", kind, V([m, 64]), V([5, 64]).t(), seed=10 + m, rscale=rs, expect_kernel=KINDS[kind])


@pytest.mark.parametrize("kind", list(KINDS))
def test_batched_rows_fold_or_stay_batched(no_gemv, kind):
    ctx = no_gemv
    rs = 2.0 if "f8" in kind else None
    # [4, 1, K] x shared weight: the batch folds into 4 rows
    check_product(ctx, "matmul", kind, V([4, 1, 256]), V([40, 256]).t().broadcast_to([4, 256, 40]), seed=1, rscale=rs,
                  expect_kernel=KINDS[kind])
    # per-batch weights: stays a batch of GEMVs
    check_product(ctx, "matmul", kind, V([3, 2, 256]), V([3, 40, 256]).t(), seed=2, rscale=rs, expect_kernel=KINDS[kind])
    # row-sliced weight (leading dimension > K) and an aligned offset
    check_product(ctx, "dot", kind, V([2, 512]).slice(1, 128, 384), V([24, 512], offset=64).slice(1, 64, 320).t(), seed=3,
                  rscale=rs, expect_kernel=KINDS[kind])


@pytest.mark.parametrize("kind", list(KINDS))
@pytest.mark.parametrize("shape", [35, 36, 37, 39])
def test_workgroup_shapes(ctx, kind, shape):
    """1, 2 or 4 blocks of 16 weight rows per workgroup, and (39) one block with the left operand read in place
    instead of staged in LDS: N ragged against all of them, M from 5 to 16"""
    rs = 2.0 if "f8" in kind else None
    ctx.force_tile(shape)
    try:
        for m in (5, 16):
            check_product(ctx, "dot", kind, V([m, 1040]), V([203, 1040]).t(), seed=m, rscale=rs, expect_kernel=KINDS[kind])
        check_product(ctx, "matmul", kind, V([3, 9, 256]), V([3, 40, 256]).t(), seed=2, rscale=rs, expect_kernel=KINDS[kind])
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("kind", list(KINDS))
def test_left_operand_too_large_for_lds(ctx, kind):
    """16 rows of 9216 k do not fit the staging buffer: the one-pass kernel reads its left fragments in place (the
    path hook value 39 pins at any size); K leaves an uneven split over the wavefronts, N is ragged"""
    rs = 2.0 if "f8" in kind else None
    check_product(ctx, "dot", kind, V([16, 9232]), V([40, 9232]).t(), seed=3, scale=0.5, rscale=rs, expect_kernel=KINDS[kind])
    check_product(ctx, "dot", kind, V([13, 18432]), V([21, 18432]).t(), seed=4, scale=0.5, rscale=rs, expect_kernel=KINDS[kind])


@pytest.mark.parametrize("kind", list(KINDS))
@pytest.mark.parametrize("m", [5, 16])
def test_split_k_across_workgroups(ctx, kind, m):
    """wide and deep products with 5..16 rows: 128 weight rows and one slice of K per workgroup, the last workgroup
    of a column block to arrive adds the slices; N ragged against 128, K ragged against the slice; run twice in a
    row (the arrival counters must be back at zero) and compared bit for bit"""
    rs = 2.0 if "f8" in kind else None
    ctx.force_tile(38)  # the automatic choice keeps products this small on the one-pass kernel
    try:
        for _ in range(2):
            check_product(ctx, "dot", kind, V([m, 2064]), V([1100, 2064]).t(), seed=m, rscale=rs,
                          expect_kernel=KINDS[kind] + "_splitk")
        # row-sliced operands at aligned offsets
        check_product(ctx, "dot", kind, V([m, 4096]).slice(1, 1024, 3072),
                      V([1030, 4096], offset=64).slice(1, 512, 2560).t(), seed=20 + m, rscale=rs,
                      expect_kernel=KINDS[kind] + "_splitk")
        # deep K: more slices than the last workgroup adds in one round of loads
        check_product(ctx, "dot", kind, V([m, 4224]), V([1030, 4224]).t(), seed=40 + m, rscale=rs,
                      expect_kernel=KINDS[kind] + "_splitk")
    finally:
        ctx.force_tile(-1)


def test_not_applicable_layouts_fall_through(ctx):
    # weight with n dense ([K, N] row-major): not this kernel's layout; still correct via the tile kernel
    check_product(ctx, "dot", "bf16_f8e4m3w", V([1, 256]), V([256, 64]), seed=4, rscale=2.0, expect_kernel="mfma_")
    # misaligned activation rows
    check_product(ctx, "dot", "bf16", V([2, 100], offset=1), V([32, 100]).t(), seed=5, expect_kernel="mfma_")


# ---- row-streaming GEMV kernel (M <= 4, bf16 activations, bf16 or f8e4m3 weights) ---------------------
@pytest.mark.parametrize("kind", list(GEMV_KINDS))
@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("rows", [-1, 31, 32, 33, 34])
def test_gemv_rowstream(ctx, kind, m, rows):
    rs = 2.0 if "f8" in kind else None
    name = GEMV_KINDS[kind]
    ctx.force_tile(rows)
    try:
        # ragged N (not a multiple of the rows per wavefront or per workgroup), ragged last 1 KB piece
        check_product(ctx, "dot", kind, V([m, 1040]), V([203, 1040]).t(), seed=m, rscale=rs, expect_kernel=name)
        # K shorter than one piece; tiny N
        check_product(ctx, "dot", kind, V([m, 64]), V([5, 64]).t(), seed=10 + m, rscale=rs, expect_kernel=name)
        # K longer than what a wavefront keeps in flight (several passes, ragged tail)
        check_product(ctx, "dot", kind, V([m, 4112]), V([37, 4112]).t(), seed=20 + m, rscale=rs, expect_kernel=name)
        # row-sliced weight and activations (leading dimension > K) at aligned offsets
        check_product(ctx, "dot", kind, V([m, 512]).slice(1, 128, 384), V([24, 512], offset=64).slice(1, 64, 320).t(),
                      seed=30 + m, rscale=rs, expect_kernel=name)
        if rows in (-1, 33):
            # more row groups than wavefronts in the grid: a wavefront walks up to three groups, the last round ragged
            # (from 4096 rows on this is the kernel chosen without a pin); K of one pass, of a long pass, of several
            check_product(ctx, "dot", kind, V([m, 1040]), V([5001, 1040]).t(), seed=40 + m, rscale=rs, expect_kernel=name + "_walk")
            check_product(ctx, "dot", kind, V([m, 4112]), V([4100, 4112]).t(), seed=50 + m, rscale=rs, expect_kernel=name + "_walk")
            check_product(ctx, "dot", kind, V([m, 8720]), V([4099, 8720]).t(), seed=60 + m, rscale=rs, expect_kernel=name + "_walk")
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("kind", list(GEMV_KINDS))
def test_gemv_batch_folding_and_fallbacks(ctx, kind):
    rs = 2.0 if "f8" in kind else None
    # [4, 1, K] x shared weight: the batch folds into 4 rows of one GEMV
    check_product(ctx, "matmul", kind, V([4, 1, 256]), V([40, 256]).t().broadcast_to([4, 256, 40]), seed=1, rscale=rs,
                  expect_kernel=GEMV_KINDS[kind])
    # per-batch weights: not one product; the MFMA skinny kernel takes it
    check_product(ctx, "matmul", kind, V([3, 2, 256]), V([3, 40, 256]).t(), seed=2, rscale=rs, expect_kernel=KINDS[kind])
    # K not a multiple of the 16-byte vector: falls through
    k = 72 if "f8" in kind else 68
    check_product(ctx, "dot", kind, V([1, k]), V([16, k]).t(), seed=3, rscale=rs, expect_kernel="")


ROWS_KINDS = {"bf16": ("gemv_rows_bf16", 4), "f16": ("gemv_rows_f16", 4), "f32": ("gemv_rows_f32", 16)}


@pytest.mark.parametrize("kind", list(ROWS_KINDS))
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 13, 16])
def test_row_dense_weight(ctx, kind, m):
    """x [m, K] times W stored [K, N] (N contiguous): the kernel that sums weight rows, K cut into chunks -- f32 up to 16
    rows, bf16 / f16 up to 4 (beyond, and for the other kinds, the tile kernels); K that leaves a ragged last chunk, N
    that leaves a partly empty last workgroup, a column-strided x"""
    name, m_max = ROWS_KINDS[kind]
    expect = name if m <= m_max else "mfma_"
    check_product(ctx, "dot", kind, V([m, 1000]), V([1000, 320]), seed=m, expect_kernel=expect)
    k = 2048 if kind == "f32" else 4096  # (f32 against the sequential-k oracle at 1e-5: the orders differ, keep K moderate)
    check_product(ctx, "dot", kind, V([m, k]), V([k, 1024]), seed=20 + m, expect_kernel=expect)
    check_product(ctx, "dot", kind, V([m, 200]).slice(1, 0, 200, 2), V([100, 64]), seed=40 + m, expect_kernel=expect)


@pytest.mark.parametrize("kind", list(ROWS_KINDS))
def test_row_dense_weight_views_and_fallbacks(ctx, kind):
    name, _ = ROWS_KINDS[kind]
    # a column slice of a wider weight (row pitch > N) at an aligned offset
    check_product(ctx, "dot", kind, V([4, 256]), V([256, 512], offset=64).slice(1, 64, 320), seed=1, expect_kernel=name)
    # N not a multiple of the 8-byte vector, a misaligned offset, a batch: other kernels take these
    check_product(ctx, "dot", kind, V([2, 256]), V([256, 100 + 3]), seed=2)
    assert not ctx.last_kernel().startswith("gemv_rows")
    check_product(ctx, "dot", kind, V([2, 256]), V([256, 128], offset=1), seed=3)
    assert not ctx.last_kernel().startswith("gemv_rows")
    check_product(ctx, "matmul", kind, V([3, 2, 256]), V([3, 256, 128]), seed=4)
    assert not ctx.last_kernel().startswith("gemv_rows")


def test_row_dense_weight_other_kinds_keep_the_tile_kernels(ctx):
    check_product(ctx, "dot", "bf16_f8e4m3w", V([1, 256]), V([256, 64]), seed=4, rscale=2.0, expect_kernel="mfma_")
    check_product(ctx, "dot", "i32_i8i8", V([2, 256]), V([256, 64]), seed=5, expect_kernel="mfma_")


def test_split_k_arrival_protocol_over_thousands_of_launches(ctx):
    """Config 3 at M = 16 (the automatic choice is the split-K kernel) 3072 times back to back over 48 weight buffers
    whose rows are rotated by a different amount each -- so a partial sum left over from the previous launch, or one
    read before its writer's store was visible, gives a different output -- into a ring of 64 output buffers, every one
    of them compared bit for bit with the one-pass kernel's result on the unrotated weight, stopping at the first
    mismatch."""
    import numpy as np
    m, n, k = 16, 4096, 4096
    x = H.random_storage("bf16", m * k, 71)
    w = H.random_storage("f8e4m3", n * k, 72, 30.0)
    md = H.dot_md(V([m, k]), V([n, k]).t())
    dx, dw = ctx.upload(x), ctx.upload(w)
    ref = ctx.alloc(m * n * 2)
    ctx.force_tile(36)
    try:
        ctx.product("dot", "bf16_f8e4m3w", dx, dw, ref, md)
        assert not ctx.last_kernel().endswith("_splitk")
    finally:
        ctx.force_tile(-1)
    base = ctx.download(ref, np.uint16).reshape(m, n)
    copies, ring = 48, 64
    shifts = [(128 * c + 16 * (c // 32)) % n for c in range(copies)]  # W_c[j] = W[(j + shift_c) % n]
    ws = []
    for s in shifts:
        buf = ctx.alloc(n * k)
        ctx._check(ctx.lib.hodu_rocm_memcpy_d2d(ctx.handle, buf.ptr, dw.ptr + s * k, (n - s) * k))
        if s:
            ctx._check(ctx.lib.hodu_rocm_memcpy_d2d(ctx.handle, buf.ptr + (n - s) * k, dw.ptr, s * k))
        ws.append(buf)
    outs = [ctx.alloc(m * n * 2) for _ in range(ring)]
    launch = 0
    try:
        for _ in range(3072 // ring):
            used = []
            for slot in range(ring):
                c = launch % copies
                ctx.product("dot", "bf16_f8e4m3w", dx, ws[c], outs[slot], md)
                used.append(c)
                launch += 1
            assert ctx.last_kernel() == "skinny_bf16_f8w_splitk"
            for slot, c in enumerate(used):
                got = ctx.download(outs[slot], np.uint16).reshape(m, n)
                want = np.roll(base, -shifts[c], axis=1)
                assert np.array_equal(got, want), f"launch {launch - ring + slot} (weight copy {c}) differs"
    finally:
        for b in [dx, dw, ref] + ws + outs:
            b.free()
