"""GPU parity of the MFMA tile kernels: every compiled variant (dtype kind x tile x load-mode pair)
is driven through the C ABI at ragged sizes and compared with the oracle."""
import numpy as np
import pytest

import helpers as H
from gpu_util import check_product
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View

KINDS = {
    # name: (kernel prefix, K multiple for the k-dense path, row multiple for the row-dense path)
    "bf16": ("mfma_bf16", 8, 8),
    "f16": ("mfma_f16", 8, 8),
    "f32": ("mfma_f32", 4, 4),
    "bf16_f8e4m3w": ("mfma_bf16_f8w", 8, 8),
    "i32_i8i8": ("mfma_i32_i8i8", 16, 8),
}
TILES = {0: "256x256w8", 1: "256x256", 2: "128x128", 3: "64x64"}


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.force_tile(-1)
    c.close()


def views(combo, M, K, N):
    lv = V([M, K]) if combo[0] == "K" else V([K, M]).t()
    rv = V([N, K]).t() if combo[1] == "K" else V([K, N])
    return lv, rv


@pytest.mark.parametrize("kind", list(KINDS))
@pytest.mark.parametrize("tile", [0, 1, 2, 3])
def test_every_variant_ragged(ctx, kind, tile):
    prefix, kmul, rmul = KINDS[kind]
    ctx.force_tile(tile)
    M, N = 296, 200  # not multiples of any tile
    # K = 400: full K steps (through the LDS-DMA path where the layout allows) and a ragged last one
    K = 400
    scale = 1.0
    for combo in ("KK", "KM", "MK", "MM"):
        lv, rv = views(combo, M, K, N)
        # the 8-wavefront variant exists for k-dense left operands only; others use the 4-wavefront one
        name = TILES[1] if (tile == 0 and combo[0] == "M") else TILES[tile]
        check_product(ctx, "dot", kind, lv, rv, seed=tile, scale=scale, rscale=2.0 if "f8" in kind else None,
                      expect_kernel=f"{prefix}_{name}_{combo}")
    ctx.force_tile(-1)


@pytest.mark.parametrize("kind", ["bf16", "f16", "f32", "i32_i8i8"])
@pytest.mark.parametrize("tile,name", [(10, "pipe256x256w8"), (11, "pipe256x256"), (12, "pipe128x128"), (13, "pipe64x64")])
def test_pipelined_kk_variants(ctx, kind, tile, name):
    """the software-pipelined kernel (both operands k-dense): 1 to 11 stages of 64 bytes, ragged M and N"""
    prefix = KINDS[kind][0]
    ctx.force_tile(tile)
    es = {"bf16": 2, "f16": 2, "f32": 4, "i32_i8i8": 1}[kind]
    for stages in (1, 2, 3, 4, 5, 11):
        K = stages * 128 // es
        check_product(ctx, "dot", kind, V([296, K]), V([200, K]).t(), seed=stages, expect_kernel=f"{prefix}_{name}_KK")
    # batched, with a row-sliced operand (leading dimension > K) and an offset
    K = 6 * 128 // es
    check_product(ctx, "matmul", kind, V([3, 72, 2 * K]).slice(2, K, 2 * K), V([3, 80, K], offset=64).t(), seed=7,
                  expect_kernel=f"{prefix}_{name}_KK")
    ctx.force_tile(-1)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
def test_pipelined_kk_16x16_instruction(ctx, kind):
    """the 256 x 256 tile on the 16 x 16 x 32 matrix instruction (two k-dense 16-bit operands): the shapes of
    test_pipelined_kk_variants"""
    prefix = KINDS[kind][0]
    ctx.force_tile(15)
    try:
        for stages in (1, 2, 3, 4, 5, 11):
            K = stages * 64
            check_product(ctx, "dot", kind, V([296, K]), V([200, K]).t(), seed=stages, expect_kernel=f"{prefix}_pipe256x256mi16_KK")
        K = 6 * 64
        check_product(ctx, "matmul", kind, V([3, 72, 2 * K]).slice(2, K, 2 * K), V([3, 80, K], offset=64).t(), seed=7,
                      expect_kernel=f"{prefix}_pipe256x256mi16_KK")
        check_product(ctx, "dot", kind, V([1000, 1024]), V([777, 1024]).t(), seed=8, expect_kernel=f"{prefix}_pipe256x256mi16_KK")
        # a row-dense right operand ([K, N] row-major, read through the LDS transpose): the shapes of
        # test_pipelined_row_dense_variants
        km = f"{prefix}_pipe256x256mi16_KM"
        for stages in (1, 2, 3, 5):
            K = stages * 64
            check_product(ctx, "dot", kind, V([19 * 16 - 8, K]), V([K, 13 * 16 - 8]), seed=stages, expect_kernel=km)
        check_product(ctx, "dot", kind, V([24, 128]), V([128, 40]), seed=9, expect_kernel=km)
        check_product(ctx, "matmul", kind, V([3, 72, 128], offset=64), V([128, 80], offset=128).broadcast_to([3, 128, 80]), seed=10,
                      expect_kernel=km)
        check_product(ctx, "dot", kind, V([72, 128]), V([128, 160]).slice(1, 16, 16 + 6 * 16), seed=11, expect_kernel=km)
        check_product(ctx, "dot", kind, V([1000, 512]), V([512, 776]), seed=12, expect_kernel=km)
        # a row-dense left operand (a transposed view), against both kinds of right operand
        for combo in ("MK", "MM"):
            name = f"{prefix}_pipe256x256mi16_{combo}"
            for stages in (1, 2, 3, 5):
                lv, rv = views(combo, 19 * 16 - 8, stages * 64, 13 * 16 - 8)
                check_product(ctx, "dot", kind, lv, rv, seed=stages, expect_kernel=name)
            lv, rv = views(combo, 24, 128, 40)
            check_product(ctx, "dot", kind, lv, rv, seed=9, expect_kernel=name)
            lv, rv = views(combo, 1000, 512, 776)
            check_product(ctx, "dot", kind, lv, rv, seed=13, expect_kernel=name)
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("kind", ["bf16", "f16", "i32_i8i8"])
@pytest.mark.parametrize("tile,name", [(10, "pipe256x256w8"), (11, "pipe256x256"), (12, "pipe128x128")])
@pytest.mark.parametrize("combo", ["KM", "MK", "MM"])
def test_pipelined_row_dense_variants(ctx, kind, tile, name, combo):
    """the pipelined kernel with row-dense operands (LDS transpose reads): 1 to 5 stages of 128 bytes of k; M
    and N ragged against every tile but multiples of the 16-byte row chunk, as the layout requires"""
    prefix = KINDS[kind][0]
    es = 1 if kind == "i32_i8i8" else 2
    epc = 16 // es
    ctx.force_tile(tile)
    try:
        for stages in (1, 2, 3, 5):
            K = stages * 128 // es
            lv, rv = views(combo, 19 * 16 - (0 if es == 1 else 8), K, 13 * 16 - (0 if es == 1 else 8))
            check_product(ctx, "dot", kind, lv, rv, seed=stages, expect_kernel=f"{prefix}_{name}_{combo}")
        # fewer rows than one tile, and a tile edge that cuts through a 16-column group
        lv, rv = views(combo, 3 * epc, 256 // es, 5 * epc)
        check_product(ctx, "dot", kind, lv, rv, seed=9, expect_kernel=f"{prefix}_{name}_{combo}")
        if combo == "KM":
            K = 256 // es
            # batched with a shared row-dense weight (stride-0 batch) and offsets into larger buffers
            check_product(ctx, "matmul", kind, V([3, 72, K], offset=64), V([K, 80], offset=128).broadcast_to([3, K, 80]),
                          seed=10, expect_kernel=f"{prefix}_{name}_{combo}")
            # column-sliced weight: leading dimension larger than N
            check_product(ctx, "dot", kind, V([72, K]), V([K, 160]).slice(1, 16, 16 + 6 * 16), seed=11,
                          expect_kernel=f"{prefix}_{name}_{combo}")
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("tile,name", [(10, "pipe256x256w8"), (11, "pipe256x256"), (12, "pipe128x128")])
@pytest.mark.parametrize("combo", ["KK", "KM"])
def test_pipelined_f8_weight_variants(ctx, tile, name, combo):
    """fused f8e4m3 weights in the pipelined kernel: raw bytes through LDS-DMA, widened between fragment read and
    MFMA.  k-dense weights move 128 k per buffer (pairs of stages: 1, 2, 3 and 5 pairs), row-dense ones 64 k-rows
    per stage (odd and even stage counts)."""
    kind, prefix = "bf16_f8e4m3w", KINDS["bf16_f8e4m3w"][0]
    ctx.force_tile(tile)
    try:
        for K in ((128, 256, 384, 640) if combo == "KK" else (64, 128, 192, 320)):
            lv, rv = views(combo, 296, K, 208)
            check_product(ctx, "dot", kind, lv, rv, seed=K, rscale=2.0, expect_kernel=f"{prefix}_{name}_{combo}")
        lv, rv = views(combo, 24, 256, 48)
        check_product(ctx, "dot", kind, lv, rv, seed=9, rscale=2.0, expect_kernel=f"{prefix}_{name}_{combo}")
        # weight shared across a batch (stride 0), at a 16-byte-aligned offset, with a leading dimension larger
        # than its extent
        if combo == "KK":
            w = V([80, 512], offset=64).slice(1, 128, 384).t().broadcast_to([3, 256, 80])
        else:
            w = V([256, 160], offset=32).slice(1, 16, 112).broadcast_to([3, 256, 96])
        check_product(ctx, "matmul", kind, V([3, 72, 256]), w, seed=10, rscale=2.0, expect_kernel=f"{prefix}_{name}_{combo}")
    finally:
        ctx.force_tile(-1)


def test_pipelined_f8_weight_16x16_instruction(ctx):
    """fused f8e4m3 weights on the 256 x 256 tile of the 16 x 16 x 32 instruction (hook value 15, the default for large
    products): 1, 2, 3 and 5 pairs of stages, ragged and tiny M and N, a shared weight at an offset
    with a leading dimension larger than its extent, a full grid of tiles"""
    kind, prefix = "bf16_f8e4m3w", KINDS["bf16_f8e4m3w"][0]
    name = f"{prefix}_pipe256x256mi16_KK"
    ctx.force_tile(15)
    try:
        for K in (128, 256, 384, 640):
            check_product(ctx, "dot", kind, V([296, K]), V([208, K]).t(), seed=K, rscale=2.0, expect_kernel=name)
        check_product(ctx, "dot", kind, V([24, 256]), V([48, 256]).t(), seed=9, rscale=2.0, expect_kernel=name)
        w = V([80, 512], offset=64).slice(1, 128, 384).t().broadcast_to([3, 256, 80])
        check_product(ctx, "matmul", kind, V([3, 72, 256]), w, seed=10, rscale=2.0, expect_kernel=name)
        check_product(ctx, "dot", kind, V([1000, 1024]), V([777, 1024]).t(), seed=11, rscale=2.0, expect_kernel=name)
        # row-dense weights ([K, N] bytes, read through the 8-bit LDS transpose): odd and even stage counts
        km = f"{prefix}_pipe256x256mi16_KM"
        for K in (64, 128, 192, 320):
            check_product(ctx, "dot", kind, V([296, K]), V([K, 208]), seed=K, rscale=2.0, expect_kernel=km)
        check_product(ctx, "dot", kind, V([24, 256]), V([256, 48]), seed=12, rscale=2.0, expect_kernel=km)
        w = V([256, 160], offset=32).slice(1, 16, 112).broadcast_to([3, 256, 96])
        check_product(ctx, "matmul", kind, V([3, 72, 256]), w, seed=13, rscale=2.0, expect_kernel=km)
        check_product(ctx, "dot", kind, V([1000, 512]), V([512, 784]), seed=14, rscale=2.0, expect_kernel=km)
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("kind", list(KINDS))
def test_scalar_load_variant(ctx, kind):
    prefix, _, _ = KINDS[kind]
    # odd K, odd strides, odd offsets: nothing is vector-loadable
    lv = V([45, 77], offset=1)
    rv = V([77, 2 * 31]).slice(1, 1, 62, 2)
    ctx.force_tile(3)  # (a small f32 product would go to the kernel that needs no vector loads at all)
    try:
        check_product(ctx, "dot", kind, lv, rv, seed=3, rscale=2.0 if "f8" in kind else None,
                      expect_kernel=f"{prefix}_64x64_scalar")
    finally:
        ctx.force_tile(-1)


@pytest.mark.parametrize("kind", ["bf16", "f16", "f32", "i32_i8i8"])
def test_unaligned_operands(ctx, kind):
    """operands whose vectors do not start on 16-byte boundaries: k-dense rows with an odd K or stride or offset (one
    unaligned vector load per chunk), row-dense operands with an odd row count or offset (the row-dense scheme with
    unaligned loads and a guarded last vector), both at once, tiny and degenerate extents"""
    cases = [
        (V([70, 197]), V([67, 197]).t()),                         # odd K, both k-dense
        (V([3, 40, 100], offset=1), V([3, 50, 100], offset=3).t()),   # misaligned bases, batched
        (V([70, 96]), V([96, 67])),                               # right operand row-dense, odd N
        (V([70, 96]), V([96, 67], offset=1)),
        (V([96, 71]).t(), V([96, 67])),                           # both row-dense and odd
        (V([96, 71]).t(), V([61, 96]).t()),                       # left row-dense odd, right k-dense
        (V([33, 101]), V([101, 3])),                              # fewer columns than one vector holds
        (V([5, 1]), V([1, 13])),                                  # K = 1
        (V([64, 200]), V([200, 500]).slice(1, 3, 260)),           # a column slice: row pitch 500, 257 columns
        (V([2, 45, 130]), V([130, 75]).broadcast_to([2, 130, 75])),
    ]
    ctx.force_tile(3 if kind == "f32" else -1)  # (small f32 products have a kernel of their own: pin the tile kernel)
    try:
        for n, (lv, rv) in enumerate(cases):
            check_product(ctx, "matmul" if len(lv.shape) > 2 else "dot", kind, lv, rv, seed=n, expect_kernel="mfma_")
            assert "scalar" in ctx.last_kernel(), ctx.last_kernel()
    finally:
        ctx.force_tile(-1)
    # large enough for several K steps and workgroups, at the sizes the paths were written for
    check_product(ctx, "matmul", kind, V([2, 3, 197, 197]), V([2, 3, 197, 64]), seed=20)
    check_product(ctx, "dot", kind, V([300, 520]), V([520, 1031]), seed=21)
    # enough 128 x 128 tiles to fill the chip: the large-tile variant of the same loaders
    check_product(ctx, "dot", kind, V([2048, 264]), V([264, 2051]), seed=22, expect_kernel="mfma_")
    assert ctx.last_kernel().endswith("_128x128_scalar"), ctx.last_kernel()
    check_product(ctx, "dot", kind, V([2049, 197]), V([2048, 197]).t(), seed=23, expect_kernel="mfma_")
    assert ctx.last_kernel().endswith("_128x128_scalar"), ctx.last_kernel()


@pytest.mark.parametrize("kind", list(KINDS))
def test_batched_and_broadcast(ctx, kind):
    prefix, _, _ = KINDS[kind]
    rs = 2.0 if "f8" in kind else None
    ctx.force_tile(2 if kind == "f32" else -1)  # (small f32 products have a kernel of their own: pin the tile kernel)
    try:
        # strided batch on both sides, rhs a transposed view (BASELINE config 2 in small)
        check_product(ctx, "matmul", kind, V([3, 72, 64]), V([3, 80, 64]).t(), seed=11, rscale=rs, expect_kernel=prefix)
        # weight shared across the batch (stride 0) and transposed: folds into one tall product
        check_product(ctx, "matmul", kind, V([4, 40, 96]), V([56, 96]).t().broadcast_to([4, 96, 56]), seed=12, rscale=rs,
                      expect_kernel=prefix)
        # 2-D rhs, two batch dims on the lhs
        check_product(ctx, "matmul", kind, V([2, 3, 24, 32]), V([32, 40]), seed=13, rscale=rs, expect_kernel=prefix)
        # lhs broadcast over the batch, batched rhs (cannot fold: stays batched with a stride-0 operand)
        check_product(ctx, "matmul", kind, V([24, 32]).broadcast_to([3, 24, 32]), V([3, 32, 40]), seed=14, rscale=rs,
                      expect_kernel=prefix)
        # aligned offsets into larger buffers
        check_product(ctx, "dot", kind, V([40, 64], offset=64), V([64, 48], offset=128), seed=15, rscale=rs,
                      expect_kernel=prefix)
        # row slices: leading dimension larger than the extent
        check_product(ctx, "dot", kind, V([40, 128]).slice(1, 32, 96), V([64, 96]).slice(1, 16, 64), seed=16, rscale=rs,
                      expect_kernel=prefix)
    finally:
        ctx.force_tile(-1)


def test_deep_k_accumulation(ctx):
    """K = 4096 products at ordinary magnitudes: f32 accumulation keeps bf16 results inside 2e-2"""
    check_product(ctx, "dot", "bf16", V([64, 4096]), V([96, 4096]).t(), seed=21, scale=1.0)
    check_product(ctx, "dot", "f32", V([64, 4096]), V([4096, 96]), seed=22, scale=1.0)
    check_product(ctx, "dot", "bf16_f8e4m3w", V([64, 4096]), V([96, 4096]).t(), seed=23, scale=1.0, rscale=100.0)


@pytest.mark.parametrize("kind", ["bf16", "f16", "f32", "i32_i8i8", "bf16_f8e4m3w"])
@pytest.mark.parametrize("splits", [2, 3, 8])
def test_split_k(ctx, kind, splits):
    """K cut into ranges, one workgroup each, partial sums added by a second kernel: same numbers as one pass"""
    prefix = KINDS[kind][0]
    es = {"bf16": 2, "f16": 2, "f32": 4, "i32_i8i8": 1, "bf16_f8e4m3w": 2}[kind]
    rs = 2.0 if "f8" in kind else None
    ctx.force_splitk(splits)
    try:
        for tile, name in ((10, "pipe256x256w8"), (12, "pipe128x128")):
            ctx.force_tile(tile)
            K = 10 * 128 // es  # ten stages: uneven ranges for 3 and 8 ways
            check_product(ctx, "dot", kind, V([296, K]), V([200, K]).t(), seed=splits, rscale=rs,
                          expect_kernel=f"{prefix}_{name}_KK_splitk")
            if kind in ("bf16", "bf16_f8e4m3w"):
                check_product(ctx, "matmul", kind, V([2, 72, K]), V([K, 80]).broadcast_to([2, K, 80]), seed=splits + 10,
                              rscale=rs, expect_kernel=f"{prefix}_{name}_KM_splitk")
        # automatic: a product too small for 128x128 tiles to fill the machine is cut along K
        ctx.force_tile(-1)
        ctx.force_splitk(-1)
        K = 32 * 128 // es
        check_product(ctx, "dot", kind, V([256, K]), V([384, K]).t(), seed=5, rscale=rs,
                      expect_kernel="small_f32_KK" if kind == "f32" else f"{prefix}_pipe128x128_KK_splitk")
    finally:
        ctx.force_tile(-1)
        ctx.force_splitk(-1)


@pytest.mark.parametrize("dt", ["f8e4m3", "f8e5m2"])
@pytest.mark.parametrize("tile,name", [(11, "pipe256x256"), (12, "pipe128x128"), (15, "pipe256x256mi16")])
def test_native_f8_products(ctx, dt, tile, name):
    """f8e4m3 x f8e4m3 -> f8e4m3 (and the same for f8e5m2) on the 8-bit matrix instruction: 1 to 5 stages of 128 k, ragged M
    and N, batches,
    row slices and offsets; K not a multiple of 128 or a row-dense operand stay with the generic kernel"""
    ctx.force_tile(tile)
    try:
        for K in (128, 256, 384, 640):
            check_product(ctx, "dot", dt, V([296, K]), V([200, K]).t(), seed=K, scale=0.5,
                          expect_kernel=f"mfma_{dt}_{name}_KK")
        check_product(ctx, "matmul", dt, V([3, 72, 512]).slice(2, 128, 384), V([3, 80, 256], offset=64).t(), seed=7,
                      scale=0.5, expect_kernel=f"mfma_{dt}_{name}_KK")
        check_product(ctx, "matmul", dt, V([4, 40, 256]), V([56, 256]).t().broadcast_to([4, 256, 56]), seed=8, scale=0.5,
                      expect_kernel=f"mfma_{dt}_{name}_KK")
        if tile != 15:  # (the 16 x 16 x 128 tile is never cut along K)
            ctx.force_splitk(3)
            check_product(ctx, "dot", dt, V([296, 1280]), V([200, 1280]).t(), seed=9, scale=0.3,
                          expect_kernel=f"mfma_{dt}_{name}_KK_splitk3")
            ctx.force_splitk(-1)
        else:
            check_product(ctx, "dot", dt, V([1000, 1280]), V([777, 1280]).t(), seed=9, scale=0.3,
                          expect_kernel=f"mfma_{dt}_{name}_KK")
        check_product(ctx, "dot", dt, V([64, 200]), V([48, 200]).t(), seed=10, scale=0.5, expect_kernel="generic")
        check_product(ctx, "dot", dt, V([64, 256]), V([256, 48]), seed=11, scale=0.5, expect_kernel="generic")
    finally:
        ctx.force_tile(-1)
        ctx.force_splitk(-1)


@pytest.mark.parametrize("dt", ["i8", "u8"])
def test_eight_bit_integer_products_wrap(ctx, dt):
    """hodu's own i8 x i8 -> i8 and u8 x u8 -> u8 products (the accumulator has the operands' type and wraps) on the i8
    matrix instruction: the low byte of the exact sum, bit for bit the reference's result -- every tile variant, row-dense
    and unaligned operands, batches, K cut across workgroups"""
    prefix = f"mfma_{dt}_"
    for tile in (10, 11, 12, 13, 0, 2, 3):
        ctx.force_tile(tile)
        try:
            check_product(ctx, "dot", dt, V([296, 384]), V([200, 384]).t(), seed=tile, expect_kernel=prefix)
            check_product(ctx, "dot", dt, V([150, 128]), V([128, 272]), seed=20 + tile, expect_kernel=prefix)
        finally:
            ctx.force_tile(-1)
    check_product(ctx, "matmul", dt, V([3, 72, 256]), V([3, 80, 256]).t(), seed=40, expect_kernel=prefix)
    check_product(ctx, "matmul", dt, V([4, 40, 96]), V([56, 96]).t().broadcast_to([4, 96, 56]), seed=41, expect_kernel=prefix)
    check_product(ctx, "dot", dt, V([70, 197]), V([67, 197]).t(), seed=42, expect_kernel=prefix)          # odd K
    check_product(ctx, "dot", dt, V([33, 101], offset=1), V([101, 35]), seed=43, expect_kernel=prefix)    # odd everything
    check_product(ctx, "dot", dt, V([256, 4096]), V([384, 4096]).t(), seed=44, expect_kernel=prefix)      # cut along K
    assert "splitk" in ctx.last_kernel(), ctx.last_kernel()
    check_product(ctx, "dot", dt, V([2, 512]), V([64, 512]).t(), seed=45, expect_kernel=prefix)           # two rows


@pytest.mark.parametrize("dt", ["i8", "u8"])
def test_eight_bit_integer_products_full_range(ctx, dt):
    """every byte value on both sides (u8 values from 128 up are negative numbers to the matrix core: the low byte of
    the sum does not care), against the reference-faithful oracle bit for bit"""
    from gpu_util import run_product
    import oracle
    np_dt = np.int8 if dt == "i8" else np.uint8
    g = H.rng(77)
    for (m, k, n), rt in (((200, 384, 136), True), ((96, 1000, 72), False)):
        a = g.integers(0, 256, m * k).astype(np.uint8).view(np_dt)
        b = g.integers(0, 256, k * n).astype(np.uint8).view(np_dt)
        a[:256] = np.arange(256, dtype=np.uint8).view(np_dt)
        md = H.dot_md(V([m, k]), V([n, k]).t() if rt else V([k, n]))
        got = run_product(ctx, "dot", dt, a, b, md)
        assert ctx.last_kernel().startswith(f"mfma_{dt}_")
        assert np.array_equal(got, oracle.dot_asis(dt, a, b, md))
