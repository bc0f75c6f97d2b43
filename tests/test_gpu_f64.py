"""f64 products on the f64 matrix-core instruction (operands straight from memory, both tile sizes, every layout), against
the reference's sequential f64 arithmetic through the C ABI at 1e-12."""
import pytest

import helpers as H
from gpu_util import check_product
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


LAYOUTS = {
    "KM": lambda m, k, n: (V([m, k]), V([k, n])),
    "KK": lambda m, k, n: (V([m, k]), V([n, k]).t()),
    "MK": lambda m, k, n: (V([k, m]).t(), V([n, k]).t()),
    "MM": lambda m, k, n: (V([k, m]).t(), V([k, n])),
}


@pytest.mark.parametrize("tile,size", [(41, "128x128"), (42, "64x64"), (43, "32x32")])
@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_layouts_and_edges(ctx, tile, size, layout):
    ctx.force_tile(tile)
    try:
        for seed, (m, k, n) in enumerate([(128, 64, 128), (200, 96, 136),   # whole tiles; ragged rows and columns
                                          (33, 70, 45),                    # a rest of 6 k after 8 chunks
                                          (17, 7, 31),                     # K shorter than one chunk
                                          (70, 259, 36),                   # many rings of chunks, odd N (element stores)
                                          (16, 16, 16), (5, 3, 2)]):       # one tile; less than a tile
            lv, rv = LAYOUTS[layout](m, k, n)
            check_product(ctx, "dot", "f64", lv, rv, seed=seed, expect_kernel=f"mfma_f64_{size}_{layout}")
    finally:
        ctx.force_tile(-1)


def test_views_batches_and_selection(ctx):
    # row-sliced operands at odd offsets, a column-strided x
    check_product(ctx, "dot", "f64", V([48, 300], offset=3).slice(1, 5, 261), V([256, 131], offset=1).slice(1, 0, 99),
                  seed=1, expect_kernel="mfma_f64_32x32_KM")
    check_product(ctx, "dot", "f64", V([48, 400]).slice(1, 0, 400, 2), V([200, 64]), seed=2, expect_kernel="mfma_f64_32x32_MM")
    # batched; one operand shared across the batch
    check_product(ctx, "matmul", "f64", V([3, 2, 40, 64]), V([64, 72]).broadcast_to([3, 2, 64, 72]), seed=3,
                  expect_kernel="mfma_f64_32x32_KM")
    check_product(ctx, "matmul", "f64", V([5, 96, 128]), V([5, 80, 128]).t(1, 2), seed=4, expect_kernel="mfma_f64_32x32_KK")
    check_product(ctx, "dot", "f64", V([1024, 40]), V([40, 1100]), seed=8, expect_kernel="mfma_f64_64x64_KM")
    # enough 128 x 128 tiles to fill the chip: the large tile
    check_product(ctx, "dot", "f64", V([2048, 40]), V([40, 2048]), seed=5, expect_kernel="mfma_f64_128x128_KM")
    # thinner than a tile, a matrix times a vector, a single output
    check_product(ctx, "dot", "f64", V([4, 256]), V([256, 64]), seed=6, expect_kernel="mfma_f64_32x32_KM")
    check_product(ctx, "dot", "f64", V([1, 1000]), V([333, 1000]).t(), seed=9, expect_kernel="mfma_f64_32x32_KK")
    check_product(ctx, "dot", "f64", V([77, 130]), V([130, 1]), seed=10, expect_kernel="mfma_f64_32x32")
    check_product(ctx, "dot", "f64", V([1, 50]), V([50, 1]), seed=11, expect_kernel="mfma_f64_32x32")
