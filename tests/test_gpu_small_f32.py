"""Small f32 products: the kernel that feeds the matrix cores straight from memory (a 32 x 32 tile per workgroup, K cut
four ways inside it), against the oracle through the C ABI at the 1e-5 bar of f32 products."""
import numpy as np
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
    "KM": lambda m, k, n: (V([m, k]), V([k, n])),                      # two contiguous matrices (Tensor::dot)
    "KK": lambda m, k, n: (V([m, k]), V([n, k]).t()),                  # x . W^T
    "MK": lambda m, k, n: (V([k, m]).t(), V([n, k]).t()),
    "MM": lambda m, k, n: (V([k, m]).t(), V([k, n])),                  # a weight gradient: x^T . g
}


@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_layouts_and_edges(ctx, layout):
    name = "small_f32_" + layout
    for seed, (m, k, n) in enumerate([(512, 512, 512),    # hodu's own CPU-sized benchmark case
                                      (64, 256, 96),
                                      (33, 70, 45),       # ragged rows, columns and k (a rest of 6 after 8 chunks)
                                      (17, 7, 31),        # K shorter than one chunk: the last wavefront's element loads
                                      (100, 1031, 36),    # many rings of chunks, ragged
                                      (40, 64, 40)]):     # one ring exactly for two of the wavefronts
        lv, rv = LAYOUTS[layout](m, k, n)
        check_product(ctx, "dot", "f32", lv, rv, seed=seed, expect_kernel=name)


def test_views_batches_and_broadcasts(ctx):
    # row-sliced operands at odd offsets (k-dense loads from 4-byte-aligned addresses), column-strided x
    check_product(ctx, "dot", "f32", V([48, 300], offset=3).slice(1, 5, 261), V([256, 131], offset=1).slice(1, 0, 99),
                  seed=1, expect_kernel="small_f32_KM")
    check_product(ctx, "dot", "f32", V([48, 400]).slice(1, 0, 400, 2), V([200, 64]), seed=2, expect_kernel="small_f32_MM")
    # batched, one operand shared across the batch
    check_product(ctx, "matmul", "f32", V([3, 2, 40, 64]), V([64, 72]).broadcast_to([3, 2, 64, 72]), seed=3,
                  expect_kernel="small_f32_KM")
    check_product(ctx, "matmul", "f32", V([5, 96, 128]), V([5, 80, 128]).t(1, 2), seed=4, expect_kernel="small_f32_KK")


def test_large_products_keep_the_tile_kernels(ctx):
    check_product(ctx, "dot", "f32", V([2048, 256]), V([256, 2048]), seed=5, expect_kernel="mfma_")
    check_product(ctx, "dot", "bf16", V([512, 512]), V([512, 512]), seed=6, expect_kernel="mfma_")
    check_product(ctx, "dot", "f32", V([8, 512]), V([512, 512]), seed=7, expect_kernel="gemv_rows_f32")
