"""NOT collected (the file name keeps pytest off it): the respaced-issue form of the 256 x 256 tile on the 16 x 16 x 32
instruction (testing hook 16, mfma_pipe16r_kernel) has been compiled and its code inspected but has never run on a
GPU.  Run it by naming the file, after a probe has confirmed on the hardware that the immediate offset of
global_load_lds_dwordx4 moves the LDS address and the global address alike:

    python -u -m pytest tests/wip_pipe16r.py -x -v --timeout 120 --timeout-method thread

It holds the kernel to the oracle on the shapes of test_pipelined_kk_16x16_instruction with an even number of stages,
and to the integer product bit for bit on exact-valued operands, the left edge of the first tile included (the
biased lane offsets of that tile are the ones closest to the start of the operand's buffer)."""
import numpy as np
import pytest

import helpers as H
from gpu_util import check_product
from hodu_amd import ffi
from test_gpu_exact import run_exact
from test_gpu_mfma import KINDS, views

pytestmark = pytest.mark.gpu
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.force_tile(-1)
    c.close()


@pytest.mark.parametrize("kind", ["bf16", "f16"])
def test_respaced_16x16_instruction_all_layouts(ctx, kind):
    prefix = KINDS[kind][0]
    ctx.force_tile(16)
    try:
        kk = f"{prefix}_pipe256x256mi16_KK_r"
        for stages in (2, 4, 6, 12):
            K = stages * 64
            check_product(ctx, "dot", kind, V([296, K]), V([200, K]).t(), seed=stages, expect_kernel=kk)
        K = 6 * 64
        check_product(ctx, "matmul", kind, V([3, 72, 2 * K]).slice(2, K, 2 * K), V([3, 80, K], offset=64).t(), seed=7, expect_kernel=kk)
        check_product(ctx, "dot", kind, V([1000, 1024]), V([777, 1024]).t(), seed=8, expect_kernel=kk)
        km = f"{prefix}_pipe256x256mi16_KM_r"
        for stages in (2, 4):
            K = stages * 64
            check_product(ctx, "dot", kind, V([19 * 16 - 8, K]), V([K, 13 * 16 - 8]), seed=stages, expect_kernel=km)
        check_product(ctx, "dot", kind, V([24, 128]), V([128, 40]), seed=9, expect_kernel=km)
        check_product(ctx, "matmul", kind, V([3, 72, 128], offset=64), V([128, 80], offset=128).broadcast_to([3, 128, 80]), seed=10,
                      expect_kernel=km)
        check_product(ctx, "dot", kind, V([1000, 512]), V([512, 776]), seed=12, expect_kernel=km)
        for combo in ("MK", "MM"):
            name = f"{prefix}_pipe256x256mi16_{combo}_r"
            for stages in (2, 4):
                lv, rv = views(combo, 19 * 16 - 8, stages * 64, 13 * 16 - 8)
                check_product(ctx, "dot", kind, lv, rv, seed=stages, expect_kernel=name)
            lv, rv = views(combo, 1000, 512, 776)
            check_product(ctx, "dot", kind, lv, rv, seed=13, expect_kernel=name)
    finally:
        ctx.force_tile(-1)


def test_respaced_is_exact_on_exact_operands(ctx):
    ctx.force_tile(16)
    try:
        for k in (128, 256, 1024, 2304 + 128):
            run_exact(ctx, "dot", "bf16", V([296, k]), V([384, k]).t(), k, "mfma_bf16_pipe256x256mi16_KK_r")
        run_exact(ctx, "dot", "bf16", V([4096, 256]), V([4096, 256]).t(), 8, "mfma_bf16_pipe256x256mi16_KK_r")
        run_exact(ctx, "dot", "bf16", V([4096, 128]), V([128, 4096]), 12, "mfma_bf16_pipe256x256mi16_KM_r")
    finally:
        ctx.force_tile(-1)


def test_respaced_f8_weight_tile_is_exact(ctx):
    """mfma_pipe16r_f8w_kernel: the shapes of test_16x16_instruction_tile_with_f8_weights_is_exact"""
    name = "mfma_bf16_f8w_pipe256x256mi16_KK_r"
    ctx.force_tile(16)
    try:
        for k in (128, 256, 384, 1024, 2304):
            run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, k]), V([384, k]).t(), k, name)
        run_exact(ctx, "dot", "bf16_f8e4m3w", V([17, 256]), V([5, 256]).t(), 5, name)
        run_exact(ctx, "matmul", "bf16_f8e4m3w", V([2, 160, 512]), V([520, 512]).t().broadcast_to([2, 512, 520]), 6, name)
        km = name.replace("_KK_r", "_KM_r")  # row-dense weights
        for k in (64, 192, 1024):
            run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, k]), V([k, 384]), k + 1, km)
        run_exact(ctx, "matmul", "bf16_f8e4m3w", V([2, 160, 512]), V([512, 528]).broadcast_to([2, 512, 528]), 7, km)
        run_exact(ctx, "dot", "bf16_f8e4m3w", V([4096, 256]), V([4096, 256]).t(), 8, name)
        # N(0,1) data against the comparator as well
        check_product(ctx, "dot", "bf16_f8e4m3w", V([1000, 1024]), V([777, 1024]).t(), seed=8, rscale=2.0, expect_kernel=name)
    finally:
        ctx.force_tile(-1)
