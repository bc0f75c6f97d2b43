"""The matrix-core tile kernels of bf16, f16 and f8e4m3 weights in their CPU build (tests/emu_util.py, EmuContext):
the kernels' unmodified source, run workgroup by workgroup with lanes as host threads, against CPU models of the
gfx950 instructions they are written in (tests/emu/gfx950_insn_emu.hpp: the 16 x 16 x 32 and 32 x 32 x 16 MFMA lane
layouts, LDS-DMA with M0 and the instruction's immediate offset, the LDS transpose reads, vmcnt, v_perm, the 8-bit
float conversions), through the real entry points and the real variant selection.

Two things are checked, in this order:

1. The models.  Kernels that pass their tests on the hardware must pass the same tests here: every variant the
   testing hook can pin (the general tile kernel at four sizes, the pipelined kernels on both instruction shapes, the
   f8e4m3-weight kernels, a product cut along K with the arrival counters) in all four operand layouts, bit for bit on
   exact-valued operands.  A wrong lane layout, transpose pattern, byte permutation or swizzle in a model fails here.
   A model of LDS-DMA arrival that is LATER than the hardware allows by one load must fail these kernels, or the
   as-late-as-allowed model would prove nothing about a kernel's waits.

2. The respaced-issue kernels (testing hook 16: mfma_pipe16r_kernel, mfma_pipe16r_f8w_kernel), which regroup the
   LDS-DMA instructions four to an M0 write through the immediate offset and peel the last two stages.  They are
   held to the same results as the kernels they derive from: all layouts, ragged edges (clamped rows), batches with
   offsets, both 16-bit types, f8e4m3 weights k-dense and row-dense, fused element-wise steps, under both models of
   DMA arrival (at issue; only at the s_waitcnt that retires it), with operands placed tight against an inaccessible
   page at their end and at their start (a read outside an operand faults here instead of on a GPU).

What this does not show: timing, and anything about the hardware the models do not say -- in particular that the
immediate offset of global_load_lds_dwordx4 moves the LDS address as well as the global one, which is the models'
reading of the ISA document and is what the respaced kernels rest on."""
import numpy as np
import pytest

import emu_util
import helpers as H
from gpu_util import check_product
from test_gpu_epilogue import LINEAR, SPECS, check_fused
from test_gpu_exact import run_exact
from test_gpu_mfma import views

V = H.View
pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")


@pytest.fixture(scope="module")
def ctx():
    c = emu_util.EmuContext(tight="end")
    yield c
    c.close()


@pytest.fixture(autouse=True)
def _reset(ctx):
    ctx.force_tile(-1)
    ctx.force_splitk(-1)
    ctx.dma_lazy(1)
    ctx.tight = "end"
    ctx.lds_fill(0xAB)  # a kernel that reads LDS it has not filled does not find the previous launch's operands
    yield
    ctx.force_tile(-1)
    ctx.force_splitk(-1)
    ctx.dma_lazy(0)


# ---- 1. the models, on kernels the hardware has run ------------------------------------------------------------------

@pytest.mark.parametrize("hook,name", [(0, "256x256w8"), (1, "256x256"), (2, "128x128"), (3, "64x64")])
def test_general_tile_kernel_on_the_32x32x16_instruction(ctx, hook, name):
    ctx.force_tile(hook)
    for combo in ("KK", "KM", "MK", "MM"):
        lv, rv = views(combo, 136, 200, 72)  # K = 200: full steps through LDS-DMA where the layout allows, and a ragged one
        shape = "256x256" if (hook == 0 and combo[0] == "M") else name
        run_exact(ctx, "dot", "bf16", lv, rv, hook, f"mfma_bf16_{shape}_{combo}")
    run_exact(ctx, "dot", "bf16_f8e4m3w", V([136, 200]), V([72, 200]).t(), hook, f"mfma_bf16_f8w_{name}_KK")


def test_pipelined_kernels_on_the_32x32x16_instruction(ctx):
    for hook, name in ((10, "pipe256x256w8"), (11, "pipe256x256"), (12, "pipe128x128"), (14, "pipe256x128")):
        ctx.force_tile(hook)
        run_exact(ctx, "dot", "bf16", V([296, 192]), V([136, 192]).t(), hook, f"mfma_bf16_{name}_KK")
        run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, 256]), V([136, 256]).t(), hook, f"mfma_bf16_f8w_{name}_KK")
    ctx.force_tile(11)
    run_exact(ctx, "dot", "bf16", V([296, 192]), V([192, 136]), 5, "mfma_bf16_pipe256x256_KM")
    check_product(ctx, "dot", "f16", V([192, 296]).t(), V([192, 136]), seed=6, expect_kernel="mfma_f16_pipe256x256_MM")


def test_product_cut_along_k_with_arrival_counters(ctx):
    ctx.force_tile(11)
    ctx.force_splitk(2)
    run_exact(ctx, "dot", "bf16", V([296, 512]), V([136, 512]).t(), 3, "mfma_bf16_pipe256x256_KK_splitk2")
    ctx.force_splitk(3)
    run_exact(ctx, "dot", "bf16", V([40, 448]), V([136, 448]).t(), 4, "mfma_bf16_pipe256x256_KK_splitk3")


def test_16x16x32_instruction_kernels(ctx):
    ctx.force_tile(15)
    for combo in ("KK", "KM", "MK", "MM"):
        lv, rv = views(combo, 296, 192, 136)  # three stages: an odd count
        run_exact(ctx, "dot", "bf16", lv, rv, 3, f"mfma_bf16_pipe256x256mi16_{combo}")
    check_product(ctx, "dot", "f16", V([296, 128]), V([128, 136]), seed=4, expect_kernel="mfma_f16_pipe256x256mi16_KM")
    run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, 256]), V([136, 256]).t(), 5, "mfma_bf16_f8w_pipe256x256mi16_KK")
    run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, 192]), V([192, 144]), 6, "mfma_bf16_f8w_pipe256x256mi16_KM")


@pytest.mark.parametrize("hook,kernel", [(15, "mfma_bf16_pipe256x256mi16_KK"), (16, "mfma_bf16_pipe256x256mi16_KK_r"),
                                         (11, "mfma_bf16_pipe256x256_KK")])
def test_a_dma_model_one_load_too_late_fails_them(ctx, hook, kernel):
    """the waits of these kernels are exact: were a load allowed to stay out one wait longer, a stage would be read
    before its last 1 KB piece has arrived"""
    ctx.force_tile(hook)
    ctx.dma_lazy(2)
    with pytest.raises(AssertionError, match="outputs differ"):
        run_exact(ctx, "dot", "bf16", V([256, 256]), V([256, 256]).t(), 7, kernel)
    ctx.dma_lazy(1)
    run_exact(ctx, "dot", "bf16", V([256, 256]), V([256, 256]).t(), 7, kernel)


# ---- 2. the respaced-issue kernels -----------------------------------------------------------------------------------

@pytest.mark.parametrize("model,tight", [(1, "end"), (0, "start")])
def test_respaced_all_layouts(ctx, model, tight):
    ctx.force_tile(16)
    ctx.dma_lazy(model)
    ctx.tight = tight
    for combo in ("KK", "KM", "MK", "MM"):
        name = f"mfma_bf16_pipe256x256mi16_{combo}_r"
        lv, rv = views(combo, 296, 256, 136)  # four stages: the loop body once, then the peeled pair; clamped rows in both operands
        run_exact(ctx, "dot", "bf16", lv, rv, 3, name)
        lv, rv = views(combo, 19 * 16 - 8, 128, 13 * 16 - 8)  # two stages: only the peeled pair
        run_exact(ctx, "dot", "bf16", lv, rv, 4, name)


def test_respaced_longer_k_batches_and_offsets(ctx):
    ctx.force_tile(16)
    kk = "mfma_bf16_pipe256x256mi16_KK_r"
    run_exact(ctx, "dot", "bf16", V([40, 768]), V([24, 768]).t(), 5, kk)  # twelve stages
    K = 384
    run_exact(ctx, "matmul", "bf16", V([3, 72, 2 * K]).slice(2, K, 2 * K), V([3, 80, K], offset=64).t(), 7, kk)
    run_exact(ctx, "matmul", "bf16", V([3, 72, 128], offset=64), V([128, 80], offset=128).broadcast_to([3, 128, 80]), 10,
              "mfma_bf16_pipe256x256mi16_KM_r")
    # an odd number of stages is not this kernel's, and the hook pins nothing else: the generic kernel takes the product
    run_exact(ctx, "dot", "bf16", V([40, 192]), V([24, 192]).t(), 6, "generic")


def test_respaced_f16_against_the_oracle(ctx):
    ctx.force_tile(16)
    for combo in ("KK", "MM"):
        lv, rv = views(combo, 296, 256, 136)
        check_product(ctx, "dot", "f16", lv, rv, seed=8, expect_kernel=f"mfma_f16_pipe256x256mi16_{combo}_r")
    check_product(ctx, "dot", "bf16", V([296, 384]), V([384, 136]), seed=9, expect_kernel="mfma_bf16_pipe256x256mi16_KM_r")


@pytest.mark.parametrize("model,tight", [(1, "end"), (0, "start")])
def test_respaced_f8_weights(ctx, model, tight):
    ctx.force_tile(16)
    ctx.dma_lazy(model)
    ctx.tight = tight
    kk, km = "mfma_bf16_f8w_pipe256x256mi16_KK_r", "mfma_bf16_f8w_pipe256x256mi16_KM_r"
    for k in (128, 256, 384):  # a weight buffer holds two stages: one pair, two, three
        run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, k]), V([136, k]).t(), k, kk)
    run_exact(ctx, "dot", "bf16_f8e4m3w", V([17, 256]), V([5, 256]).t(), 5, kk)
    for k in (64, 192, 256):
        run_exact(ctx, "dot", "bf16_f8e4m3w", V([296, k]), V([k, 144]), k + 1, km)
    if model == 1:
        run_exact(ctx, "matmul", "bf16_f8e4m3w", V([2, 160, 512]), V([264, 512]).t().broadcast_to([2, 512, 264]), 6, kk)
        run_exact(ctx, "matmul", "bf16_f8e4m3w", V([2, 160, 128]), V([128, 272]).broadcast_to([2, 128, 272]), 7, km)
        check_product(ctx, "dot", "bf16_f8e4m3w", V([296, 256]), V([136, 256]).t(), seed=8, rscale=2.0, expect_kernel=kk)


def test_respaced_with_fused_steps(ctx):
    ctx.force_tile(16)
    for n, spec in enumerate((LINEAR, SPECS[3])):
        check_fused(ctx, "dot", "bf16", V([296, 128]), V([136, 128]).t(), spec, seed=n, expect_kernel="mfma_bf16_pipe256x256mi16_KK_r")
    check_fused(ctx, "dot", "f16", V([40, 128]), V([128, 264]), SPECS[3], seed=3, expect_kernel="mfma_f16_pipe256x256mi16_KM_r")
    check_fused(ctx, "dot", "bf16_f8e4m3w", V([40, 128]), V([264, 128]).t(), LINEAR, seed=4,
                expect_kernel="mfma_bf16_f8w_pipe256x256mi16_KK_r")
