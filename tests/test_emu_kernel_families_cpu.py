"""Every other product kernel family in its CPU build (tests/emu_util.py, EmuContext; instruction models in
tests/emu/gfx950_insn_emu.hpp): the row-streaming GEMV for M <= 4 (v_dot2_f32_bf16, DPP row reductions, readlane), the
M <= 16 kernels with and without a cut K, the few-rows kernel of the other dtypes, the transposed matrix-vector route,
the f32 / i8 / u8 / native 8-bit-float matrix-core tiles (32 x 32 x 2 and 16 x 16 x 4 f32, 32 x 32 x 32 and 16 x 16 x 64
i8, 32 x 32 x 64 and 16 x 16 x 128 f8f6f4 with unit scales), the small-f32 kernel and the f64 matrix-core kernel
(whose accumulator registers step through the rows by four, unlike the others').

These kernels pass their tests on the hardware; here the same helpers (tests/gpu_util.py, tests/test_gpu_exact.py)
drive the same source against the models, at sizes a workgroup-as-threads run finishes quickly.  What it is for:
the models are pinned by kernels the hardware has run (a wrong lane layout fails here), the kernels' indexing and
edge handling are checked where no GPU is at hand (operands lie between inaccessible pages), and a change to one of
them is caught on the CPU first."""
import pytest

import emu_util
import helpers as H
from gpu_util import check_product
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
    ctx.lds_fill(0xAB)
    yield
    ctx.force_tile(-1)
    ctx.force_splitk(-1)
    ctx.dma_lazy(0)


@pytest.mark.parametrize("name", ["bf16_f8e4m3w", "bf16"])
def test_row_streaming_gemv(ctx, name):
    pre = "gemv_bf16_f8w" if name == "bf16_f8e4m3w" else "gemv_bf16"
    for m in (1, 2, 4):
        run_exact(ctx, "dot", name, V([m, 4112]), V([67, 4112]).t(), 10 + m, pre)  # a ragged last pass, rows past N
    run_exact(ctx, "dot", name, V([4, 2048]), V([136, 2048]).t(), 4, pre)
    k = run_exact(ctx, "dot", name, V([1, 128]), V([4100, 128]).t(), 21, pre)  # many rows: a wavefront walks row groups
    assert k.endswith("_walk"), k


def test_matrix_times_vector_takes_the_transposed_route(ctx):
    check_product(ctx, "dot", "bf16", V([300, 512]), V([512, 1]), seed=4, expect_kernel="gemv_bf16")


@pytest.mark.parametrize("name", ["bf16_f8e4m3w", "bf16"])
def test_few_rows_kernels_one_pass_and_cut_k(ctx, name):
    pre = "skinny_bf16_f8w" if name == "bf16_f8e4m3w" else "skinny_bf16"
    for hook, m in ((35, 16), (36, 5), (37, 16), (39, 5)):  # the one-pass kernel's three shapes; x not staged in LDS
        ctx.force_tile(hook)
        run_exact(ctx, "dot", name, V([m, 1024]), V([264, 1024]).t(), hook + m, pre)
    ctx.force_tile(38)
    k = run_exact(ctx, "dot", name, V([16, 4224]), V([1040, 4224]).t(), 20, pre)  # arrival counters, the last workgroup adds
    assert k.endswith("_splitk"), k
    ctx.force_tile(-1)
    run_exact(ctx, "dot", name, V([12, 1024]), V([200, 1024]).t(), 3, pre)


def test_few_rows_kernel_of_the_other_dtypes(ctx):
    check_product(ctx, "dot", "f32", V([3, 1000]), V([1000, 70]), seed=1, expect_kernel="gemv_rows_f32")
    check_product(ctx, "dot", "f16", V([2, 512]), V([512, 300]), seed=2, expect_kernel="gemv_rows_f16")
    check_product(ctx, "dot", "f64", V([4, 300]), V([300, 65]), seed=3)


@pytest.mark.parametrize("kind,k", [("f32", 200), ("i32_i8i8", 208), ("i8", 208), ("u8", 208)])
def test_matrix_core_tiles_of_the_other_kinds(ctx, kind, k):
    prefix = {"f32": "mfma_f32", "i32_i8i8": "mfma_i32_i8i8", "i8": "mfma_i8", "u8": "mfma_u8"}[kind]
    for hook, shape in ((1, "256x256"), (2, "128x128"), (3, "64x64")):
        ctx.force_tile(hook)
        for combo in ("KK", "KM", "MK", "MM") if hook == 2 or kind != "f32" else ("KM", "MK"):
            lv, rv = views(combo, 136, k, 80)
            check_product(ctx, "dot", kind, lv, rv, seed=hook, expect_kernel=f"{prefix}_{shape}_{combo}")
    ctx.force_tile(12)
    lv, rv = views("KK", 136, 256, 80)
    check_product(ctx, "dot", kind, lv, rv, seed=9, expect_kernel=f"{prefix}_pipe128x128_KK")


@pytest.mark.parametrize("kind", ["f8e4m3", "f8e5m2"])
def test_native_8_bit_float_tiles(ctx, kind):
    lv, rv = V([296, 384]), V([264, 384]).t()
    for hook, name in ((-1, "pipe128x128"), (11, "pipe256x256"), (15, "pipe256x256mi16")):
        ctx.force_tile(hook)
        check_product(ctx, "dot", kind, lv, rv, seed=5, expect_kernel=f"mfma_{kind}_{name}_KK")
    ctx.force_tile(-1)
    check_product(ctx, "dot", kind, V([40, 200]), V([200, 24]), seed=6, expect_kernel="generic")  # not k-dense: no tile


def test_small_f32_and_f64(ctx):
    check_product(ctx, "dot", "f32", V([64, 512]), V([512, 10]), seed=1, expect_kernel="small_f32_KM")
    check_product(ctx, "dot", "f32", V([33, 100]), V([20, 100]).t(), seed=2, expect_kernel="small_f32_KK")
    for lv, rv in ((V([100, 70]), V([70, 90])), (V([100, 72]), V([90, 72]).t()), (V([70, 200]).t(), V([70, 300])),
                   (V([17, 9]), V([9, 5]))):
        check_product(ctx, "dot", "f64", lv, rv, seed=3, expect_kernel="mfma_f64")
    check_product(ctx, "matmul", "f64", V([3, 40, 24]), V([24, 36]).broadcast_to([3, 24, 36]), seed=4, expect_kernel="mfma_f64")
