"""The GPU test files, run unmodified against the CPU build.

tests/emu_util.EmuContext is hodu_amd.ffi.Context over the CPU build of the kernels (their unmodified source against
CPU models of the gfx950 instructions, tests/emu/gfx950_insn_emu.hpp), so a GPU test function that takes the `ctx`
fixture can be handed one: same inputs, same entry points, same variant selection, same comparison with the oracle,
same expected kernel names.  This file collects those functions from the GPU test modules, expands their
parametrisations, and runs each case as a test of its own.

Two uses.  Every one of these cases passes on the hardware, so each is a check of the instruction models against a
kernel the hardware has run (a model that disagrees with the hardware fails the kernel written for the hardware).  And
with the models pinned that way, the same run is a regression test of the kernels' indexing, edge handling and
selection logic where no GPU is at hand.

By default the cases that take more than a few seconds each are skipped; HODU_EMU_ALL=1 runs them too (about a
third of an hour on 8 cores).  The debug library's hooks, timing loops and graph replay are part of the CPU build, so
tests that use them run too (a graph is recorded and replayed by the stand-in runtime; times are the host's).  Not run here:
one test of thousands of large launches, the Tensor-level tests (tests/test_emu_host_mirror_cpu.py runs those) and
tests/test_gpu_large_extents.py (operands of several GiB).  BASELINE's five configurations run at their full sizes
(tests/test_gpu_configs.py): 1, 2, 3 up to M = 256 and 4 with HODU_EMU_ALL=1, config 3 at M = 4096 and config 5 -- three
minutes and a quarter of an hour per case -- with HODU_EMU_ALL=2."""
import importlib
import inspect
import itertools
import os

import pytest

import emu_util
from hodu_amd import ffi

pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")

SUITES = ["test_gpu_products", "test_gpu_mfma", "test_gpu_exact", "test_gpu_epilogue", "test_gpu_skinny", "test_gpu_small_f32",
          "test_gpu_f64", "test_gpu_casts", "test_gpu_sum", "test_gpu_softmax", "test_gpu_attention", "test_zz_no_alloc",
          "test_zx_softmax_masked", "test_zx_attention_masked", "test_zy_reference_sums",
          "test_gpu_configs",  # BASELINE's five configurations at their full sizes
          # the GPU test of kernels that have not run on a GPU, kept under a name pytest does not collect: it runs here
          "wip_pipe16r"]
EXCLUDED = {"test_gpu_skinny.test_split_k_arrival_protocol_over_thousands_of_launches",  # (thousands of large launches)
            "test_zx_softmax_masked.test_attention_with_a_padding_mask_against_float64",  # (the host mirror: these two
            "test_zx_softmax_masked.test_a_mask_of_another_dtype_is_its_nonzero_pattern"}  #  run in test_emu_host_mirror_cpu.py)
# more than a few seconds per case in the CPU build
HEAVY = {
    "test_gpu_mfma.test_every_variant_ragged", "test_gpu_mfma.test_native_f8_products",
    "test_gpu_mfma.test_pipelined_f8_weight_16x16_instruction", "test_gpu_mfma.test_pipelined_kk_16x16_instruction",
    "test_gpu_mfma.test_pipelined_kk_variants", "test_gpu_mfma.test_pipelined_row_dense_variants", "test_gpu_mfma.test_split_k",
    "test_gpu_mfma.test_unaligned_operands",
    "test_gpu_exact.test_16x16_instruction_tile_is_exact_and_equals_the_32x32_one",
    "test_gpu_exact.test_16x16_instruction_tile_with_f8_weights_is_exact",
    "test_gpu_exact.test_config3_m16_takes_the_split_k_kernel_exactly", "test_gpu_exact.test_f8_weight_pipelined_tiles",
    "test_gpu_exact.test_native_f8_products_narrow_the_exact_sum_once", "test_gpu_exact.test_one_pass_and_split_k_skinny",
    "test_gpu_exact.test_pipelined_split_k_through_the_workspace", "test_gpu_exact.test_row_streaming_gemv",
    "test_gpu_epilogue.test_16x16_instruction_tiles", "test_gpu_epilogue.test_linear_layer_of_config3",
    "test_gpu_epilogue.test_pipelined_kernels", "test_gpu_epilogue.test_small_m_kernels",
    "test_gpu_skinny.test_gemv_rowstream", "test_gpu_skinny.test_row_dense_weight", "test_gpu_skinny.test_split_k_across_workgroups",
    "test_gpu_small_f32.test_large_products_keep_the_tile_kernels",
    "test_gpu_softmax.test_causal_mask", "test_gpu_softmax.test_long_and_strided_rows",
    "test_zz_no_alloc.test_two_calls_in_a_row_the_second_smaller", "test_zz_no_alloc.test_a_fresh_context_allocates_nothing_for_it",
    "test_zz_no_alloc.test_scratch_beyond_the_limit_is_refused", "test_zz_no_alloc.test_shapes_without_scratch",
    "test_zz_no_alloc.test_captured_into_a_graph_and_replayed",
    "test_gpu_configs.test_config2_bf16_batched_transposed", "test_gpu_configs.test_config3_fp8_weight_linear",
    "test_gpu_configs.test_config4_int8_valued_i32",
    "wip_pipe16r.test_respaced_16x16_instruction_all_layouts", "wip_pipe16r.test_respaced_is_exact_on_exact_operands",
    "wip_pipe16r.test_respaced_f8_weight_tile_is_exact",
}
# a quarter of an hour and more per case: config 5 (2 x 4096 x 4096 x 14336 per weight kind: 16 and 18 minutes on 8 cores)
# and config 3 at M = 4096 (3 minutes per scale)
VERY_HEAVY = {"test_gpu_configs.test_config5_mlp_broadcast", "test_gpu_configs.test_config3_fp8_weight_linear[4096-448.0]",
              "test_gpu_configs.test_config3_fp8_weight_linear[4096-240.0]"}
LEVEL = int(os.environ.get("HODU_EMU_ALL", "0") or 0)
RUN_ALL = LEVEL >= 1


def _expansions(fn):
    names, lists = [], []
    for mark in getattr(fn, "pytestmark", []):
        if mark.name != "parametrize":
            continue
        argnames = [a.strip() for a in mark.args[0].split(",")] if isinstance(mark.args[0], str) else list(mark.args[0])
        names.append(argnames)
        lists.append(list(mark.args[1]))
    for combo in itertools.product(*lists):
        kwargs = {}
        for argnames, value in zip(names, combo):
            if hasattr(value, "values") and hasattr(value, "marks"):  # pytest.param
                values = value.values
            else:
                values = value if len(argnames) > 1 else (value,)
            kwargs.update(zip(argnames, values))
        yield kwargs


def _cases():
    for modname in SUITES:
        mod = importlib.import_module(modname)
        for name, fn in inspect.getmembers(mod, inspect.isfunction):
            full = f"{modname}.{name}"
            if not name.startswith("test_") or fn.__module__ != modname or full in EXCLUDED:
                continue
            params = list(inspect.signature(fn).parameters)
            for kwargs in _expansions(fn):
                if set(params) - {"ctx"} != set(kwargs):
                    continue  # wants a fixture this file does not provide
                case = full + "[" + "-".join(str(v) for v in kwargs.values()) + "]"
                if case in EXCLUDED:
                    continue
                ident = full.replace("test_gpu_", "", 1).replace("wip_", "unrun_on_gpu_", 1) + ("[" + "-".join(str(v) for v in kwargs.values()) + "]" if kwargs else "")
                marks = []
                if (full in VERY_HEAVY or case in VERY_HEAVY) and LEVEL < 2:
                    marks = [pytest.mark.skip(reason="a quarter of an hour and more in the CPU build: set HODU_EMU_ALL=2")]
                elif full in HEAVY and not RUN_ALL:
                    marks = [pytest.mark.skip(reason="slow in the CPU build: set HODU_EMU_ALL=1")]
                yield pytest.param(fn, kwargs, id=ident, marks=marks)


@pytest.fixture(scope="module")
def ctx():
    c = emu_util.EmuContext(tight="end")
    c.dma_lazy(1)
    yield c
    c.close()


def _collected():
    """(a failure to collect must not take the other test files' collection down with it: it becomes one failing case)"""
    try:
        return list(_cases())
    except Exception as e:  # noqa: BLE001
        message = f"{type(e).__name__}: {e}"

        def collection_failed():
            raise RuntimeError(f"collecting the GPU test functions failed: {message}")
        return [pytest.param(collection_failed, {}, id="collection")]


@pytest.mark.parametrize("fn,kwargs", _collected())
def test_gpu_test_passes_in_the_cpu_build(ctx, fn, kwargs, monkeypatch):
    ctx.force_tile(-1)
    ctx.force_splitk(-1)
    monkeypatch.setattr(ffi, "Context", emu_util.EmuContext)  # (a test that makes a context of its own gets this one)
    if "ctx" in inspect.signature(fn).parameters:
        kwargs = dict(kwargs, ctx=ctx)
    try:
        fn(**kwargs)
    finally:
        ctx.force_tile(-1)
        ctx.force_splitk(-1)
        ctx.set_reference_sums(False)
