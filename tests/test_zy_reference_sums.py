"""GPU parity of hodu_rocm_ctx_set_reference_sums: narrow-float products in the reference's own arithmetic must store
the reference's bytes.  The kernel (hodu_amd/csrc/gemm_refsum.hip) is held bit for bit to the oracle's
reference-faithful products and to the compiled reference in the CPU build (tests/test_emu_reference_sums_cpu.py); the
file name sorts this test behind those of the kernels with a longer history on the hardware.

What the GPU run adds to the CPU one: that the device's frexpf / ldexpf / float-to-int conversions and its f32 multiply
and add (denormals kept, no contraction into an FMA) give the reference's bytes."""
import numpy as np
import pytest

import helpers as H
import oracle
from gpu_util import run_product
from hodu_amd import ffi
from test_emu_reference_sums_cpu import NARROW, every_pattern, same_bytes, tame

pytestmark = pytest.mark.gpu
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.set_reference_sums(False)
    c.close()


@pytest.fixture(autouse=True)
def _mode_off_afterwards(ctx):
    yield
    ctx.set_reference_sums(False)


@pytest.mark.parametrize("dt", NARROW)
def test_reference_bytes(ctx, dt):
    ctx.set_reference_sums(True)
    cases = [("dot", V([37, 29]), V([29, 41]), True), ("dot", V([33, 64]), V([20, 64]).t(), False),
             ("dot", V([70, 50]).t(), V([70, 9], offset=5), False),
             ("matmul", V([3, 2, 9, 12]), V([12, 7]).broadcast_to([3, 2, 12, 7]), False),
             ("dot", V([300, 512]), V([260, 512]).t(), False), ("dot", V([4, 0]), V([0, 6]), False)]
    for n, (op, lv, rv, wild) in enumerate(cases):
        gen = every_pattern if wild else (lambda d, k, s: tame(d, k, s, 0.5 if d == "f8e4m3" else 1.0))
        a, b = gen(dt, max(lv.span(), 1), 100 + n), gen(dt, max(rv.span(), 1), 200 + n)
        md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
        got = run_product(ctx, op, dt, a, b, md)
        assert ctx.last_kernel() == f"reference_sums_{dt}"
        want = (oracle.dot_asis if op == "dot" else oracle.matmul_asis)(dt, a, b, md)
        bad = same_bytes(dt, got, want)
        assert bad.size == 0, f"{op} {dt} case {n}: {bad.size} of {got.size} outputs differ, first at {bad[:5]}"


def test_switching_off_restores_the_f32_sums(ctx):
    ctx.set_reference_sums(True)
    lv, rv = V([300, 512]), V([260, 512]).t()
    a, b = tame("bf16", lv.span(), 7), tame("bf16", rv.span(), 8)
    md = H.dot_md(lv, rv)
    ref_bytes = run_product(ctx, "dot", "bf16", a, b, md)
    ctx.set_reference_sums(False)
    try:
        own = run_product(ctx, "dot", "bf16", a, b, md)
        assert ctx.last_kernel().startswith("mfma_bf16")
        assert not np.array_equal(own, ref_bytes)
    finally:
        ctx.set_reference_sums(True)
