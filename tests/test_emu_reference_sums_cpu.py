"""hodu_rocm_ctx_set_reference_sums: products of f8e4m3, f8e5m2, bf16 and f16 in the reference's own arithmetic -- the
running sum kept in the narrow type, re-rounded by the type's routine after every multiply and every add
(kernels/ops_matrix.c:196-240, :351-354, :556-600, :713-716) -- must store the reference's bytes.

The kernel (hodu_amd/csrc/gemm_refsum.hip) runs here from its unmodified source in the CPU build, through the real
entry points, and is compared BIT FOR BIT with
  * the oracle's reference-faithful products (oracle.dot_asis / matmul_asis), and
  * where oracle/_ref is built, the reference's own compiled hodu_cpu_dot_<dt> / hodu_cpu_matmul_<dt>,
on operands drawn from every bit pattern of the type (NaNs, infinities, subnormals, the f8e4m3 codes above 240 that the
reference's decoder reads as infinity), on strided, transposed, offset, batched and broadcast layouts, and on K = 0.
What the CPU build cannot show is that frexpf / ldexpf / the float-to-int conversion behave the same on the GPU; the
reference's f16 narrowing, built from the same three, is held bit for bit on the hardware by tests/test_gpu_epilogue.py.
"""
import numpy as np
import pytest

import emu_util
import helpers as H
import oracle

V = H.View
pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")
NARROW = ("f8e4m3", "f8e5m2", "bf16", "f16")


@pytest.fixture(scope="module")
def emu():
    e = emu_util.Emu()
    e.set_reference_sums(True)
    yield e
    e.close()


@pytest.fixture(scope="module")
def ref():
    return oracle.RefLib() if oracle.RefLib.available() else None


def every_pattern(dt, n, seed):
    bits = 8 if dt.startswith("f8") else 16
    return H.rng(seed).integers(0, 1 << bits, n).astype(oracle.STORAGE[dt])


def tame(dt, n, seed, scale=1.0):
    """values whose sums stay finite, so that the comparison is not mostly NaN == NaN"""
    return H.random_storage(dt, n, seed, scale)


def same_bytes(dt, got, want):
    """bit for bit -- except that bf16, whose narrowing keeps a NaN's sign and payload, may hold ANY NaN where the
    other holds one: which NaN an addition of two NaNs or an inf - inf produces is the FPU's choice (x86 and Arm
    differ for the reference itself, and so does a GPU).  The other three types narrow every NaN to one code."""
    if dt != "bf16":
        return np.flatnonzero(got != want)
    nan_g, nan_w = np.isnan(H.widen(dt, got)), np.isnan(H.widen(dt, want))
    return np.flatnonzero((nan_g != nan_w) | (~nan_g & (got != want)))


def run(emu, ref, op, dt, lv, rv, a, b):
    md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
    want = (oracle.dot_asis if op == "dot" else oracle.matmul_asis)(dt, a, b, md)
    got = np.full(want.size, 0xFF, dtype=want.dtype)
    emu.product(op, dt, a, b, got, md)
    assert emu.last_kernel() == f"reference_sums_{dt}"
    bad = same_bytes(dt, got, want)
    assert bad.size == 0, f"{op} {dt}: {bad.size} of {got.size} outputs differ from the oracle, first at {bad[:5]}"
    if ref is not None:
        real = (ref.dot if op == "dot" else ref.matmul)(dt, a, b, md)
        assert same_bytes(dt, got, real).size == 0, f"{op} {dt}: differs from the compiled reference"
    return got


@pytest.mark.parametrize("dt", NARROW)
def test_every_bit_pattern(emu, ref, dt):
    lv, rv = V([37, 29]), V([29, 41])
    for seed in (1, 2):
        run(emu, ref, "dot", dt, lv, rv, every_pattern(dt, lv.span(), seed), every_pattern(dt, rv.span(), 10 + seed))


@pytest.mark.parametrize("dt", NARROW)
def test_finite_sums_and_layouts(emu, ref, dt):
    scale = 0.5 if dt == "f8e4m3" else 1.0
    cases = [("dot", V([33, 64]), V([20, 64]).t()),                                   # weights as stored by Linear
             ("dot", V([70, 50]).t(), V([70, 9], offset=5)),                           # transposed left operand, offset
             ("dot", V([17, 40]).slice(1, 1, 39, 2), V([19, 30]).slice(0, 0, 19, 1)),  # strided k
             ("matmul", V([3, 2, 9, 12]), V([12, 7]).broadcast_to([3, 2, 12, 7])),     # stride-0 batch
             ("matmul", V([2, 5, 16], offset=3), V([2, 16, 6]).t(1, 2).t(1, 2)),
             ("dot", V([4, 0]), V([0, 6]))]                                            # K = 0: zeros
    got_any_finite = False
    for n, (op, lv, rv) in enumerate(cases):
        a, b = tame(dt, max(lv.span(), 1), 100 + n, scale), tame(dt, max(rv.span(), 1), 200 + n, scale)
        got = run(emu, ref, op, dt, lv, rv, a, b)
        got_any_finite |= bool(np.isfinite(H.widen(dt, got)).any()) if got.size else False
    assert got_any_finite


def test_differs_from_the_f32_accumulated_product_and_switches_back(emu):
    """the mode does something, and turning it off restores the library's own arithmetic"""
    lv, rv = V([24, 256]), V([16, 256]).t()
    a, b = tame("bf16", lv.span(), 7), tame("bf16", rv.span(), 8)
    md = H.dot_md(lv, rv)
    ref_bytes = np.zeros(24 * 16, np.uint16)
    emu.product("dot", "bf16", a, b, ref_bytes, md)
    assert emu.last_kernel() == "reference_sums_bf16"
    emu.set_reference_sums(False)
    try:
        own = np.zeros(24 * 16, np.uint16)
        emu.product("dot", "bf16", a, b, own, md)
        assert emu.last_kernel() == "generic"
        o32, _, _ = oracle.dot_spec("bf16", "bf16", a, b, md)
        assert np.array_equal(own, H.f32_to_bf16_rne(o32)) or np.max(np.abs(H.widen("bf16", own) - o32)) < 0.05
        assert not np.array_equal(own, ref_bytes)  # 256 truncating adds do not land on the rounded f32 sum
    finally:
        emu.set_reference_sums(True)


def test_other_dtypes_are_untouched(emu):
    for dt in ("f32", "i32", "u8", "f64"):
        lv, rv = V([9, 12]), V([12, 7])
        a, b = H.random_storage(dt, lv.span(), 3), H.random_storage(dt, rv.span(), 4)
        got = np.zeros(63, oracle.STORAGE[dt])
        emu.product("dot", dt, a, b, got, H.dot_md(lv, rv))
        assert emu.last_kernel() == "generic"


def test_f8_weight_kind_is_the_cast_then_the_bf16_product(emu, ref):
    lv, rv = V([10, 48]), V([14, 48]).t()
    a = tame("bf16", lv.span(), 5)
    w = every_pattern("f8e4m3", rv.span(), 6)
    md = H.dot_md(lv, rv)
    got = np.zeros(140, np.uint16)
    emu.product("dot", "bf16_f8e4m3w", a, w, got, md)
    assert emu.last_kernel() == "reference_sums_bf16_f8w"
    w16 = oracle.cast("f8e4m3", "bf16", w, H.cast_md(V([rv.span()])), decode=oracle.F8_OCP)
    assert np.array_equal(got, oracle.dot_asis("bf16", a, w16, md))


def test_fused_steps_follow_the_reference_sum(emu):
    """_ex in this mode: the reference's product bytes pushed through the reference's add / relu, as a caller that runs
    hodu's kernels one after the other would get them"""
    import ctypes
    from hodu_amd import ffi
    lv, rv = V([12, 40]), V([18, 40]).t()
    for dt in ("bf16", "f16"):
        a, b = tame(dt, lv.span(), 11), tame(dt, rv.span(), 12)
        bias = tame(dt, 18, 13, 4.0)
        md = H.dot_md(lv, rv)
        plain = oracle.dot_asis(dt, a, b, md)
        full = V([12, 18])
        want = oracle.relu(dt, oracle.add(dt, plain, bias, H.binary_md(full, V([18]).broadcast_to([12, 18]))), H.cast_md(full))
        steps = (ffi.EpilogueStep * 2)(ffi.EpilogueStep(ffi.EPI_ADD_ROW, bias.ctypes.data, 1, 0, (ctypes.c_ubyte * 8)()), ffi.relu())
        fn = getattr(emu.lib, f"hodu_rocm_dot_{dt}_ex")
        fn.argtypes = [ctypes.c_void_p] * 4 + [ctypes.POINTER(ctypes.c_size_t), ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t]
        arr, n = emu._md(md)
        got = np.zeros(12 * 18, np.uint16)
        assert fn(emu.ctx, a.ctypes.data, b.ctypes.data, got.ctypes.data, arr, n, ctypes.cast(steps, ctypes.c_void_p), 2) == 0
        assert emu.last_kernel() == f"reference_sums_{dt}"
        assert np.array_equal(got, want)
