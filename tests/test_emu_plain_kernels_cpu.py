"""Casts, gathers, sums and the generic product: the kernels' unmodified source in its CPU build (tests/emu,
tests/emu_util.py), through the real entry points, against the oracle.  The same comparisons as the GPU tests make on
the hardware (tests/test_gpu_casts.py, test_gpu_sum.py, test_gpu_products.py), at sizes a workgroup-as-threads run
finishes quickly: bit for bit for casts, gathers and integer arithmetic, the parity tolerances for floating sums and
products (the 8-bit float conversion instructions are written out in the CPU build's shim and are held to the oracle's
tables by the pairs that touch f8).  With the matrix-core launchers answering UNSUPPORTED, every product here runs on
generic_product_kernel -- the kernel of the dtypes and layouts nothing else takes."""
import numpy as np
import pytest

import emu_util
import helpers as H
import oracle

V = H.View
pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")
ALL = list(oracle.DTYPE_ID)


@pytest.fixture(scope="module")
def emu():
    e = emu_util.Emu()
    yield e
    e.close()


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


def in_domain(src, dst, x):
    """inputs for which the reference's C conversion is defined (negative floats to unsigned are not)"""
    if dst[0] == "u" or dst == "bool":
        if src in ("f32", "f64"):
            return np.abs(x)
        if src in ("bf16", "f16"):
            return x & 0x7FFF
    return x


def same(got, want, dst):
    if dst in ("f32", "f64"):
        nan = np.isnan(want)
        return np.array_equal(np.isnan(got), nan) and np.array_equal(_bits(got[~nan]), _bits(want[~nan]))
    return np.array_equal(_bits(got), _bits(want))


def test_cast_pairs_dense_and_strided(emu):
    views = [V([1031]), V([7, 9, 5], offset=3).t(0, 2), V([1, 9]).broadcast_to([5, 9]), V([6, 10, 12], offset=7).slice(2, 1, 11, 3),
             V([70, 130]).t()]
    kernels = set()
    for v in views:
        md = H.cast_md(v)
        for src in ALL:
            for dst in ALL:
                x = in_domain(src, dst, H.random_storage(src, v.span(), 77, 3.0))
                want = oracle.cast(src, dst, x, md, decode=oracle.F8_OCP)
                got = np.zeros(int(md[0]), dtype=oracle.STORAGE[dst])
                emu.cast(src, dst, x, got, md)
                kernels.add(emu.last_kernel())
                assert same(got, want, dst), (src, dst, v.shape, emu.last_kernel())
    assert {"cast_dense_vec", "cast_transpose_vec"} <= kernels, kernels


def test_contiguous_of_views(emu):
    for dt in ("bf16", "f32", "i8", "u64", "bool"):
        for n, v in enumerate((V([9, 70, 66]).t(1, 2), V([5, 6, 7], offset=2).t(0, 2), V([4, 1, 8]).broadcast_to([4, 3, 8]),
                               V([300]), V([130, 70]).t())):
            x = H.random_storage(dt, v.span(), 80 + n)
            md = H.cast_md(v)
            got = np.zeros(int(md[0]), dtype=oracle.STORAGE[dt])
            emu.contiguous(dt, x, got, md)
            assert np.array_equal(_bits(got), _bits(oracle.contiguous(dt, x, md))), (dt, v.shape, emu.last_kernel())


def test_sums(emu):
    cases = [(V([6, 40, 50]), [0, 1], False), (V([6, 40, 50]), [2], False), (V([6, 40, 50]), [1], True), (V([3000]), [0], False),
             (V([40, 70]).t(), [1], False), (V([2, 300, 130]), [0, 1], False), (V([5, 4100]), [1], False)]
    kernels = set()
    for n, (v, dims, keep) in enumerate(cases):
        md = H.reduce_md(v, dims, keep)
        n_out = oracle.reduce_out_elems(md)
        # integers: wrap-around sums, bit for bit
        for dt in ("i32", "u8", "i64"):
            x = H.random_storage(dt, v.span(), 300 + n)
            got = np.zeros(n_out, dtype=oracle.STORAGE[dt])
            emu.sum(dt, x, got, md)
            assert np.array_equal(got, oracle.sum_asis(dt, x, md)), (dt, v.shape, dims, emu.last_kernel())
        # floats: against the f32- / f64-accumulated comparator
        for dt, tol in (("bf16", 2e-2), ("f32", 1e-5), ("f64", 1e-12)):
            x = H.random_storage(dt, v.span(), 310 + n)
            got = np.zeros(n_out, dtype=oracle.STORAGE[dt])
            emu.sum(dt, x, got, md)
            kernels.add(emu.last_kernel())
            _, o64, oabs = oracle.sum_spec(dt, x, md)
            k = v.size // max(n_out, 1)
            H.assert_close(H.widen(dt, got), o64, oabs, k, tol, f"sum {dt} {v.shape} {dims}", eps_acc=H.EPS_F64 if dt == "f64" else H.EPS_F32)
    assert len(kernels) >= 3, kernels   # the by-output, chunked and by-row forms were all reached


def test_generic_product_integer_dtypes_bit_exact(emu):
    for dt in ("i16", "u16", "i32", "u32", "i64", "u64", "i8", "u8"):
        for n, (lv, rv) in enumerate(((V([37, 50]), V([50, 29])), (V([50, 37]).t(), V([29, 50]).t()),
                                      (V([3, 20, 16], offset=5), V([16, 24]).broadcast_to([3, 16, 24])))):
            a, b = H.random_storage(dt, lv.span(), 400 + n), H.random_storage(dt, rv.span(), 410 + n)
            op = "dot" if lv.ndim == 2 else "matmul"
            md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
            want = oracle.dot_asis(dt, a, b, md) if op == "dot" else oracle.matmul_asis(dt, a, b, md)
            got = np.zeros(want.size, dtype=oracle.STORAGE[dt])
            emu.product(op, dt, a, b, got, md)
            assert emu.last_kernel() == "generic"
            assert np.array_equal(got, want), (dt, n)


def test_generic_product_floats_and_fused_cast_entries(emu):
    lv, rv = V([45, 96]), V([33, 96]).t()
    md = H.dot_md(lv, rv)
    for dt, tol, eps in (("f32", 1e-5, H.EPS_F32), ("f64", 1e-12, H.EPS_F64), ("bf16", 2e-2, H.EPS_F32), ("f16", 2e-2, H.EPS_F32)):
        a, b = H.random_storage(dt, lv.span(), 500), H.random_storage(dt, rv.span(), 501)
        got = np.zeros(45 * 33, dtype=oracle.STORAGE[dt])
        emu.product("dot", dt, a, b, got, md)
        if dt == "f64":
            want = oracle.dot_asis("f64", a, b, md).astype(np.float64)
            sumabs = np.abs(lv.take(a)) @ np.abs(rv.take(b))
            H.assert_close(got, want, sumabs.ravel(), 96, tol, "generic f64", eps_acc=eps)
        else:
            _, o64, sumabs = oracle.dot_spec(dt, dt, a, b, md)
            H.assert_close(H.widen(dt, got), o64, sumabs, 96, tol, f"generic {dt}", eps_acc=eps)
    # i8 storage multiplied as i32 (the deferred to_dtype(i32) of both operands): exact
    a8, b8 = H.random_storage("i8", lv.span(), 502), H.random_storage("i8", rv.span(), 503)
    got = np.zeros(45 * 33, dtype=np.int32)
    emu.product("dot", "i32_i8i8", a8, b8, got, md)
    assert np.array_equal(got, oracle.dot_asis("i32", a8.astype(np.int32), b8.astype(np.int32), md))


def test_reference_known_answers_and_edge_shapes(emu):
    """the reference's own known-answer tests (crates/hodu_cpu_kernels/tests/ops_matrix.rs:8-147) through the entry
    points of the CPU build; K = 0 writes zeros; an empty output writes nothing"""
    a = np.arange(1, 7, dtype=np.float32)
    b = np.arange(7, 13, dtype=np.float32)
    out = np.zeros(4, np.float32)
    emu.product("dot", "f32", a, b, out, [2, 3, 2, 3, 1, 2, 1, 0, 0])
    assert out.tolist() == [58, 64, 139, 154]
    out = np.zeros(4, np.float32)
    emu.product("matmul", "f32", a, b, out, [4, 2, 2, 0, 2, 3, 3, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2])
    assert out.tolist() == [58, 64, 139, 154]
    out = np.full(35, 7, np.int32)
    emu.product("dot", "i32", np.zeros(1, np.int32), np.zeros(1, np.int32), out, [5, 0, 7, 0, 1, 7, 1, 0, 0])
    assert np.all(out == 0)
    keep = np.full(1, 0x5A5A5A5A, np.uint32)
    ones = np.ones(16, np.float32)
    for md in ([0, 4, 3, 4, 1, 3, 1, 0, 0], [3, 4, 0, 4, 1, 1, 1, 0, 0]):
        emu.product("dot", "f32", ones, ones, keep.view(np.float32), md)
    emu.product("matmul", "f32", ones, ones, keep.view(np.float32), [0, 3, 3, 1, 0, 2, 4, 0, 4, 2, 0, 8, 4, 1, 8, 2, 1, 0, 0, 2, 4, 2])
    assert keep[0] == 0x5A5A5A5A


def test_errors_are_status_codes_not_launches(emu):
    a, b, o = np.zeros(16, np.float32), np.zeros(16, np.float32), np.zeros(16, np.float32)
    bad = [
        ("dot", a, b, o, [2, 3, 2, 3, 1, 2, 1, 0]),                                     # 8 words
        ("matmul", a, b, o, [4, 2, 2, 0, 2, 3, 4, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2]),       # K mismatch
        ("matmul", a, b, o, [4, 1, 2, 0, 3, 3, 2, 1, 2, 1, 0, 0, 2, 3, 2]),             # 1-D operand
        ("matmul", a, b, o, [5, 2, 2, 0, 2, 3, 3, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2]),       # num_els inconsistent
        ("dot", a, b, a, [2, 3, 2, 3, 1, 2, 1, 0, 0]),                                  # out aliases an input
    ]
    for op, x, y, out, md in bad:
        with pytest.raises(RuntimeError, match="status 1"):
            emu.product(op, "f32", x, y, out, md)
    with pytest.raises(RuntimeError, match="status 1"):
        emu.cast("f32", "bf16", a, o.view(np.uint16), [4, 1, 5, 1, 0])                  # num_els != prod(shape)
    with pytest.raises(RuntimeError, match="status 2"):
        emu._check(emu.lib.hodu_rocm_cast(emu.ctx, 99, 3, a.ctypes.data, o.ctypes.data, *emu._md([4, 1, 4, 1, 0])), "cast")
    emu.product("dot", "f32", a, b, o, [2, 3, 2, 3, 1, 2, 1, 0, 0])                     # the context is still usable
