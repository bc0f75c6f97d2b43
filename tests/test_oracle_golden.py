"""Pins the CPU oracle: against the fixtures produced from the reference's own C kernels
(tests/golden/*.npz, written by tests/golden/make_fixtures.py), against the literal known-answer
vectors of the reference's kernel tests, and against what the mathematics fixes."""
import os

import numpy as np
import pytest

import helpers as H
import oracle

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


@pytest.fixture(scope="module")
def products():
    return np.load(os.path.join(GOLD, "products.npz"))


@pytest.fixture(scope="module")
def casts():
    return np.load(os.path.join(GOLD, "casts.npz"))


@pytest.fixture(scope="module")
def tables():
    return np.load(os.path.join(GOLD, "tables.npz"))


def test_products_bit_exact_vs_reference_fixtures(products):
    index = [s.split("|") for s in products["index"]]
    assert len(index) >= 100
    for key, op, dt in index:
        a, b, md = products[key + "__lhs"], products[key + "__rhs"], products[key + "__md"]
        fn = oracle.dot_asis if op == "dot" else oracle.matmul_asis
        got = fn(dt, a, b, md)
        assert np.array_equal(_bits(got), _bits(products[key + "__out"])), key


def test_casts_bit_exact_vs_reference_fixtures(casts):
    for entry in casts["index"]:
        key, src, dst = entry.split("|")
        x, md, want = casts[key + "__in"], casts[key + "__md"], casts[key + "__out"]
        got = oracle.contiguous(dst, x, md) if src == "contiguous" else oracle.cast(src, dst, x, md)
        assert np.array_equal(_bits(got), _bits(want)), key


def test_scalar_tables_vs_reference_fixtures(tables):
    one = lambda n: H.cast_md(H.View([n]))  # noqa: E731
    codes = np.arange(256, dtype=np.uint8)
    h = np.arange(65536, dtype=np.uint16)
    x = tables["f32_samples"].view(np.float32)
    checks = [
        ("f8e4m3_to_f32", oracle.cast("f8e4m3", "f32", codes, one(256)).view(np.uint32)),
        ("f8e5m2_to_f32", oracle.cast("f8e5m2", "f32", codes, one(256)).view(np.uint32)),
        ("f8e4m3_to_bf16", oracle.cast("f8e4m3", "bf16", codes, one(256))),
        ("f8e4m3_to_f16", oracle.cast("f8e4m3", "f16", codes, one(256))),
        ("f16_to_f32", oracle.cast("f16", "f32", h, one(65536)).view(np.uint32)),
        ("bf16_to_f16", oracle.cast("bf16", "f16", h, one(65536))),
        ("bf16_to_f8e4m3", oracle.cast("bf16", "f8e4m3", h, one(65536))),
        ("bf16_to_f8e5m2", oracle.cast("bf16", "f8e5m2", h, one(65536))),
        ("f16_to_f8e4m3", oracle.cast("f16", "f8e4m3", h, one(65536))),
    ] + [(f"f32_to_{d}", oracle.cast("f32", d, x, one(x.size))) for d in ("bf16", "f16", "f8e4m3", "f8e5m2")]
    for name, got in checks:
        want = tables[name]
        if want.dtype == np.uint32:  # float results: NaN payloads may differ, compare NaN-ness there
            gf, wf = got.view(np.float32), want.view(np.float32)
            nan = np.isnan(wf)
            assert np.array_equal(np.isnan(gf), nan), name
            assert np.array_equal(got[~nan], want[~nan]), name
        else:
            assert np.array_equal(got, want), name


def test_f8e4m3_decoders_differ_on_exactly_the_14_exp15_codes():
    hodu, ocp = oracle.f8e4m3_table(oracle.F8_HODU), oracle.f8e4m3_table(oracle.F8_OCP)
    diff = [b for b in range(256) if not (hodu[b] == ocp[b] or (np.isnan(hodu[b]) and np.isnan(ocp[b])))]
    assert diff == list(range(0x78, 0x7F)) + list(range(0xF8, 0xFF))
    assert ocp[0x7E] == 448.0 and ocp[0xFE] == -448.0 and np.isnan(ocp[0x7F]) and np.isinf(hodu[0x78])
    # OCP column against an independent statement of the format
    assert np.array_equal(np.nan_to_num(ocp, nan=7.0), np.nan_to_num(H.ocp_e4m3_decode(np.arange(256)), nan=7.0))


def test_ocp_table_matches_torch_float8_e4m3fn():
    torch = pytest.importorskip("torch")
    if not hasattr(torch, "float8_e4m3fn"):
        pytest.skip("torch without float8_e4m3fn")
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    ocp = oracle.f8e4m3_table(oracle.F8_OCP)
    assert np.array_equal(np.isnan(t), np.isnan(ocp))
    assert np.array_equal(t[~np.isnan(t)], ocp[~np.isnan(ocp)])


def test_bf16_widen_is_shift_and_narrow_truncates():
    g = H.rng(5)
    x = g.standard_normal(1000).astype(np.float32)
    got = oracle.cast("f32", "bf16", x, H.cast_md(H.View([1000])))
    assert np.array_equal(got, (x.view(np.uint32) >> 16).astype(np.uint16))
    # 1 + 2^-8 + 2^-9 rounds up under RNE but hodu truncates
    v = np.array([1.005859375], dtype=np.float32)
    assert oracle.cast("f32", "bf16", v, H.cast_md(H.View([1])))[0] == 0x3F80
    assert H.f32_to_bf16_rne(v)[0] == 0x3F81
    back = oracle.cast("bf16", "f32", got, H.cast_md(H.View([1000])))
    assert np.array_equal(back.view(np.uint32), got.astype(np.uint32) << 16)


# literal vectors of the reference's kernel tests -------------------------------------------------
def test_reference_known_answers_matmul_dot():
    f = np.float32
    # crates/hodu_cpu_kernels/tests/ops_matrix.rs:8-61
    a = np.array([1, 2, 3, 4, 5, 6], f); b = np.array([7, 8, 9, 10, 11, 12], f)
    md = [4, 2, 2, 0, 2, 3, 3, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2]
    assert oracle.matmul_asis("f32", a, b, md).tolist() == [58, 64, 139, 154]
    # :63-117
    a = np.array([1, 2, 3, 4, 2, 3, 4, 5], f); b = np.array([5, 6, 7, 8, 6, 7, 8, 9], f)
    md = [8, 3, 3, 1, 2, 2, 2, 2, 2, 2, 2, 4, 2, 1, 4, 2, 1, 0, 0, 2, 2, 2]
    assert oracle.matmul_asis("f32", a, b, md).tolist() == [19, 22, 43, 50, 36, 41, 64, 73]
    # :119-147
    a = np.array([1, 2, 3, 4, 5, 6], f); b = np.array([7, 8, 9, 10, 11, 12], f)
    assert oracle.dot_asis("f32", a, b, [2, 3, 2, 3, 1, 2, 1, 0, 0]).tolist() == [58, 64, 139, 154]
    # crates/hodu_cuda_kernels/tests/ops_matrix.rs:103-151 (3x3 square)
    a = np.arange(1, 10).astype(f); b = np.arange(9, 0, -1).astype(f)
    md = [9, 2, 2, 0, 3, 3, 3, 3, 3, 1, 3, 1, 0, 0, 3, 3, 3]
    assert oracle.matmul_asis("f32", a, b, md).tolist() == [30, 24, 18, 84, 69, 54, 138, 114, 90]
    # :153-186 (identity)
    eye = np.eye(3, dtype=f).ravel()
    assert oracle.dot_asis("f32", eye, eye, [3, 3, 3, 3, 1, 3, 1, 0, 0]).tolist() == eye.tolist()
    # :188-262 (lhs [2,2,3] x shared 2-D rhs)
    a = np.arange(1, 13).astype(f); b = np.array([1, 0, 0, 1, 1, 1], f)
    md = [8, 3, 2, 1, 2, 2, 3, 3, 2, 2, 6, 3, 1, 2, 1, 0, 0, 2, 3, 2]
    assert oracle.matmul_asis("f32", a, b, md).tolist() == [4, 5, 10, 11, 16, 17, 22, 23]
    # crates/hodu_metal_kernels/tests/ops_matrix.rs:141-228 (batched)
    a = np.array([1, 2, 3, 4, 5, 6, 13, 14, 15, 16, 17, 18], f)
    b = np.array([7, 8, 9, 10, 11, 12, 19, 20, 21, 22, 23, 24], f)
    md = [8, 3, 3, 1, 2, 2, 3, 2, 3, 2, 2, 6, 3, 1, 6, 2, 1, 0, 0, 2, 3, 2]
    assert oracle.matmul_asis("f32", a, b, md).tolist() == [58, 64, 139, 154, 886, 928, 1075, 1126]
    # :230-313 (broadcast)
    a = np.arange(1, 13).astype(f); b = np.arange(1, 7).astype(f)
    md = [8, 3, 2, 1, 2, 2, 3, 3, 2, 2, 6, 3, 1, 2, 1, 0, 0, 2, 3, 2]
    assert oracle.matmul_asis("f32", a, b, md).tolist() == [22, 28, 49, 64, 76, 100, 103, 136]


def test_reference_known_answers_casts():
    # crates/hodu_cuda_kernels/tests/ops_cast.rs:48-89
    one = lambda n: [n, 1, n, 1, 0]  # noqa: E731
    assert oracle.cast("f32", "i32", np.array([1.5, -2.7, 3.2, -4.9], np.float32), one(4)).tolist() == [1, -2, 3, -4]
    assert oracle.cast("i32", "f32", np.array([1, -2, 3, -4], np.int32), one(4)).tolist() == [1.0, -2.0, 3.0, -4.0]
    assert oracle.cast("f32", "u32", np.array([1.5, 2.7, 3.2, 4.9], np.float32), one(4)).tolist() == [1, 2, 3, 4]
    assert oracle.cast("u32", "f32", np.array([1, 2, 3, 4], np.uint32), one(4)).tolist() == [1.0, 2.0, 3.0, 4.0]
    x64 = np.array([1.5, 2.7, 3.2, 4.9])
    assert np.array_equal(oracle.cast("f64", "f32", x64, one(4)), x64.astype(np.float32))
    assert np.array_equal(oracle.cast("f32", "f64", x64.astype(np.float32), one(4)), x64.astype(np.float32).astype(np.float64))


def test_metadata_helpers_reproduce_reference_literals():
    V = H.View
    assert H.dot_md(V([2, 3]), V([3, 2])) == [2, 3, 2, 3, 1, 2, 1, 0, 0]
    assert H.matmul_md(V([2, 3]), V([3, 2])) == [4, 2, 2, 0, 2, 3, 3, 2, 3, 1, 2, 1, 0, 0, 2, 3, 2]
    assert H.matmul_md(V([2, 2, 2]), V([2, 2, 2])) == [8, 3, 3, 1, 2, 2, 2, 2, 2, 2, 2, 4, 2, 1, 4, 2, 1, 0, 0, 2, 2, 2]
    assert H.matmul_md(V([2, 2, 3]), V([3, 2])) == [8, 3, 2, 1, 2, 2, 3, 3, 2, 2, 6, 3, 1, 2, 1, 0, 0, 2, 3, 2]
    assert H.cast_md(V([4])) == [4, 1, 4, 1, 0]


# what the mathematics fixes ----------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64"])
def test_integer_products_equal_exact_arithmetic_mod_width(dt):
    lv, rv = H.View([3, 17, 40]), H.View([23, 40]).t().broadcast_to([3, 40, 23])
    a, b = H.random_storage(dt, lv.span(), 11), H.random_storage(dt, rv.span(), 12)
    got = oracle.matmul_asis(dt, a, b, H.matmul_md(lv, rv)).reshape(3, 17, 23)
    A = lv.take(a).astype(object); B = rv.take(b).astype(object)
    exact = np.array([[[sum(int(A[n, i, k]) * int(B[n, k, j]) for k in range(40)) for j in range(23)]
                       for i in range(17)] for n in range(3)], dtype=object)
    bits = np.dtype(oracle.STORAGE[dt]).itemsize * 8
    wrapped = exact % (1 << bits)
    assert np.array_equal(got.astype(object) % (1 << bits), wrapped)


def test_i32_product_of_i8_valued_inputs_matches_numpy_int64():
    g = H.rng(401)
    a = g.integers(-127, 128, (64, 256)).astype(np.int32)
    b = g.integers(-127, 128, (256, 48)).astype(np.int32)
    got = oracle.dot_asis("i32", a.ravel(), b.ravel(), H.dot_md(H.View([64, 256]), H.View([256, 48])))
    assert np.array_equal(got.reshape(64, 48).astype(np.int64), a.astype(np.int64) @ b.astype(np.int64))


@pytest.mark.parametrize("l_dt,r_dt", [("bf16", "bf16"), ("f16", "f16"), ("bf16", "f8e4m3"), ("f32", "f32"),
                                       ("f8e4m3", "f8e4m3")])
def test_spec_comparator_against_float64_ground_truth(l_dt, r_dt):
    lv, rv = H.View([2, 31, 200]), H.View([45, 200]).t().broadcast_to([2, 200, 45])
    a, b = H.random_storage(l_dt, lv.span(), 21), H.random_storage(r_dt, rv.span(), 22, 30.0)
    o32, o64, oabs = oracle.matmul_spec(l_dt, r_dt, a, b, H.matmul_md(lv, rv))
    A, B = H.widen(l_dt, lv.take(a)), H.widen(r_dt, rv.take(b))
    truth = np.einsum("bik,bkj->bij", A, B).ravel()
    sumabs = np.einsum("bik,bkj->bij", np.abs(A), np.abs(B)).ravel()
    assert np.allclose(o64, truth, rtol=1e-12, atol=1e-9)
    assert np.allclose(oabs, sumabs, rtol=1e-12)
    # f32 sequential accumulation: |err| <= K * 2^-24 * sum|a b|
    assert np.all(np.abs(o32 - truth) <= 200 * 2.0 ** -24 * sumabs + 1e-30)


def test_spec_bf16_matches_torch_bfloat16_semantics():
    torch = pytest.importorskip("torch")
    a = H.random_storage("bf16", 24 * 64, 31); b = H.random_storage("bf16", 64 * 20, 32)
    o32, _, _ = oracle.dot_spec("bf16", "bf16", a, b, H.dot_md(H.View([24, 64]), H.View([64, 20])))
    ta = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).reshape(24, 64).float()
    tb = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).reshape(64, 20).float()
    assert np.allclose(o32.reshape(24, 20), (ta.double() @ tb.double()).numpy(), rtol=1e-5, atol=1e-5)


def test_layout_invariants():
    dt = "bf16"
    # transposed view == contiguous copy of the transpose
    w = H.random_storage(dt, 23 * 40, 41)
    x = H.random_storage(dt, 9 * 40, 42)
    wt_view = H.View([23, 40]).t()
    wt_copy = oracle.contiguous(dt, w, H.cast_md(wt_view))
    r1 = oracle.dot_asis(dt, x, w, H.dot_md(H.View([9, 40]), wt_view))
    r2 = oracle.dot_asis(dt, x, wt_copy, H.dot_md(H.View([9, 40]), H.View([40, 23])))
    assert np.array_equal(r1, r2)
    # offset slice == explicit sub-array
    big = H.random_storage(dt, 20 * 40, 43)
    sl = H.View([20, 40]).slice(0, 5, 14)
    r3 = oracle.dot_asis(dt, big, w, H.dot_md(sl, wt_view))
    r4 = oracle.dot_asis(dt, np.ascontiguousarray(big.reshape(20, 40)[5:14]).ravel(), w, H.dot_md(H.View([9, 40]), wt_view))
    assert np.array_equal(r3, r4)
    # stride-0 batch == explicit repeat; matmul on a single batch == dot
    xb = H.random_storage(dt, 3 * 9 * 40, 44)
    r5 = oracle.matmul_asis(dt, xb, w, H.matmul_md(H.View([3, 9, 40]), wt_view.broadcast_to([3, 40, 23])))
    wrep = np.tile(wt_copy, 3)
    r6 = oracle.matmul_asis(dt, xb, wrep, H.matmul_md(H.View([3, 9, 40]), H.View([3, 40, 23])))
    assert np.array_equal(r5, r6)
    r7 = oracle.dot_asis(dt, xb[9 * 40:2 * 9 * 40], w, H.dot_md(H.View([9, 40]), wt_view))
    assert np.array_equal(r5.reshape(3, -1)[1], r7)


def test_narrow_accumulate_differs_from_f32_accumulate():
    """hodu's bf16 CPU product truncates after every multiply and add; at K=1024 the result is far
    from the f32-accumulated value, which is why the parity gate uses the SPEC comparator."""
    a = H.random_storage("bf16", 8 * 1024, 51, 1 / 32); b = H.random_storage("bf16", 1024 * 8, 52, 1 / 32)
    md = H.dot_md(H.View([8, 1024]), H.View([1024, 8]))
    narrow = H.bf16_to_f32(oracle.dot_asis("bf16", a, b, md)).astype(np.float64)
    o32, o64, oabs = oracle.dot_spec("bf16", "bf16", a, b, md)
    rel = np.abs(narrow - o64) / np.maximum(np.abs(o64), 1e-30)
    assert np.median(rel) > 0.05


def test_reference_thread_policy():
    # thread_utils.h:46-58
    assert oracle.reference_threads(511, 256, 64) == 1
    assert oracle.reference_threads(512, 256, 64) == 2
    assert oracle.reference_threads(2048, 256, 64) == 8
    assert oracle.reference_threads(4096, 128, 8) == 8


# ---------------------------------------------------------------------------------------------
# element-wise kernels the callers of the product run on its output (add, mul_scalar, relu)
# ---------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def elementwise():
    return np.load(os.path.join(GOLD, "elementwise.npz"))


def _elementwise_got(ew, key, op, dt):
    if op == "add":
        return oracle.add(dt, ew[key + "__lhs"], ew[key + "__rhs"], ew[key + "__md"])
    if op == "mul_scalar":
        return oracle.mul_scalar(dt, ew[key + "__in"], ew[key + "__md"], ew[key + "__scalar"])
    return oracle.relu(dt, ew[key + "__in"], ew[key + "__md"])


def test_elementwise_bit_exact_vs_reference_fixtures(elementwise):
    index = [s.split("|") for s in elementwise["index"]]
    assert len(index) == 90
    for key, op, dt in index:
        got, want = _elementwise_got(elementwise, key, op, dt), elementwise[key + "__out"]
        if dt in ("f32", "f64"):  # NaN payloads are not part of the contract
            assert np.array_equal(np.isnan(got), np.isnan(want)), key
            got, want = np.nan_to_num(got, nan=0.0), np.nan_to_num(want, nan=0.0)
        assert np.array_equal(_bits(got), _bits(want)), key


def test_elementwise_known_answers_of_the_reference_tests():
    """crates/hodu_cpu_kernels/tests/ops_binary.rs:68-73, tests/ops_unary.rs:143-147, :503-507"""
    one = lambda n: H.cast_md(H.View([n]))  # noqa: E731
    f = lambda *v: np.array(v, dtype=np.float32)  # noqa: E731
    md = H.binary_md(H.View([4]), H.View([4]))
    assert np.array_equal(oracle.add("f32", f(1, 2, 3, 4), f(5, 6, 7, 8), md), f(6, 8, 10, 12))
    assert np.array_equal(oracle.relu("f32", f(-2, -1, 0, 1, 2), one(5)), f(0, 0, 0, 1, 2))
    assert np.array_equal(oracle.mul_scalar("f32", f(1, 2, 3, 4), one(4), f(3)), f(3, 6, 9, 12))


def test_elementwise_against_independent_arithmetic():
    """bf16: the exact f32 sum / product with its low 16 bits cut (kernels/t_bf16.h:35-39); integers: numpy's
    modular arithmetic; relu: NaN and -0 become +0"""
    g = H.rng(5)
    a = g.integers(0, 1 << 16, 4096).astype(np.uint16)
    b = g.integers(0, 1 << 16, 4096).astype(np.uint16)
    a[(a & 0x7F80) == 0x7F80] = 0x3F80  # keep inf / NaN out of the random operands
    b[(b & 0x7F80) == 0x7F80] = 0xBF80
    af, bf = H.bf16_to_f32(a), H.bf16_to_f32(b)
    with np.errstate(over="ignore", invalid="ignore"):
        want = ((af + bf).view(np.uint32) >> 16).astype(np.uint16)
    md = H.binary_md(H.View([4096]), H.View([4096]))
    assert np.array_equal(oracle.add("bf16", a, b, md), want)
    c = np.array([0x4049], dtype=np.uint16)  # 3.140625
    with np.errstate(over="ignore", invalid="ignore"):
        want = ((af * H.bf16_to_f32(c)[0]).view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(oracle.mul_scalar("bf16", a, H.cast_md(H.View([4096])), c), want)
    x = g.integers(-2 ** 31, 2 ** 31, 4096).astype(np.int32)
    y = g.integers(-2 ** 31, 2 ** 31, 4096).astype(np.int32)
    assert np.array_equal(oracle.add("i32", x, y, md), (x.astype(np.int64) + y.astype(np.int64)).astype(np.int32))
    s = np.array([-77777], dtype=np.int32)
    assert np.array_equal(oracle.mul_scalar("i32", x, H.cast_md(H.View([4096])), s),
                          (x.astype(np.int64) * int(s[0])).astype(np.int32))
    r = oracle.relu("bf16", np.array([0x7FC0, 0x8000, 0xBF80, 0x3F80, 0xFF80, 0x7F80], dtype=np.uint16), H.cast_md(H.View([6])))
    assert list(r) == [0, 0, 0, 0x3F80, 0, 0x7F80]


# ---------------------------------------------------------------------------------------------
# sum over dims (what sum_to_shape runs on a matmul's gradients)
# ---------------------------------------------------------------------------------------------
def test_sums_bit_exact_vs_reference_fixtures():
    sums = np.load(os.path.join(GOLD, "sums.npz"))
    index = [s.split("|") for s in sums["index"]]
    assert len(index) == 14 * 8
    for key, dt in index:
        got, want = oracle.sum_asis(dt, sums[key + "__in"], sums[key + "__md"]), sums[key + "__out"]
        if dt in ("f32", "f64") and key.startswith("sum_last__"):
            # the reference adds lane-wise (SIMD) when only the last, dense dim is reduced: same numbers, other order
            assert np.allclose(got, want, rtol=1e-5 if dt == "f32" else 1e-13, atol=1e-5 if dt == "f32" else 1e-13), key
            continue
        assert np.array_equal(_bits(got), _bits(want)), key


def test_sums_against_numpy():
    """integers: numpy's modular sum; floats: the f32-accumulated comparator against a float64 sum; keep_dim only
    changes the shape; bf16 accumulates in bf16 (kernels/ops_reduce.c:129): summing 1.0 513 times stalls at 256"""
    V = H.View
    g = H.rng(31)
    v = V([6, 5, 7])
    x = g.integers(-2 ** 31, 2 ** 31, v.size).astype(np.int32)
    want = x.reshape(6, 5, 7).astype(np.int64).sum(axis=0).astype(np.int32).ravel()
    assert np.array_equal(oracle.sum_asis("i32", x, H.reduce_md(v, [0], False)), want)
    assert np.array_equal(oracle.sum_asis("i32", x, H.reduce_md(v, [0], True)), want)
    want = x.reshape(6, 5, 7).astype(np.int64).sum(axis=(0, 2)).astype(np.int32).ravel()
    assert np.array_equal(oracle.sum_asis("i32", x, H.reduce_md(v, [0, 2], False)), want)
    f = g.standard_normal(v.size).astype(np.float32)
    o32, o64, oabs = oracle.sum_spec("f32", f, H.reduce_md(v, [1], False))
    assert np.allclose(o64, f.reshape(6, 5, 7).astype(np.float64).sum(axis=1).ravel(), rtol=1e-14)
    assert np.allclose(o32, o64, rtol=1e-5, atol=1e-6) and np.allclose(oabs, np.abs(f.reshape(6, 5, 7)).sum(axis=1).ravel())
    ones = np.full(513, 0x3F80, dtype=np.uint16)
    assert oracle.sum_asis("bf16", ones, H.reduce_md(V([513]), [0], False))[0] == 0x4380  # 256.0
    assert oracle.sum_spec("bf16", ones, H.reduce_md(V([513]), [0], False))[0][0] == 513.0


# ---------------------------------------------------------------------------------------------
# softmax (the step between attention's two products)
# ---------------------------------------------------------------------------------------------
def test_softmax_comparator_against_numpy_and_invariants():
    V = H.View
    g = H.rng(41)
    x = (g.standard_normal(3 * 5 * 17) * 3).astype(np.float32)
    md = H.reduce_md(V([3, 5, 17]), [2], True)
    o32, o64 = oracle.softmax_spec("f32", x, md)
    a = x.astype(np.float64).reshape(3, 5, 17)
    e = np.exp(a - a.max(-1, keepdims=True))
    want = (e / e.sum(-1, keepdims=True)).ravel()
    assert np.allclose(o64, want, rtol=1e-14, atol=0) and np.allclose(o32, want, rtol=2e-6, atol=1e-12)
    assert np.allclose(o64.reshape(15, 17).sum(1), 1.0, rtol=1e-14)
    # shift invariance: softmax(x + c) == softmax(x)
    assert np.allclose(oracle.softmax_spec("f32", x + np.float32(7.0), md)[1], o64, rtol=1e-5)
    # a dim that is not the last one, through a transposed view
    vt = V([3, 5, 17]).t(1, 2)  # [3, 17, 5] strided, softmax over what used to be the last dim
    o64t = oracle.softmax_spec("f32", x, H.reduce_md(vt, [1], True))[1]
    assert np.allclose(o64t.reshape(3, 17, 5), want.reshape(3, 5, 17).transpose(0, 2, 1), rtol=1e-14)
    # causal (crates/hodu_nn/src/modules/attention.rs:73-86: masked where j > i): row i is a softmax of its first i + 1 entries
    s = (g.standard_normal(2 * 6 * 6)).astype(np.float32)
    c64 = oracle.softmax_spec("f32", s, H.reduce_md(V([2, 6, 6]), [2], True), causal=True)[1].reshape(2, 6, 6)
    b = s.astype(np.float64).reshape(2, 6, 6)
    for i in range(6):
        row = np.exp(b[:, i, :i + 1] - b[:, i, :i + 1].max(-1, keepdims=True))
        assert np.allclose(c64[:, i, :i + 1], row / row.sum(-1, keepdims=True), rtol=1e-14)
        assert np.all(c64[:, i, i + 1:] == 0.0)
    # bf16 inputs are widened exactly
    xb = H.f32_to_bf16_rne(x)
    assert np.allclose(oracle.softmax_spec("bf16", xb, md)[1], oracle.softmax_spec("f32", H.bf16_to_f32(xb), md)[1], rtol=0, atol=0)
