"""Randomly drawn Tensor-level programs through the host mirror (hodu_amd.tensor over hodu_amd/host/capi.cpp, linked
against the CPU build of the kernels) against numpy.

A program is a pair of tensors, each taken through a random chain of view operations (transpose, slice with a step,
unsqueeze + broadcast, reshape of a contiguous tensor), then a matmul -- ranks 1 to 4 on either side, batch dims
broadcast the way Tensor::matmul broadcasts them (crates/hodu_core/src/tensor/ops/matrix.rs:14-120) -- optionally
followed by sum over random dims and the matmul's VJP (a vector against a batched matrix is refused, as it is there).  Values are small integers in i32 and f32, so every product,
sum and gradient is exact and compared for equality; numpy applies the same view operations to its own arrays."""
import numpy as np
import pytest

import emu_util
from hodu_amd import tensor as T

pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")
NP = {"i32": np.int32, "f32": np.float32, "i64": np.int64}
BITS = {"i32": np.uint32, "f32": np.uint32, "i64": np.uint64}
BITS_BY_SIZE = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}


@pytest.fixture(scope="module", autouse=True)
def host_mirror_over_the_cpu_build():
    saved_path, saved_lib = T.HOST_LIB_PATH, T._lib
    T.HOST_LIB_PATH, T._lib = emu_util.build_host(), None
    yield
    T.HOST_LIB_PATH, T._lib = saved_path, saved_lib


def make(g, dt, shape):
    a = g.integers(-4, 5, size=shape).astype(NP[dt])
    return T.Tensor.from_bits(a.reshape(-1).view(BITS[dt]), dt, list(shape)), a


def values(t, dt):
    return t.to_bits().view(NP[dt]).reshape(t.shape)


def random_views(g, t, a, want_shape):
    """takes (tensor, array) of any shape whose size is that of a padded want_shape to a view of want_shape"""
    # start: storage holds want_shape with every dim padded and in a random order
    n = len(want_shape)
    for d in range(n):                                   # slice every dim back to its extent, some with a step
        have = a.shape[d]
        step = 2 if have >= 2 * want_shape[d] and want_shape[d] > 0 else 1
        start = int(g.integers(0, have - (want_shape[d] - 1) * step)) if want_shape[d] > 0 else 0
        end = start + (want_shape[d] - 1) * step + 1 if want_shape[d] > 0 else start
        t, a = t.slice(d, start, end, step), a[(slice(None),) * d + (slice(start, end, step),)]
    return t, a


def operand(g, dt, shape):
    """a tensor of logical `shape` reached through random views of a larger, permuted storage"""
    n = len(shape)
    perm = list(g.permutation(n))
    padded = [s * int(g.choice([1, 1, 2])) + int(g.choice([0, 0, 1, 3])) for s in shape]
    t, a = make(g, dt, [padded[p] for p in perm])        # stored in permuted order
    inv = [perm.index(d) for d in range(n)]
    # undo the permutation with transposes (a sequence of swaps)
    order = list(perm)
    for d in range(n):
        j = order.index(d)
        if j != d:
            t, a = t.transpose(d, j), np.swapaxes(a, d, j)
            order[d], order[j] = order[j], order[d]
    t, a = random_views(g, t, a, shape)
    assert list(a.shape) == list(shape) and inv is not None
    return t, a


def broadcastable_batches(g):
    nb = int(g.integers(0, 3))
    full = [int(g.integers(1, 4)) for _ in range(nb)]
    def side():
        keep = int(g.integers(0, nb + 1))
        return [b if g.random() < 0.7 else 1 for b in full[nb - keep:]]
    return side(), side()


@pytest.fixture(params=["nocopy", "reference"])
def mode(request):
    """'reference' copies non-contiguous operands and materialises broadcast batches the way hodu does today, 'nocopy'
    hands the views to the kernels: the same values either way"""
    T.set_matmul_mode(request.param)
    yield request.param
    T.set_matmul_mode("nocopy")


@pytest.mark.parametrize("dt", ["i32", "f32", "i64"])
def test_matmul_programs(dt, mode):
    g = np.random.default_rng(11000 + sum(map(ord, dt)))
    for n in range(120):
        m, k, cols = (int(g.choice([1, 2, 3, 8, 16, 17, 33, 64])) for _ in range(3))
        lb, rb = broadcastable_batches(g)
        kind = int(g.integers(0, 10))
        if kind == 0:
            ls, rs = [k], [k]                            # two vectors
        elif kind == 1:
            ls, rs = [k], [k, cols]                      # vector x matrix
        elif kind == 2:
            ls, rs = [m, k], [k]                         # matrix x vector
        elif kind == 3:                                  # a vector against a batched matrix: the reference refuses
            (ta, _), (tb, _) = operand(g, dt, [2, m, k]), operand(g, dt, [k])
            with pytest.raises(T.HoduError, match="IncompatibleShapes"):
                ta.matmul(tb)
            with pytest.raises(T.HoduError, match="IncompatibleShapes"):
                tb.matmul(operand(g, dt, [2, k, cols])[0])
            continue
        else:
            ls, rs = lb + [m, k], rb + [k, cols]
        (ta, a), (tb, b) = operand(g, dt, ls), operand(g, dt, rs)
        what = f"{dt} case {n}: {ls} {ta.layout()} x {rs} {tb.layout()}"
        out = ta.matmul(tb)
        want = np.matmul(a.astype(np.float64), b.astype(np.float64))
        assert np.abs(want).max(initial=0) < 2 ** 24
        assert list(out.shape) == list(want.shape), what
        assert np.array_equal(values(out, dt).astype(np.float64), want), what
        if want.ndim >= 1 and g.random() < 0.5:          # a sum over some dims of the product
            dims = sorted(int(d) for d in g.choice(want.ndim, size=int(g.integers(1, want.ndim + 1)), replace=False))
            keep = bool(g.integers(2))
            got = out.sum(dims, keep)
            assert np.array_equal(values(got, dt).astype(np.float64), want.sum(axis=tuple(dims), keepdims=keep)), what + f" sum {dims} {keep}"
        if len(ls) >= 2 and len(rs) >= 2 and g.random() < 0.5:  # the gradient of sum(out * grad) w.r.t. both operands
            tg, grad = make(g, dt, list(want.shape))
            da, db = T.matmul_vjp(ta, tb, tg)
            g64, a64, b64 = grad.astype(np.float64), a.astype(np.float64), b.astype(np.float64)
            want_a = np.matmul(g64, np.swapaxes(b64, -1, -2))
            want_b = np.matmul(np.swapaxes(a64, -1, -2), g64)
            # summed back to the operand's shape where matmul had broadcast it
            def to_shape(x, shape):
                while x.ndim > len(shape):
                    x = x.sum(axis=0)
                for d, s in enumerate(shape):
                    if s == 1 and x.shape[d] != 1:
                        x = x.sum(axis=d, keepdims=True)
                return x
            assert np.array_equal(values(da, dt).astype(np.float64), to_shape(want_a, ls)), what + " dA"
            assert np.array_equal(values(db, dt).astype(np.float64), to_shape(want_b, rs)), what + " dB"


def test_linear_layers_with_deferred_f8_weights():
    """hodu_nn's Linear on random shapes -- input [batch.., rows, K] in bf16, weight [N, K] stored as f8e4m3 and cast with a
    deferred to_dtype, an optional bias and ReLU in the product's store -- from one row (the GEMV kernels) over few rows
    to tiles: integer values, so the product is exact and every step is the reference kernel's own arithmetic on it"""
    import helpers as H
    from test_gpu_host_tensor import _oracle_after
    g = np.random.default_rng(12000)
    for n in range(60):
        lead = [int(g.integers(1, 4)) for _ in range(int(g.integers(0, 3)))]
        rows, k, cols = int(g.choice([1, 2, 4, 5, 16, 33, 130])), int(g.choice([64, 128, 200, 512, 1024])), int(g.choice([16, 48, 100, 256, 520]))
        x = H.f32_to_bf16_rne(g.integers(-4, 5, size=int(np.prod(lead + [rows, k]))).astype(np.float32))
        w8 = H.f32_to_ocp_e4m3_rne(g.integers(-8, 9, size=cols * k).astype(np.float64))
        b = H.f32_to_bf16_rne(g.integers(-100, 101, size=cols).astype(np.float32))
        tx = T.Tensor.from_bits(x, "bf16", lead + [rows, k])
        tw = T.Tensor.from_bits(w8, "f8e4m3", [cols, k]).to_dtype("bf16")
        assert tw.physical_dtype == "f8e4m3"
        with_bias, relu = bool(g.integers(2)), bool(g.integers(2))
        exact = H.bf16_to_f32(x).astype(np.float64).reshape(-1, k) @ H.ocp_e4m3_decode(w8).astype(np.float64).reshape(cols, k).T
        assert np.abs(exact).max() < 2 ** 24
        plain = H.f32_to_bf16_rne(exact.astype(np.float32).ravel())
        what = f"case {n}: {lead + [rows, k]} x [{cols}, {k}]^T bias {with_bias} relu {relu}"
        assert np.array_equal(tx.matmul(tw.t()).to_bits(), plain), what
        steps = ([("add", b, H.View([cols]))] if with_bias else []) + ([("relu",)] if relu else [])
        got = T.Linear(tw, T.Tensor.from_bits(b, "bf16", [cols]) if with_bias else None).forward(tx, relu=relu)
        assert list(got.shape) == lead + [rows, cols], what
        assert np.array_equal(got.to_bits(), _oracle_after("bf16", plain, lead + [rows, cols], steps)), what


@pytest.mark.parametrize("dt", ["i32", "f32"])
def test_weight_gradients_with_the_batch_folded_into_the_contraction(dt, mode):
    """matmul_vjp of a batched contiguous input against a 2-D weight (every Linear): the weight's gradient is ONE product
    over batch x rows in 'nocopy' mode, the batched product followed by sums in 'reference' mode -- the same integers"""
    g = np.random.default_rng(14000 + sum(map(ord, dt)))
    for n in range(40):
        lead = [int(g.integers(1, 5)) for _ in range(int(g.integers(1, 3)))]
        m, k, cols = (int(g.choice([1, 3, 8, 16, 33, 64])) for _ in range(3))
        (ta, a), (tb, b), (tg, grad) = make(g, dt, lead + [m, k]), make(g, dt, [k, cols]), make(g, dt, lead + [m, cols])
        T.stats(reset=True)
        da, db = T.matmul_vjp(ta, tb, tg)
        st = T.stats()
        a64, b64, g64 = (x.astype(np.float64) for x in (a, b, grad))
        what = f"{dt} {mode} case {n}: {lead + [m, k]} x {[k, cols]}"
        assert np.array_equal(values(da, dt).astype(np.float64), g64 @ b64.T), what
        want_b = a64.reshape(-1, k).T @ g64.reshape(-1, cols)
        assert list(db.shape) == [k, cols] and np.array_equal(values(db, dt).astype(np.float64), want_b), what
        if mode == "nocopy":
            assert st["sum_kernels"] == 0, (what, st)  # folded: no [B, K, N] intermediate to sum


def test_to_dtype_of_random_views_matches_the_cast_oracle():
    """to_dtype of a transposed, stepped-slice view for random dtype pairs (the deferred pairs f8e4m3 -> bf16 and i8 -> i32
    included: read back, they must be the cast's values), against the oracle's cast of the same logical elements"""
    import helpers as H
    import oracle
    from test_gpu_casts import in_domain, same
    g = np.random.default_rng(15000)
    names = list(oracle.DTYPE_ID)
    for n in range(150):
        src, dst = names[int(g.integers(len(names)))], names[int(g.integers(len(names)))]
        nd = int(g.integers(1, 4))
        stored = [int(g.choice([1, 2, 5, 8, 17, 40])) for _ in range(nd)]
        bits = in_domain(src, dst, H.random_storage(src, int(np.prod(stored)), 50 + n, 3.0))
        t, a = T.Tensor.from_bits(bits.view(BITS_BY_SIZE[bits.dtype.itemsize]), src, stored), bits.reshape(stored)
        if nd >= 2 and g.random() < 0.6:
            d1, d2 = (int(x) for x in g.choice(nd, size=2, replace=False))
            t, a = t.transpose(d1, d2), np.swapaxes(a, d1, d2)
        for d in range(nd):
            if a.shape[d] >= 4 and g.random() < 0.5:
                start, step = int(g.integers(0, 2)), int(g.choice([1, 2]))
                t, a = t.slice(d, start, a.shape[d], step), a[(slice(None),) * d + (slice(start, None, step),)]
        logical = np.ascontiguousarray(a).reshape(-1)
        want = oracle.cast(src, dst, logical, H.cast_md(H.View(list(a.shape))), decode=oracle.F8_OCP)
        got = t.to_dtype(dst)
        assert list(got.shape) == list(a.shape)
        assert same(got.to_bits().view(oracle.STORAGE[dst]), want, dst), (n, src, dst, list(a.shape), t.layout())


def test_attention_programs_with_random_masks():
    """scaled_dot_product_attention through the Tensor API: q against k / v that lack or repeat batch dims, an optional
    attn_mask of any broadcastable shape and of u8 / bool / f32 dtype, is_causal or not; bf16 at head dims 64 / 128 (the
    one kernel) and 32 (three launches), f32 (three launches); against the float64 function, a masked score filled with
    what the reference's masked_fill writes in the dtype"""
    import helpers as H
    g = np.random.default_rng(16000)
    for n in range(40):
        dt = "bf16" if g.random() < 0.75 else "f32"
        d = int(g.choice([32, 64, 128])) if dt == "bf16" else int(g.choice([16, 64]))
        batch = [int(g.integers(1, 4)) for _ in range(int(g.integers(0, 3)))]
        sq, sk = int(g.choice([1, 7, 33, 64, 100])), int(g.choice([1, 9, 32, 65, 130]))
        kv_batch = [b if g.random() < 0.6 else 1 for b in batch][int(g.integers(0, len(batch) + 1)):]
        def bits(shape, seed):
            x = np.random.default_rng(seed).standard_normal(shape).astype(np.float32)
            if dt == "bf16":
                b = H.f32_to_bf16_rne(x.ravel())
                return T.Tensor.from_bits(b, "bf16", list(shape)), H.bf16_to_f32(b).astype(np.float64).reshape(shape)
            return T.Tensor.from_bits(x.ravel().view(np.uint32), "f32", list(shape)), x.astype(np.float64)
        (tq, q), (tk, k), (tv, v) = bits(batch + [sq, d], 3 * n), bits(kv_batch + [sk, d], 3 * n + 1), bits(kv_batch + [sk, d], 3 * n + 2)
        causal, masked = bool(g.integers(2)), bool(g.integers(3))
        keep, tm = None, None
        if masked:
            full = batch + [sq, sk]
            mshape = [e if g.random() < 0.6 else 1 for e in full[int(g.integers(0, len(full))):]]
            keep = (g.random(mshape) < 0.7).astype(np.uint8)
            keep[..., 0] = 1
            mdt = str(g.choice(["u8", "bool", "f32"]))
            mbits = keep.astype(np.float32).ravel().view(np.uint32) if mdt == "f32" else keep.ravel()
            tm = T.Tensor.from_bits(mbits, mdt, mshape)
        got_t = T.scaled_dot_product_attention(tq, tk, tv, causal, tm)
        scale = float(H.bf16_to_f32(T.scalar_bits("bf16", 1.0 / np.sqrt(float(d))))[0]) if dt == "bf16" else float(np.float32(1.0 / np.sqrt(float(d))))
        s = q @ np.swapaxes(k, -1, -2) * scale
        filled = np.zeros(s.shape, bool)
        if masked:
            filled |= np.broadcast_to(keep == 0, s.shape)
        if causal:
            filled |= np.arange(sk)[None, :] > np.arange(sq)[:, None]
        s = np.where(filled, -65536.0 if dt == "bf16" else -np.inf, s)
        p = np.exp(s - s.max(-1, keepdims=True))
        p = p / p.sum(-1, keepdims=True)
        want = p @ v
        raw = got_t.to_bits()
        got = (H.bf16_to_f32(raw) if dt == "bf16" else raw.view(np.float32)).astype(np.float64).reshape(want.shape)
        tol = 2e-2 if dt == "bf16" else 1e-4
        size = np.maximum(np.abs(want), p @ np.abs(np.broadcast_to(v, want.shape[:-2] + v.shape[-2:])))
        assert list(got_t.shape) == list(want.shape)
        assert np.all(np.abs(got - want) <= tol * size + 1e-30), (n, dt, d, batch, kv_batch, sq, sk, causal, masked, float(np.abs(got - want).max()))
