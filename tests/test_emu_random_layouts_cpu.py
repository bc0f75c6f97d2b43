"""Randomly drawn layouts through the C ABI of the CPU build, against the oracle.

The hand-picked layouts of the GPU test files name the cases somebody thought of.  Here shapes, storage orders,
slices with steps, offsets, size-1 and stride-0 broadcasts are drawn at random (seeded: the same cases every run), so
that the host's classification of an operand (dense along k, dense along rows, element-wise; aligned or not), the
choice of kernel family, ragged edges and batch decomposition meet combinations nobody listed -- with every operand
allocated tight against an inaccessible page at its end or, every other case, at its start, so a kernel variant that
reads one element outside what its layout addresses faults instead of passing.  The comparison is the GPU tests' own
(tests/gpu_util.py, test_gpu_sum.py, test_gpu_softmax.py, test_gpu_casts.py): bit for bit for integers and casts,
the stated tolerances for floats."""
import os

import numpy as np
import pytest

import emu_util
import helpers as H
import oracle
from gpu_util import FUSED, check_product
from hodu_amd import ffi

pytestmark = pytest.mark.skipif(emu_util.compiler() is None, reason="no host clang++ for the CPU build")
V = H.View
MORE = int(os.environ.get("HODU_EMU_ALL", "0") or 0) > 0
ROUNDS = 40 if MORE else 6  # multiplies the cases per dtype and family


@pytest.fixture(scope="module")
def contexts():
    made = {"end": emu_util.EmuContext(tight="end"), "start": emu_util.EmuContext(tight="start")}
    yield made
    for c in made.values():
        c.close()


def random_view(g, shape, may_broadcast=(), tame=False, inner=None):
    """a view of logical `shape` over some storage: dims stored in a random order, each possibly a slice (with a step)
    of a longer storage dim, a random offset; dims listed in may_broadcast may get stride 0.  tame: the innermost
    stored dim is dense and every other stride and the offset are multiples of 16 elements, the layouts the
    vector-loading kernels take; inner: the dim that is stored innermost"""
    n = len(shape)
    order = list(g.permutation(n))                      # storage order, outermost first
    if inner is not None:                               # this dim innermost
        i = order.index(inner)
        order[i], order[-1] = order[-1], order[i]
    elif tame and n >= 2 and order[-1] < n - 2:         # a matrix dim innermost, batch dims anywhere outside
        i = order.index(n - 1 if g.random() < 0.5 else n - 2)
        order[i], order[-1] = order[-1], order[i]
    step = [int(g.choice([1, 1, 1, 2, 3])) for _ in range(n)]
    extra = [int(g.choice([0, 0, 16, 32] if tame else [0, 0, 8, 3, 1])) for _ in range(n)]
    if tame and n:
        step[order[-1]] = 1
    stored = [(shape[d] - 1) * step[d] + 1 + extra[d] if shape[d] > 0 else extra[d] + 1 for d in range(n)]
    if tame and n:
        stored[order[-1]] = -(-stored[order[-1]] // 16) * 16
    strides, acc = [0] * n, 1
    for d in reversed(order):
        strides[d] = acc * step[d]
        acc *= stored[d]
    for d in may_broadcast:
        if g.random() < 0.35:
            strides[d] = 0
    return V(list(shape), strides, int(g.choice([0, 0, 16, 48] if tame else [0, 0, 8, 16, 3, 5])))


def dims(g, choices):
    return int(g.choice(choices))


M_CHOICES = [1, 2, 3, 4, 5, 16, 17, 31, 33, 64, 65, 100, 128, 130, 257, 300]
K_CHOICES = [1, 7, 8, 16, 31, 64, 65, 128, 136, 192, 200, 256, 260, 512]


def product_case(g):
    m, n, k = dims(g, M_CHOICES), dims(g, M_CHOICES), dims(g, K_CHOICES)
    while m * n * k > 6_000_000:
        m = max(1, m // 2)
    tame = g.random() < 0.65
    if tame and g.random() < 0.75:  # .. and extents in whole vectors, as the vector-loading kernels need them
        m, n, k = (v if v == 1 and g.random() < 0.5 else -(-v // 16) * 16 for v in (m, n, k))
    if g.random() < 0.5:
        return "dot", random_view(g, [m, k], tame=tame), random_view(g, [k, n], tame=tame)
    nb = int(g.integers(0, 3))
    batch = [int(g.integers(1, 4)) for _ in range(nb)]
    while int(np.prod(batch + [m, n, k], dtype=np.int64)) > 6_000_000 and batch:
        batch.pop()
    # either side may lack leading batch dims or hold extent 1 where the other has more (broadcast by shape), or hold
    # the full extent with stride 0 (broadcast by stride)
    def side(rows, cols):
        keep = int(g.integers(0, len(batch) + 1))
        shape = [b if g.random() < 0.7 else 1 for b in batch[len(batch) - keep:]] + [rows, cols]
        return random_view(g, shape, may_broadcast=range(len(shape) - 2), tame=tame)
    return "matmul", side(m, k), side(k, n)


@pytest.mark.parametrize("dt", ffi.PRODUCT_DTYPES + list(FUSED))
def test_products_over_random_layouts(contexts, dt):
    g = np.random.default_rng(1000 + sum(map(ord, dt)))
    scale = 2.0 if dt.startswith("f8") else 1.0
    for n in range(3 * ROUNDS):
        op, lv, rv = product_case(g)
        ctx = contexts["end" if n % 2 == 0 else "start"]
        try:
            check_product(ctx, op, dt, lv, rv, seed=n, scale=scale)
        except AssertionError as e:
            raise AssertionError(f"{op} {dt} case {n}: lhs {lv.shape} {lv.strides} +{lv.offset}, rhs {rv.shape} {rv.strides} +{rv.offset}, "
                                 f"kernel {ctx.last_kernel()}: {e}") from None


def test_casts_and_gathers_over_random_layouts(contexts):
    from test_gpu_casts import gpu_cast, in_domain, same
    g = np.random.default_rng(2024)
    names = list(oracle.DTYPE_ID)
    for n in range(20 * ROUNDS):
        nd = int(g.integers(1, 5))
        shape = [dims(g, [1, 2, 3, 5, 8, 17, 33, 64, 70]) for _ in range(nd)]
        while int(np.prod(shape, dtype=np.int64)) > 200_000:
            shape[int(np.argmax(shape))] //= 2
        v = random_view(g, shape, may_broadcast=range(nd))
        md = H.cast_md(v)
        src, dst = names[int(g.integers(len(names)))], names[int(g.integers(len(names)))]
        ctx = contexts["end" if n % 2 == 0 else "start"]
        x = in_domain(src, dst, H.random_storage(src, max(v.span(), 1), 77 + n, 3.0))
        want = oracle.cast(src, dst, x, md, decode=oracle.F8_OCP)
        assert same(gpu_cast(ctx, src, dst, x, md), want, dst), (n, src, dst, v.shape, v.strides, v.offset, ctx.last_kernel())
        want = oracle.contiguous(src, x, md)
        assert same(gpu_cast(ctx, "contiguous", src, x, md), want, src), (n, src, v.shape, v.strides, v.offset, ctx.last_kernel())


@pytest.mark.parametrize("dt", ["bf16", "f32", "f64", "i32", "u8", "f8e4m3"])
def test_sums_over_random_layouts(contexts, dt):
    from test_gpu_sum import check_sum
    g = np.random.default_rng(3000 + sum(map(ord, dt)))
    for n in range(4 * ROUNDS):
        nd = int(g.integers(1, 5))
        shape = [dims(g, [1, 2, 3, 5, 8, 17, 33, 64, 130]) for _ in range(nd)]
        while int(np.prod(shape, dtype=np.int64)) > 150_000:
            shape[int(np.argmax(shape))] //= 2
        v = random_view(g, shape, may_broadcast=range(nd))
        reduced = sorted(int(d) for d in g.choice(nd, size=int(g.integers(1, nd + 1)), replace=False))
        ctx = contexts["end" if n % 2 == 0 else "start"]
        try:
            check_sum(ctx, dt, v, reduced, bool(g.integers(2)), seed=n)
        except AssertionError as e:
            raise AssertionError(f"sum {dt} case {n}: {v.shape} {v.strides} +{v.offset} over {reduced}, kernel {ctx.last_kernel()}: {e}") from None


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_softmax_over_random_layouts(contexts, dt):
    from test_gpu_softmax import check_softmax
    g = np.random.default_rng(4000 + sum(map(ord, dt)))
    for n in range(4 * ROUNDS):
        nd = int(g.integers(1, 5))
        shape = [dims(g, [1, 2, 3, 5, 8, 17, 33, 64, 130, 700]) for _ in range(nd)]
        while int(np.prod(shape, dtype=np.int64)) > 100_000:
            shape[int(np.argmax(shape))] //= 2
        v = random_view(g, shape)
        dim = int(g.integers(nd))
        causal = dim == nd - 1 and nd >= 2 and bool(g.integers(2))
        ctx = contexts["end" if n % 2 == 0 else "start"]
        try:
            check_softmax(ctx, dt, v, dim, causal, seed=n)
        except AssertionError as e:
            raise AssertionError(f"softmax {dt} case {n}: {v.shape} {v.strides} +{v.offset} dim {dim} causal {causal}, "
                                 f"kernel {ctx.last_kernel()}: {e}") from None


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_attention_over_random_layouts(contexts, dt):
    """the one-kernel attention with and without an attn_mask: q, k, v as views with the head dim innermost and
    everything else in any order (heads interleaved with positions, k and v shared across batch dims by stride 0), the
    mask as any view that broadcasts against the scores"""
    from test_gpu_attention import check_attention
    from test_zx_attention_masked import check as check_masked
    g = np.random.default_rng(5000 + sum(map(ord, dt)))
    for n in range(3 * ROUNDS):
        d = int(g.choice([64, 128]))
        batch = [int(g.integers(1, 4)) for _ in range(int(g.integers(0, 3)))]
        sq, sk = dims(g, [1, 2, 31, 33, 64, 100, 128, 130, 200]), dims(g, [1, 5, 32, 63, 64, 65, 127, 129, 200, 300])
        while int(np.prod(batch, dtype=np.int64)) * sq * sk > 150_000 and batch:
            batch.pop()
        nb = len(batch)
        qv = random_view(g, batch + [sq, d], tame=True, inner=nb + 1)
        kv = random_view(g, batch + [sk, d], may_broadcast=range(nb), tame=True, inner=nb + 1)
        vv = random_view(g, batch + [sk, d], may_broadcast=range(nb), tame=True, inner=nb + 1)
        causal = bool(g.integers(2))
        ctx = contexts["end" if n % 2 == 0 else "start"]
        what = f"attention {dt} case {n}: batch {batch} {sq}x{sk} d {d} causal {causal}, q {qv.strides} +{qv.offset}, k {kv.strides} +{kv.offset}, v {vv.strides} +{vv.offset}"
        try:
            if n % 3 == 0:
                check_attention(ctx, dt, batch, sq, sk, causal, seed=n, qv=qv, kv=kv, vv=vv, d=d)
            else:
                keep = int(g.integers(1, nb + 3))  # trailing dims of the scores the mask has
                mshape = [e if g.random() < 0.6 else 1 for e in (batch + [sq, sk])[nb + 2 - keep:]]
                mv = random_view(g, mshape, may_broadcast=range(len(mshape)))
                what += f", mask {mv.shape} {mv.strides} +{mv.offset}"
                check_masked(ctx, dt, batch, sq, sk, mv, causal, seed=n, d=d, density=float(g.choice([0.05, 0.5, 0.9])),
                             close_key0=bool(g.integers(2)), qv=qv, kv=kv, vv=vv)
        except AssertionError as e:
            raise AssertionError(f"{what}: {e}") from None


@pytest.mark.parametrize("dt", ffi.EPILOGUE_DTYPES + ["bf16_f8e4m3w"])
def test_fused_steps_over_random_layouts(contexts, dt):
    """the product with add(bias) / mul_scalar / relu in its store equals the plain product followed by the reference's
    own kernels, bit for bit, whatever kernel family the layout selects"""
    from test_gpu_epilogue import FLOATS, SPECS, check_fused
    g = np.random.default_rng(6000 + sum(map(ord, dt)))
    for n in range(2 * ROUNDS):
        op, lv, rv = product_case(g)
        if 0 in lv.shape or 0 in rv.shape:
            continue
        spec = SPECS[int(g.integers(len(SPECS)))]
        if dt not in FLOATS and dt != "bf16_f8e4m3w" and ("relu",) in spec:
            spec = SPECS[0]
        ctx = contexts["end" if n % 2 == 0 else "start"]
        # every other case with a tile (and a number of K ranges) pinned, for the kinds that have matrix-core tiles
        hook = int(g.choice([0, 1, 2, 3, 10, 11, 12, 13, 15, 16])) if n % 2 and dt in ("bf16", "f16", "f32", "i8", "u8", "bf16_f8e4m3w") else -1
        cuts = int(g.choice([-1, 1, 2, 3])) if hook >= 0 else -1
        ctx.force_tile(hook)
        ctx.force_splitk(cuts)
        try:
            check_fused(ctx, op, dt, lv, rv, spec, seed=n, must_change=False)
        except AssertionError as e:
            raise AssertionError(f"{op} {dt} + {spec} case {n}, hook {hook}, {cuts} K ranges: lhs {lv.shape} {lv.strides} +{lv.offset}, "
                                 f"rhs {rv.shape} {rv.strides} +{rv.offset}, kernel {ctx.last_kernel()}: {e}") from None
        finally:
            ctx.force_tile(-1)
            ctx.force_splitk(-1)


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64", "i8", "u8", "f8e4m3", "f8e5m2", "bf16_f8e4m3w", "i32_i8i8"])
def test_pinned_tiles_and_k_cuts_over_random_layouts(contexts, dt):
    """the same draw with the testing hooks pinning a tile of the matrix-core kernels (general and pipelined, 256 x 256
    down to 64 x 64, the 16 x 16 x 32 tile and its respaced form, the GEMV and few-rows kernels' shapes, the small-f32 kernel at any size,
    the f64 tiles) and a number of K ranges: the large tiles on small,
    ragged, oddly laid out products, where the automatic choice never puts them.  A hook that does not apply to a
    layout leaves the choice to the dispatcher; whatever runs must be right"""
    g = np.random.default_rng(7000 + sum(map(ord, dt)))
    for n in range(4 * ROUNDS):
        op, lv, rv = product_case(g)
        ctx = contexts["end" if n % 2 == 0 else "start"]
        hooks = {"f64": [41, 42, 43], "f32": [0, 1, 2, 3, 10, 11, 12, 13, 40]}.get(dt, [0, 1, 2, 3, 10, 11, 12, 13, 14, 15, 16, 30, 31, 32, 33, 34, 35, 36, 37, 38, 39])
        hook, cuts = int(g.choice(hooks)), int(g.choice([-1, -1, 1, 2, 3]))
        ctx.force_tile(hook)
        ctx.force_splitk(cuts)
        try:
            check_product(ctx, op, dt, lv, rv, seed=n, scale=2.0 if dt.startswith("f8") else 1.0)
        except AssertionError as e:
            raise AssertionError(f"{op} {dt} case {n}, hook {hook}, {cuts} K ranges: lhs {lv.shape} {lv.strides} +{lv.offset}, rhs {rv.shape} "
                                 f"{rv.strides} +{rv.offset}, kernel {ctx.last_kernel()}: {e}") from None
        finally:
            ctx.force_tile(-1)
            ctx.force_splitk(-1)


@pytest.mark.parametrize("dt", ["f8e4m3", "f8e5m2", "bf16", "f16"])
def test_reference_sums_over_random_layouts(contexts, dt):
    """with the context switched to the reference's arithmetic, narrow-float products store the reference's bytes
    (the oracle's reference-faithful product) over any layout"""
    from gpu_util import run_product
    from test_emu_reference_sums_cpu import same_bytes
    g = np.random.default_rng(8000 + sum(map(ord, dt)))
    for n in range(2 * ROUNDS):
        op, lv, rv = product_case(g)
        ctx = contexts["end" if n % 2 == 0 else "start"]
        a = H.random_storage(dt, max(lv.span(), 1), 100 + n, 0.5 if dt == "f8e4m3" else 1.0)
        b = H.random_storage(dt, max(rv.span(), 1), 200 + n, 0.5 if dt == "f8e4m3" else 1.0)
        md = H.dot_md(lv, rv) if op == "dot" else H.matmul_md(lv, rv)
        ctx.set_reference_sums(True)
        try:
            got = run_product(ctx, op, dt, a, b, md)
            kernel = ctx.last_kernel()
        finally:
            ctx.set_reference_sums(False)
        want = (oracle.dot_asis if op == "dot" else oracle.matmul_asis)(dt, a, b, md)
        bad = same_bytes(dt, got, want)
        assert kernel == f"reference_sums_{dt}" or got.size == 0, kernel
        assert bad.size == 0, (f"{op} {dt} case {n}: lhs {lv.shape} {lv.strides} +{lv.offset}, rhs {rv.shape} {rv.strides} +{rv.offset}: "
                               f"{bad.size} of {got.size} outputs differ, first at {bad[:5]}")


def test_the_entry_point_that_allocates_nothing_over_random_shapes(contexts):
    """hodu_rocm_dot_bf16_f8e4m3w_noalloc against the allocating entry point: the same kernel and the same bytes, from
    one row against a small weight to shapes that are cut along K through the static scratch"""
    from test_zz_no_alloc import both
    g = np.random.default_rng(9000)
    for n in range(2 * ROUNDS):
        m = dims(g, [1, 2, 4, 5, 12, 16, 17, 64, 128, 200])
        k = dims(g, [64, 128, 192, 256, 512, 1024, 4096])
        n_cols = dims(g, [16, 48, 128, 200, 256, 512, 1040])
        while m * k * n_cols > 40_000_000:
            n_cols = max(16, n_cols // 2)
        both(contexts["end" if n % 2 == 0 else "start"], m, n_cols, k, 10 * n)


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_masked_softmax_over_random_layouts(contexts, dt):
    from test_zx_softmax_masked import check as check_masked_softmax
    g = np.random.default_rng(9500 + sum(map(ord, dt)))
    for n in range(3 * ROUNDS):
        nd = int(g.integers(1, 5))
        shape = [dims(g, [1, 2, 3, 5, 8, 17, 33, 64, 130, 700]) for _ in range(nd)]
        while int(np.prod(shape, dtype=np.int64)) > 60_000:
            shape[int(np.argmax(shape))] //= 2
        v = random_view(g, shape)
        keep = int(g.integers(1, nd + 1))
        mask_shape = [e if g.random() < 0.6 else 1 for e in shape[nd - keep:]]
        mask_shape[-1] = shape[-1]  # (the helper opens entry 0 of every mask row)
        causal = nd >= 2 and bool(g.integers(2))
        ctx = contexts["end" if n % 2 == 0 else "start"]
        try:
            check_masked_softmax(ctx, dt, v, mask_shape, causal=causal, seed=n)
        except AssertionError as e:
            raise AssertionError(f"masked softmax {dt} case {n}: {v.shape} {v.strides} +{v.offset}, mask {mask_shape}, causal {causal}: {e}") from None


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "bf16_f8e4m3w", "i32_i8i8"])
def test_decode_shapes_over_random_sizes_and_pinned_variants(contexts, dt):
    """one to sixteen rows against a weight stored [N, K] (a Linear layer at decode) or [K, N]: the GEMV, few-rows and
    row-dense GEMV kernels at random sizes and offsets, automatic and with every shape of theirs pinned"""
    g = np.random.default_rng(10000 + sum(map(ord, dt)))
    for n in range(4 * ROUNDS):
        m = int(g.integers(1, 17))
        k = int(g.choice([64, 128, 200, 256, 520, 1024, 2048, 4096]))
        cols = int(g.choice([1, 16, 33, 128, 200, 256, 1040]))
        while m * k * cols > 8_000_000:
            cols = max(1, cols // 2)
        off = int(g.choice([0, 0, 16, 64, 3]))
        lv = V([m, k], offset=int(g.choice([0, 16, 5])))
        rv = V([cols, k], offset=off).t() if g.random() < 0.7 else V([k, cols], offset=off)
        hook = int(g.choice([-1, -1, 30, 31, 32, 33, 34, 35, 36, 37, 38, 39]))
        ctx = contexts["end" if n % 2 == 0 else "start"]
        ctx.force_tile(hook)
        try:
            check_product(ctx, "dot", dt, lv, rv, seed=n)
        except AssertionError as e:
            raise AssertionError(f"dot {dt} case {n}, hook {hook}: [{m}, {k}] +{lv.offset} x {rv.shape} {rv.strides} +{rv.offset}, "
                                 f"kernel {ctx.last_kernel()}: {e}") from None
        finally:
            ctx.force_tile(-1)


@pytest.mark.parametrize("dt", ffi.PRODUCT_DTYPES)
def test_products_of_two_long_vectors_over_random_lengths_and_strides(contexts, dt):
    """[1, K] x [K, 1] (Tensor::matmul of two 1-D tensors): K cut into chunks across workgroups, dense and strided
    vectors, ragged last chunks, offsets"""
    g = np.random.default_rng(13000 + sum(map(ord, dt)))
    scale = 0.25 if dt in ("f8e4m3", "f8e5m2") else 1.0
    for n in range(ROUNDS):
        k = int(g.integers(5000, 150_000))
        sa, sb = int(g.choice([1, 1, 2, 3])), int(g.choice([1, 1, 2, 5]))
        lv = V([1, k], [0, sa], int(g.choice([0, 16, 3])))
        rv = V([k, 1], [sb, 0], int(g.choice([0, 16, 7])))
        ctx = contexts["end" if n % 2 == 0 else "start"]
        try:
            check_product(ctx, "dot", dt, lv, rv, seed=n, scale=scale)
        except AssertionError as e:
            raise AssertionError(f"dot {dt} case {n}: K {k}, strides {sa} / {sb}, offsets {lv.offset} / {rv.offset}, "
                                 f"kernel {ctx.last_kernel()}: {e}") from None
