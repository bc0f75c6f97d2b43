"""GPU parity of hodu_rocm_attention_masked: scaled_dot_product_attention with an attn_mask
(crates/hodu_nn/src/modules/attention.rs:50-56) as one kernel, against the function in float64 on the exactly widened
inputs.  (The file name sorts it behind the tests of the kernels that have a longer history on the hardware; these cases
also run against the CPU build of the same kernel source, tests/test_emu_gpu_suites_cpu.py.)

The float64 function fills a masked score -- attn_mask == 0, or key > query with is_causal -- with what the reference's
masked_fill writes in the tensor's dtype (get_neg_inf, attention.rs:88-96, through full_like: -65504 in f16, -65536 in
bf16) and runs the softmax over every key, so a row masked entirely is the uniform average of v.  Tolerance as in
test_gpu_attention.py: 2e-2 relative to max(|want|, mean |v| / sqrt(n_eff))."""
import numpy as np
import pytest

import helpers as H
from hodu_amd import ffi
from test_gpu_attention import attention_md

pytestmark = pytest.mark.gpu
V = H.View
FILL = {"bf16": -65536.0, "f16": -65504.0}


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def reference(q, k, v, scale, causal, keep, fill):
    s = q @ np.swapaxes(k, -1, -2) * scale
    filled = np.broadcast_to(keep == 0, s.shape).copy()
    if causal:
        i, j = np.arange(s.shape[-2])[:, None], np.arange(s.shape[-1])[None, :]
        filled |= j > i
    s = np.where(filled, fill, s)
    e = np.exp(s - s.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    return p @ v, 1.0 / (p * p).sum(-1), p, filled


def check(ctx, dt, batch, sq, sk, mask_view, causal=False, seed=0, d=128, density=0.6, closed_rows=(), close_key0=False,
          mask_dt="u8", qv=None, kv=None, vv=None, edit=None):
    """mask_view: a helpers.View over the mask's storage whose shape broadcasts (right-aligned) against
    batch + [sq, sk]; closed_rows: rows of the flattened mask view masked entirely"""
    qv = qv or V(list(batch) + [sq, d])
    kv = kv or V(list(batch) + [sk, d])
    vv = vv or V(list(batch) + [sk, d])
    q, k, v = (H.random_storage(dt, view.span(), base + seed, 1.0) for view, base in ((qv, 100), (kv, 200), (vv, 300)))
    g = np.random.default_rng(500 + seed)
    keep_logical = (g.random(mask_view.shape) < density).astype(np.uint8)
    if not close_key0:
        keep_logical[..., 0] = 1
    for r in closed_rows:
        keep_logical.reshape(-1, mask_view.shape[-1])[r, :] = 0
    if edit:
        edit(keep_logical)
    storage = np.zeros(max(mask_view.span(), 1), np.uint8)
    storage[mask_view.take(np.arange(storage.size)).ravel()] = keep_logical.ravel()  # scatter the logical mask into its storage
    scores_shape = list(batch) + [sq, sk]
    full = mask_view.broadcast_to(scores_shape)
    scale_bits = (H.f32_to_bf16_rne if dt == "bf16" else H.f16_bits)(np.array([1.0 / np.sqrt(d)], dtype=np.float32))
    scale = float(H.widen(dt, scale_bits)[0])
    n_out = int(np.prod(list(batch) + [sq, d]))
    dq, dk, dv, dm = ctx.upload(q), ctx.upload(k), ctx.upload(v), ctx.upload(storage)
    dout = ctx.alloc(n_out * 2)
    ctx.fill(dout, 0xFF)
    ctx.attention(dt, dq, dk, dv, dout, attention_md(batch, sq, sk, d, qv, kv, vv), scale_bits, causal,
                  mask=dm, mask_strides=full.strides, mask_offset=full.offset, mask_dt=mask_dt)
    assert ctx.last_kernel() == f"attention_masked_fwd_{dt}" + ("_d64" if d == 64 else "")
    got = H.widen(dt, ctx.download(dout, np.uint16, n_out)).reshape(list(batch) + [sq, d]).astype(np.float64)
    for b in (dq, dk, dv, dm, dout):
        b.free()
    qa, ka, va = (H.widen(dt, view.take(x)).reshape(view.shape).astype(np.float64) for view, x in ((qv, q), (kv, k), (vv, v)))
    keep = full.take(storage).reshape(scores_shape)
    want, attended, p, filled = reference(qa, ka, va, scale, causal, keep, FILL[dt])
    assert np.all(np.isfinite(got))
    floor = np.abs(va).mean() / np.sqrt(attended)[..., None]
    rel = np.abs(got - want) / np.maximum(np.abs(want), floor)
    assert rel.max() <= 2e-2, f"masked attention {dt} {batch} {sq}x{sk} causal={causal}: max rel err {rel.max():.3e}"
    return p, filled


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("causal", [False, True])
def test_masks_of_every_broadcast_shape(ctx, dt, causal):
    batch, sq, sk = [2, 3], 100, 150
    for n, shape in enumerate(([2, 3, sq, sk], [2, 1, 1, sk], [1, 1, sq, sk], [sq, sk], [sk], [2, 3, 1, sk])):
        check(ctx, dt, batch, sq, sk, V(shape), causal, seed=n)


@pytest.mark.parametrize("d", [64, 128])
def test_ragged_and_tiny_shapes(ctx, d):
    check(ctx, "bf16", [], 1, 1, V([1, 1]), seed=10, d=d)
    check(ctx, "bf16", [1], 33, 31, V([33, 31]), seed=11, d=d)          # less than one key half
    check(ctx, "f16", [2], 130, 65, V([2, 1, 65]), True, seed=12, d=d)  # one key past a block; causal with Sq > Sk
    check(ctx, "bf16", [3], 77, 203, V([3, 77, 203]), True, seed=13, d=d)
    check(ctx, "bf16", [2], 300, 1000, V([2, 1, 1000]), seed=14, d=d)   # many key blocks


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_rows_masked_entirely_average_every_key(ctx, dt):
    """all of a row's keys filled with the same finite value: uniform weights, over the keys behind the diagonal too"""
    sq, sk = 70, 96
    p, filled = check(ctx, dt, [2], sq, sk, V([2, sq, sk]), seed=20, closed_rows=(0, 5, 69, 70, 139))
    assert np.allclose(p[0, 5], 1.0 / sk) and np.allclose(p[1, 69], 1.0 / sk)
    # with the causal mask: row 3 attends keys 0..3 and row 40 keys 0..40; a mask that closes exactly those (and leaves
    # the keys behind the diagonal open) closes the row
    def close_what_the_diagonal_leaves(keep):
        keep[3, :4] = 0
        keep[3, 4:] = 1
        keep[40, :41] = 0
        keep[40, 41:] = 1
    pc, filled = check(ctx, dt, [1], sq, sk, V([sq, sk]), True, seed=21, edit=close_what_the_diagonal_leaves)
    assert np.allclose(pc[0, 3], 1.0 / sk) and np.allclose(pc[0, 40], 1.0 / sk) and not np.allclose(pc[0, 41], 1.0 / sk)
    # rows whose first key is masked, and masks that leave few keys
    check(ctx, dt, [2], sq, sk, V([2, 1, sk]), seed=22, close_key0=True, density=0.1)
    check(ctx, dt, [2], sq, 200, V([2, sq, 200]), True, seed=23, close_key0=True, density=0.05)


def test_strided_masks_views_and_byte_dtypes(ctx):
    sq, sk = 96, 130
    check(ctx, "bf16", [4], sq, sk, V([sk, sq]).t(), seed=30)                        # keys strided, rows dense
    check(ctx, "bf16", [4], sq, sk, V([4, sq, sk], offset=7), seed=31, mask_dt="bool")
    check(ctx, "f16", [4], sq, sk, V([sq, 4, sk]).t(0, 1), True, seed=32, mask_dt="i8")
    qv = V([sq, 4, 128], offset=128).t(0, 1)  # heads interleaved in memory
    kv = V([sk, 4, 128]).t(0, 1)
    vv = V([sk, 4, 128], offset=256).t(0, 1)
    check(ctx, "bf16", [4], sq, sk, V([1, sq, sk]), True, seed=33, qv=qv, kv=kv, vv=vv)


def test_refusals(ctx):
    d = 128
    q = ctx.upload(H.random_storage("bf16", 64 * d, 1, 1.0))
    out, m = ctx.alloc(64 * d * 2), ctx.upload(np.ones(64 * 64, np.uint8))
    scale = H.f32_to_bf16_rne(np.array([0.1], np.float32))
    md = attention_md([], 64, 64, d, V([64, d]), V([64, d]), V([64, d]))
    with pytest.raises(ffi.HoduRocmError) as e:
        ctx.attention("bf16", q, q, q, out, md, scale, False, mask=m, mask_strides=[64, 1], mask_dt="f32")
    assert e.value.status == ffi.UNSUPPORTED
    with pytest.raises(ffi.HoduRocmError) as e:
        ctx.attention("bf16", q, q, q, out, md, scale, False, mask=m, mask_strides=[64, 2])  # reaches past the mask
    assert e.value.status == ffi.INVALID_ARG
    with pytest.raises(ffi.HoduRocmError) as e:
        ctx.attention("bf16", q, q, q, out, md, scale, False, mask=m, mask_strides=[1])
    assert e.value.status == ffi.INVALID_ARG
    for b in (q, out, m):
        b.free()
