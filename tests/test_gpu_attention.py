"""GPU parity of hodu_rocm_attention (softmax(q k^T * scale [causal]) v as one kernel) against the function computed in
float64 on the exactly widened inputs, with the scale the kernel receives (the scalar in the storage type).
Tolerance: the output is a convex combination of v rows delivered in bf16 / f16; probabilities are rounded to the
storage type once as the second product's operand (relative 2^-9 / 2^-11) and the output once more, so the bar is the
products' 2e-2, relative to max(|want|, mean |v| / sqrt(n_eff)) with n_eff = 1 / sum p^2 the effective number of keys
the row attends -- the size of a sum of n_eff weighted v rows that may cancel, which is what a relative error of
every p scales with."""
import numpy as np
import pytest

import helpers as H
from hodu_amd import ffi

pytestmark = pytest.mark.gpu
V = H.View


@pytest.fixture(scope="module")
def ctx():
    c = ffi.Context(0)
    yield c
    c.close()


def attention_md(batch, sq, sk, d, qv, kv, vv):
    nb = len(batch)
    return [nb] + list(batch) + [sq, sk, d] + qv.strides + kv.strides + vv.strides + [qv.offset, kv.offset, vv.offset]


def reference(q, k, v, scale, causal):
    s = q @ np.swapaxes(k, -1, -2) * scale
    if causal:
        i, j = np.arange(s.shape[-2])[:, None], np.arange(s.shape[-1])[None, :]
        s = np.where(j > i, -np.inf, s)
    e = np.exp(s - s.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    return p @ v, 1.0 / (p * p).sum(-1)  # the effective number of keys a row attends


def narrow(dt, x):
    return (H.f32_to_bf16_rne if dt == "bf16" else H.f16_bits)(np.ascontiguousarray(x, dtype=np.float32))


def check_attention(ctx, dt, batch, sq, sk, causal, seed=0, qv=None, kv=None, vv=None, vscale=1.0, qscale=1.0, ramp=None, d=128):
    """ramp: logits that grow along the keys (contiguous operands only) -- q rows all point along one direction and
    key j is that direction times ramp * f(j), f rising from 0 to 1 (or falling, ramp < 0), plus noise"""
    qv = qv or V(list(batch) + [sq, d])
    kv = kv or V(list(batch) + [sk, d])
    vv = vv or V(list(batch) + [sk, d])
    q = H.random_storage(dt, qv.span(), 100 + seed, qscale)
    k = H.random_storage(dt, kv.span(), 200 + seed, 1.0)
    v = H.random_storage(dt, vv.span(), 300 + seed, vscale)
    if ramp is not None:
        rng = np.random.default_rng(400 + seed)
        u = np.ones(d, np.float32)
        qa = u + 0.1 * rng.standard_normal((int(np.prod(batch, dtype=int)) * sq, d)).astype(np.float32)
        f = np.arange(sk, dtype=np.float32) / max(sk - 1, 1)
        f = f if ramp > 0 else 1.0 - f
        # q . k_j * d^-1/2 ~ sqrt(d) * |ramp| * f(j)
        ka = (abs(ramp) * f)[:, None] * u[None, :] + 0.1 * rng.standard_normal((sk, d)).astype(np.float32)
        q = narrow(dt, qa).reshape(-1)
        k = narrow(dt, np.tile(ka, (int(np.prod(batch, dtype=int)), 1))).reshape(-1)
    scale_bits = (H.f32_to_bf16_rne if dt == "bf16" else H.f16_bits)(np.array([1.0 / np.sqrt(d)], dtype=np.float32))
    scale = float(H.widen(dt, scale_bits)[0])
    n_out = int(np.prod(list(batch) + [sq, d]))
    dq, dk, dv = ctx.upload(q), ctx.upload(k), ctx.upload(v)
    dout = ctx.alloc(n_out * 2)
    ctx.fill(dout, 0xFF)
    ctx.attention(dt, dq, dk, dv, dout, attention_md(batch, sq, sk, d, qv, kv, vv), scale_bits, causal)
    assert ctx.last_kernel() == f"attention_fwd_{dt}" + ("_d64" if d == 64 else "")
    got = H.widen(dt, ctx.download(dout, np.uint16, n_out)).reshape(list(batch) + [sq, d])
    for b in (dq, dk, dv, dout):
        b.free()
    qa, ka, va = (H.widen(dt, view.take(x)).reshape(view.shape) for view, x in ((qv, q), (kv, k), (vv, v)))
    want, attended = reference(qa, ka, va, scale, causal)
    assert np.all(np.isfinite(got))
    floor = np.abs(va).mean() / np.sqrt(attended)[..., None]
    rel = np.abs(got - want) / np.maximum(np.abs(want), floor)
    assert rel.max() <= 2e-2, f"attention {dt} {batch} {sq}x{sk} causal={causal}: max rel err {rel.max():.3e}"


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("causal", [False, True])
def test_small_shapes(ctx, dt, causal):
    check_attention(ctx, dt, [], 32, 64, causal, seed=1)        # one wavefront's rows, one key block
    check_attention(ctx, dt, [2], 128, 128, causal, seed=2)     # a full query block, two key blocks
    check_attention(ctx, dt, [3], 100, 70, causal, seed=3)      # ragged in both directions
    check_attention(ctx, dt, [2, 2], 300, 260, causal, seed=4)  # several query blocks, two batch dims


@pytest.mark.parametrize("causal", [False, True])
def test_views(ctx, causal):
    """heads interleaved in memory ([S, H, D] storage viewed as [H, S, D]), a shared k / v across a batch dim, offsets"""
    sq = sk = 96
    qv = V([sq, 4, 128], offset=128).t(0, 1)  # [4, sq, 128] with row stride 4 * 128
    kv = V([sk, 4, 128]).t(0, 1)
    vv = V([sk, 4, 128], offset=256).t(0, 1)
    check_attention(ctx, "bf16", [4], sq, sk, causal, seed=5, qv=qv, kv=kv, vv=vv)
    kb = V([sk, 128]).broadcast_to([3, sk, 128])
    check_attention(ctx, "bf16", [3], 64, sk, causal, seed=6, kv=kb, vv=V([sk, 128], offset=8).broadcast_to([3, sk, 128]))


def test_long_sequences(ctx):
    check_attention(ctx, "bf16", [2], 1024, 1024, True, seed=7)
    check_attention(ctx, "bf16", [2], 200, 2048, False, seed=8)
    check_attention(ctx, "bf16", [1], 2048, 300, True, seed=9)   # Sq > Sk with the mask: late rows see every key


def test_large_logits_and_values(ctx):
    check_attention(ctx, "bf16", [2], 128, 192, False, seed=10, vscale=100.0)


@pytest.mark.parametrize("causal", [False, True])
def test_maxima_that_keep_moving(ctx, causal):
    """the exponent reference of a row follows its maximum lazily (it moves only when a block exceeds it by 2^8): logits
    that climb a little with every block (below the threshold per block, far above it in total), that climb steeply,
    and that fall from a large first value; and logits with a large spread"""
    check_attention(ctx, "bf16", [2], 160, 1024, causal, seed=11, ramp=6.0)     # ~ +2 per 32 keys, 68 in total
    check_attention(ctx, "bf16", [2], 160, 512, causal, seed=12, ramp=40.0)     # ~ +28 per 32 keys
    check_attention(ctx, "f16", [1], 96, 512, causal, seed=13, ramp=-10.0)      # the first keys dominate
    check_attention(ctx, "bf16", [2], 128, 640, causal, seed=14, qscale=6.0)    # random logits of std ~ 6


@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("causal", [False, True])
def test_head_dim_64(ctx, dt, causal):
    check_attention(ctx, dt, [2], 128, 128, causal, seed=20, d=64)
    check_attention(ctx, dt, [3], 77, 203, causal, seed=21, d=64)      # ragged rows and keys
    check_attention(ctx, dt, [2, 2], 300, 1000, causal, seed=22, d=64)  # many key blocks: the fast loop and its tail
    check_attention(ctx, dt, [1], 1, 1, causal, seed=23, d=64)
    check_attention(ctx, dt, [2], 128, 640, causal, seed=24, qscale=6.0, d=64)
    check_attention(ctx, dt, [1], 200, 777, causal, seed=25, ramp=2.0, d=64)  # the reference maximum keeps moving


def test_head_dim_64_strided_views(ctx):
    sq, sk = 130, 190
    qv = V([sq, 4, 64], offset=64).t(0, 1)  # [4, sq, 64] with row stride 4 * 64
    kv = V([sk, 4, 64]).t(0, 1)
    vv = V([sk, 4, 64], offset=128).t(0, 1)
    check_attention(ctx, "bf16", [4], sq, sk, True, seed=26, qv=qv, kv=kv, vv=vv, d=64)


def test_unsupported_calls_are_refused(ctx):
    q, out = ctx.upload(np.zeros(64 * 64, np.uint16)), ctx.alloc(64 * 64 * 2)
    one = np.array([0x3F80], np.uint16)
    with pytest.raises(ffi.HoduRocmError, match="head dim 64 or 128"):
        ctx.attention("bf16", q, q, q, out, attention_md([], 64, 64, 32, V([64, 32]), V([64, 32]), V([64, 32])), one)
    with pytest.raises(ffi.HoduRocmError, match="dense"):
        ctx.attention("bf16", q, q, q, out, attention_md([], 8, 8, 128, V([8, 128], [1, 8]), V([8, 128]), V([8, 128])), one)
    with pytest.raises(ffi.HoduRocmError, match="words"):
        ctx.attention("bf16", q, q, q, out, [0, 8, 8, 128, 128, 1], one)
    ok = attention_md([], 8, 8, 128, V([8, 128]), V([8, 128]), V([8, 128]))
    for bits in (0xBF80, 0x0000, 0x7F80, 0x7FC0):  # -1, 0, inf, nan: the kernel takes the row maximum before scaling
        with pytest.raises(ffi.HoduRocmError, match="positive finite scale"):
            ctx.attention("bf16", q, q, q, out, ok, np.array([bits], np.uint16))
    q.free(); out.free()
