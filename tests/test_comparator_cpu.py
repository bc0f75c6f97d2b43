"""The float parity gate must bite: helpers.assert_close, the comparator of every bf16 / f16 / fp8 GPU parity test,
accepts a correctly f32-accumulated result and rejects three plausible kernel bugs at the sizes of the BASELINE
configurations -- one dropped k-term, one row accumulated in bf16 instead of f32 (what the reference's own narrow
path does, crates/hodu_cpu_kernels/kernels/ops_matrix.c:572-573), and one mis-decoded f8e4m3 code.

No GPU: the "kernel" here is numpy (float32 sgemm, whose summation order differs from the comparator's float64
one, like a real kernel's), sliced to a few hundred rows so the whole file runs in seconds.
"""
import numpy as np
import pytest

import helpers as H

TOL = 2e-2


def bf16_round(x):
    return H.bf16_to_f32(H.f32_to_bf16_rne(np.asarray(x, dtype=np.float32))).astype(np.float64)


def bf16_values(seed, shape, scale=1.0):
    return H.bf16_to_f32(H.f32_to_bf16_rne((H.rng(seed).standard_normal(shape) * scale).astype(np.float32)))


def fp8_weight_codes(seed, n, k):
    """N(0, 0.02) scaled so that max|W| maps to 448, OCP e4m3 codes (BASELINE configs 3 and 5)"""
    w = H.rng(seed).standard_normal((n, k)).astype(np.float32) * 0.02
    return H.f32_to_ocp_e4m3_rne(np.clip(w * (448.0 / np.abs(w).max()), -448, 448))


def exact(a, b):
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    return a64 @ b64, np.abs(a64) @ np.abs(b64)


# (name, rows of the slice, K, N, activation scale, weight kind)
SHAPES = [
    ("config 2: one batch, 1024^3, N(0,1)/32", 256, 1024, 1024, 1 / 32, "bf16/32"),
    ("config 3: M = 256 against the f8e4m3 weight", 256, 4096, 4096, 1.0, "f8"),
    ("config 5 down: 128 rows, K = 14336", 128, 14336, 4096, 0.3, "bf16*0.02"),
    ("config 5 up, f8e4m3 weight: 128 rows, K = 4096", 128, 4096, 14336, 1.0, "f8"),
]


def operands(m, k, n, xscale, wkind):
    x = bf16_values(11, (m, k), xscale)
    if wkind == "f8":
        codes = fp8_weight_codes(12, n, k)
        return x, H.ocp_e4m3_decode(codes).T.copy(), codes
    w = bf16_values(12, (k, n), 1 / 32 if wkind == "bf16/32" else 0.02)
    return x, w, None


@pytest.mark.parametrize("name,m,k,n,xscale,wkind", SHAPES, ids=[s[0].split(":")[0] for s in SHAPES])
def test_gate_accepts_f32_accumulation_and_rejects_three_bugs(name, m, k, n, xscale, wkind):
    x, w, codes = operands(m, k, n, xscale, wkind)
    want, sumabs = exact(x, w)
    good = bf16_round(x @ w)  # f32 accumulate (sgemm's blocked order), one rounding
    H.assert_close(good, want, sumabs, k, TOL, name)
    frac = H.floor_fraction(want, sumabs, k, TOL)
    assert frac < 0.02, f"{100 * frac:.1f} % of elements on the floor: the gate is not per-element any more"

    # (1) k-term k0 missing from ONE output row
    k0, row = k // 3, m // 2
    dropped = good.copy()
    dropped[row] = bf16_round((x[row] @ w) - x[row, k0] * w[k0])
    with pytest.raises(AssertionError):
        H.assert_close(dropped, want, sumabs, k, TOL, name)

    # (2) ONE row accumulated in bf16, truncating after every multiply and add like hodu_cpu_dot_bf16
    def trunc(v):
        return (np.asarray(v, dtype=np.float32).view(np.uint32) & 0xFFFF0000).view(np.float32)
    acc = np.zeros(n, dtype=np.float32)
    for kk in range(k):
        acc = trunc(acc + trunc(x[row, kk] * w[kk]))
    narrow = good.copy()
    narrow[row] = acc
    with pytest.raises(AssertionError):
        H.assert_close(narrow, want, sumabs, k, TOL, name)

    # (3) the largest f8e4m3 code (0x7E = 448, sign either way) decoded as its neighbour 0x7D = 416
    if codes is not None:
        hit = np.argwhere((codes & 0x7F) == 0x7E)
        assert len(hit) >= 1  # the scaling puts max|W| exactly there
        w_bad = w.copy()
        for nn, kk in hit:
            w_bad[kk, nn] = np.sign(w[kk, nn]) * 416.0
        wrong = bf16_round(x @ w_bad)
        assert np.count_nonzero(wrong != good) <= m * len(hit)
        with pytest.raises(AssertionError):
            H.assert_close(wrong, want, sumabs, k, TOL, name)


def test_f32_gate_at_config1_size():
    """1e-5 for f32: a float32 sum in another order passes, a dropped term in one row does not"""
    g = H.rng(5)
    a, b = g.standard_normal((512, 512)).astype(np.float32), g.standard_normal((512, 512)).astype(np.float32)
    want, sumabs = exact(a, b)
    good = (a @ b).astype(np.float64)
    H.assert_close(good, want, sumabs, 512, 1e-5, "f32 512^3")
    seq = np.zeros((512, 512), dtype=np.float32)  # the reference's ascending-k order
    for kk in range(512):
        seq += np.outer(a[:, kk], b[kk])
    H.assert_close(good, seq.astype(np.float64), sumabs, 512, 1e-5, "sgemm against sequential-k")
    bad = good.copy()
    bad[7] = ((a[7] @ b) - a[7, 100] * b[100]).astype(np.float64)
    with pytest.raises(AssertionError):
        H.assert_close(bad, want, sumabs, 512, 1e-5, "f32 512^3")
