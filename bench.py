#!/usr/bin/env python3
"""Benchmark of the MI355X matmul / dot / to_dtype backend on BASELINE.json's five configurations.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs c1,c2,c3,c4,c5,...] [--no-cpu] [--only KEY]

A "step" is one pass of the hot path over one batch of synthetic input: one matmul / dot call through the C ABI
with operands resident in HBM.  The headline (`value`, `ms_per_step`, `roofline`, `cpu_baseline`) is the largest
configuration, BASELINE.json configs[4] (the transformer-MLP-shaped broadcast matmul), on its down projection with
bf16 weights: X[8,512,14336] x W_down (a transposed view of [4096,14336], broadcast over the batch), 481 GFLOP per
step; it is timed over exactly K launches after W untimed ones.  Every other configuration -- the 4096^3-class
products and the M = 1 GEMV the targets are stated on among them -- is measured in the same run (at least 20 timed
launches after at least 10 untimed ones, whatever K and W are) and reported, one compact row each, under
`roofline.per_config`: TFLOP/s against the MFMA dense peak of the type the matrix cores consume, or GB/s against the
HBM peak for the M <= 16 shapes; `config.north_star` repeats the three rows the targets name.

Timing: HIP events recorded on the stream the kernels are launched on (the context's stream), launches issued back
to back from C; `achieved` = algorithmic flops (or bytes) per launch / average launch duration.  The M <= 16
configurations rotate through enough distinct weight buffers to exceed the 256 MB Infinity Cache, so their reads
come from HBM.  Before a row is reported, rows of the output buffer the timed launches wrote are downloaded and
compared with the CPU oracle on the same inputs (bit-exact for integers, 1e-5 for f32, 2e-2 for bf16 / fp8, with the
comparator of the parity tests); a mismatch aborts the run.

cpu_baseline: hodu's CPU path for the same configuration, timed on this host on a bounded sample under the
reference's own threading policy: the reference's C kernels compiled by oracle/Makefile where that library is
present (kind "reference"), this repository's restatement otherwise (kind "port").  `cpu_baseline.per_config` holds
one row per configuration.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

# published MI355X peaks (dense)
PEAK = {"bf16": 2500.0, "f16": 2500.0, "fp8": 5000.0, "int8": 5000.0, "f32": 157.3, "f64": 78.6}  # TFLOP/s or TOP/s
HBM_PEAK_GBS = 8000.0
INFINITY_CACHE_BYTES = 256 << 20

# HBM bytes per launch from the rocprofv3 --pmc runs summarised under profiles/ (FETCH_SIZE + WRITE_SIZE, each scaled
# by what the counter reads for a plain copy of known size).  A figure is reported only for the (kernel, configuration)
# pair it was measured on, together with the file that holds the measurement; anything else reports null.
_TRAFFIC_FILE = "profiles/traffic_counters_all_bench_rows.txt"
MEASURED_TRAFFIC = {
    # "kernel@config": (bytes per launch: FETCH_SIZE + WRITE_SIZE, each scaled by what it reads for a plain copy; summary file)
    "mfma_bf16_pipe256x256mi16_KK@c5_down_bf16": (734.63e6, _TRAFFIC_FILE),
    "mfma_bf16_pipe256x256mi16_KM@c5_up_bf16": (884.02e6, _TRAFFIC_FILE),
    "mfma_bf16_f8w_pipe256x256mi16_KK@c3_m4096": (200.56e6, _TRAFFIC_FILE),
    "mfma_bf16_f8w_pipe128x128_KK_splitk4@c3_m256": (68.94e6, _TRAFFIC_FILE),
    "skinny_bf16_f8w_splitk@c3_m16": (22.19e6, _TRAFFIC_FILE),
    "gemv_bf16_f8w_walk@c3_m1": (16.89e6, _TRAFFIC_FILE),
    "gemv_bf16_f8w_walk@gemv_14336x4096": (58.67e6, _TRAFFIC_FILE),
    "mfma_f8e4m3_pipe256x256mi16_KK@f8_4096": (117.08e6, _TRAFFIC_FILE),
    "mfma_i32_i8i8_pipe128x128_KM@c4": (41.78e6, _TRAFFIC_FILE),
    "mfma_bf16_pipe256x256mi16_KK@c2": (100.43e6, _TRAFFIC_FILE),
}


def traffic_of(kernel, key):
    hit = MEASURED_TRAFFIC.get(f"{kernel}@{key}")
    return (hit[0], hit[1]) if hit else (None, None)


def bf16(x):
    import helpers as H
    return H.f32_to_bf16_rne(np.asarray(x, dtype=np.float32))


def normal(seed, n, scale=1.0):
    g = np.random.default_rng(seed)
    out = g.standard_normal(n, dtype=np.float32)
    if scale != 1.0:
        out *= np.float32(scale)
    return out


def fp8_weights(seed, n, top=448.0):
    import helpers as H
    w = normal(seed, n, 0.02)
    s = top / float(np.abs(w).max())
    return H.f32_to_ocp_e4m3_rne(np.clip(w * s, -448, 448))


class Case:
    """one timed launch shape"""

    def __init__(self, key, label, op, name, lv, rv, make_a, make_b, flops, alg_bytes, bound, peak_key, rotate=False,
                 fused=()):
        self.key, self.label, self.op, self.name = key, label, op, name
        self.lv, self.rv, self.make_a, self.make_b = lv, rv, make_a, make_b
        self.flops, self.alg_bytes, self.bound, self.peak_key, self.rotate = flops, alg_bytes, bound, peak_key, rotate
        self.fused = tuple(fused)  # element-wise steps fused into the store: "bias", "scale", "relu"

    def with_steps(self, key, label, fused):
        """the same launch with the caller's next element-wise kernels fused in (not a BASELINE configuration)"""
        return Case(key, label, self.op, self.name, self.lv, self.rv, self.make_a, self.make_b, self.flops,
                    self.alg_bytes, self.bound, self.peak_key, self.rotate, fused)


def build_cases(which):
    import helpers as H
    V = H.View
    cases = []
    if "c1" in which:
        n = 512
        cases.append(Case("c1", "C1 f32 dot 512x512x512", "dot", "f32", V([n, n]), V([n, n]),
                          lambda n=n: normal(101, n * n), lambda n=n: normal(102, n * n),
                          2.0 * n ** 3, 3 * n * n * 4, "mfma", "f32"))
    if "c2" in which:
        B, n = 16, 1024
        cases.append(Case("c2", "C2 bf16 matmul [16,1024,1024]x[16,1024,1024]^T-view", "matmul", "bf16",
                          V([B, n, n]), V([B, n, n]).t(),
                          lambda B=B, n=n: bf16(normal(201, B * n * n, 1 / 32)),
                          lambda B=B, n=n: bf16(normal(202, B * n * n, 1 / 32)),
                          2.0 * B * n ** 3, 3 * B * n * n * 2, "mfma", "bf16"))
    if "c3" in which:
        n = k = 4096
        for m in (1, 16, 256, 4096):
            cases.append(Case(f"c3_m{m}", f"C3 bf16[{m},4096] x f8e4m3[4096,4096]^T-view (fused to_dtype)", "dot",
                              "bf16_f8e4m3w", V([m, k]), V([n, k]).t(),
                              (lambda m=m, k=k: bf16(normal(302, m * k))), (lambda n=n, k=k: fp8_weights(301, n * k)),
                              2.0 * m * n * k, n * k + m * k * 2 + m * n * 2,
                              "hbm" if m <= 16 else "mfma", "bf16", rotate=(m <= 16)))
    if "c3" in which:
        # not a BASELINE configuration: the same M = 1 product against the 14336 x 4096 weight of config 5, where the
        # launch and ramp-up that dominate a 2 us transfer are a smaller share
        n, k = 14336, 4096
        cases.append(Case("gemv_14336x4096", "bf16[1,4096] x f8e4m3[14336,4096]^T-view (fused to_dtype; not a BASELINE config)",
                          "dot", "bf16_f8e4m3w", V([1, k]), V([n, k]).t(),
                          (lambda k=k: bf16(normal(302, k))), (lambda n=n, k=k: fp8_weights(303, n * k)),
                          2.0 * n * k, n * k + k * 2 + n * 2, "hbm", "bf16", rotate=True))
    if "f8" in which:
        # not a BASELINE configuration: hodu's own f8e4m3 x f8e4m3 -> f8e4m3 product at 4096^3 on the native 8-bit
        # matrix instruction, reported against the fp8 dense peak
        n = 4096
        cases.append(Case("f8_4096", "f8e4m3 dot 4096^3 (native fp8 MFMA), rhs a transposed view", "dot", "f8e4m3",
                          V([n, n]), V([n, n]).t(), lambda n=n: fp8_weights(601, n * n, top=8.0),
                          lambda n=n: fp8_weights(602, n * n, top=8.0), 2.0 * n ** 3, 3 * n * n, "mfma", "fp8"))
        # the plain bf16 product at 4096^3 (the size the bf16 target is stated on; config 3's M = 4096 case with the
        # weight already in bf16)
        cases.append(Case("bf16_4096", "bf16 dot 4096^3, rhs a transposed view (the target's size; not a BASELINE config)",
                          "dot", "bf16", V([n, n]), V([n, n]).t(), lambda n=n: bf16(normal(611, n * n)),
                          lambda n=n: bf16(normal(612, n * n, 0.02)), 2.0 * n ** 3, 3 * n * n * 2, "mfma", "bf16"))
    if "f64" in which:
        # not a BASELINE configuration: hodu's f64 dot at 2048^3 on the f64 matrix instruction
        n = 2048
        cases.append(Case("f64_2048", "f64 dot 2048^3 (not a BASELINE config)", "dot", "f64", V([n, n]), V([n, n]),
                          lambda n=n: normal(701, n * n).astype(np.float64), lambda n=n: normal(702, n * n).astype(np.float64),
                          2.0 * n ** 3, 3 * n * n * 8, "mfma", "f64"))
    if "c4" in which:
        n = 2048
        ints = lambda seed, n=n: np.random.default_rng(seed).integers(-127, 128, n * n).astype(np.int8)  # noqa: E731
        cases.append(Case("c4", "C4 i8-valued i32 dot 2048^3 (fused to_dtype)", "dot", "i32_i8i8", V([n, n]), V([n, n]),
                          lambda: ints(401), lambda: ints(402), 2.0 * n ** 3, 2 * n * n + n * n * 4, "mfma", "int8"))
    if "c5" in which:
        b, s, d, f = 8, 512, 4096, 14336
        for wk in ("bf16", "f8e4m3"):
            name = "bf16" if wk == "bf16" else "bf16_f8e4m3w"
            wbytes = d * f * (2 if wk == "bf16" else 1)
            mk_w = (lambda seed, d=d, f=f: (lambda: bf16(normal(seed, d * f, 0.02)))) if wk == "bf16" else \
                (lambda seed, d=d, f=f: (lambda: fp8_weights(seed, d * f)))
            cases.append(Case(f"c5_up_{wk}", f"C5 up   bf16[8,512,4096] x {wk}[4096,14336] (batch-broadcast)", "matmul",
                              name, V([b, s, d]), V([d, f]).broadcast_to([b, d, f]),
                              lambda b=b, s=s, d=d: bf16(normal(501, b * s * d)), mk_w(502),
                              2.0 * b * s * d * f, b * s * d * 2 + wbytes + b * s * f * 2, "mfma", "bf16"))
            cases.append(Case(f"c5_down_{wk}", f"C5 down bf16[8,512,14336] x {wk}[4096,14336]^T-view (batch-broadcast)",
                              "matmul", name, V([b, s, f]), V([d, f]).t().broadcast_to([b, f, d]),
                              lambda b=b, s=s, f=f: bf16(normal(504, b * s * f, 0.3)), mk_w(503),
                              2.0 * b * s * d * f, b * s * f * 2 + wbytes + b * s * d * 2, "mfma", "bf16"))
    if "bwd" in which:
        # not a BASELINE configuration: the weight gradient of config 5's up projection, dW = X^T . dY with the batch
        # folded into the contraction (K = 8 * 512): both operands row-dense, the layout pair the forward never uses
        b, s_, d, f = 8, 512, 4096, 14336
        cases.append(Case("c5_up_dw_bf16", "C5 up weight gradient: bf16[4096,4096]^T-view x bf16[4096,14336] (not a BASELINE config)",
                          "dot", "bf16", V([b * s_, d]).t(), V([b * s_, f]),
                          lambda: bf16(normal(801, b * s_ * d)), lambda: bf16(normal(802, b * s_ * f, 0.05)),
                          2.0 * d * b * s_ * f, (b * s_ * d + b * s_ * f + d * f) * 2, "mfma", "bf16"))
    if "fused" in which:
        base = {c.key: c for c in build_cases({"c2", "c3", "c5"})}
        cases.append(base["c3_m1"].with_steps("c3_m1_linear", "C3 M=1 as a Linear layer: + bias fused", ("bias",)))
        cases.append(base["c3_m16"].with_steps("c3_m16_linear", "C3 M=16 as a Linear layer: + bias fused", ("bias",)))
        cases.append(base["c2"].with_steps("c2_scaled", "C2 as attention scores: * scalar fused", ("scale",)))
        cases.append(base["c5_up_bf16"].with_steps("c5_up_bf16_bias_relu", "C5 up as Linear + ReLU: + bias, relu fused",
                                                   ("bias", "relu")))
    return cases


def out_bytes(case):
    import helpers as H
    md = H.dot_md(case.lv, case.rv) if case.op == "dot" else H.matmul_md(case.lv, case.rv)
    n = md[0] * md[2] if case.op == "dot" else md[0]
    return md, n * {"f32": 4, "f64": 8, "bf16": 2, "bf16_f8e4m3w": 2, "i32_i8i8": 4, "f8e4m3": 1}[case.name]


MIN_LAUNCHES, MIN_WARMUP, SPREAD_BATCHES = 20, 10, 10


class ParityError(AssertionError):
    pass


def _sub2d(view, bshape, bidx):
    """the [rows, cols] matrix of batch `bidx` (flat index into the broadcast batch shape) of a >= 2-D view"""
    import helpers as H
    full = view.broadcast_to(list(bshape) + view.shape[-2:])
    off, rem = full.offset, bidx
    for d in range(len(bshape) - 1, -1, -1):
        off += (rem % bshape[d]) * full.strides[d]
        rem //= bshape[d]
    return H.View(full.shape[-2:], full.strides[-2:], off)


def verify_case(ctx, case, a_host, b_host, out, bias_host=None, scale_host=None):
    """Rows of the buffer the timed launches wrote, against the CPU oracle on the same inputs.  Six (batch, row)
    pairs spread over the output; every column of each.  Raises ParityError on a mismatch; returns what was held."""
    import helpers as H
    import oracle
    name = case.name
    l_dt, r_dt, out_dt = {"bf16_f8e4m3w": ("bf16", "f8e4m3", "bf16"), "i32_i8i8": ("i8", "i8", "i32")}.get(name, (name,) * 3)
    lv, rv = case.lv, case.rv
    M, K, N = lv.shape[-2], lv.shape[-1], rv.shape[-1]
    bshape = list(np.broadcast_shapes(tuple(lv.shape[:-2]), tuple(rv.shape[:-2])))
    nb = int(np.prod(bshape)) if bshape else 1
    pairs = sorted({(0, 0), (nb - 1, M - 1), (nb // 2, M // 2), (0, M - 1), (nb - 1, 0), (nb // 3, (2 * M) // 3)})
    store = {"bf16": np.uint16, "f16": np.uint16, "f8e4m3": np.uint8, "f32": np.float32, "f64": np.float64, "i32": np.int32}[out_dt]
    worst = 0.0
    for bi, r in pairs:
        a2, b2 = _sub2d(lv, bshape, bi), _sub2d(rv, bshape, bi)
        a_row = np.ascontiguousarray(H.View([1, K], [0, a2.strides[1]], a2.offset + r * a2.strides[0]).take(a_host)).ravel()
        md = H.dot_md(H.View([1, K]), b2)
        got = ctx.download(out, store, N, first=(bi * M + r) * N)
        where = f"{case.key}: batch {bi}, row {r}"
        if out_dt == "i32":
            want = oracle.dot_asis("i32", a_row.astype(np.int32), b_host.astype(np.int32), md)
            if not np.array_equal(got, want):
                raise ParityError(f"{where}: integer result differs from the oracle")
            continue
        if out_dt == "f64":
            want = oracle.dot_asis("f64", a_row, b_host, md).astype(np.float64)
            sumabs = np.abs(a_row) @ np.abs(b2.take(b_host))
            tol, eps = 1e-12, H.EPS_F64
            gotf = got.astype(np.float64)
        else:
            o32, o64, sumabs = oracle.dot_spec(l_dt, r_dt, a_row, b_host, md)
            want, gotf = o64, H.widen(out_dt, got)
            tol, eps = (1e-5 if out_dt == "f32" else 2e-2), H.EPS_F32
        if not np.all(np.isfinite(gotf)):
            raise ParityError(f"{where}: non-finite output")
        if out_dt == "f8e4m3":
            # delivered in an 8-bit float: within one rounding step of the f32-accumulated value
            lim = np.clip(want, -448.0, 448.0)
            if not np.all(np.abs(gotf - lim) <= 2.0 ** -3 * np.abs(lim) + 2.0 ** -9 + 1e-3 * sumabs / np.sqrt(K)):
                raise ParityError(f"{where}: f8e4m3 output is more than one rounding step from the f32 sum")
            continue
        if scale_host is not None:
            sc = float(H.bf16_to_f32(np.asarray(scale_host, dtype=np.uint16).reshape(1))[0])
            want, sumabs = want * sc, sumabs * abs(sc)
        for what in case.fused:  # the fused steps start from the rounded product: one more bf16 rounding each
            if what == "bias":
                bvals = H.bf16_to_f32(bias_host).astype(np.float64)
                want, sumabs = want + bvals, sumabs + np.abs(bvals)
            elif what == "relu":
                want = np.maximum(want, 0.0)
        try:
            H.assert_close(gotf, want, sumabs, K, tol, where, eps_acc=eps if not case.fused else 2.0 ** -9)
        except AssertionError as e:
            raise ParityError(str(e)) from None
        worst = max(worst, float(H.rel_err(gotf, want, sumabs, K, tol, eps if not case.fused else 2.0 ** -9).max()))
    return {"rows_checked": len(pairs), "against": "oracle dot_asis (bit-exact)" if out_dt == "i32" else
            f"oracle f32-accumulated comparator, tol {2e-2 if out_dt in ('bf16', 'f16') else 1e-5 if out_dt == 'f32' else 'one f8 step' if out_dt == 'f8e4m3' else 1e-12}",
            "max_rel_err": worst}


def time_case(ctx, case, steps, warmup, graph=False, exact_steps=False, verify=True, headline=None):
    """returns a result dict; operands are uploaded before the timed region starts.  exact_steps: time exactly
    `steps` launches after exactly `warmup` untimed ones; otherwise at least MIN_LAUNCHES after at least MIN_WARMUP.
    headline = (K, W): once the row is measured and with the operands still resident, W more untimed launches and
    then exactly K timed ones -- the figure the bench line's `value` is made of.  (Timed cold, after the seconds of
    host-side data generation that precede every case, the first batch of a large product runs about 15 % slower
    than every later one while the clocks ramp up; that batch is reported as first_batch_us.)"""
    if not exact_steps:
        steps, warmup = max(steps, MIN_LAUNCHES), max(warmup, MIN_WARMUP)
    md, obytes = out_bytes(case)
    a_host = case.make_a()
    a = ctx.upload(a_host)
    w_host = case.make_b()
    copies = 1
    if case.rotate:
        copies = max(2, int(3 * INFINITY_CACHE_BYTES // max(w_host.nbytes, 1)) + 1)
    ws = [ctx.upload(w_host)]
    for i in range(1, copies):
        # distinct buffers with the same contents: what matters is that the addresses differ
        extra = ctx.alloc(w_host.nbytes)
        ctx.lib.hodu_rocm_memcpy_d2d(ctx.handle, extra.ptr, ws[0].ptr, w_host.nbytes)
        ws.append(extra)
    out = ctx.alloc(obytes)
    ctx.fill(out, 0xFF)
    from hodu_amd import ffi
    fused_steps, bias, bias_host, scale_host = [], None, None, None
    for what in case.fused:
        if what == "bias":
            bias_host = bf16(normal(700, case.rv.shape[-1], 0.1))
            bias = ctx.upload(bias_host)
            fused_steps.append(ffi.add_row(bias))
        elif what == "scale":
            scale_host = bf16(np.array([0.125], dtype=np.float32))
            fused_steps.append(ffi.mul_scalar(scale_host))
        else:
            fused_steps.append(ffi.relu())
    ctx.sync()
    for i in range(warmup):
        if fused_steps:
            ctx.product_ex(case.op, case.name, a, ws[i % copies], out, md, fused_steps)
        else:
            ctx.product(case.op, case.name, a, ws[i % copies], out, md)
    ctx.sync()
    kernel = ctx.last_kernel()
    # the K timed launches are issued back to back from C (hodu_rocm_debug_time_product) so that a
    # 3 us GEMV is not hidden behind the interpreter's per-call cost; HIP events on the same stream
    ms = ctx.time_product(case.op, case.name, a, ws, out, md, steps, graph=graph, steps=fused_steps)
    # spread: further batches of the same launches (outside the K timed steps), each timed the same way
    spread = sorted(ctx.time_product(case.op, case.name, a, ws, out, md, steps, graph=graph, steps=fused_steps) * 1e3 / steps
                    for _ in range(SPREAD_BATCHES))
    head_ms = None
    if headline is not None:
        k_steps, w_steps = headline
        for i in range(w_steps):
            ctx.product(case.op, case.name, a, ws[i % copies], out, md)
        head_ms = ctx.time_product(case.op, case.name, a, ws, out, md, k_steps)
    parity = verify_case(ctx, case, a_host, w_host, out, bias_host, scale_host) if verify else None
    for buf in [a, out] + ws + ([bias] if bias else []):
        buf.free()
    med = 0.5 * (spread[len(spread) // 2 - 1] + spread[len(spread) // 2])
    first_batch_us = ms * 1e3 / steps
    # the row's figure is the median batch (for --only, which asks for exactly K launches, the K launches themselves)
    per_launch_s = (first_batch_us if exact_steps else med) * 1e-6
    tflops = case.flops / per_launch_s / 1e12
    gbs = case.alg_bytes / per_launch_s / 1e9
    if case.bound == "hbm":
        roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS}
    else:
        peak = PEAK[case.peak_key]
        roof = {"bound": "mfma", "achieved": tflops, "peak": peak, "unit": "TFLOP/s", "frac": tflops / peak}
    roof["traffic"], roof["traffic_source"] = traffic_of(kernel, case.key)
    roof["kernel"] = kernel
    return {"config": case.key, "label": case.label, "kernel": kernel, "us_per_launch": per_launch_s * 1e6,
            "first_batch_us": first_batch_us, "launches_timed": steps, "warmup_launches": warmup,
            "headline_ms_total": head_ms,
            "tflops": tflops, "algorithmic_gbs": gbs, "weight_buffers_rotated": copies, "roofline": roof,
            "flops": case.flops, "alg_bytes": case.alg_bytes, "peak_key": case.peak_key, "parity": parity,
            "us_batches": {"launches_per_batch": steps, "batches": SPREAD_BATCHES, "p10": spread[1], "median": med,
                           "p90": spread[-2]}}


def compact_row(r):
    """one row of roofline.per_config: the median over the extra batches is the figure"""
    us = r["us_batches"]["median"]
    roof = r["roofline"]
    if roof["bound"] == "hbm":
        ach = r["alg_bytes"] / us / 1e3 if "alg_bytes" in r else roof["achieved"]
    else:
        ach = r["flops"] / us / 1e6 if "flops" in r else roof["achieved"]
    # unit is TFLOP/s (TOP/s for integers) where bound is mfma, GB/s where it is hbm; p10 / p90 are in bench_full.json
    row = {"key": r["config"], "us": round(us, 2), "bound": roof["bound"], "achieved": round(ach, 1), "peak": roof["peak"],
           "frac": round(ach / roof["peak"], 4), "kernel": r["kernel"]}
    return row


def attention_probe(ctx, steps, d=128, heads=32, s_len=2048):
    """not a BASELINE configuration: hodu_nn's scaled_dot_product_attention (causal, bf16, 32 heads x 2048 x d) as
    the one fused kernel, and as the three launches the host mirror falls back to -- Q K^T with the scale in its
    store, masked softmax, P V -- each timed with HIP events around `steps` back-to-back launches; and, beside them,
    the same function with a [1, Sk] padding attn_mask (a quarter of the keys masked, no causal mask) as one kernel and
    its middle launch of the three"""
    import helpers as H
    from hodu_amd import ffi
    V = H.View
    q, k, v = (ctx.upload(bf16(normal(950 + i, heads * s_len * d))) for i in range(3))
    scores, probs = ctx.alloc(heads * s_len * s_len * 2), ctx.alloc(heads * s_len * s_len * 2)
    out = ctx.alloc(heads * s_len * d * 2)
    md_qk = H.matmul_md(V([heads, s_len, d]), V([heads, s_len, d]).t())
    md_pv = H.matmul_md(V([heads, s_len, s_len]), V([heads, s_len, d]))
    md_sm = H.reduce_md(V([heads, s_len, s_len]), [2], True)
    scale = [ffi.mul_scalar(bf16(np.array([1.0 / np.sqrt(d)], dtype=np.float32)))]
    legs = {
        "qk_scaled": lambda: ctx.product_ex("matmul", "bf16", q, k, scores, md_qk, scale),
        "softmax_causal": lambda: ctx.softmax("bf16", scores, probs, md_sm, True),
        "pv": lambda: ctx.product("matmul", "bf16", probs, v, out, md_pv),
    }
    md_at = [1, heads, s_len, s_len, d] + [s_len * d, d, 1] * 3 + [0, 0, 0]
    scale_bits = bf16(np.array([1.0 / np.sqrt(d)], dtype=np.float32))
    legs["fused_one_kernel"] = lambda: ctx.attention("bf16", q, k, v, out, md_at, scale_bits, True)
    keep = np.ones(s_len, np.uint8)
    keep[s_len - s_len // 4:] = 0
    mask = ctx.upload(keep)
    legs["softmax_padding_mask"] = lambda: ctx.softmax_masked("bf16", scores, probs, md_sm, mask, [0, 0, 1])
    legs["fused_padding_mask"] = lambda: ctx.attention("bf16", q, k, v, out, md_at, scale_bits, False, mask=mask, mask_strides=[0, 0, 1])
    beside = ("fused_one_kernel", "softmax_padding_mask", "fused_padding_mask")  # not part of the three-launch total
    res, total = {}, 0.0
    for name, fn in legs.items():
        for _ in range(3):
            fn()
        ctx.sync()
        t = ctx.timer()
        t.start()
        for _ in range(steps):
            fn()
        us = t.stop_ms() * 1e3 / steps
        res[name] = {"us": us, "kernel": ctx.last_kernel()}
        total += us if name not in beside else 0.0
    flops = 2 * 2.0 * heads * s_len * s_len * d
    res["qk_scaled"]["tflops"] = flops / 2 / res["qk_scaled"]["us"] / 1e6
    res["pv"]["tflops"] = flops / 2 / res["pv"]["us"] / 1e6
    res["softmax_causal"]["gbs"] = 2.0 * heads * s_len * s_len * 2 / res["softmax_causal"]["us"] / 1e3
    for b in (q, k, v, scores, probs, out, mask):
        b.free()
    # the causal mask halves the useful work; rates count the unmasked half only for the fused kernel
    res["fused_one_kernel"]["tflops_useful"] = flops / 2 / res["fused_one_kernel"]["us"] / 1e6
    return {"config": "attention", "shape": f"bf16 q,k,v [{heads},{s_len},{d}], causal", "us_three_launches": total,
            "us_fused": res["fused_one_kernel"]["us"], "us_fused_padding_mask": res["fused_padding_mask"]["us"], "legs": res}


def cast_cases():
    """the to_dtype / contiguous passes the path takes when a cast is NOT deferred into the product, at the sizes of
    the BASELINE configurations: (key, label, src, dst, view, elements)"""
    import helpers as H
    V = H.View
    return [
        ("cast_f8e4m3_bf16_c3w", "to_dtype f8e4m3 -> bf16, config 3's weight [4096,4096]", "f8e4m3", "bf16", V([4096 * 4096])),
        ("cast_f8e4m3_bf16_c5w", "to_dtype f8e4m3 -> bf16, config 5's weight [4096,14336]", "f8e4m3", "bf16", V([4096 * 14336])),
        ("cast_i8_i32_c4", "to_dtype i8 -> i32, one operand of config 4 [2048,2048]", "i8", "i32", V([2048 * 2048])),
        ("contiguous_bf16_c2_bt", "contiguous of config 2's transposed operand [16,1024,1024]^T", "bf16", "bf16",
         V([16, 1024, 1024]).t()),
        ("contiguous_bf16_c5_wdown", "contiguous of config 5's W_down view [4096,14336]^T", "bf16", "bf16",
         V([4096, 14336]).t()),
    ]


def time_cast_case(ctx, key, label, src, dst, view, steps, warmup):
    """HBM-bound: algorithmic bytes = elements x (source + destination element size); inputs and outputs rotate
    through enough buffer pairs to exceed three times the Infinity Cache"""
    import helpers as H
    from hodu_amd import ffi
    n = int(np.prod(view.shape))
    in_bytes, out_bytes_ = view.span() * ffi.DTYPE_SIZE[src], n * ffi.DTYPE_SIZE[dst]
    pairs = max(2, int(3 * INFINITY_CACHE_BYTES // (in_bytes + out_bytes_)) + 1)
    host = np.random.default_rng(77).integers(0, 120, size=in_bytes, dtype=np.uint8)  # finite in every dtype used here
    ins = [ctx.upload(host)]
    for _ in range(1, pairs):
        extra = ctx.alloc(in_bytes)
        ctx.lib.hodu_rocm_memcpy_d2d(ctx.handle, extra.ptr, ins[0].ptr, in_bytes)
        ins.append(extra)
    outs = [ctx.alloc(out_bytes_) for _ in range(pairs)]
    md = H.cast_md(view)
    steps, warmup = max(steps, MIN_LAUNCHES), max(warmup, MIN_WARMUP)
    ctx.time_cast(src, dst, ins, outs, md, warmup)
    kernel = ctx.last_kernel()
    ms = ctx.time_cast(src, dst, ins, outs, md, steps)
    spread = sorted(ctx.time_cast(src, dst, ins, outs, md, steps) * 1e3 / steps for _ in range(SPREAD_BATCHES))
    # parity on the buffer the timed launches wrote: three rows of the last dim (first, middle, last of the leading
    # index space), bit for bit against the oracle's cast / gather of the same view
    import oracle
    lead = view.shape[:-1]
    n_lead, last = int(np.prod(lead)) if lead else 1, view.shape[-1]
    host_typed = host.view(oracle.STORAGE[src])
    for flat in sorted({0, n_lead // 2, n_lead - 1}):
        off, rem = view.offset, flat
        for d in range(len(lead) - 1, -1, -1):
            off += (rem % lead[d]) * view.strides[d]
            rem //= lead[d]
        sub = H.View([min(last, 1 << 20)], [view.strides[-1]], off)
        want = (oracle.contiguous(src, host_typed, H.cast_md(sub)) if src == dst else
                oracle.cast(src, dst, host_typed, H.cast_md(sub), decode=oracle.F8_OCP))
        got = ctx.download(outs[0], oracle.STORAGE[dst], sub.shape[0], first=flat * last)
        if not np.array_equal(got, want):
            raise ParityError(f"{key}: row {flat} of the output differs from the oracle")
    for b in ins + outs:
        b.free()
    s_per = ms / 1e3 / steps
    alg = n * (ffi.DTYPE_SIZE[src] + ffi.DTYPE_SIZE[dst])
    gbs = alg / s_per / 1e9
    return {"config": key, "label": label, "kernel": kernel, "us_per_launch": s_per * 1e6, "tflops": 0.0,
            "algorithmic_gbs": gbs, "weight_buffers_rotated": pairs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "traffic": None, "traffic_source": None, "kernel": kernel},
            "alg_bytes": alg, "parity": {"rows_checked": 3, "against": "oracle cast / contiguous, bit-exact"},
            "us_batches": {"launches_per_batch": steps, "batches": SPREAD_BATCHES, "p10": spread[1],
                           "median": 0.5 * (spread[4] + spread[5]), "p90": spread[-2]}}


def sum_cases():
    """sum_to_shape of the backward pass at the sizes of configuration 5: (key, label, view, reduced dims)"""
    import helpers as H
    V = H.View
    return [
        ("sum_bias_grad_c5_up", "sum_to_shape: bias gradient of C5 up, bf16 [8,512,14336] -> [14336]", V([8, 512, 14336]), [0, 1]),
        ("sum_bias_grad_c5_down", "sum_to_shape: bias gradient of C5 down, bf16 [8,512,4096] -> [4096]", V([8, 512, 4096]), [0, 1]),
        ("sum_rows_c5", "row sums, bf16 [4096,14336] -> [4096]", V([4096, 14336]), [1]),
    ]


def time_sum_case(ctx, key, label, view, dims, steps, warmup):
    """HBM-bound: algorithmic bytes = (input + output elements) x element size; buffers rotate past the Infinity Cache"""
    import helpers as H
    n = int(np.prod(view.shape))
    n_out = n // int(np.prod([view.shape[d] for d in dims]))
    pairs = max(2, int(3 * INFINITY_CACHE_BYTES // (2 * (n + n_out))) + 1)
    host = bf16(normal(61, n))
    ins = [ctx.upload(host)]
    for _ in range(1, pairs):
        extra = ctx.alloc(2 * n)
        ctx.lib.hodu_rocm_memcpy_d2d(ctx.handle, extra.ptr, ins[0].ptr, 2 * n)
        ins.append(extra)
    outs = [ctx.alloc(2 * n_out) for _ in range(pairs)]
    md = H.reduce_md(view, dims, False)
    steps, warmup = max(steps, MIN_LAUNCHES), max(warmup, MIN_WARMUP)
    ctx.time_sum("bf16", ins, outs, md, warmup)
    kernel = ctx.last_kernel()
    ms = ctx.time_sum("bf16", ins, outs, md, steps)
    spread = sorted(ctx.time_sum("bf16", ins, outs, md, steps) * 1e3 / steps for _ in range(SPREAD_BATCHES))
    # parity: every output of the buffer the timed launches wrote, against the oracle's f32-accumulated sums
    import oracle
    o32, o64, oabs = oracle.sum_spec("bf16", host, md)
    got = H.bf16_to_f32(ctx.download(outs[0], np.uint16, n_out)).astype(np.float64)
    try:
        H.assert_close(got, o64, oabs, n // n_out, 2e-2, key)
    except AssertionError as e:
        raise ParityError(str(e)) from None
    for b in ins + outs:
        b.free()
    s_per = ms / 1e3 / steps
    gbs = 2 * (n + n_out) / s_per / 1e9
    return {"config": key, "label": label, "kernel": kernel, "us_per_launch": s_per * 1e6, "tflops": 0.0,
            "algorithmic_gbs": gbs, "weight_buffers_rotated": pairs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "traffic": None, "traffic_source": None, "kernel": kernel},
            "alg_bytes": 2 * (n + n_out), "parity": {"rows_checked": n_out, "against": "oracle f32-accumulated sums, tol 2e-2"},
            "us_batches": {"launches_per_batch": steps, "batches": SPREAD_BATCHES, "p10": spread[1],
                           "median": 0.5 * (spread[4] + spread[5]), "p90": spread[-2]}}


def host_buffers_probe(ctx, key, reps=5):
    """one configuration with the operands starting and the result ending in host memory (pageable numpy arrays through
    hodu_rocm_memcpy_h2d / _d2h, buffers allocated beforehand): what a caller pays who hands host buffers over per
    product instead of keeping tensors on the device.  Never the headline value."""
    import time
    case = next(c for c in build_cases({"c2", "c5"}) if c.key == key)
    md, obytes = out_bytes(case)
    a_host, b_host = np.ascontiguousarray(case.make_a()), np.ascontiguousarray(case.make_b())
    a, b, out = ctx.alloc(a_host.nbytes), ctx.alloc(b_host.nbytes), ctx.alloc(obytes)
    res = np.empty(obytes // 2, dtype=np.uint16)

    def once():
        ctx._check(ctx.lib.hodu_rocm_memcpy_h2d(ctx.handle, a.ptr, a_host.ctypes.data, a_host.nbytes))
        ctx._check(ctx.lib.hodu_rocm_memcpy_h2d(ctx.handle, b.ptr, b_host.ctypes.data, b_host.nbytes))
        ctx.product(case.op, case.name, a, b, out, md)
        ctx._check(ctx.lib.hodu_rocm_memcpy_d2h(ctx.handle, res.ctypes.data, out.ptr, res.nbytes))

    once()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(reps):
        once()
    ctx.sync()
    s_per = (time.perf_counter() - t0) / reps
    for buf in (a, b, out):
        buf.free()
    moved = a_host.nbytes + b_host.nbytes + res.nbytes
    return {"config": key + "_host_buffers", "ms_per_product": s_per * 1e3, "tflops": case.flops / s_per / 1e12,
            "bytes_over_pcie": moved, "gbs_over_pcie": moved / s_per / 1e9, "host_memory": "pageable"}


def vendor_yardstick(steps):
    """NOT this library: what the vendor's own GEMM kernels reach on the bench's large 2-D bf16 shapes with operands of
    the same distribution (torch.matmul, i.e. hipBLASLt / rocBLAS behind it, timed with events around `steps`
    back-to-back calls, median of five batches).  A yardstick for how close the hand-written kernels are to what the
    hardware allows on this data; never part of `value`.  Only plain 2-D products are run."""
    import torch
    torch.manual_seed(0)
    dev = "cuda:0"
    rows = []

    def gemm(key, m, n, k, b_transposed_view):
        a = torch.randn((m, k), device=dev, dtype=torch.float32).to(torch.bfloat16)
        if b_transposed_view:
            b = (torch.randn((n, k), device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16).t()
        else:
            b = (torch.randn((k, n), device=dev, dtype=torch.float32) * 0.02).to(torch.bfloat16)
        out = torch.empty((m, n), device=dev, dtype=torch.bfloat16)
        for _ in range(MIN_WARMUP):
            torch.matmul(a, b, out=out)
        torch.cuda.synchronize()
        times = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                torch.matmul(a, b, out=out)
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) / steps * 1e3)
        us = sorted(times)[2]
        rows.append({"config": key, "us_per_launch": us, "tflops": 2.0 * m * n * k / us / 1e6,
                     "frac_of_bf16_peak": 2.0 * m * n * k / us / 1e6 / (PEAK["bf16"])})

    gemm("c5_down_bf16 shape: [4096,14336] x [4096,14336]^T-view", 4096, 4096, 14336, True)
    gemm("c5_up_bf16 shape: [4096,4096] x [4096,14336]", 4096, 14336, 4096, False)
    gemm("bf16 4096^3, rhs a transposed view", 4096, 4096, 4096, True)
    return {"config": "yardstick", "what": "torch.matmul (the vendor's GEMM library), NOT this library", "launches": steps, "rows": rows}


def read_floor_probe(ctx):
    """what a kernel that does nothing but read can reach at the sizes of the M = 1 configurations (weight buffers
    rotated past the Infinity Cache like the GEMV's), and the launch cadence of an empty kernel"""
    out = []
    for label, nbytes in (("16.8 MB (config 3 weight)", 4096 * 4096), ("58.7 MB (config 5 weight)", 14336 * 4096)):
        copies = max(2, int(3 * INFINITY_CACHE_BYTES // nbytes) + 1)
        bufs = [ctx.alloc(nbytes) for _ in range(copies)]
        for b in bufs:
            ctx.fill(b, 0x5A)
        ctx.sync()
        r = ctx.read_floor(bufs, nbytes, 200)
        for b in bufs:
            b.free()
        out.append({"bytes": nbytes, "label": label, "buffers_rotated": copies, "read_us": r["read_us"],
                    "read_gbs": nbytes / r["read_us"] / 1e3, "frac_of_hbm_peak": nbytes / r["read_us"] / 1e3 / HBM_PEAK_GBS,
                    "empty_kernel_us": r["empty_us"]})
    return out


def mfma_clock_probe(ctx):
    """what the matrix cores sustain from registers (no LDS, no memory traffic), and at which shader clock, on
    constant and on N(0,1) operands, for both shapes of the bf16 and of the f8 instruction: the clock under full MFMA
    load depends on the data and on the instruction's shape"""
    import helpers as H
    out = []
    for kind, name, peak in ((0, "bf16 32x32x16", PEAK["bf16"]), (2, "bf16 16x16x32", PEAK["bf16"]),
                             (1, "f8e4m3 32x32x64 (unit scales)", PEAK["fp8"]), (3, "f8e4m3 16x16x128 (unit scales)", PEAK["fp8"])):
        for data in ("constant", "normal"):
            if kind in (0, 2):
                bits = bf16(np.full(8192, 0.0111, dtype=np.float32) if data == "constant" else normal(900, 8192))
            else:
                vals = np.full(16384, 0.5, dtype=np.float32) if data == "constant" else normal(901, 16384)
                bits = H.f32_to_ocp_e4m3_rne(np.clip(vals, -448, 448))
            buf = ctx.upload(bits)
            r = ctx.mfma_clock(kind, buf, 20000)
            buf.free()
            out.append({"instruction": name, "operands": data, "tflops": r["tflops"], "shader_mhz": r["shader_mhz"],
                        "frac_of_datasheet_peak": r["tflops"] / peak})
    return out


# ------------------------------------------------------------------------------------------------
# CPU baselines: hodu's CPU path per configuration, on bounded samples
# ------------------------------------------------------------------------------------------------
class CpuKernels:
    """hodu's CPU kernels for the baseline: the reference's own C files compiled by oracle/Makefile when that
    library is present (kind "reference"), else this repository's restatement (kind "port", OpenMP threads set to
    what the reference's pthread policy would use: kernels/thread_utils.h:28-58, ops_matrix.c:102-109, :455-462)."""

    def __init__(self):
        import oracle
        self.oracle = oracle
        self.ref = None
        if oracle.RefLib.available():
            try:
                self.ref = oracle.RefLib()
            except OSError:
                self.ref = None
        self.kind = "reference" if self.ref is not None else "port"
        self.online = os.cpu_count() or 1

    def threads(self, rows, min_rows, dense):
        """threads the reference would use: one for batched / strided operands, else rows / min_rows capped"""
        if not dense:
            return 1
        return max(1, min(32, self.oracle.reference_threads(rows, min_rows, self.online)))

    def dot(self, dt, a, b, md, threads):
        if self.ref is not None:
            return self.ref.dot(dt, a, b, md)
        self.oracle.set_threads(threads)
        try:
            return self.oracle.dot_asis(dt, a, b, md)
        finally:
            self.oracle.set_threads(self.online)

    def matmul(self, dt, a, b, md, threads):
        if self.ref is not None:
            return self.ref.matmul(dt, a, b, md)
        self.oracle.set_threads(threads)
        try:
            return self.oracle.matmul_asis(dt, a, b, md)
        finally:
            self.oracle.set_threads(self.online)

    def cast(self, src, dst, x, md):
        if self.ref is not None:
            return self.ref.cast(src, dst, x, md)
        return self.oracle.cast(src, dst, x, md)


def _timed(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


def _rows_for_budget(run_rows, probe_rows, max_rows, budget_s, multiple=1):
    """times run_rows(probe_rows), then one run sized to the budget; returns (rows, seconds)"""
    t = _timed(lambda: run_rows(probe_rows))
    rows = int(min(max_rows, max(probe_rows, budget_s / max(t, 1e-9) * probe_rows)))
    rows = max(multiple, rows // multiple * multiple)
    if rows <= probe_rows:
        return probe_rows, t
    return rows, _timed(lambda: run_rows(rows))


def _sgemm_rate(m, k, n, seconds=0.6):
    """numpy's OpenBLAS sgemm on all host cores: the f32-upcast comparator path (to_dtype(f32) + matmul_f32, which is
    cblas_sgemm with hodu's openblas feature, kernels/ops_matrix_openblas.c:19-153, :286-340)"""
    g = np.random.default_rng(1)
    a, b = g.standard_normal((m, k), dtype=np.float32), g.standard_normal((k, n), dtype=np.float32)
    a @ b
    t0, reps = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        a @ b
        reps += 1
    return 2.0 * m * k * n * reps / (time.perf_counter() - t0)


def cpu_baselines(which, headline_key, headline_budget_s=10.0, budget_s=2.0):
    """One row per configuration: hodu's CPU path timed on a bounded sample (full size where that takes under a
    second), the rate extrapolated linearly to the whole job where the sample is a slice, and the f32-upcast
    comparator path (sgemm) beside it.  Returns (rows, row of the headline)."""
    import helpers as H
    V = H.View
    cpu = CpuKernels()
    rows, head = [], None
    blas = "numpy's bundled OpenBLAS sgemm, all host cores"

    def row(key, what, flops_sample, secs, cores, sample, flops_full, extra=None):
        rate = flops_sample / secs
        r = {"key": key, "path": what, "value": rate / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": cpu.kind,
             "sample": sample, "seconds_sampled": round(secs, 3),
             "whole_job_seconds": round(flops_full / rate, 3),
             "whole_job_is": "measured" if abs(flops_sample - flops_full) < 1 else "linear extrapolation of the sample"}
        if extra:
            r.update(extra)
        rows.append(r)
        return r

    if "c1" in which:
        n = 512
        a, b = normal(101, n * n), normal(102, n * n)
        md = H.dot_md(V([n, n]), V([n, n]))
        th = cpu.threads(n, 256, True)
        cpu.dot("f32", a, b, md, th)
        secs = min(_timed(lambda: cpu.dot("f32", a, b, md, th)) for _ in range(3))
        row("c1", "hodu_cpu_dot_f32_fallback (sequential k, kernels/ops_matrix.c:399-549)", 2.0 * n ** 3, secs, th,
            "full size, best of 3", 2.0 * n ** 3,
            {"openblas_sgemm_tflops": _sgemm_rate(n, n, n, 0.3) / 1e12,
             "openblas_note": f"hodu's openblas feature path (kernels/ops_matrix_openblas.c:286-340) through {blas}"})
    if "c2" in which:
        n = 1024
        a, b = bf16(normal(201, n * n, 1 / 32)), bf16(normal(202, n * n, 1 / 32))

        def run(r):
            cpu.matmul("bf16", a[:r * n], b, H.matmul_md(V([1, r, n]), V([1, n, n]).t()), 1)
        r_, secs = _rows_for_budget(run, 32, n, budget_s, 32)
        row("c2", "hodu_cpu_matmul_bf16 (bf16 accumulate, batched path: one thread, kernels/ops_matrix.c:292-337)",
            2.0 * r_ * n * n, secs, 1, f"{r_} of 1024 rows of one of the 16 batches against its full [1024,1024]^T-view",
            16 * 2.0 * n ** 3, {"f32_comparator_sgemm_tflops": _sgemm_rate(n, n, n, 0.4) / 1e12})
    if "c3" in which:
        n = k = 4096
        w8 = fp8_weights(301, n * k)
        t_cast = _timed(lambda: cpu.cast("f8e4m3", "bf16", w8, H.cast_md(V([n * k]))))
        wb = cpu.cast("f8e4m3", "bf16", w8, H.cast_md(V([n * k])))
        x = bf16(normal(302, 512 * k))
        sg = _sgemm_rate(512, k, n, 0.5) / 1e12
        for m in (1, 16, 256, 4096):
            # the right operand is a transposed view: the reference's dot takes its strided branch on one thread
            if m <= 16:
                md = H.dot_md(V([m, k]), V([n, k]).t())
                secs = _timed(lambda: cpu.dot("bf16", x[:m * k], wb, md, 1))
                fl, sample = 2.0 * m * n * k, "full size"
            else:
                ns = 1024 if m == 4096 else n  # M = 4096: a quarter of the weight rows as well

                def run(r, ns=ns):
                    cpu.dot("bf16", x[:r * k], wb, H.dot_md(V([r, k]), V([ns, k]).t()), 1)
                r_, secs = _rows_for_budget(run, 4, min(m, 512), budget_s, 4)
                fl, sample = 2.0 * r_ * ns * k, f"{r_} of {m} rows against {ns} of 4096 weight rows"
            row(f"c3_m{m}", "hodu_cpu_cast_f8e4m3_to_bf16 (kernels/ops_cast.c:130) + hodu_cpu_dot_bf16 (bf16 accumulate, "
                "strided branch: one thread, kernels/ops_matrix.c:556-701); the cast is timed apart",
                fl, secs, 1, sample, 2.0 * m * n * k,
                {"cast_seconds_whole_weight": round(t_cast, 4), "f32_comparator_sgemm_tflops": sg})
    if "c4" in which:
        n = 2048
        g = np.random.default_rng(401)
        a8 = g.integers(-127, 128, n * n).astype(np.int8)
        b8 = np.random.default_rng(402).integers(-127, 128, n * n).astype(np.int8)
        md1 = H.cast_md(V([n * n]))
        t_cast = _timed(lambda: cpu.cast("i8", "i32", a8, md1)) + _timed(lambda: cpu.cast("i8", "i32", b8, md1))
        a32, b32 = a8.astype(np.int32), b8.astype(np.int32)

        def run(r):
            th = cpu.threads(r, 256, True)
            cpu.dot("i32", a32[:r * n], b32, H.dot_md(V([r, n]), V([n, n])), th)
        r_, secs = _rows_for_budget(run, 64, n, budget_s, 64)
        th = cpu.threads(r_, 256, True)
        th_full = cpu.threads(n, 256, True)
        r = row("c4", "hodu_cpu_cast_i8_to_i32 x 2 (kernels/ops_cast.c:330) + hodu_cpu_dot_i32 (kernels/ops_matrix.c:399-549, :719); "
                "the casts are timed apart", 2.0 * r_ * n * n, secs, th, f"{r_} of 2048 rows ({th} thread(s); the whole product "
                f"would run on {th_full})", 2.0 * n ** 3, {"cast_seconds_both_operands": round(t_cast, 4), "unit": "TOP/s"})
        if th_full != th:
            r["whole_job_seconds"] = round(r["whole_job_seconds"] * th / th_full, 3)
            r["whole_job_is"] = f"linear extrapolation of the sample, scaled to {th_full} threads"
    if "c5" in which:
        d, f = 4096, 14336
        sg = _sgemm_rate(512, d, f // 4, 0.5) / 1e12
        for leg, kdim, ndim, xs, ws in (("down", f, d, 0.3, 503), ("up", d, f, 1.0, 502)):
            key = f"c5_{leg}_bf16"
            x = bf16(normal(504 if leg == "down" else 501, 64 * kdim, xs))
            w = bf16(normal(ws, d * f, 0.02))
            # the weight as the configuration hands it over: [4096, 14336] broadcast over the batch, transposed for "down"
            wv = V([d, f]).t() if leg == "down" else V([d, f])

            def run(r, wv=wv, x=x, w=w, kdim=kdim, ndim=ndim):
                cpu.matmul("bf16", x[:r * kdim], w, H.matmul_md(V([1, r, kdim]), wv.broadcast_to([1, kdim, ndim])), 1)
            budget = headline_budget_s if key == headline_key else budget_s
            r_, secs = _rows_for_budget(run, 2, 64, budget, 2)
            fl_full = 2.0 * 8 * 512 * d * f
            rr = row(key, "hodu_cpu_matmul_bf16 (bf16 accumulate, batched / broadcast path: one thread, kernels/ops_matrix.c:292-337)",
                     2.0 * r_ * kdim * ndim, secs, 1, f"{r_} of the 8 x 512 rows against the whole weight", fl_full,
                     {"f32_comparator_sgemm_tflops": sg})
            if key == headline_key:
                head = rr
            # f8e4m3 weights: to_dtype(bf16) first (one more pass over 58.7 M elements), then the same kernel
            if leg == "down":
                w8 = fp8_weights(503, d * f)
                t_cast = _timed(lambda: cpu.cast("f8e4m3", "bf16", w8, H.cast_md(V([d * f]))))
            r8 = dict(rr)
            r8.update({"key": f"c5_{leg}_f8e4m3", "path": "hodu_cpu_cast_f8e4m3_to_bf16 over the whole weight, then the "
                       "bf16 product above (the same kernel on the same shapes: its rate is not timed twice)",
                       "cast_seconds_whole_weight": round(t_cast, 4)})
            rows.append(r8)
    for r in rows:
        r["host_cores_online"] = cpu.online
    return rows, head


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--configs", default="c1,c2,c3,c4,c5,f8,f64,fused,bwd,casts")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--only", default="", help="time exactly one case key (e.g. c5_down_bf16) and print its result")
    ap.add_argument("--force-tile", type=int, default=-1, help="testing hook: pin a kernel variant (include/hodu_rocm_debug.h; 15 and 16: the 16 x 16 x 32 tile and its respaced form)")
    ap.add_argument("--graph", action="store_true", help="with --only: replay the K launches as one HIP graph")
    ap.add_argument("--force-splitk", type=int, default=-1, help="testing hook: pin the number of K ranges")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU: it has no collective or sharded path, and `value` is the one "
              "GPU's throughput. Re-run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    if args.only == "yardstick":
        # (before this library touches the GPU: torch brings a HIP runtime of its own, and the two do not share a process)
        print(json.dumps(vendor_yardstick(max(args.steps, MIN_LAUNCHES))))
        return
    from hodu_amd import ffi
    ctx = ffi.Context(0)
    info = ctx.device_info()
    ctx.force_tile(args.force_tile)
    ctx.force_splitk(args.force_splitk)
    if args.only == "copy":
        # calibration for the rocprofv3 FETCH_SIZE / WRITE_SIZE counters: a plain dense copy of known size
        # (hodu_rocm_contiguous on a contiguous f32 buffer reads n bytes and writes n bytes)
        import helpers as H
        n = 64 << 20
        src, dst = ctx.alloc(4 * n), ctx.alloc(4 * n)
        ctx.fill(src, 0)
        md = H.cast_md(H.View([n]))
        for _ in range(args.steps):
            ctx.contiguous("f32", src, dst, md)
        ctx.sync()
        print(json.dumps({"config": "copy", "kernel": ctx.last_kernel(), "bytes_read": 4 * n, "bytes_written": 4 * n,
                          "launches": args.steps}))
        ctx.close()
        return
    if args.only in ("attention", "attention_d64"):
        print(json.dumps(attention_probe(ctx, args.steps, 64 if args.only == "attention_d64" else 128)))
        ctx.close()
        return
    if args.only == "pcie":
        print(json.dumps({"config": "pcie", "rows": [host_buffers_probe(ctx, k) for k in ("c5_down_bf16", "c2")]}))
        ctx.close()
        return
    if args.only == "clock":
        print(json.dumps({"config": "clock", "register_only_mfma": mfma_clock_probe(ctx), "streaming_read": read_floor_probe(ctx)}))
        ctx.close()
        return
    if args.only in [c[0] for c in sum_cases()]:
        print(json.dumps(time_sum_case(ctx, *next(c for c in sum_cases() if c[0] == args.only), args.steps, args.warmup)))
        ctx.close()
        return
    if args.only in [c[0] for c in cast_cases()]:
        print(json.dumps(time_cast_case(ctx, *next(c for c in cast_cases() if c[0] == args.only), args.steps, args.warmup)))
        ctx.close()
        return
    if args.only:
        case = next(c for c in build_cases({"c1", "c2", "c3", "c4", "c5", "f8", "f64", "fused", "bwd"}) if c.key == args.only)
        print(json.dumps(time_case(ctx, case, args.steps, args.warmup, graph=args.graph, exact_steps=True)))
        ctx.close()
        return
    HEAD = "c5_down_bf16"
    which = set(args.configs.split(",")) | {"c5"}
    results = []

    def note(r):
        roof = r["roofline"]
        rate = f"{r['tflops']:.1f} TFLOP/s" if roof["bound"] == "mfma" else f"{r['algorithmic_gbs']:.0f} GB/s"
        print(f"# {r['label']}: {r['us_batches']['median']:.1f} us (p10 {r['us_batches']['p10']:.1f}, p90 {r['us_batches']['p90']:.1f}; "
              f"first batch {r.get('first_batch_us', r['us_per_launch']):.1f})  {rate}  [{r['kernel']}] {100 * roof['frac']:.1f}% of {roof['bound']} peak"
              f"  parity {'ok' if r.get('parity') else 'not checked'}", file=sys.stderr, flush=True)

    cases = build_cases(which)
    head_case = next(c for c in cases if c.key == HEAD)
    for case in cases:
        results.append(time_case(ctx, case, args.steps, args.warmup,
                                 headline=(args.steps, args.warmup) if case.key == HEAD else None))
        note(results[-1])
    if "casts" in which:
        for cc in cast_cases():
            results.append(time_cast_case(ctx, *cc, args.steps, args.warmup))
            note(results[-1])
    if "bwd" in which:
        for sc in sum_cases():
            results.append(time_sum_case(ctx, *sc, args.steps, args.warmup))
            note(results[-1])
    head = next(r for r in results if r["config"] == HEAD)
    probes = {"register_only_mfma": mfma_clock_probe(ctx), "streaming_read": read_floor_probe(ctx), "device": info}
    ctx.close()
    cpu_rows, cpu_head = (None, None) if args.no_cpu else cpu_baselines(which, HEAD)
    line, full = assemble_line(args.steps, args.warmup, HEAD, head_case.flops, head_case.alg_bytes, results, cpu_rows,
                               cpu_head, probes)
    # what does not fit the one-line contract (every row in full, the probes, the CPU rows' descriptions) goes to a file
    try:
        os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
        with open(os.path.join(ROOT, "gpurun_out", "bench_full.json"), "w") as f:
            json.dump(full, f)
    except OSError as e:
        print(f"# bench_full.json not written: {e}", file=sys.stderr)
    text = json.dumps(line, separators=(",", ":"))
    assert len(text) < LINE_LIMIT, f"the bench line is {len(text)} characters; its reader needs it under {LINE_LIMIT}"
    sys.stderr.flush()
    print(text, flush=True)


ROW_COLUMNS = ("key", "us", "bound", "achieved", "peak", "frac", "kernel")
LINE_LIMIT = 6000  # characters of the final stdout line: what reads it keeps only a tail of stdout


def _target(by_key, key, need):
    r = by_key.get(key)
    if r is None:
        return None
    row = compact_row(r)
    return {"key": key, "us": row["us"], "frac": row["frac"], "target": need, "met": row["frac"] >= need}


def assemble_line(steps, warmup, head_key, head_flops, head_bytes, results, cpu_rows, cpu_head, probes=None):
    """(line, full): `line` is the one JSON object printed last on stdout -- the contract's scalar keys, the workload,
    the headline's roofline with one compact row per measured configuration, and the CPU baseline with one short row
    per configuration -- kept under LINE_LIMIT characters; `full` adds every row unabridged, the probe tables and the
    CPU rows' descriptions, and is written to gpurun_out/bench_full.json."""
    by_key = {r["config"]: r for r in results}
    head = by_key[head_key]
    head_us = head["headline_ms_total"] * 1e3 / steps
    head_tflops = head_flops / head_us / 1e6
    line = {
        "metric": "TFLOP/s & % MFMA peak per dtype; M=1 GEMV GB/s & % HBM peak",
        "value": round(head_tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(head_us / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[4] (largest), down projection: X[8,512,14336] bf16 x W_down = transposed "
                               "view of bf16 [4096,14336] broadcast over the batch; f32 accumulate, bf16 out; 1 matmul per step",
                   "flop_per_step": head_flops, "algorithmic_bytes_per_step": head_bytes,
                   "parity_checked_in_this_run": bool(head.get("parity")),
                   # `value` is timed on a warm clock; the first batch after host-side work runs on a ramping clock
                   "cold_first_batch_us": round(head["first_batch_us"], 1),
                   # the rows the targets are stated on (bf16-rate 4096^3-class GEMM, native fp8 4096^3, M = 1 GEMV)
                   "north_star": [t for t in (_target(by_key, "c3_m4096", 0.60), _target(by_key, "c5_down_bf16", 0.60),
                                              _target(by_key, "c5_up_bf16", 0.60), _target(by_key, "bf16_4096", 0.60),
                                              _target(by_key, "f8_4096", 0.60), _target(by_key, "c3_m1", 0.70)) if t]},
        "roofline": {"bound": "mfma", "achieved": round(head_tflops, 2), "peak": PEAK["bf16"], "unit": "TFLOP/s",
                     "frac": round(head_tflops / PEAK["bf16"], 4), "traffic": head["roofline"]["traffic"],
                     "traffic_source": head["roofline"]["traffic_source"], "kernel": head["kernel"],
                     "launch_us": round(head_us, 2),
                     # rows whose timed output buffer was compared with the oracle inside this run (a mismatch aborts)
                     "parity_rows_ok": sum(1 for r in results if r.get("parity") is not None), "rows": len(results),
                     # every configuration of this run, one array per row in the order of per_config_columns:
                     # us = median over 10 batches of back-to-back launches; achieved and peak in TFLOP/s (TOP/s for
                     # integers) where bound is mfma, in GB/s where it is hbm
                     "per_config_columns": list(ROW_COLUMNS),
                     "per_config": [[compact_row(r)[c] for c in ROW_COLUMNS] for r in results]},
    }
    full = dict(line)
    full["all_configs"] = results
    if probes:
        full.update(probes)
    if cpu_rows is not None:
        how = lambda r: "measured" if r["whole_job_is"] == "measured" else "extrapolated"  # noqa: E731
        line["cpu_baseline"] = {
            "value": float(f"{cpu_head['value']:.4g}"), "unit": "TFLOP/s", "cores": cpu_head["cores"], "kind": cpu_head["kind"],
            "sample": (f"hodu_cpu_matmul_bf16, {cpu_head['sample']}: {cpu_head['seconds_sampled']} s of CPU work; "
                       f"whole step {cpu_head['whole_job_seconds']} s ({how(cpu_head)})")[:200],
            "host_cores_online": cpu_head["host_cores_online"],
            "f32_comparator_sgemm_tflops": round(cpu_head.get("f32_comparator_sgemm_tflops") or 0.0, 2),
            "per_config": [{"key": r["key"], "value": float(f"{r['value']:.4g}"), "cores": r["cores"], "kind": r["kind"],
                            "whole_job_is": how(r)} for r in cpu_rows]}
        full["cpu_baseline"] = dict(line["cpu_baseline"], per_config=cpu_rows,
                                    sample=f"{cpu_head['path']}: {cpu_head['sample']}; {cpu_head['seconds_sampled']} s of CPU "
                                           f"work; the whole step would take {cpu_head['whole_job_seconds']} s "
                                           f"({cpu_head['whole_job_is']})")
    return line, full


if __name__ == "__main__":
    main()
