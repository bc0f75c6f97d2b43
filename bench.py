#!/usr/bin/env python3
"""Benchmark of the MI355X matmul / dot / to_dtype backend on BASELINE.json's five configurations.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs c1,c2,c3,c4,c5] [--no-cpu]

A "step" is one pass of the hot path over one batch of synthetic input: one matmul/dot call through
the C ABI with operands resident in HBM.  The headline (`value`, `roofline`, `cpu_baseline`) is
BASELINE.json configs[1]: bf16 batched matmul [16,1024,1024] x [16,1024,1024] with the right
operand a transposed view.  Every other configuration is measured in the same run and reported
under "all_configs" with its own roofline fraction (TFLOP/s against the MFMA dense peak of the
type the matrix cores consume, GB/s against HBM peak for the M <= 16 GEMV shapes).

Timing: HIP events recorded on the stream the kernels are launched on (the context's stream),
W untimed warm-up launches, then K launches back to back; `achieved` = algorithmic flops (or
bytes) per launch / average launch duration.  The GEMV configurations rotate through enough
distinct weight buffers to exceed the 256 MB Infinity Cache so that reads come from HBM.

cpu_baseline: the oracle (a restatement of hodu's CPU kernels, kind "port") timed on this host on
a bounded sample of the same workload, under the reference's own threading policy.
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

# HBM bytes per launch of the dominant kernel, from the rocprofv3 --pmc runs summarised under
# profiles/ (FETCH_SIZE + WRITE_SIZE scaled by the copy-kernel calibration); None = not measured
MEASURED_TRAFFIC = {
    "mfma_bf16_pipe256x256w8_KK@c2": 100.2e6,
    "gemv_bf16_f8w@c3_m1": 16.83e6,
    "gemv_bf16_f8w@gemv_14336x4096": 58.6e6,
    "skinny_bf16_f8w_splitk@c3_m16": 22.2e6,
    "mfma_bf16_pipe256x256w8_KK@c5_down_bf16": 734.5e6,
    "mfma_f8e4m3_pipe256x256_KK@f8_4096": 124.1e6,
}


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


def time_case(ctx, case, steps, warmup, graph=False):
    """returns a result dict; operands are uploaded before the timed region starts"""
    md, obytes = out_bytes(case)
    a = ctx.upload(case.make_a())
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
    from hodu_amd import ffi
    fused_steps, bias = [], None
    for what in case.fused:
        if what == "bias":
            bias = ctx.upload(bf16(normal(700, case.rv.shape[-1], 0.1)))
            fused_steps.append(ffi.add_row(bias))
        elif what == "scale":
            fused_steps.append(ffi.mul_scalar(bf16(np.array([0.125], dtype=np.float32))))
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
    # spread: ten more batches of the same launches (outside the K timed steps), each timed the same way
    batch = steps
    spread = sorted(ctx.time_product(case.op, case.name, a, ws, out, md, batch, graph=graph, steps=fused_steps) * 1e3 / batch
                    for _ in range(10))
    for buf in [a, out] + ws + ([bias] if bias else []):
        buf.free()
    per_launch_s = ms / 1e3 / steps
    tflops = case.flops / per_launch_s / 1e12
    gbs = case.alg_bytes / per_launch_s / 1e9
    if case.bound == "hbm":
        roof = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS}
    else:
        peak = PEAK[case.peak_key]
        roof = {"bound": "mfma", "achieved": tflops, "peak": peak, "unit": "TFLOP/s", "frac": tflops / peak}
    roof["traffic"] = MEASURED_TRAFFIC.get(f"{kernel}@{case.key}")
    roof["kernel"] = kernel
    return {"config": case.key, "label": case.label, "kernel": kernel, "us_per_launch": per_launch_s * 1e6,
            "tflops": tflops, "algorithmic_gbs": gbs, "weight_buffers_rotated": copies, "roofline": roof,
            "us_batches": {"launches_per_batch": batch, "p10": spread[1], "median": 0.5 * (spread[4] + spread[5]),
                           "p90": spread[8]}}


def attention_probe(ctx, steps, d=128):
    """not a BASELINE configuration: hodu_nn's scaled_dot_product_attention (causal, bf16, 32 heads x 2048 x d) as
    the one fused kernel, and as the three launches the host mirror falls back to -- Q K^T with the scale in its
    store, masked softmax, P V -- each timed with HIP events around `steps` back-to-back launches"""
    import helpers as H
    from hodu_amd import ffi
    V = H.View
    heads, s_len = 32, 2048
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
        total += us if name != "fused_one_kernel" else 0.0
    flops = 2 * 2.0 * heads * s_len * s_len * d
    res["qk_scaled"]["tflops"] = flops / 2 / res["qk_scaled"]["us"] / 1e6
    res["pv"]["tflops"] = flops / 2 / res["pv"]["us"] / 1e6
    res["softmax_causal"]["gbs"] = 2.0 * heads * s_len * s_len * 2 / res["softmax_causal"]["us"] / 1e3
    for b in (q, k, v, scores, probs, out):
        b.free()
    # the causal mask halves the useful work; rates count the unmasked half only for the fused kernel
    res["fused_one_kernel"]["tflops_useful"] = flops / 2 / res["fused_one_kernel"]["us"] / 1e6
    return {"config": "attention", "shape": f"bf16 q,k,v [{heads},{s_len},{d}], causal", "us_three_launches": total,
            "us_fused": res["fused_one_kernel"]["us"], "legs": res}


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
    ctx.time_cast(src, dst, ins, outs, md, max(warmup, 1))
    kernel = ctx.last_kernel()
    ms = ctx.time_cast(src, dst, ins, outs, md, steps)
    spread = sorted(ctx.time_cast(src, dst, ins, outs, md, steps) * 1e3 / steps for _ in range(10))
    for b in ins + outs:
        b.free()
    s_per = ms / 1e3 / steps
    alg = n * (ffi.DTYPE_SIZE[src] + ffi.DTYPE_SIZE[dst])
    gbs = alg / s_per / 1e9
    return {"config": key, "label": label, "kernel": kernel, "us_per_launch": s_per * 1e6, "tflops": 0.0,
            "algorithmic_gbs": gbs, "weight_buffers_rotated": pairs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "traffic": None, "kernel": kernel},
            "us_batches": {"launches_per_batch": steps, "p10": spread[1], "median": 0.5 * (spread[4] + spread[5]),
                           "p90": spread[8]}}


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
    ins = [ctx.upload(bf16(normal(61, n)))]
    for _ in range(1, pairs):
        extra = ctx.alloc(2 * n)
        ctx.lib.hodu_rocm_memcpy_d2d(ctx.handle, extra.ptr, ins[0].ptr, 2 * n)
        ins.append(extra)
    outs = [ctx.alloc(2 * n_out) for _ in range(pairs)]
    md = H.reduce_md(view, dims, False)
    ctx.time_sum("bf16", ins, outs, md, max(warmup, 1))
    kernel = ctx.last_kernel()
    ms = ctx.time_sum("bf16", ins, outs, md, steps)
    spread = sorted(ctx.time_sum("bf16", ins, outs, md, steps) * 1e3 / steps for _ in range(10))
    for b in ins + outs:
        b.free()
    s_per = ms / 1e3 / steps
    gbs = 2 * (n + n_out) / s_per / 1e9
    return {"config": key, "label": label, "kernel": kernel, "us_per_launch": s_per * 1e6, "tflops": 0.0,
            "algorithmic_gbs": gbs, "weight_buffers_rotated": pairs,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "traffic": None, "kernel": kernel},
            "us_batches": {"launches_per_batch": steps, "p10": spread[1], "median": 0.5 * (spread[4] + spread[5]),
                           "p90": spread[8]}}


def host_buffers_probe(ctx, reps=5):
    """config 2 with the operands starting and the result ending in host memory (pageable numpy arrays through
    hodu_rocm_memcpy_h2d / _d2h, buffers allocated beforehand): what a caller pays who hands host buffers over per
    product instead of keeping tensors on the device.  Never the headline value."""
    import time
    case = build_cases(["c2"])[0]
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
    return {"config": "c2_host_buffers", "ms_per_product": s_per * 1e3, "tflops": case.flops / s_per / 1e12,
            "bytes_over_pcie": moved, "gbs_over_pcie": moved / s_per / 1e9, "host_memory": "pageable"}


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
    constant and on N(0,1) operands: the clock under full MFMA load depends on the data"""
    import helpers as H
    out = []
    for kind, name, peak in ((0, "bf16 32x32x16", PEAK["bf16"]), (1, "f8e4m3 32x32x64 (unit scales)", PEAK["fp8"])):
        for data in ("constant", "normal"):
            if kind == 0:
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


def cpu_baseline_c2(budget_s=15.0):
    """hodu's CPU path for config 2, timed on a bounded sample.

    hodu routes a >= 3-D matmul to hodu_cpu_matmul_bf16, whose batched path runs on ONE thread and
    accumulates in bf16 (crates/hodu_cpu_kernels/kernels/ops_matrix.c:292-337); through the public
    API the transposed operand is first copied (tensor/ops/shape.rs:232-237), which is not timed.
    The sample is the first few of the 16 batches (all 1024 rows of each, or fewer rows of one batch
    on a slow host), sized by a short probe to about `budget_s` seconds; the rate is per flop, so it
    scales linearly to the whole job.
    """
    import helpers as H
    import oracle
    n = 1024
    a = bf16(normal(201, n * n, 1 / 32))
    b = bf16(normal(202, n * n, 1 / 32))
    oracle.set_threads(1)
    # a short probe fixes the rate, then one run sized to the budget: `rows` rows of each of `nb` batches
    lv, rv = H.View([1, 32, n]), H.View([1, n, n]).t()
    t0 = time.perf_counter()
    oracle.matmul_asis("bf16", a[:32 * n], b, H.matmul_md(lv, rv))
    probe = time.perf_counter() - t0
    rows_total = max(32, int(budget_s / (probe / 32)))
    nb = max(1, min(16, rows_total // n))
    rows = n if rows_total >= n else rows_total
    lv, rv = H.View([nb, rows, n]), H.View([nb, n, n]).t()
    a_s, b_s = np.tile(a[:rows * n], nb), np.tile(b, nb)
    t0 = time.perf_counter()
    oracle.matmul_asis("bf16", a_s, b_s, H.matmul_md(lv, rv))
    t_used = time.perf_counter() - t0
    rate = 2.0 * nb * rows * n * n / t_used
    # the f32-accumulated comparator path (to_dtype(f32) + sgemm), all cores, for scale
    af = H.bf16_to_f32(a).reshape(n, n)
    bfm = H.bf16_to_f32(b).reshape(n, n)
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 1.5:
        af @ bfm.T
        reps += 1
    sgemm_rate = 2.0 * n ** 3 * reps / (time.perf_counter() - t0)
    oracle.set_threads(os.cpu_count() or 1)
    return {"value": rate / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"hodu_cpu_matmul_bf16 semantics (bf16-accumulate, batched path, 1 thread) on {nb} of the 16 "
                      f"batches, {rows} of 1024 rows each, x full [1024,1024]^T-view; {t_used:.1f} s of CPU work",
            "host_cores_online": os.cpu_count(),
            "f32_comparator_sgemm_tflops": sgemm_rate / 1e12,
            "f32_comparator_note": "to_dtype(f32) inputs through numpy's OpenBLAS sgemm on all host cores (1024^3)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--configs", default="c1,c2,c3,c4,c5,f8,f64,fused,bwd,casts")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--only", default="", help="time exactly one case key (e.g. c5_down_bf16) and print its result")
    ap.add_argument("--force-tile", type=int, default=-1, help="testing hook: pin the MFMA tile variant (0..3)")
    ap.add_argument("--graph", action="store_true", help="with --only: replay the K launches as one HIP graph")
    ap.add_argument("--force-splitk", type=int, default=-1, help="testing hook: pin the number of K ranges")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU: it has no collective or sharded path, and `value` is the one "
              "GPU's throughput. Re-run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

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
        print(json.dumps(host_buffers_probe(ctx)))
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
        print(json.dumps(time_case(ctx, case, args.steps, args.warmup, graph=args.graph)))
        ctx.close()
        return
    which = set(args.configs.split(",")) | {"c2"}
    results = []
    for case in build_cases(which):
        steps = args.steps if case.flops < 4e11 else max(5, args.steps // 5)
        results.append(time_case(ctx, case, steps, args.warmup))
        print(f"# {results[-1]['label']}: {results[-1]['us_per_launch']:.1f} us  {results[-1]['tflops']:.1f} TFLOP/s  "
              f"{results[-1]['algorithmic_gbs']:.0f} GB/s  [{results[-1]['kernel']}] "
              f"{100 * results[-1]['roofline']['frac']:.1f}% of {results[-1]['roofline']['bound']} peak",
              file=sys.stderr, flush=True)
    if "casts" in which:
        for cc in cast_cases():
            results.append(time_cast_case(ctx, *cc, args.steps, args.warmup))
            print(f"# {results[-1]['label']}: {results[-1]['us_per_launch']:.1f} us  {results[-1]['algorithmic_gbs']:.0f} GB/s  "
                  f"[{results[-1]['kernel']}] {100 * results[-1]['roofline']['frac']:.1f}% of hbm peak", file=sys.stderr, flush=True)
    if "bwd" in which:
        for sc in sum_cases():
            results.append(time_sum_case(ctx, *sc, args.steps, args.warmup))
            print(f"# {results[-1]['label']}: {results[-1]['us_per_launch']:.1f} us  {results[-1]['algorithmic_gbs']:.0f} GB/s  "
                  f"[{results[-1]['kernel']}] {100 * results[-1]['roofline']['frac']:.1f}% of hbm peak", file=sys.stderr, flush=True)
    head = next(r for r in results if r["config"] == "c2")
    # the headline is re-timed with exactly the requested step count
    case2 = [c for c in build_cases({"c2"})][0]
    head = time_case(ctx, case2, args.steps, args.warmup)
    line = {
        "metric": "TFLOP/s & % MFMA peak per dtype; M=1 GEMV GB/s & % HBM peak",
        "value": head["tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["us_per_launch"] / 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: bf16 batched matmul A[16,1024,1024] x B[16,1024,1024], "
                               "B a transposed (non-contiguous) view, f32 accumulate, bf16 out; one matmul call per step",
                   "flop_per_step": case2.flops, "algorithmic_bytes_per_step": case2.alg_bytes},
        "roofline": {k: head["roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")},
        "dominant_kernel": head["kernel"],
        # not part of the roofline (whose peak is the datasheet's): the rate a register-only MFMA loop sustains on
        # this box, by operand data
        "register_only_mfma": mfma_clock_probe(ctx),
        # likewise for the HBM-bound rows: a kernel that only reads, at the M = 1 configurations' sizes
        "streaming_read": read_floor_probe(ctx),
        "device": info,
        "all_configs": results,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_c2()
    ctx.close()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
