"""The one JSON line bench.py prints last must stay small: whatever reads it keeps only a tail of stdout, and a line
that outgrows that tail loses its head (metric, value, roofline).  Built here from canned rows, no GPU."""
import json
import os
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), ".."))
import bench  # noqa: E402


def _row(key, bound, peak, us, kernel):
    return {"config": key, "label": key + " " + "x" * 60, "kernel": kernel, "us_per_launch": us, "first_batch_us": us * 1.2,
            "headline_ms_total": us * 20 / 1e3, "flops": 4.81e11, "alg_bytes": 2.684e8, "parity": {"rows_checked": 6},
            "roofline": {"bound": bound, "peak": peak, "unit": "GB/s" if bound == "hbm" else "TFLOP/s", "achieved": 1.0,
                         "frac": 0.5, "traffic": 7.3463e8, "traffic_source": "profiles/traffic_counters_all_bench_rows.txt",
                         "kernel": kernel},
            "us_batches": {"launches_per_batch": 20, "batches": 10, "p10": us * 0.99, "median": us, "p90": us * 1.01}}


def _canned(extra_rows=0):
    long_name = "mfma_bf16_f8w_pipe256x256mi16_KK_splitk4"
    keys = ["c1", "c2", "c3_m1", "c3_m16", "c3_m256", "c3_m4096", "gemv_14336x4096", "f8_4096", "bf16_4096", "f64_2048",
            "c4", "c5_up_bf16", "c5_down_bf16", "c5_up_f8e4m3", "c5_down_f8e4m3", "c5_up_dw_bf16", "c3_m1_linear",
            "c3_m16_linear", "c2_scaled", "c5_up_bf16_bias_relu", "cast_f8e4m3_bf16_c3w", "cast_f8e4m3_bf16_c5w",
            "cast_i8_i32_c4", "contiguous_bf16_c2_bt", "contiguous_bf16_c5_wdown", "sum_bias_grad_c5_up",
            "sum_bias_grad_c5_down", "sum_rows_c5"] + [f"extra_configuration_{i}" for i in range(extra_rows)]
    results = [_row(k, "hbm" if ("m1" in k or "cast" in k or "sum" in k) else "mfma", 8000.0 if "m1" in k else 2500.0,
                    294.123456, long_name) for k in keys]
    cpu_rows = [{"key": k, "path": "hodu_cpu_matmul_bf16 " + "y" * 100, "value": 0.00085924641, "unit": "TFLOP/s", "cores": 1,
                 "kind": "reference", "sample": "64 of the 8 x 512 rows against the whole weight", "seconds_sampled": 8.747,
                 "whole_job_seconds": 559.835, "whole_job_is": "linear extrapolation of the sample",
                 "f32_comparator_sgemm_tflops": 2.97222691, "host_cores_online": 16}
                for k in ("c1", "c2", "c3_m1", "c3_m16", "c3_m256", "c3_m4096", "c4", "c5_down_bf16", "c5_down_f8e4m3",
                          "c5_up_bf16", "c5_up_f8e4m3")]
    return results, cpu_rows


def test_line_is_small_and_round_trips():
    results, cpu_rows = _canned(extra_rows=4)  # room for rows added later, every kernel name at the longest
    head = next(r for r in cpu_rows if r["key"] == "c5_down_bf16")
    line, full = bench.assemble_line(20, 10, "c5_down_bf16", 4.81e11, 2.684e8, results, cpu_rows, head,
                                     {"device": {"name": "x"}, "register_only_mfma": [], "streaming_read": []})
    text = json.dumps(line, separators=(",", ":"))
    assert "\n" not in text
    assert len(text) < bench.LINE_LIMIT <= 6000, len(text)
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in back, key
    assert back["vs_baseline"] is None and back["n_gpus"] == 1
    roof = back["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(back["value"] - 4.81e11 / (back["ms_per_step"] * 1e-3) / 1e12) < 0.05
    cols = roof["per_config_columns"]
    assert cols[0] == "key" and all(len(r) == len(cols) for r in roof["per_config"])
    assert len(roof["per_config"]) == len(results) == roof["rows"] == roof["parity_rows_ok"]
    cpu = back["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    assert len(cpu["sample"]) <= 200
    assert {tuple(sorted(r)) for r in cpu["per_config"]} == {("cores", "key", "kind", "value", "whole_job_is")}
    assert [t["key"] for t in back["config"]["north_star"]] == ["c3_m4096", "c5_down_bf16", "c5_up_bf16", "bf16_4096",
                                                                 "f8_4096", "c3_m1"]
    # the unabridged record keeps what the line drops
    assert full["all_configs"] is results and full["cpu_baseline"]["per_config"] is cpu_rows and "device" in full


def test_line_without_cpu_leg():
    results, _ = _canned()
    line, _ = bench.assemble_line(5, 2, "c5_down_bf16", 4.81e11, 2.684e8, results, None, None)
    assert "cpu_baseline" not in line and line["steps"] == 5 and line["warmup"] == 2


@pytest.mark.skipif(os.environ.get("HODU_EMU_ALL", "0") in ("", "0"), reason="slow in the CPU build: set HODU_EMU_ALL=1")
def test_timed_cases_and_the_line_against_the_cpu_build():
    """bench.py's own per-case routine -- buffers, the timing loop of the debug library, the in-run parity check of a
    timed output buffer -- on config 1 and config 3 at M = 1 at their full sizes against the CPU build of the library
    (tests/emu_util.py), and the JSON line assembled from those rows.  The times are the emulation's and mean nothing."""
    import emu_util
    if emu_util.compiler() is None:
        pytest.skip("no host clang++ for the CPU build")
    ctx = emu_util.EmuContext()
    try:
        cases = {c.key: c for c in bench.build_cases({"c1", "c3"})}
        rows = [bench.time_case(ctx, cases["c1"], 2, 1, exact_steps=True), bench.time_case(ctx, cases["c3_m1"], 2, 1, headline=(2, 1))]
    finally:
        ctx.close()
    assert [r["kernel"] for r in rows] == ["small_f32_KM", "gemv_bf16_f8w_walk"]
    assert all(r["parity"] and r["parity"]["rows_checked"] >= 1 for r in rows)
    line, _ = bench.assemble_line(2, 1, "c3_m1", cases["c3_m1"].flops, cases["c3_m1"].alg_bytes, rows, None, None)
    text = json.dumps(line, separators=(",", ":"))
    assert len(text) < bench.LINE_LIMIT
    per_config = json.loads(text)["roofline"]["per_config"]
    assert [(row[0], row[2], row[6]) for row in per_config] == [("c1", "mfma", "small_f32_KM"), ("c3_m1", "hbm", "gemv_bf16_f8w_walk")]


def test_attention_probe_against_the_cpu_build():
    """`bench.py --only attention`'s routine at a reduced size against the CPU build: every leg launches the kernel it
    names (the times are the emulation's and mean nothing)"""
    import emu_util
    if emu_util.compiler() is None:
        pytest.skip("no host clang++ for the CPU build")
    ctx = emu_util.EmuContext()
    try:
        res = bench.attention_probe(ctx, 1, 64, heads=2, s_len=128)
    finally:
        ctx.close()
    kernels = {name: leg["kernel"] for name, leg in res["legs"].items()}
    assert kernels["fused_one_kernel"] == "attention_fwd_bf16_d64" and kernels["fused_padding_mask"] == "attention_masked_fwd_bf16_d64"
    assert kernels["softmax_causal"].startswith("softmax_") and kernels["softmax_padding_mask"] == "softmax_masked"
    assert res["us_three_launches"] == pytest.approx(sum(res["legs"][n]["us"] for n in ("qk_scaled", "softmax_causal", "pv")))
