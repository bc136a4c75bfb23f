"""The last stdout line of bench.py is what a harness parses: it must stay small (a harness that keeps only the tail of
stdout otherwise starts mid-object) and carry the headline, its roofline and the CPU baseline."""
import json

import bench


def _roofline(bound, unit, n):
    return {"bound": bound, "achieved": 1038.637059950548, "peak": 2516.6, "unit": unit, "frac": 0.4127144003618168,
            "traffic": 710652928.0, "traffic_source": "constant from profiles/" + "x" * 200, "kernel": "k" * 60,
            "algorithmic_flops_per_launch": 549890031616.0, "launch_ms_mean": 0.5294342488050461,
            "launch_ms_median": 0.5276944935321808, "launch_ms_min": 0.5232549905776978, "extra": list(range(n))}


def _stub():
    cpu = {"value": 0.004632295403535066, "unit": "TFLOP/s", "cores": 16, "kind": "port", "sample": "s" * 900}
    big = {"leg%d" % i: {"workload": "w" * 120, "roofline": _roofline("hbm", "GB/s", 30)} for i in range(40)}
    return {
        "metric": bench.METRIC, "value": 1032.4270033578005, "unit": "TFLOP/s", "n_gpus": 1, "steps": 20, "warmup": 5,
        "ms_per_step": 0.5326187999999732, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: Q,K,V i.i.d. N(0,1) from numpy PCG64(seed 20261125+config), rounded to bf16",
        "config": {"workload": "BASELINE config 3: bf16 causal prefill B=8 H=16 S_q=S_kv=4096 D=128, scale=1/sqrt(128), "
                               "f32 accumulate, bf16 out", "step": "one incin_rocm_sdpa_fwd launch"},
        "device": {"name": "", "arch": "gfx950:sramecc+:xnack-", "compute_units": 256, "clock_khz": 2400000},
        "roofline": _roofline("mfma", "TFLOP/s", 10), "cpu_baseline": cpu, "parity_max_abs_err": 0.0014135241508483887,
        "prefill_with_dense_mask_tensor": {"what": "x" * 300},
        "prefill_long": {"workload": "w" * 400, "value": 1250.0, "unit": "TFLOP/s", "ms_per_step": 5.1,
                         "roofline": _roofline("mfma", "TFLOP/s", 10), "parity_max_abs_err": 1e-3},
        "decode": {"workload": "BASELINE config 4: bf16 decode MHA B=32 H=32 S_q=1 KV=8192 D=128", "value": 7100.0, "unit": "GB/s",
                   "ms_per_step": 0.605, "roofline": _roofline("hbm", "GB/s", 10), "cpu_baseline": dict(cpu, unit="GB/s"),
                   "parity_max_abs_err": 2e-4, "vector_alu_kernel": {"x": "y" * 500}, "decode_step_graph": {"x": "y" * 500}},
        "prefill_chunk": big, "decode_gqa": big, "head_dims": big, "f32_c1": big, "f32_c2": big, "matrix_rate": big,
        "backward": {"value": 561.8, "unit": "TFLOP/s", "ms_per_step": 2.447, "frac_of_bf16_mfma_peak": 0.223, "workload": "w" * 300},
    }


def test_compact_line_is_small_and_complete():
    line = bench.compact_line(_stub())
    assert "\n" not in line
    assert len(line) < 4096
    d = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity_max_abs_err"):
        assert key in d, key
    assert d["config"]["workload"].startswith("BASELINE config 3")
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic", "launch_ms_mean"):
        assert key in d["roofline"], key
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / d["roofline"]["peak"]) < 1e-4
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in d["cpu_baseline"], key
    assert d["decode"]["roofline"]["bound"] == "hbm" and "cpu_baseline" in d["decode"]
    assert "frac" in d["prefill_long"]["roofline"]
    # the legs that made the line too long for a tail-reading harness are not on it
    for key in ("prefill_chunk", "decode_gqa", "head_dims", "f32_c1", "matrix_rate"):
        assert key not in d


def test_compact_line_of_a_single_leg_run():
    """`--only decode` (profiling) has no headline figures: the line still parses."""
    d = json.loads(bench.compact_line({"metric": bench.METRIC, "value": None, "decode": {"value": 1.0, "roofline": {"frac": 0.5}}}))
    assert d["value"] is None and d["decode"]["roofline"]["frac"] == 0.5
