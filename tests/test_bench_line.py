"""The benchmark's final stdout line: small, one JSON object, and carrying what a reader of it needs.

A canned record shaped like a real run (30 rows with long kernel descriptions) goes through
bench.final_line(); nothing here touches a GPU or the library.
"""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("wkf_bench", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _row(key, frac, unit="GB/s"):
    detail = "rows=256 n=262144 vec=4 threads_per_row=256 vectors_per_lane=8 stages=2 operands=2, " * 3
    return {"name": "configuration " + key + " with a long descriptive name " * 2, "dtype": "f32", "unit": unit, "work_per_step": 1 << 30,
            "kernels": [{"kind": "row", "detail": detail, "us": 100.0, "min_us": 99.0}] * 3,
            "median_us_per_step": 100.0, "min_us_per_step": 99.0, "achieved": 5000.0, "peak": 8000.0, "frac": frac, "min_frac": frac,
            "batch_us_per_step": 101.0, "batch_achieved": 4990.0, "batch_frac": frac,
            "roofline": {"bound": "hbm", "kernel": "row " + detail, "kernels_per_step": 1, "avg_us": 101.0, "achieved": 4990.0,
                         "peak": 8000.0, "unit": unit, "frac": frac},
            "wall_ms_per_step": 0.1, "wall_rate": 4900.0, "key": key,
            "cpu_baseline": {"value": 1.0, "unit": unit, "cores": 16, "kind": "port", "sample": "a bounded sample " * 8}}


def _canned(bench, rows):
    return {"metric": bench.METRIC, "value": 6739.5, "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 0.0797,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "config2: row max(x) and row sum(exp(x-1)), f32 [8192,8192]", "seed": "SplitMix64", "rotating_inputs": 4,
                       "kernels_per_step": 2, "algorithmic_bytes_per_step": 536936448,
                       "kernel_us": {"row_max": 39.0, "row_sum_exp": 39.7, "per_launch_event_pairs_median": [38.5, 38.9]},
                       "device": "gfx950:sramecc+:xnack-", "compute_units": 256, "clock_khz": 2400000},
            "roofline": {"bound": "hbm", "achieved": 6753.9, "peak": 8000.0, "unit": "GB/s", "frac": 0.8442, "traffic": 268700000,
                         "traffic_source": "profiles/traffic.json " * 3, "kernel": "red_row " + "x" * 120, "avg_us": 39.75,
                         "algorithmic_bytes_per_launch": 268468224},
            "value_frac_of_hbm_peak": 0.8424,
            "cpu_baseline": {"value": 36.66, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "the full config-2 step " * 4},
            "reference_cpu_path": {"available": False, "probe": {"cargo": None, "rustc": None, "vulkan_icds": ["/x.json"] * 20},
                                   "note": "the reference's wgpu path on a CPU adapter needs cargo + rustc + a Vulkan CPU ICD"},
            "copy_kernel_GBs": 6334.0,
            "all_configs": rows}


def test_final_line_is_small_and_round_trips():
    bench = _bench()
    keys = ["c1", "c2_one_pass", "c2a", "c2b", "c3", "c3_reference_rules", "c4_rmsnorm", "c4_rope", "c4_softmax", "c5_f32", "c5_f16",
            "c5_mlp"] + ["more_%d" % i for i in range(28)]
    rows = [_row(k, 0.3 + 0.01 * i) for i, k in enumerate(keys)]
    rows[10] = _row("c5_f16", 0.21, "TFLOP/s")
    text, full = bench.final_line(_canned(bench, rows))
    assert "\n" not in text and len(text) <= bench.MAX_LINE_BYTES <= 4096
    line = json.loads(text)
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
              "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in line, k
    assert "all_configs" not in line and len(full["all_configs"]) == len(keys)
    assert line["config"]["workload"].startswith("config2")
    assert set(line["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    assert set(line["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"}
    assert line["worst_config"]["key"] == "c5_f16" and line["worst_config"]["frac"] == 0.21
    assert line["fracs"]["c1"] == [0.3, 101.0] and len(line["fracs"]) == len(keys)
    assert json.loads(json.dumps(full))["all_configs"][0]["key"] == "c1"


def test_final_line_drops_optional_parts_before_it_grows():
    bench = _bench()
    rows = [_row("c_%04d_with_a_long_key_name" % i, 0.5) for i in range(400)]
    text, _ = bench.final_line(_canned(bench, rows))
    assert len(text) <= bench.MAX_LINE_BYTES
    line = json.loads(text)
    assert "fracs" not in line and "roofline" in line and "cpu_baseline" in line


def test_headline_only_run_has_no_detail():
    bench = _bench()
    rec = _canned(bench, [])
    del rec["all_configs"]
    text, full = bench.final_line(rec)
    line = json.loads(text)
    assert "fracs" not in line and "all_configs" not in full and line["value"] == 6739.5
