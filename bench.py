#!/usr/bin/env python3
"""Benchmark of the fused hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-detail] [--no-cpu]

Prints ONE JSON line.  The headline (`value`) is BASELINE.json's metric on its
configuration 2: one step = the two fused row-reduce kernels of a softmax,
row max(x) and row sum(exp(x - 1)), over f32 [8192, 8192]; value = algorithmic
GB/s of the whole step by the wall clock, inputs resident in HBM, steps rotating
over several input tensors so that the 256 MB Infinity Cache cannot serve them.
`roofline` is the dominant kernel (the exp-sum reduce) timed with hipEvent pairs
on the stream it runs on; `cpu_baseline` is the CPU port of the reference's
decomposition (oracle/port.c) on this box's host cores; `all_configs` carries
every BASELINE configuration (GB/s or TFLOP/s and the fraction of the roofline).

Everything runs on one GPU: `--gpus N` with N > 1 is refused.
"""
import argparse
import importlib.util
import json
import os
import subprocess
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
F16_MFMA_PEAK_TFLOPS = 2500.0  # dense f16 MFMA, published
F32_MFMA_PEAK_TFLOPS = 157.3   # f32, published
METRIC = "fused-op HBM GB/s (% of peak) + matmul TFLOP/s (% MFMA peak), 1 MI355X"


def load_package():
    # the benchmark loads what is built; only a tree with no built library at all is built first
    if not os.path.exists(os.path.join(ROOT, "wgpu-kernal-fusion_amd", "libwkf_hip.so")):
        subprocess.check_call(["bash", os.path.join(ROOT, "wgpu-kernal-fusion_amd", "build.sh")])
    if not os.path.exists(os.path.join(ROOT, "oracle", "libwkf_port.so")):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    path = os.path.join(ROOT, "wgpu-kernal-fusion_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location("wgpu_kernal_fusion_amd", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules["wgpu_kernal_fusion_amd"] = mod
    spec.loader.exec_module(mod)
    mod.load()  # raises when the library is not built: there is no fallback path
    return mod


def rope_tables(seq, dim, theta=10000.0):
    inv = theta ** (-np.arange(0, dim, 2, dtype=np.float64) / dim)
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


class Workload:
    """`variants`: the same expression over different input tensors (rotated step by step)."""

    def __init__(self, name, variants, work, unit, peak, dtype="f32", joint=None):
        self.name, self.variants, self.work, self.unit, self.peak, self.dtype = name, variants, work, unit, peak, dtype
        self.joint = joint  # the package's materialize_many: the tensors of a step are materialised in ONE pass

    def step(self, i):
        """Launches step i; returns the tensors whose kernel records describe it."""
        ts = self.variants[i % len(self.variants)]
        if self.joint:
            self.joint(ts)
            return ts[:1]
        for t in ts:
            t.materialize()
        return ts


def measure_kernels(dev, wl, steps, warmup):
    """Per-kernel GPU time (hipEvent pair around each launch), averaged over `steps` steps."""
    dev.set_timing(True)
    for i in range(warmup):
        wl.step(i)
    dev.sync()
    sums, kinds, details = None, None, None
    for i in range(steps):
        ns = []
        ks = []
        for t in wl.step(i):
            ks += t.kernels()
        ns = np.array([k.elapsed_ns for k in ks], dtype=np.float64)
        sums = ns if sums is None else sums + ns
        kinds = [k.kind for k in ks]
        details = [k.detail for k in ks]
    avg = sums / steps
    return [{"kind": k, "detail": d, "us": round(float(a) / 1e3, 2)} for k, d, a in zip(kinds, details, avg)]


def measure_batch(w, dev, wl, steps, warmup):
    """Average GPU time per step from ONE hipEvent pair around `steps` back-to-back steps on the
    library's stream (no per-launch events, so neither their cost nor host gaps are counted twice)."""
    import ctypes
    lib = w.load()
    timer = ctypes.c_void_p()
    assert lib.wkf_timer_create(dev._h, ctypes.byref(timer)) == 0
    dev.set_timing(False)
    try:
        for i in range(warmup):
            wl.step(i)
        dev.sync()
        assert lib.wkf_timer_begin(timer) == 0
        for i in range(steps):
            wl.step(i)
        assert lib.wkf_timer_end(timer) == 0
        ns = ctypes.c_uint64()
        assert lib.wkf_timer_elapsed_ns(timer, ctypes.byref(ns)) == 0
        return ns.value / steps / 1e3  # us per step
    finally:
        dev.set_timing(True)
        lib.wkf_timer_destroy(timer)


def measure_wall(dev, wl, steps, warmup):
    """Wall-clock seconds for `steps` steps, no per-launch events, synchronised on both sides."""
    dev.set_timing(False)
    try:
        for i in range(warmup):
            wl.step(i)
        dev.sync()
        t0 = time.perf_counter()
        for i in range(steps):
            wl.step(i)
        dev.sync()
        return time.perf_counter() - t0
    finally:
        dev.set_timing(True)


def summarise(wl, kernels, wall_s, steps, batch_us):
    gpu_us = sum(k["us"] for k in kernels)
    scale = 1e-3 if wl.unit == "GB/s" else 1e-6  # bytes/us -> GB/s ; flop/us -> TFLOP/s
    return {"name": wl.name, "dtype": wl.dtype, "unit": wl.unit, "work_per_step": wl.work,
            "kernels": kernels, "gpu_us_per_step": round(gpu_us, 2),
            "achieved": round(wl.work / gpu_us * scale, 1), "peak": wl.peak,
            "frac": round(wl.work / gpu_us * scale / wl.peak, 4), "batch_us_per_step": batch_us,
            "batch_achieved": round(wl.work / batch_us * scale, 1) if batch_us else None,
            "batch_frac": round(wl.work / batch_us * scale / wl.peak, 4) if batch_us else None,
            "wall_ms_per_step": round(wall_s / steps * 1e3, 4),
            "wall_rate": round(wl.work * steps / wall_s * (1e-9 if wl.unit == "GB/s" else 1e-12), 1)}


def build_workloads(w, dev, seeded, which):
    T = w.Tensor
    out = {}
    if "c2" in which:
        xs = [T.new(dev, seeded(2, r, (8192, 8192), "normal")) for r in range(4)]
        out["c2"] = Workload("config2: row max(x) + row sum(exp(x-1)), f32 [8192,8192]",
                             [[x.max(1), (x.clone() - 1.0).exp().sum(1)] for x in xs], 2 * 268468224, "GB/s", HBM_PEAK_GBS)
        # the same two results from ONE pass over the matrix (the reference lists this fusion as to-do, README.md:20):
        # algorithmic bytes = the matrix once + both result vectors
        out["c2_one_pass"] = Workload("config2 in one pass: row max(x) and row sum(exp(x-1)) together, f32 [8192,8192]",
                                      [[x.max(1), (x.clone() - 1.0).exp().sum(1)] for x in xs], 8192 * 8192 * 4 + 2 * 8192 * 4,
                                      "GB/s", HBM_PEAK_GBS, joint=w.materialize_many)
        out["c2a"] = Workload("config2a: row max(x), f32 [8192,8192]", [[x.max(1)] for x in xs], 268468224, "GB/s", HBM_PEAK_GBS)
        out["c2b"] = Workload("config2b: row sum(exp(x-1)), f32 [8192,8192]", [[(x.clone() - 1.0).exp().sum(1)] for x in xs],
                              268468224, "GB/s", HBM_PEAK_GBS)
    if "c1" in which:
        xs = [T.new(dev, seeded(1, r, (4096, 4096), "uniform")) for r in range(8)]
        out["c1"] = Workload("config1: exp(sin(x*2+1)), f32 [4096,4096]", [[((x * 2.0) + 1.0).sin().exp()] for x in xs],
                             134217728, "GB/s", HBM_PEAK_GBS)
    if "c3" in which:
        variants = []
        bias = T.new(dev, seeded(3, 2, (4096,), "normal", std=0.02))
        bias3 = bias.broadcast([1024, 4096]).broadcast([32, 1024, 4096])
        for r in range(2):
            a = T.new(dev, seeded(3, 4 * r, (32, 1024, 4096), "uniform"))
            b = T.new(dev, seeded(3, 4 * r + 1, (32, 1024, 4096), "uniform"))
            variants.append([a.silu() * (b + bias3)])
        out["c3"] = Workload("config3: silu(a)*(b+bias), f32 [32,1024,4096]", variants, 1610629120, "GB/s", HBM_PEAK_GBS)
    if "c4" in which:
        w4 = T.new(dev, seeded(4, 1, (4096,), "normal", mean=1.0, std=0.02))
        xs = [T.new(dev, seeded(4, 8 + r, (2048, 4096), "normal")) for r in range(8)]
        out["c4_rmsnorm"] = Workload("config4: RMSNorm f32 [2048,4096]", [[x.layer_norm(w4, 1e-5)] for x in xs], 67125248, "GB/s", HBM_PEAK_GBS)
        cos, sin = rope_tables(2048, 128)
        tc, ts = T.new(dev, cos), T.new(dev, sin)
        qs = [T.new(dev, seeded(4, 16 + r, (32, 2048, 128), "normal")) for r in range(8)]
        out["c4_rope"] = Workload("config4: RoPE f32 [32,2048,128]", [[q.rope(tc, ts)] for q in qs], 69206016, "GB/s", HBM_PEAK_GBS)
        ss = [T.new(dev, seeded(4, 24 + r, (32, 2048, 2048), "normal")) for r in range(2)]
        out["c4_softmax"] = Workload("config4: softmax f32 [32,2048,2048]", [[s.softmax_last_dim()] for s in ss], 1073741824, "GB/s", HBM_PEAK_GBS)
    if "c5" in which:
        a32 = T.new(dev, seeded(5, 0, (4096, 4096), "normal", std=0.02))
        b32 = T.new(dev, seeded(5, 1, (4096, 4096), "normal", std=0.02))
        out["c5_f32"] = Workload("config5a: GEMM f32 4096^3", [[a32.mat_mul(b32)]], 137438953472, "TFLOP/s", F32_MFMA_PEAK_TFLOPS)
        a16 = T.new(dev, seeded(5, 0, (4096, 4096), "normal", dtype=np.float16, std=0.02))
        b16 = T.new(dev, seeded(5, 1, (4096, 4096), "normal", dtype=np.float16, std=0.02))
        out["c5_f16"] = Workload("config5b: GEMM f16 4096^3", [[a16.mat_mul(b16)]], 137438953472, "TFLOP/s", F16_MFMA_PEAK_TFLOPS, "f16")
        am = T.new(dev, seeded(5, 2, (2048, 4096), "normal", dtype=np.float16, std=0.02))
        bm = T.new(dev, seeded(5, 3, (4096, 11008), "normal", dtype=np.float16, std=0.02))
        out["c5_mlp"] = Workload("config5c: GEMM f16 [2048x4096]x[4096x11008]", [[am.mat_mul(bm)]], 184683593728, "TFLOP/s",
                                 F16_MFMA_PEAK_TFLOPS, "f16")
    return out


def copy_ceiling(w, dev):
    """Achieved GB/s of a plain device copy kernel (1 GiB read + 1 GiB write), for scale."""
    x = w.Tensor.new(dev, np.zeros((1 << 28,), dtype=np.float32))
    t = x.resize([1 << 28])  # resize to the same shape = one dense copy kernel
    wl = Workload("copy", [[t]], 2 * (1 << 30), "GB/s", HBM_PEAK_GBS)
    k = measure_kernels(dev, wl, 10, 3)
    return round(wl.work / k[0]["us"] * 1e-3, 1)


def cpu_baseline(seeded):
    """The CPU port (oracle/port.c), timed on this box's host cores: config 2, full size."""
    from oracle import port
    port.load()
    x = seeded(2, 0, (8192, 8192), "normal")
    out = np.empty(8192, dtype=np.float32)
    port.row_max(x, out)
    port.row_sum_exp_sub(x, 1.0, out)
    times = []
    t_end = time.perf_counter() + 15.0
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 40):
        t0 = time.perf_counter()
        port.row_max(x, out)
        port.row_sum_exp_sub(x, 1.0, out)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(2 * 268468224 / med * 1e-9, 2), "unit": "GB/s", "cores": port.threads(), "kind": "port",
            "sample": f"the full config-2 step (row max + row sum(exp(x-1)) on f32 [8192,8192]), median of {len(times)} runs, "
                      "oracle/port.c with OpenMP (the reference's wgpu path cannot run: no Rust toolchain, no Vulkan ICD)"}


def plan_only(w):
    """Plans (and so JIT-compiles for gfx950) every kernel this benchmark launches, at the benchmark's shapes, on a
    device that has no GPU behind it.  Nothing is computed or timed; the inputs are zeros."""
    dev = w.Device.planner()

    def zeros(config, tensor, shape, dist, dtype=np.float32, **kw):
        return np.zeros(shape, dtype=dtype)

    before = dev.module_stats()
    copy = w.Tensor.new(dev, np.zeros((1 << 28,), dtype=np.float32)).resize([1 << 28])
    copy.materialize()
    del copy
    for gname in ("c1", "c2", "c3", "c4", "c5"):
        wls = build_workloads(w, dev, zeros, {gname})
        for one in wls.values():
            for mode in ((w.FUSION_TREE, w.FUSION_REFERENCE) if gname in ("c3", "c4") else (w.FUSION_TREE,)):
                dev.set_fusion(mode)
                one.step(0)
            dev.set_fusion(w.FUSION_TREE)
        del wls
    after = dev.module_stats()
    print(json.dumps({"plan_only": True, "kernels_compiled": after["compiled"] - before["compiled"],
                      "kernels_from_disk_cache": after["disk_hits"] - before["disk_hits"]}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-detail", action="store_true", help="only the headline configuration")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only", default="", help="comma-separated subset of c1,c2,c3,c4,c5 for the detail table")
    ap.add_argument("--plan-only", action="store_true",
                    help="no GPU: plan every workload on a plan-only device so that each kernel is JIT-compiled into the cache")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every kernel, no collectives); --gpus must be 1.")

    w = load_package()
    dg_spec = importlib.util.spec_from_file_location("wkf_datagen", os.path.join(ROOT, "wgpu-kernal-fusion_amd", "datagen.py"))
    datagen = importlib.util.module_from_spec(dg_spec)
    dg_spec.loader.exec_module(datagen)
    seeded = datagen.seeded
    if args.plan_only:
        plan_only(w)
        return
    dev = w.Device.new(0)
    props = dev.props()
    if args.only == "copy":
        # calibration run for the rocprofv3 counters: nothing but the 1 GiB -> 1 GiB copy kernel
        print(json.dumps({"copy_kernel_GBs": copy_ceiling(w, dev), "bytes_read": 1 << 30, "bytes_written": 1 << 30}))
        return

    head = build_workloads(w, dev, seeded, {"c2"})
    wl = head["c2"]
    kernels = measure_kernels(dev, wl, args.steps, args.warmup)
    wall = measure_wall(dev, wl, args.steps, args.warmup)
    ms_per_step = wall / args.steps * 1e3
    value = wl.work * args.steps / wall * 1e-9
    # the dominant kernel alone, timed with one event pair over `steps` consecutive launches
    dom_us = measure_batch(w, dev, head["c2b"], args.steps, args.warmup)
    max_us = measure_batch(w, dev, head["c2a"], args.steps, args.warmup)
    dominant = dict(max(kernels, key=lambda k: k["us"]))
    dominant["us"] = round(dom_us, 2)
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get("config2b_red_row_bytes_per_launch")
    result = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": wl.name, "seed": "SplitMix64 0x5EED0020+r", "rotating_inputs": len(wl.variants),
                   "kernels_per_step": len(kernels), "algorithmic_bytes_per_step": wl.work,
                   "kernel_us": {"row_max": round(max_us, 2), "row_sum_exp": round(dom_us, 2),
                                 "per_launch_event_pairs": [k["us"] for k in kernels]},
                   "device": props.arch.decode(), "compute_units": props.compute_units, "clock_khz": props.clock_khz},
        "roofline": {"bound": "hbm", "achieved": round(268468224 / dominant["us"] * 1e-3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(268468224 / dominant["us"] * 1e-3 / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "kernel": dominant["kind"] + " " + dominant["detail"], "avg_us": dominant["us"],
                     "algorithmic_bytes_per_launch": 268468224},
        "value_frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
    }
    del head, wl
    dev.trim()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(seeded)
    else:
        result["cpu_baseline"] = None
    if not args.no_detail:
        detail = []
        result["copy_kernel_GBs"] = copy_ceiling(w, dev)
        dev.trim()
        groups = [g for g in ("c1", "c2", "c3", "c4", "c5") if not args.only or g in args.only.split(",")]
        steps = max(10, min(args.steps, 50))
        for gname in groups:
            wls = build_workloads(w, dev, seeded, {gname})
            for key, one in wls.items():
                if key == "c2":
                    continue
                ks = measure_kernels(dev, one, steps, 5)
                wall_s = measure_wall(dev, one, steps, 5)
                batch_us = round(measure_batch(w, dev, one, steps, 5), 2)
                detail.append(summarise(one, ks, wall_s, steps, batch_us))
                if gname in ("c3", "c4"):
                    # the same graph under the reference's own fusion rules (its kernel decomposition):
                    # same algorithmic work, more passes over memory
                    dev.set_fusion(w.FUSION_REFERENCE)
                    try:
                        ks = measure_kernels(dev, one, steps, 5)
                        wall_s = measure_wall(dev, one, steps, 5)
                        row = summarise(one, ks, wall_s, steps, None)
                        row["name"] += " -- reference kernel decomposition"
                        detail.append(row)
                    finally:
                        dev.set_fusion(w.FUSION_TREE)
            del wls
            dev.trim()
        result["all_configs"] = detail
    print(json.dumps(result))


if __name__ == "__main__":
    main()
