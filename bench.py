#!/usr/bin/env python3
"""Benchmark of the fused hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-detail] [--no-cpu] [--only c1,c5,f16]
    python bench.py --profile c5_f16 [--launches N]     (one workload only, for rocprofv3)

Prints ONE JSON line.  The headline (`value`) is BASELINE.json's metric on its
configuration 2: one step = the two fused row-reduce kernels of a softmax,
row max(x) and row sum(exp(x - 1)), over f32 [8192, 8192]; value = algorithmic
GB/s of the whole step by the wall clock, inputs resident in HBM, steps rotating
over several input tensors so that the 256 MB Infinity Cache cannot serve them.
`roofline` is the dominant kernel (the exp-sum reduce) timed with hipEvent pairs
on the stream it runs on; `cpu_baseline` is the CPU port of the reference's
decomposition (oracle/port.c) on this box's host cores; the line also carries `fracs`, one
[fraction of roofline, microseconds per step] pair per configuration, and stays below 4 KB.  The rows behind it
(`all_configs`) are written to the file `--detail-out` names:
every BASELINE configuration (GB/s or TFLOP/s, the fraction of its roofline, the median and the minimum of the
per-launch times after at least 100 warm launches, and the CPU port timed on a bounded sample of the same
configuration), plus f16 rows of the memory-bound kernels.

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
    """`variants`: the same expression over different input tensors (rotated step by step).
    `cpu`: (callable, work, text) -- the CPU port of the same computation on a bounded sample of it: calling the
    callable runs the sample once, `work` is the sample's algorithmic bytes or flops, `text` says what it was."""

    def __init__(self, name, variants, work, unit, peak, dtype="f32", joint=None, cpu=None):
        self.name, self.variants, self.work, self.unit, self.peak, self.dtype = name, variants, work, unit, peak, dtype
        self.joint = joint  # the package's materialize_many: the tensors of a step are materialised in ONE pass
        self.cpu = cpu

    def step(self, i, fresh=False):
        """Launches step i; returns the tensors whose kernel records describe it.  `fresh`: through new handles on the same
        graph nodes, so that the records of earlier steps stay readable while later ones are already enqueued."""
        ts = self.variants[i % len(self.variants)]
        if fresh:
            ts = [t.clone() for t in ts]
        if self.joint:
            self.joint(ts)
            return ts[:1]
        for t in ts:
            t.materialize()
        return ts


def measure_kernels(dev, wl, steps, warmup):
    """Per-kernel GPU time (a hipEvent pair carried by each dispatch: the kernel's own begin to end) over `steps` steps after `warmup` untimed ones:
    the median and the minimum per kernel, and of the step's total."""
    dev.set_timing(True)
    for i in range(warmup):
        wl.step(i)
    dev.sync()
    samples, kinds, details = [], None, None
    # Sixteen steps are enqueued ahead of the step whose times are read, each through handles of its own (its kernel
    # records stay readable, its result lives until it has been read): reading a time waits for its kernel, and on some
    # machines a GPU that waits for the host between two short kernels drops its clocks (seen: 28-30 us per launch read
    # one by one against 23 us for a 128 MiB map kernel whose vector ALUs are busy 60 % of the time).
    depth = 16

    def read(outs):
        nonlocal kinds, details
        ks = []
        for t in outs:
            ks += t.kernels()
        samples.append([k.elapsed_ns for k in ks])
        kinds = [k.kind for k in ks]
        details = [k.detail for k in ks]

    pending = []
    for i in range(steps):
        pending.append(wl.step(i, fresh=True))
        if len(pending) > depth:
            read(pending.pop(0))
    while pending:
        read(pending.pop(0))
    arr = np.array(samples, dtype=np.float64) / 1e3  # [step][kernel] in us
    med, mn = np.median(arr, axis=0), arr.min(axis=0)
    total = arr.sum(axis=1)
    kernels = [{"kind": k, "detail": d, "us": round(float(a), 2), "min_us": round(float(b), 2)}
               for k, d, a, b in zip(kinds, details, med, mn)]
    return kernels, round(float(np.median(total)), 2), round(float(total.min()), 2)


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


def settle(dev, wl, seconds=0.3):
    """Runs the workload untimed for `seconds`: after uploads and an idle spell the GPU takes tens of milliseconds to
    reach its working clocks.  Not part of any measurement (the W warm-up steps of each measurement still run)."""
    dev.set_timing(False)
    t_end = time.perf_counter() + seconds
    i = 0
    while time.perf_counter() < t_end:
        wl.step(i)
        i += 1
        if i % 50 == 0:
            dev.sync()
    dev.sync()
    dev.set_timing(True)


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


def summarise(wl, measured, wall_s, steps, batch_us):
    kernels, med_us, min_us = measured
    scale = 1e-3 if wl.unit == "GB/s" else 1e-6  # bytes/us -> GB/s ; flop/us -> TFLOP/s
    rate = lambda us: round(wl.work / us * scale, 1) if us else None
    frac = lambda us: round(wl.work / us * scale / wl.peak, 4) if us else None
    dom = max(kernels, key=lambda k: k["us"])
    # the roofline of this configuration: its dominant kernel, timed without per-launch events when a batch figure
    # exists (one hipEvent pair around `steps` back-to-back steps on the library's stream)
    step_us = batch_us if batch_us else med_us
    return {"name": wl.name, "dtype": wl.dtype, "unit": wl.unit, "work_per_step": wl.work,
            "kernels": kernels, "median_us_per_step": med_us, "min_us_per_step": min_us,
            "achieved": rate(med_us), "peak": wl.peak, "frac": frac(med_us), "min_frac": frac(min_us),
            "batch_us_per_step": batch_us, "batch_achieved": rate(batch_us), "batch_frac": frac(batch_us),
            "roofline": {"bound": "hbm" if wl.unit == "GB/s" else "mfma", "kernel": dom["kind"] + " " + dom["detail"],
                         "kernels_per_step": len(kernels), "avg_us": step_us, "achieved": rate(step_us), "peak": wl.peak,
                         "unit": wl.unit, "frac": frac(step_us)},
            "wall_ms_per_step": round(wall_s / steps * 1e3, 4),
            "wall_rate": round(wl.work * steps / wall_s * (1e-9 if wl.unit == "GB/s" else 1e-12), 1)}


def build_workloads(w, dev, seeded, which, with_cpu=False):
    """The BASELINE configurations (c1..c5) and the f16 rows of the memory-bound kernels (f16) as workloads.
    with_cpu: also prepare the CPU port of each configuration (oracle/port.c) on a bounded sample of its inputs."""
    T = w.Tensor
    out = {}
    port = None
    if with_cpu:
        from oracle import port as port_mod
        port_mod.load()
        port = port_mod

    def cpu_of(fn, work, text):
        return (fn, work, text) if port is not None else None

    if "c2" in which:
        hosts = [seeded(2, r, (8192, 8192), "normal") for r in range(4)]
        xs = [T.new(dev, h) for h in hosts]
        h0 = hosts[0]
        del hosts
        o = np.empty(8192, dtype=np.float32)
        both = cpu_of(lambda: (port.row_max(h0, o), port.row_sum_exp_sub(h0, 1.0, o)), 2 * 268468224, "the full step")
        out["c2"] = Workload("config2: row max(x) + row sum(exp(x-1)), f32 [8192,8192]",
                             [[x.max(1), (x.clone() - 1.0).exp().sum(1)] for x in xs], 2 * 268468224, "GB/s", HBM_PEAK_GBS, cpu=both)
        # the same two results from ONE pass over the matrix (the reference lists this fusion as to-do, README.md:20):
        # algorithmic bytes = the matrix once + both result vectors
        out["c2_one_pass"] = Workload("config2 in one pass: row max(x) and row sum(exp(x-1)) together, f32 [8192,8192]",
                                      [[x.max(1), (x.clone() - 1.0).exp().sum(1)] for x in xs], 8192 * 8192 * 4 + 2 * 8192 * 4,
                                      "GB/s", HBM_PEAK_GBS, joint=w.materialize_many)
        out["c2a"] = Workload("config2a: row max(x), f32 [8192,8192]", [[x.max(1)] for x in xs], 268468224, "GB/s", HBM_PEAK_GBS,
                              cpu=cpu_of(lambda: port.row_max(h0, o), 268468224, "the full kernel"))
        out["c2b"] = Workload("config2b: row sum(exp(x-1)), f32 [8192,8192]", [[(x.clone() - 1.0).exp().sum(1)] for x in xs],
                              268468224, "GB/s", HBM_PEAK_GBS,
                              cpu=cpu_of(lambda: port.row_sum_exp_sub(h0, 1.0, o), 268468224, "the full kernel"))
    if "c1" in which:
        hosts = [seeded(1, r, (4096, 4096), "uniform") for r in range(8)]
        xs = [T.new(dev, h) for h in hosts]
        h1 = hosts[0]
        del hosts
        y1 = np.empty_like(h1)
        out["c1"] = Workload("config1: exp(sin(x*2+1)), f32 [4096,4096]", [[((x * 2.0) + 1.0).sin().exp()] for x in xs],
                             134217728, "GB/s", HBM_PEAK_GBS, cpu=cpu_of(lambda: port.c1(h1, y1), 134217728, "the full tensor"))
    if "c3" in which:
        variants = []
        hb = seeded(3, 2, (4096,), "normal", std=0.02)
        bias = T.new(dev, hb)
        bias3 = bias.broadcast([1024, 4096]).broadcast([32, 1024, 4096])
        keep = None
        for r in range(2):
            ha = seeded(3, 4 * r, (32, 1024, 4096), "uniform")
            hbb = seeded(3, 4 * r + 1, (32, 1024, 4096), "uniform")
            a, b = T.new(dev, ha), T.new(dev, hbb)
            if r == 0 and port is not None:
                keep = (np.ascontiguousarray(ha[:8]), np.ascontiguousarray(hbb[:8]))  # 8 of the 32 slabs
            variants.append([a.silu() * (b + bias3)])
        cpu3 = None
        if keep is not None:
            t1, t2 = np.empty_like(keep[0]), np.empty_like(keep[0])
            cpu3 = cpu_of(lambda: port.c3(keep[0], keep[1], hb, t1, t2), 1610629120 // 4,
                          "8 of the 32 [1024,4096] slabs, the reference's three passes (silu, add, mul)")
        out["c3"] = Workload("config3: silu(a)*(b+bias), f32 [32,1024,4096]", variants, 1610629120, "GB/s", HBM_PEAK_GBS, cpu=cpu3)
    if "c4" in which:
        hw = seeded(4, 1, (4096,), "normal", mean=1.0, std=0.02)
        w4 = T.new(dev, hw)
        hosts = [seeded(4, 8 + r, (2048, 4096), "normal") for r in range(8)]
        xs = [T.new(dev, h) for h in hosts]
        hx = hosts[0]
        del hosts
        out["c4_rmsnorm"] = Workload("config4: RMSNorm f32 [2048,4096]", [[x.layer_norm(w4, 1e-5)] for x in xs], 67125248, "GB/s",
                                     HBM_PEAK_GBS, cpu=cpu_of(lambda: port.rmsnorm(hx, hw, 1e-5), 67125248, "the full tensor"))
        cos, sin = rope_tables(2048, 128)
        tc, ts = T.new(dev, cos), T.new(dev, sin)
        hosts = [seeded(4, 16 + r, (32, 2048, 128), "normal") for r in range(8)]
        qs = [T.new(dev, h) for h in hosts]
        hq = hosts[0]
        del hosts
        cf, sf = np.ascontiguousarray(np.concatenate([cos, cos], 1)), np.ascontiguousarray(np.concatenate([sin, sin], 1))
        out["c4_rope"] = Workload("config4: RoPE f32 [32,2048,128]", [[q.rope(tc, ts)] for q in qs], 69206016, "GB/s", HBM_PEAK_GBS,
                                  cpu=cpu_of(lambda: port.rope(hq, cf, sf), 69206016, "the full tensor"))
        hosts = [seeded(4, 24 + r, (32, 2048, 2048), "normal") for r in range(2)]
        ss = [T.new(dev, h) for h in hosts]
        hs = np.ascontiguousarray(hosts[0][:8])
        del hosts
        out["c4_softmax"] = Workload("config4: softmax f32 [32,2048,2048]", [[s.softmax_last_dim()] for s in ss], 1073741824, "GB/s",
                                     HBM_PEAK_GBS, cpu=cpu_of(lambda: port.softmax_rows(hs), 1073741824 // 4,
                                                              "8 of the 32 heads, the reference's passes (max, exp-sum, divide)"))
    if "c5" in which:
        ha = seeded(5, 0, (4096, 4096), "normal", std=0.02)
        hb5 = seeded(5, 1, (4096, 4096), "normal", std=0.02)
        a32, b32 = T.new(dev, ha), T.new(dev, hb5)
        rows = np.ascontiguousarray(ha[:256])
        gemm_cpu = cpu_of(lambda: port.gemm_f32(rows, hb5), 2 * 256 * 4096 * 4096, "256 of the 4096 rows of A against all of B, f32")
        out["c5_f32"] = Workload("config5a: GEMM f32 4096^3", [[a32.mat_mul(b32)]], 137438953472, "TFLOP/s", F32_MFMA_PEAK_TFLOPS,
                                 cpu=gemm_cpu)
        a16 = T.new(dev, seeded(5, 0, (4096, 4096), "normal", dtype=np.float16, std=0.02))
        b16 = T.new(dev, seeded(5, 1, (4096, 4096), "normal", dtype=np.float16, std=0.02))
        gemm_cpu16 = cpu_of(lambda: port.gemm_f32(rows, hb5), 2 * 256 * 4096 * 4096,
                            "256 of the 4096 rows of A against all of B, in f32 arithmetic (the port has no f16 path)")
        out["c5_f16"] = Workload("config5b: GEMM f16 4096^3", [[a16.mat_mul(b16)]], 137438953472, "TFLOP/s", F16_MFMA_PEAK_TFLOPS, "f16",
                                 cpu=gemm_cpu16)
        am = T.new(dev, seeded(5, 2, (2048, 4096), "normal", dtype=np.float16, std=0.02))
        hbm = seeded(5, 3, (4096, 11008), "normal", dtype=np.float16, std=0.02)
        bm = T.new(dev, hbm)
        mlp_cpu = None
        if port is not None:
            hbm32 = hbm.astype(np.float32)
            mlp_cpu = cpu_of(lambda: port.gemm_f32(rows, hbm32), 2 * 256 * 4096 * 11008,
                             "256 rows against all of the [4096,11008] weight, in f32 arithmetic (the port has no f16 path)")
        del hbm
        out["c5_mlp"] = Workload("config5c: GEMM f16 [2048x4096]x[4096x11008]", [[am.mat_mul(bm)]], 184683593728, "TFLOP/s",
                                 F16_MFMA_PEAK_TFLOPS, "f16", cpu=mlp_cpu)
    if "attn" in which:
        # batched products of attention shape (no BASELINE configuration; batched mat_mul is the reference's
        # src/matmul.rs with leading dimensions): scores = q . k^T with k^T a transposed view, then p . v.  Both are
        # bound by the [32,2048,2048] matrix they write or read, so they are priced against HBM.
        F16 = np.float16
        q = T.new(dev, seeded(6, 0, (32, 2048, 128), "normal", dtype=F16, std=0.1))
        kk = T.new(dev, seeded(6, 1, (32, 2048, 128), "normal", dtype=F16, std=0.1))
        v = T.new(dev, seeded(6, 2, (32, 2048, 128), "normal", dtype=F16, std=0.1))
        pp = [T.new(dev, seeded(6, 3 + r, (32, 2048, 2048), "uniform", dtype=F16)) for r in range(2)]
        small, big = 32 * 2048 * 128 * 2, 32 * 2048 * 2048 * 2
        out["attn_qk"] = Workload("attention scores: q.k^T, f16 [32,2048,128]x[32,128,2048]", [[q.mat_mul(kk.transpose(1, 2))]],
                                  2 * small + big, "GB/s", HBM_PEAK_GBS, "f16")
        out["attn_pv"] = Workload("attention output: p.v, f16 [32,2048,2048]x[32,2048,128]", [[p_.mat_mul(v)] for p_ in pp],
                                  big + 2 * small, "GB/s", HBM_PEAK_GBS, "f16")
    if "more" in which:
        # shapes off the BASELINE list that have kernels of their own: a transposed operand, a ragged product, a product
        # of a few hundred rows against a wide weight
        xt = [T.new(dev, seeded(7, r, (8192, 8192), "normal")) for r in range(3)]
        out["more_transpose"] = Workload("transposed operand: x^T + 1, f32 [8192,8192]", [[x.transpose(0, 1) + 1.0] for x in xt],
                                         2 * 8192 * 8192 * 4, "GB/s", HBM_PEAK_GBS)
        del xt
        F16 = np.float16
        ar = T.new(dev, seeded(7, 4, (4000, 4096), "normal", dtype=F16, std=0.02))
        br = T.new(dev, seeded(7, 5, (4096, 4096), "normal", dtype=F16, std=0.02))
        out["more_gemm_ragged"] = Workload("ragged product: GEMM f16 [4000x4096]x[4096x4096]", [[ar.mat_mul(br)]], 2 * 4000 * 4096 * 4096,
                                           "TFLOP/s", F16_MFMA_PEAK_TFLOPS, "f16")
        am_ = T.new(dev, seeded(7, 6, (512, 4096), "normal", dtype=F16, std=0.02))
        bm_ = T.new(dev, seeded(7, 7, (4096, 11008), "normal", dtype=F16, std=0.02))
        out["more_gemm_mid"] = Workload("512 rows against a wide weight: GEMM f16 [512x4096]x[4096x11008]", [[am_.mat_mul(bm_)]],
                                        2 * 512 * 4096 * 11008, "TFLOP/s", F16_MFMA_PEAK_TFLOPS, "f16")
    if "decode" in which:
        # one row against a transposed weight (x . W^T, the linear layer at decode time; no BASELINE configuration): reading
        # W once is all the work, so the product is priced against HBM.  Three weights take turns, more bytes than
        # the last-level cache holds.
        for name, dt, key in (("f16", np.float16, "decode_f16"), ("f32", np.float32, "decode_f32")):
            xr = T.new(dev, seeded(8, 0, (1, 4096), "normal", dtype=dt))
            ws = [T.new(dev, seeded(8, 1 + r, (11008, 4096), "normal", dtype=dt, std=0.02)) for r in range(4 if dt == np.float16 else 3)]
            esz = 2 if dt == np.float16 else 4
            out[key] = Workload(f"decode: x.W^T, {name} [1x4096]x[11008x4096]^T", [[xr.mat_mul(w_.transpose(0, 1))] for w_ in ws],
                                (11008 * 4096 + 4096 + 11008) * esz, "GB/s", HBM_PEAK_GBS, name)
    if "long" in which:
        # rows longer than a block's registers (no BASELINE configuration; the reference's reduce takes any length)
        xs = [T.new(dev, seeded(4, 40 + r, (256, 262144), "normal")) for r in range(2)]
        out["long_softmax"] = Workload("long rows: softmax f32 [256,262144]", [[x.softmax_last_dim()] for x in xs], 2 * 256 * 262144 * 4,
                                       "GB/s", HBM_PEAK_GBS)
        xf = [T.new(dev, seeded(4, 44 + r, (64, 262144), "normal")) for r in range(2)]
        out["long_softmax_few"] = Workload("few long rows: softmax f32 [64,262144]", [[x.softmax_last_dim()] for x in xf],
                                           2 * 64 * 262144 * 4, "GB/s", HBM_PEAK_GBS)
    if "f16" in which:
        # the f16 forms of the memory-bound kernels (no BASELINE configuration names them; no CPU figure)
        F16 = np.float16
        xs = [T.new(dev, seeded(2, r, (8192, 8192), "normal", dtype=F16)) for r in range(4)]
        out["f16_c2"] = Workload("f16: row max(x) + row sum(exp(x-1)), f16 [8192,8192]",
                                 [[x.max(1), (x.clone() - 1.0).exp().sum(1)] for x in xs], 2 * (8192 * 8192 * 2 + 8192 * 2), "GB/s",
                                 HBM_PEAK_GBS, "f16")
        out["f16_sum"] = Workload("f16: row sum(x), f16 [8192,8192]", [[x.sum(1)] for x in xs], 8192 * 8192 * 2 + 8192 * 2, "GB/s",
                                  HBM_PEAK_GBS, "f16")
        out["f16_map"] = Workload("f16: exp(sin(x*2+1)), f16 [8192,8192]", [[((x * 2.0) + 1.0).sin().exp()] for x in xs],
                                  2 * 8192 * 8192 * 2, "GB/s", HBM_PEAK_GBS, "f16")
        # config 3 on f16: silu(a) depends on one operand only and is looked up in a table inside the fused kernel
        b16 = T.new(dev, seeded(3, 2, (4096,), "normal", dtype=F16, std=0.02)).broadcast([1024, 4096]).broadcast([32, 1024, 4096])
        ab = [(T.new(dev, seeded(3, 4 * r, (32, 1024, 4096), "uniform", dtype=F16)), T.new(dev, seeded(3, 4 * r + 1, (32, 1024, 4096), "uniform", dtype=F16)))
              for r in range(2)]
        out["f16_c3"] = Workload("f16: silu(a)*(b+bias), f16 [32,1024,4096]", [[a_.silu() * (b_ + b16)] for a_, b_ in ab],
                                 3 * 32 * 1024 * 4096 * 2 + 4096 * 2, "GB/s", HBM_PEAK_GBS, "f16")
        x32 = [T.new(dev, seeded(2, r, (8192, 8192), "normal")) for r in range(2)]
        out["f16_cast"] = Workload("cast f32 -> f16, [8192,8192]", [[x.cast(w.F16)] for x in x32], 8192 * 8192 * 6, "GB/s",
                                   HBM_PEAK_GBS, "f32->f16")
        ss = [T.new(dev, seeded(4, 24 + r, (32, 2048, 2048), "normal", dtype=F16)) for r in range(2)]
        out["f16_softmax"] = Workload("f16: softmax f16 [32,2048,2048]", [[s_.softmax_last_dim()] for s_ in ss], 2 * 32 * 2048 * 2048 * 2,
                                      "GB/s", HBM_PEAK_GBS, "f16")
        w16 = T.new(dev, seeded(4, 1, (4096,), "normal", dtype=F16, mean=1.0, std=0.02))
        x16 = [T.new(dev, seeded(4, 8 + r, (2048, 4096), "normal", dtype=F16)) for r in range(8)]
        out["f16_rmsnorm"] = Workload("f16: RMSNorm f16 [2048,4096]", [[x.layer_norm(w16, 1e-5)] for x in x16],
                                      2 * 2048 * 4096 * 2 + 4096 * 2, "GB/s", HBM_PEAK_GBS, "f16")
    return out


def time_cpu(cpu, budget_s=3.0):
    """Median seconds of the CPU port's sample over at least 2 runs (one untimed first), within about `budget_s`."""
    fn, work, text = cpu
    fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 2 or (time.perf_counter() < t_end and len(times) < 20):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times)), len(times)


def cpu_row(wl):
    """The `cpu_baseline` object of one configuration: oracle/port.c on the host cores, on a bounded sample."""
    from oracle import port
    med, n = time_cpu(wl.cpu)
    scale = 1e-9 if wl.unit == "GB/s" else 1e-12
    return {"value": round(wl.cpu[1] / med * scale, 3), "unit": wl.unit, "cores": port.threads(), "kind": "port",
            "sample": f"{wl.cpu[2]}; median of {n} runs of oracle/port.c (OpenMP)"}


def reference_cpu_path():
    """Run-time probe for what the reference's own CPU path needs (cargo / rustc and a Vulkan CPU adapter such as
    lavapipe): reported next to the CPU port's figures."""
    import glob
    import shutil
    icds = []
    for d in ("/usr/share/vulkan/icd.d", "/etc/vulkan/icd.d", "/usr/local/share/vulkan/icd.d"):
        icds += glob.glob(os.path.join(d, "*.json"))
    lvp = [p for p in icds if "lvp" in os.path.basename(p) or "lavapipe" in os.path.basename(p)]
    probe = {"cargo": shutil.which("cargo"), "rustc": shutil.which("rustc"), "vulkan_icds": icds, "lavapipe_icd": lvp[:1] or None,
             "reference_checkout": os.path.isdir("/root/reference")}
    ok = bool(probe["cargo"] and probe["rustc"] and lvp and probe["reference_checkout"])
    return {"available": ok, "probe": probe,
            "note": "the reference's wgpu path on a CPU adapter needs cargo + rustc + a Vulkan CPU ICD + its checkout; "
                    + ("all present, but this benchmark does not drive it" if ok else "unavailable on this machine, so the CPU figures are oracle/port.c")}


def copy_ceiling(w, dev):
    """Achieved GB/s of a plain device copy kernel (1 GiB read + 1 GiB write), for scale."""
    x = w.Tensor.new(dev, np.zeros((1 << 28,), dtype=np.float32))
    t = x.resize([1 << 28])  # resize to the same shape = one dense copy kernel
    wl = Workload("copy", [[t]], 2 * (1 << 30), "GB/s", HBM_PEAK_GBS)
    settle(dev, wl)
    k, med, _ = measure_kernels(dev, wl, 10, 3)
    return round(wl.work / med * 1e-3, 1)


def cpu_baseline(wl):
    """The CPU port (oracle/port.c) of the headline configuration, timed on this box's host cores at full size."""
    from oracle import port
    fn = wl.cpu[0]
    fn()
    times = []
    t_end = time.perf_counter() + 12.0
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 40):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(wl.cpu[1] / med * 1e-9, 2), "unit": "GB/s", "cores": port.threads(), "kind": "port",
            "sample": f"the full config-2 step (row max + row sum(exp(x-1)) on f32 [8192,8192]), median of {len(times)} runs, "
                      "oracle/port.c with OpenMP"}


GROUPS = ("c1", "c2", "c3", "c4", "c5", "f16", "long", "attn", "more", "decode")


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
    for gname in GROUPS:
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


def profile_one(w, dev, seeded, key, launches, warm_ms):
    """`--profile KEY`: nothing but `launches` steps of one workload, for a profiler run (rocprofv3 --kernel-trace
    --stats / --pmc ... -- python3 bench.py --profile KEY).  Before them, untimed steps for `warm_ms` milliseconds (at
    least 10 steps): after an idle spell the GPU takes tens of milliseconds to reach its working clocks."""
    group = next((g for g in GROUPS if key.startswith(g)), key)
    if key == "copy":
        x = w.Tensor.new(dev, np.zeros((1 << 28,), dtype=np.float32))
        wl = Workload("copy 1 GiB -> 1 GiB", [[x.resize([1 << 28])]], 2 * (1 << 30), "GB/s", HBM_PEAK_GBS)
    else:
        wls = build_workloads(w, dev, seeded, {group})
        if key not in wls:
            sys.exit(f"bench.py --profile: unknown workload {key!r}; group {group!r} has: " + ", ".join(wls))
        wl = wls[key]
    if warm_ms > 0:
        settle(dev, wl, warm_ms * 1e-3)
    us = measure_batch(w, dev, wl, launches, 10)
    scale = 1e-3 if wl.unit == "GB/s" else 1e-6
    print(json.dumps({"profile": key, "name": wl.name, "launches": launches, "us_per_step": round(us, 2),
                      "achieved": round(wl.work / us * scale, 1), "unit": wl.unit, "frac": round(wl.work / us * scale / wl.peak, 4),
                      "work_per_step": wl.work}))


MFMA_ONLY_SRC = r"""
// Yardstick: the MFMA work of a 256 x 256 x K tile kernel and nothing else.  Every lane takes its operand
// fragments from A and B once (real operand data: the power the matrix cores draw depends on the bits they
// toggle), then issues 64 v_mfma_f32_32x32x16_f16 per 64 columns of K, as the GEMM's loop does.
typedef unsigned int u32;
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float acc16 __attribute__((ext_vector_type(16)));
struct Args { const _Float16* a; const _Float16* b; _Float16* c; u32 m, n, k, kchunk; };
extern "C" __global__ void __launch_bounds__(256) wkf_mfma_only(const Args g) {
  const u32 tid = threadIdx.x;
  h8 fa[4], fb[4];
  for (int i = 0; i < 4; i++) fa[i] = *(const h8*)(g.a + (size_t(blockIdx.x) * 256 + tid) * 64 + i * 8);
  for (int i = 0; i < 4; i++) fb[i] = *(const h8*)(g.b + (size_t(blockIdx.x) * 256 + tid) * 64 + i * 8);
  acc16 acc[16];
  for (int i = 0; i < 16; i++) acc[i] = (acc16)(0.0f);
  for (u32 t = 0; t < g.k / 64; t++) {
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[((i >> 2) + r) & 3], fb[i & 3], acc[i], 0, 0, 0);
  }
  float s = 0;
  for (int i = 0; i < 16; i++) s += acc[i][0] + acc[i][7];
  g.c[size_t(blockIdx.x) * 256 + tid] = (_Float16)s;
}
"""

MFMA_ONLY_F32_SRC = r"""
// Yardstick: the MFMA work of the f32 256 x 256 x K tile kernel and nothing else: 256 v_mfma_f32_32x32x2_f32 per
// wave and 32 columns of K, operands taken once from A and B (real data).
typedef unsigned int u32;
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float acc16 __attribute__((ext_vector_type(16)));
struct Args { const float* a; const float* b; float* c; u32 m, n, k, kchunk; };
extern "C" __global__ void __launch_bounds__(256) wkf_mfma_only_f32(const Args g) {
  const u32 tid = threadIdx.x;
  f4 fa[4], fb[4];
  for (int i = 0; i < 4; i++) fa[i] = *(const f4*)(g.a + (size_t(blockIdx.x) * 256 + tid) * 16 + i * 4);
  for (int i = 0; i < 4; i++) fb[i] = *(const f4*)(g.b + (size_t(blockIdx.x) * 256 + tid) * 16 + i * 4);
  acc16 acc[16];
  for (int i = 0; i < 16; i++) acc[i] = (acc16)(0.0f);
  for (u32 t = 0; t < g.k / 32; t++) {
#pragma unroll
    for (int r = 0; r < 16; r++)
#pragma unroll
      for (int i = 0; i < 16; i++)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[(i >> 2)][(r + i) & 3], fb[i & 3][r & 3], acc[i], 0, 0, 0);
  }
  float s = 0;
  for (int i = 0; i < 16; i++) s += acc[i][0] + acc[i][7];
  g.c[size_t(blockIdx.x) * 256 + tid] = s;
}
"""

STREAM_SRC = r"""
// Yardstick: plain streaming kernels over 1 GiB buffers (MODE 0 copy, 1 read-only, 2 write-only, 3 two reads and
// one write: out = in + in2), U 16-byte accesses per lane and stream in flight, non-temporal bits on the loads
// (NTL) and the stores (NTS).
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;
#if NTL
#define LD(p) __builtin_nontemporal_load(p)
#else
#define LD(p) (*(p))
#endif
#if NTS
#define ST(p, v) __builtin_nontemporal_store(v, p)
#else
#define ST(p, v) (*(p) = (v))
#endif
extern "C" __global__ void __launch_bounds__(WG) wkf_stream(const f4* __restrict__ in, f4* __restrict__ out, u64 n4, const f4* __restrict__ in2) {
  const u64 chunk = u64(WG) * U;
#if PERSIST
  for (u64 base = u64(blockIdx.x) * chunk; base < n4; base += u64(gridDim.x) * chunk) {
#else
  { const u64 base = u64(blockIdx.x) * chunk;
#endif
    f4 v[U];
#if MODE == 3
    f4 v2[U];
#pragma unroll
    for (int i = 0; i < U; i++) v[i] = LD(in + base + threadIdx.x + i * WG);
#pragma unroll
    for (int i = 0; i < U; i++) v2[i] = LD(in2 + base + threadIdx.x + i * WG);
#pragma unroll
    for (int i = 0; i < U; i++) v[i] += v2[i];
#elif MODE != 2
#pragma unroll
    for (int i = 0; i < U; i++) v[i] = LD(in + base + threadIdx.x + i * WG);
#else
#pragma unroll
    for (int i = 0; i < U; i++) v[i] = (f4)(float(threadIdx.x));
#endif
#if MODE != 1
#pragma unroll
    for (int i = 0; i < U; i++) ST(out + base + threadIdx.x + i * WG, v[i]);
#else
    float s = 0;
#pragma unroll
    for (int i = 0; i < U; i++) s += v[i][0] + v[i][1] + v[i][2] + v[i][3];
    if (s == 12345.678f) out[base + threadIdx.x][0] = s;
#endif
  }
}
"""


def _raw_timed(lib, dev, fn, reps, warm):
    """us per call of `fn` (which enqueues work on the library's stream): one hipEvent pair around `reps` calls."""
    import ctypes
    timer = ctypes.c_void_p()
    assert lib.wkf_timer_create(dev._h, ctypes.byref(timer)) == 0
    for _ in range(warm):
        fn()
    dev.sync()
    assert lib.wkf_timer_begin(timer) == 0
    for _ in range(reps):
        fn()
    assert lib.wkf_timer_end(timer) == 0
    ns = ctypes.c_uint64()
    assert lib.wkf_timer_elapsed_ns(timer, ctypes.byref(ns)) == 0
    lib.wkf_timer_destroy(timer)
    return ns.value / reps / 1e3


def _smi_sample():
    """One reading of the GPU's power and clocks from rocm-smi (a child process), or the error it gave."""
    try:
        r = subprocess.run(["rocm-smi", "--showpower", "--showmaxpower", "--showclocks", "--json"], capture_output=True, text=True, timeout=10)
        card = next(iter(json.loads(r.stdout).values()))
    except Exception as e:  # no rocm-smi, no permission, no JSON: the row then says so
        return {"error": repr(e)[:200]}
    keep = {}
    for k, v in card.items():
        lk = k.lower()
        if "power" in lk or "sclk" in lk or "mclk" in lk or "fclk" in lk:
            keep[k] = v
    return keep


def power_rows(w, dev, seeded, seconds):
    """`--yardstick power`: what the chip draws and clocks at while it runs (a) the library's f16 4096^3 product,
    (b) the MFMA-only loop on the same operands, (c) the MFMA-only loop on zeros, (d) nothing.  Every phase enqueues
    its kernel back to back for `seconds` while a thread reads rocm-smi; the rows carry every reading and the rate."""
    import struct
    import threading
    from ctypes import byref, c_uint32, c_void_p
    lib = w.load()
    T = w.Tensor
    ha = seeded(5, 0, (4096, 4096), "normal", dtype=np.float16, std=0.02)
    hb = seeded(5, 1, (4096, 4096), "normal", dtype=np.float16, std=0.02)
    a16, b16 = T.new(dev, ha), T.new(dev, hb)
    prod = a16.mat_mul(b16)
    k = c_void_p()
    assert lib.wkf_module_get(dev._h, b"yardstick|mfma_only|32x32x16", MFMA_ONLY_SRC.encode(), b"wkf_mfma_only", byref(k)) == 0, lib.wkf_last_error()

    def raw(host):
        buf = c_void_p()
        assert lib.wkf_buffer_alloc(dev._h, host.nbytes, 1, byref(buf)) == 0
        assert lib.wkf_buffer_upload(buf, 0, host.ctypes.data_as(c_void_p), host.nbytes) == 0
        return buf

    ba, bb, bz, bc = raw(ha), raw(hb), raw(np.zeros((4096, 4096), np.float16)), raw(np.zeros((256, 256), np.float16))
    grid, block = (c_uint32 * 3)(256, 1, 1), (c_uint32 * 3)(256, 1, 1)

    def mfma_only(x, y):
        args = struct.pack("PPPIIII", lib.wkf_buffer_ptr(x), lib.wkf_buffer_ptr(y), lib.wkf_buffer_ptr(bc), 4096, 4096, 4096, 0)
        return lambda: lib.wkf_launch(dev._h, k, grid, block, 0, args, len(args), None)

    dev.set_timing(False)
    phases = [("library GEMM f16 4096^3, config-5 operands", lambda: prod.materialize()),
              ("MFMA only, config-5 operands", mfma_only(ba, bb)),
              ("MFMA only, zeros", mfma_only(bz, bz)),
              ("idle", None)]
    rows = []
    for name, fn in phases:
        samples, stop = [], threading.Event()

        def sampler():
            time.sleep(0.5)  # let the clocks settle under the load first
            while not stop.is_set():
                s = _smi_sample()
                s["t"] = round(time.perf_counter() - t0, 2)
                samples.append(s)
                time.sleep(0.2)

        t0 = time.perf_counter()
        th = threading.Thread(target=sampler)
        th.start()
        launches = 0
        if fn is None:
            time.sleep(seconds)
        else:
            while time.perf_counter() - t0 < seconds:
                for _ in range(200):
                    fn()
                dev.sync()
                launches += 200
        elapsed = time.perf_counter() - t0
        stop.set()
        th.join()
        row = {"phase": name, "seconds": round(elapsed, 2), "launches": launches, "smi": samples}
        if launches:
            row["us_per_launch_wall"] = round(elapsed / launches * 1e6, 2)
            row["TFLOP/s"] = round(2 * 4096 ** 3 * launches / elapsed * 1e-12, 1)
        rows.append(row)
    dev.set_timing(True)
    for bf in (ba, bb, bz, bc):
        lib.wkf_buffer_release(bf)
    return rows


def yardsticks(w, dev, seeded, which, launches):
    """`--yardstick mfma|stream`: kernels that are not part of the library, launched through its level-0 ABI, which
    bound what the library's kernels can reach on this machine: the matrix cores alone on the benchmark's operand
    data (and on zeros), and plain copy / read-only / write-only streams plus the runtime's own device copy."""
    import ctypes
    import struct
    from ctypes import byref, c_uint32, c_void_p
    lib = w.load()

    def dev_buf(nbytes, host=None):
        buf = c_void_p()
        assert lib.wkf_buffer_alloc(dev._h, nbytes, 1, byref(buf)) == 0, lib.wkf_last_error()
        if host is not None:
            assert lib.wkf_buffer_upload(buf, 0, host.ctypes.data_as(c_void_p), host.nbytes) == 0
        return buf

    def kernel(sig, src, entry):
        k = c_void_p()
        rc = lib.wkf_module_get(dev._h, sig.encode(), src.encode(), entry.encode(), byref(k))
        assert rc == 0, lib.wkf_last_error().decode()
        return k

    out = {"yardstick": which}
    if which == "mfma":
        k = kernel("yardstick|mfma_only|32x32x16", MFMA_ONLY_SRC, "wkf_mfma_only")
        rows = []
        for label, a, b in (("config-5 operands, N(0, 0.02)", seeded(5, 0, (4096, 4096), "normal", dtype=np.float16, std=0.02),
                             seeded(5, 1, (4096, 4096), "normal", dtype=np.float16, std=0.02)),
                            ("zeros", np.zeros((4096, 4096), np.float16), np.zeros((4096, 4096), np.float16))):
            ba, bb, bc = dev_buf(a.nbytes, a), dev_buf(b.nbytes, b), dev_buf(256 * 256 * 2)
            args = struct.pack("PPPIIII", lib.wkf_buffer_ptr(ba), lib.wkf_buffer_ptr(bb), lib.wkf_buffer_ptr(bc), 4096, 4096, 4096, 0)
            grid, block = (c_uint32 * 3)(256, 1, 1), (c_uint32 * 3)(256, 1, 1)
            us = _raw_timed(lib, dev, lambda: lib.wkf_launch(dev._h, k, grid, block, 0, args, len(args), None), launches, 100)
            rows.append({"data": label, "us": round(us, 2), "TFLOP/s": round(2 * 4096 ** 3 / us * 1e-6, 1),
                         "frac_of_f16_peak": round(2 * 4096 ** 3 / us * 1e-6 / F16_MFMA_PEAK_TFLOPS, 4)})
            for bf in (ba, bb, bc):
                lib.wkf_buffer_release(bf)
        out["mfma_only_4096x4096x4096_equivalent"] = rows
        # the same for the f32 kernel (v_mfma_f32_32x32x2_f32, nominal peak 157.3 TFLOP/s)
        k32 = kernel("yardstick|mfma_only|f32 32x32x2", MFMA_ONLY_F32_SRC, "wkf_mfma_only_f32")
        rows32 = []
        for label, a, b in (("config-5 operands, N(0, 0.02)", seeded(5, 0, (4096, 4096), "normal", std=0.02),
                             seeded(5, 1, (4096, 4096), "normal", std=0.02)),
                            ("zeros", np.zeros((4096, 4096), np.float32), np.zeros((4096, 4096), np.float32))):
            ba, bb, bc = dev_buf(a.nbytes, a), dev_buf(b.nbytes, b), dev_buf(256 * 256 * 4)
            args = struct.pack("PPPIIII", lib.wkf_buffer_ptr(ba), lib.wkf_buffer_ptr(bb), lib.wkf_buffer_ptr(bc), 4096, 4096, 4096, 0)
            grid, block = (c_uint32 * 3)(256, 1, 1), (c_uint32 * 3)(256, 1, 1)
            us = _raw_timed(lib, dev, lambda: lib.wkf_launch(dev._h, k32, grid, block, 0, args, len(args), None), max(5, launches // 5), 10)
            rows32.append({"data": label, "us": round(us, 2), "TFLOP/s": round(2 * 4096 ** 3 / us * 1e-6, 1),
                           "frac_of_f32_peak": round(2 * 4096 ** 3 / us * 1e-6 / F32_MFMA_PEAK_TFLOPS, 4)})
            for bf in (ba, bb, bc):
                lib.wkf_buffer_release(bf)
        out["mfma_only_f32_4096x4096x4096_equivalent"] = rows32
    elif which == "stream":
        n = 1 << 30
        src_b, dst_b, src2_b = dev_buf(n), dev_buf(n), dev_buf(n)
        us = _raw_timed(lib, dev, lambda: lib.wkf_buffer_copy(dst_b, src_b, n), 10, 3)
        rows = [{"what": "hipMemcpyAsync device to device, 1 GiB", "us": round(us, 1), "GB/s": round(2 * n / us * 1e-3)}]
        # the cost of a launch itself: the read-only kernel over 4 KiB (one block), back to back on the stream
        k0 = kernel("yardstick|stream|1|256|1|0|0|0", "#define MODE 1\n#define WG 256\n#define U 1\n#define NTL 0\n#define NTS 0\n#define PERSIST 0\n" + STREAM_SRC, "wkf_stream")
        args0 = struct.pack("PPQP", lib.wkf_buffer_ptr(src_b), lib.wkf_buffer_ptr(dst_b), 256, lib.wkf_buffer_ptr(src2_b))
        g0, b0 = (c_uint32 * 3)(1, 1, 1), (c_uint32 * 3)(256, 1, 1)
        us = _raw_timed(lib, dev, lambda: lib.wkf_launch(dev._h, k0, g0, b0, 0, args0, len(args0), None), 500, 50)
        out["launch_floor_us"] = round(us, 2)
        for mode, name in ((0, "copy"), (1, "read-only"), (2, "write-only"), (3, "two reads + one write")):
            for wg, u, persist in ((256, 4, 0), (256, 8, 0), (1024, 8, 0), (256, 8, 4)):
                for ntl, nts in ((0, 0), (1, 1)):
                    defs = f"#define MODE {mode}\n#define WG {wg}\n#define U {u}\n#define NTL {ntl}\n#define NTS {nts}\n#define PERSIST {1 if persist else 0}\n"
                    k = kernel(f"yardstick|stream|{mode}|{wg}|{u}|{ntl}|{nts}|{persist}", defs + STREAM_SRC, "wkf_stream")
                    n4 = n // 16
                    nblk = 256 * persist if persist else n4 // (wg * u)
                    args = struct.pack("PPQP", lib.wkf_buffer_ptr(src_b), lib.wkf_buffer_ptr(dst_b), n4, lib.wkf_buffer_ptr(src2_b))
                    grid, block = (c_uint32 * 3)(nblk, 1, 1), (c_uint32 * 3)(wg, 1, 1)
                    us = _raw_timed(lib, dev, lambda: lib.wkf_launch(dev._h, k, grid, block, 0, args, len(args), None), 10, 3)
                    moved = n * {0: 2, 1: 1, 2: 1, 3: 3}[mode]
                    rows.append({"what": f"{name} kernel, {wg} threads, {u} x 16 B per lane, non-temporal {'on' if ntl else 'off'}, "
                                         + (f"{nblk} persistent blocks" if persist else "one chunk per block"),
                                 "us": round(us, 1), "GB/s": round(moved / us * 1e-3)})
        out["streams_1GiB"] = rows
        # The same plain kernels at the sizes of the small BASELINE configurations (a launch's ramp and tail weigh more the
        # less it moves): 32 MiB -> 32 MiB (RMSNorm, RoPE), 64 MiB -> 64 MiB (config 1), 256 MiB read (config 2).  Each launch
        # takes the next piece of the 1 GiB buffers, so nothing is served from a cache.  `kernel_us` is the median of the
        # dispatches' own begin-to-end times (what a profiler's kernel trace shows), `batch_us` one event pair around 50
        # launches back to back.
        sized = []
        for mode, name, piece in ((0, "copy", 32 << 20), (0, "copy", 64 << 20), (1, "read-only", 256 << 20)):
            for wg, u in ((256, 4), (256, 8), (1024, 8)):
                defs = f"#define MODE {mode}\n#define WG {wg}\n#define U {u}\n#define NTL 1\n#define NTS 1\n#define PERSIST 0\n"
                k = kernel(f"yardstick|stream|{mode}|{wg}|{u}|1|1|0", defs + STREAM_SRC, "wkf_stream")
                n4 = piece // 16
                grid, block = (c_uint32 * 3)(n4 // (wg * u), 1, 1), (c_uint32 * 3)(wg, 1, 1)
                pieces = n // piece
                packed = [struct.pack("PPQP", lib.wkf_buffer_ptr(src_b) + i * piece, lib.wkf_buffer_ptr(dst_b) + i * piece, n4,
                                      lib.wkf_buffer_ptr(src2_b)) for i in range(pieces)]
                turn = [0]

                def launch(timer=None):
                    a = packed[turn[0] % pieces]
                    turn[0] += 1
                    return lib.wkf_launch(dev._h, k, grid, block, 0, a, len(a), timer)

                batch = _raw_timed(lib, dev, launch, 50, 20)
                timers = []
                for _ in range(30):
                    t = c_void_p()
                    assert lib.wkf_timer_create(dev._h, byref(t)) == 0
                    assert launch(t) == 0
                    timers.append(t)
                dev.sync()
                each = []
                for t in timers:
                    ns = ctypes.c_uint64()
                    assert lib.wkf_timer_elapsed_ns(t, byref(ns)) == 0
                    each.append(ns.value / 1e3)
                    lib.wkf_timer_destroy(t)
                moved = piece * (2 if mode == 0 else 1)
                med = float(np.median(each))
                sized.append({"what": f"{name} kernel, {piece >> 20} MiB per stream, {wg} threads, {u} x 16 B per lane, non-temporal on",
                              "moved_MiB": moved >> 20, "kernel_us": round(med, 2), "kernel_min_us": round(min(each), 2), "batch_us": round(batch, 2),
                              "GB/s_kernel": round(moved / med * 1e-3), "GB/s_batch": round(moved / batch * 1e-3)})
        out["streams_sized"] = sized
        # A second pass over what a kernel has just read: the read-only kernel over a piece, then the copy kernel over the
        # same piece (or over another one, for comparison); the copy's own begin-to-end time, median of 8.  512 MiB are read
        # elsewhere before every pair so that nothing is left from the pair before.  With ordinary loads in the first pass
        # the second finds the piece in the 256 MB Infinity Cache; with non-temporal loads it does not.
        second = []
        for piece in (64 << 20, 128 << 20):
            for ntl in (0, 1):
                ks = {}
                for mode in (0, 1):
                    defs = f"#define MODE {mode}\n#define WG 256\n#define U 8\n#define NTL {ntl}\n#define NTS 1\n#define PERSIST 0\n"
                    ks[mode] = kernel(f"yardstick|stream|{mode}|256|8|{ntl}|1|0", defs + STREAM_SRC, "wkf_stream")

                def go(k, nbytes, off_s, off_d, timer=None):
                    n4 = nbytes // 16
                    g, b = (c_uint32 * 3)(n4 // (256 * 8), 1, 1), (c_uint32 * 3)(256, 1, 1)
                    a = struct.pack("PPQP", lib.wkf_buffer_ptr(src_b) + off_s, lib.wkf_buffer_ptr(dst_b) + off_d, n4, lib.wkf_buffer_ptr(src2_b))
                    assert lib.wkf_launch(dev._h, k, g, b, 0, a, len(a), timer) == 0

                times = {"same": [], "other": []}
                for it in range(10):
                    for which in ("same", "other"):
                        go(ks[1], 512 << 20, 512 << 20, 0)
                        go(ks[1], piece, 0, 0)
                        t = c_void_p()
                        assert lib.wkf_timer_create(dev._h, byref(t)) == 0
                        go(ks[0], piece, 0 if which == "same" else (256 << 20), 0, t)
                        dev.sync()
                        ns = ctypes.c_uint64()
                        assert lib.wkf_timer_elapsed_ns(t, byref(ns)) == 0
                        lib.wkf_timer_destroy(t)
                        times[which].append(ns.value / 1e3)
                second.append({"what": f"copy of {piece >> 20} MiB after a read-only pass with {'non-temporal' if ntl else 'ordinary'} loads",
                               "after_reading_the_same_piece_us": round(float(np.median(times["same"][2:])), 2),
                               "after_reading_another_piece_us": round(float(np.median(times["other"][2:])), 2)})
        out["second_pass"] = second
        for name in ("copy", "read-only", "write-only", "two reads + one write"):
            best = max((r for r in rows if r["what"].startswith(name)), key=lambda r: r["GB/s"])
            out["best_" + name.replace("-", "_").replace(" + ", "_").replace(" ", "_")] = best
    elif which == "power":
        out["phases"] = power_rows(w, dev, seeded, max(2.0, launches / 10.0))
    else:
        sys.exit("bench.py --yardstick: mfma, stream or power")
    print(json.dumps(out))


MAX_LINE_BYTES = 4096  # the final stdout line must stay small enough for any reader of it to parse


def final_line(result):
    """(the ONE stdout line, the full record).  The line keeps the contract keys, `roofline`, `cpu_baseline`, the
    worst BASELINE configuration and one [fraction of roofline, back-to-back us per step] pair per configuration;
    the rows themselves (kernels, medians, CPU samples) are in the full record only."""
    full = dict(result)
    detail = full.get("all_configs") or []
    if detail:
        # the configuration furthest below its roofline (BASELINE configurations only, as this library fuses them)
        own = [r for r in detail if r["key"][0] == "c" and not r["key"].endswith("_reference_rules") and r["key"] != "c2_one_pass"]
        if own:
            worst = min(own, key=lambda r: r["roofline"]["frac"])
            full["worst_config"] = {"key": worst["key"], "name": worst["name"], "frac": worst["roofline"]["frac"],
                                    "achieved": worst["roofline"]["achieved"], "unit": worst["unit"]}
    line = {k: v for k, v in full.items() if k != "all_configs"}
    ref = line.get("reference_cpu_path")
    if isinstance(ref, dict):
        line["reference_cpu_path"] = {"available": ref.get("available"), "note": ref.get("note")}
    if detail:
        line["fracs"] = {r["key"]: [r["roofline"]["frac"], r["roofline"]["avg_us"]] for r in detail}
    text = json.dumps(line, separators=(",", ":"))
    if len(text) > MAX_LINE_BYTES:  # never grow past the limit: drop the optional parts, longest first
        for k in ("reference_cpu_path", "fracs"):
            line.pop(k, None)
            text = json.dumps(line, separators=(",", ":"))
            if len(text) <= MAX_LINE_BYTES:
                break
    return text, full


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-detail", action="store_true", help="only the headline configuration")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--only", default="", help="comma-separated subset of c1,c2,c3,c4,c5,f16,long,attn,more,decode for the detail table")
    ap.add_argument("--plan-only", action="store_true",
                    help="no GPU: plan every workload on a plan-only device so that each kernel is JIT-compiled into the cache")
    ap.add_argument("--profile", default="", help="run one workload only (copy, c1, c2a, c2b, c3, c4_rmsnorm, c4_rope, c4_softmax, "
                                                  "c5_f32, c5_f16, c5_mlp, f16_*), for a profiler")
    ap.add_argument("--launches", type=int, default=30, help="timed steps of --profile / launches of --yardstick mfma")
    ap.add_argument("--warm-ms", type=float, default=300.0, help="--profile: milliseconds of untimed steps before the timed ones")
    ap.add_argument("--detail-out", default="gpurun_out/bench_detail.json",
                    help="file (relative to this one) that receives the full record with every row; empty: none")
    ap.add_argument("--yardstick", default="", help="mfma | stream: bounds of the machine measured with kernels outside the library; "
                                                    "power: rocm-smi readings while the f16 product and the MFMA-only loops run (--launches/10 seconds each)")
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
    if args.profile:
        profile_one(w, dev, seeded, args.profile, args.launches, args.warm_ms)
        return
    if args.yardstick:
        yardsticks(w, dev, seeded, args.yardstick, args.launches)
        return
    if args.only == "copy":
        # calibration run for the rocprofv3 counters: nothing but the 1 GiB -> 1 GiB copy kernel
        print(json.dumps({"copy_kernel_GBs": copy_ceiling(w, dev), "bytes_read": 1 << 30, "bytes_written": 1 << 30}))
        return

    with_cpu = not args.no_cpu
    head = build_workloads(w, dev, seeded, {"c2"}, with_cpu)
    wl = head["c2"]
    settle(dev, wl)
    kernels, _, _ = measure_kernels(dev, wl, args.steps, args.warmup)
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
                                 "per_launch_event_pairs_median": [k["us"] for k in kernels]},
                   "device": props.arch.decode(), "compute_units": props.compute_units, "clock_khz": props.clock_khz},
        "roofline": {"bound": "hbm", "achieved": round(268468224 / dominant["us"] * 1e-3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(268468224 / dominant["us"] * 1e-3 / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": "profiles/traffic.json (rocprofv3 --pmc run of this kernel, calibrated with a copy kernel; not measured by this run)",
                     "kernel": dominant["kind"] + " " + dominant["detail"], "avg_us": dominant["us"],
                     "algorithmic_bytes_per_launch": 268468224},
        "value_frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
    }
    result["cpu_baseline"] = cpu_baseline(wl) if with_cpu else None
    result["reference_cpu_path"] = reference_cpu_path()
    del head, wl
    dev.trim()
    if not args.no_detail:
        detail = []
        result["copy_kernel_GBs"] = copy_ceiling(w, dev)
        dev.trim()
        groups = [g for g in GROUPS if not args.only or g in args.only.split(",")]
        steps = max(20, min(args.steps, 50))
        warm = 100  # launches before anything is timed: the first launches after an idle GPU run slower (clock ramp)
        for gname in groups:
            wls = build_workloads(w, dev, seeded, {gname}, with_cpu)
            for key, one in wls.items():
                if key == "c2":
                    continue
                settle(dev, one)  # the CPU port and the uploads before this row left the GPU idle
                measured = measure_kernels(dev, one, steps, warm)
                settle(dev, one, 0.1)  # reading the per-launch times above left the GPU waiting for the host
                wall_s = measure_wall(dev, one, steps, 5)
                settle(dev, one, 0.1)
                batch_us = round(measure_batch(w, dev, one, steps, 5), 2)
                row = summarise(one, measured, wall_s, steps, batch_us)
                row["key"] = key
                row["cpu_baseline"] = cpu_row(one) if (with_cpu and one.cpu) else None
                detail.append(row)
                if gname in ("c3", "c4"):
                    # the same graph under the reference's own fusion rules (its kernel decomposition):
                    # same algorithmic work, more passes over memory
                    dev.set_fusion(w.FUSION_REFERENCE)
                    try:
                        measured = measure_kernels(dev, one, steps, 20)
                        wall_s = measure_wall(dev, one, steps, 5)
                        row = summarise(one, measured, wall_s, steps, None)
                        row["key"] = key + "_reference_rules"
                        row["name"] += " -- reference kernel decomposition"
                        row["cpu_baseline"] = None
                        detail.append(row)
                    finally:
                        dev.set_fusion(w.FUSION_TREE)
            del wls
            dev.trim()
        result["all_configs"] = detail
    line, full = final_line(result)
    if "all_configs" in full and args.detail_out:
        path = os.path.join(ROOT, args.detail_out)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w") as f:
            json.dump(full, f, indent=1)
    print(line)


if __name__ == "__main__":
    main()
