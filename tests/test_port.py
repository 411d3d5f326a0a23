"""The CPU port that bench.py reports as `cpu_baseline` computes the same functions as the
oracle (it is f32 libm arithmetic with FMA contraction, so it is compared with tolerances,
not bit for bit).  Runs without a GPU."""
import os
import subprocess

import numpy as np
import pytest

from helpers import ROOT
from oracle.oracle import OTensor, seeded


@pytest.fixture(scope="module")
def port():
    from oracle import port as p
    if not os.path.exists(p.LIB_PATH):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    p.load()
    return p


def test_port_matches_oracle(port):
    x = seeded(1, 0, (64, 256), "uniform")
    assert np.allclose(port.c1(x), ((OTensor(x) * 2.0) + 1.0).sin().exp().to_numpy(), rtol=1e-6)
    n = seeded(2, 0, (40, 1000), "normal")
    assert np.array_equal(port.row_max(n), OTensor(n).max(1).to_numpy())
    assert np.allclose(port.row_sum_exp_sub(n, 1.0), (OTensor(n) - 1.0).exp().sum(1).to_numpy(), rtol=1e-5)
    a, b = seeded(3, 0, (4, 8, 64), "uniform"), seeded(3, 1, (4, 8, 64), "uniform")
    bias = seeded(3, 2, (64,), "normal", std=0.02)
    want = (OTensor(a).silu() * (OTensor(b) + OTensor(np.broadcast_to(bias, a.shape)))).to_numpy()
    assert np.allclose(port.c3(a, b, bias), want, rtol=1e-6, atol=1e-8)
    xs, w = seeded(4, 0, (32, 128), "normal"), seeded(4, 1, (128,), "normal", mean=1.0, std=0.02)
    assert np.allclose(port.rmsnorm(xs, w, 1e-5), OTensor(xs).layer_norm(OTensor(w), 1e-5).to_numpy(), rtol=1e-5)
    q = seeded(4, 2, (3, 16, 32), "normal")
    inv = 10000.0 ** (-np.arange(0, 32, 2, dtype=np.float64) / 32)
    ang = np.arange(16, dtype=np.float64)[:, None] * inv[None]
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    full_c, full_s = np.ascontiguousarray(np.concatenate([cos, cos], 1)), np.ascontiguousarray(np.concatenate([sin, sin], 1))
    assert np.allclose(port.rope(q, full_c, full_s), OTensor(q).rope(OTensor(cos), OTensor(sin)).to_numpy(), rtol=1e-6, atol=1e-7)
    s = seeded(4, 3, (2, 8, 100), "normal")
    assert np.allclose(port.softmax_rows(s), OTensor(s).softmax_last_dim().to_numpy(), rtol=1e-5)
    ga, gb = seeded(5, 0, (70, 130), "normal", std=0.02), seeded(5, 1, (130, 300), "normal", std=0.02)
    assert np.allclose(port.gemm_f32(ga, gb), OTensor(ga).mat_mul(OTensor(gb)).to_numpy(), rtol=1e-4, atol=1e-7)
    assert port.threads() >= 1
