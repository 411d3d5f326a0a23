"""The reference's own test vectors, run through the C ABI on the GPU: compared with
the literal expected values (at the tolerance the reference test uses) and with the
oracle (bit-exact for exact ops, <= 2 ulp where a transcendental is involved)."""
import numpy as np
import pytest

from helpers import HipAPI, OracleAPI, assert_ulp, expected_array, golden_cases, materialise_input, run_program

pytestmark = pytest.mark.gpu
CASES = golden_cases()
# cases whose value passes through a reduction (tolerance class 1e-5 relative)
REDUCTION_CLASS = {"softmax", "layer_norm"}


@pytest.mark.parametrize("mode", [1, 0], ids=["tree", "reference-rules"])
@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_reference_vector(gpu, case, mode):
    gpu.set_fusion(mode)
    try:
        inputs = {k: materialise_input(v) for k, v in case["inputs"].items()}
        got = run_program(HipAPI(gpu), case["program"], inputs)
    finally:
        gpu.set_fusion(1)
    want = expected_array(case)
    assert got.shape == want.shape, case["ref"]
    if case["tol"] == 0:
        assert np.array_equal(got.astype(np.float64), want), f"{case['name']} ({case['ref']}): {got} != {want}"
    else:
        assert np.max(np.abs(got.astype(np.float64) - want)) < case["tol"], f"{case['name']} ({case['ref']})"
    oracle = run_program(OracleAPI, case["program"], inputs)
    if case["name"] in REDUCTION_CLASS:
        assert np.allclose(got.astype(np.float64), oracle.astype(np.float64), rtol=1e-5, atol=0), case["name"]
    else:
        assert_ulp(got, oracle, 0 if case["tol"] == 0 else 2, case["name"])


def test_inplace_reuse_never_touches_a_leaf(gpu, wkf):
    # tests/inplace_clone.rs:7-37 of the reference, plus chains that DO reuse intermediates in place
    data = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    leaf = wkf.Tensor.new(gpu, data)
    for _ in range(2):
        t = ((leaf.clone() + 1.0) * 2.0).exp().sum(2)
        u = (leaf.clone() + leaf.clone()) * leaf.clone()
        gpu.set_fusion(0)
        try:
            got = [t.to_numpy(), u.to_numpy()] if not gpu.is_planner else None
            if got is None:
                t.materialize(), u.materialize()
                pytest.skip("plan-only device: kernels compiled, nothing computed")
        finally:
            gpu.set_fusion(1)
        assert np.array_equal(got[1], (data + data) * data)
        assert np.array_equal(leaf.to_numpy(), data)


def test_kernel_times_from_both_kinds_of_events(gpu):
    # PerformanceQueries / all_timing_information (src/query.rs:50-126, src/tensor.rs:556-558): every launch reports a
    # time, whether its two events ride in the dispatch (the default) or are recorded around it (WKF_TIMER_EVENTS=1,
    # also the path of grids beyond 2^32 work-items); the second kind is read once per process, hence the child process
    if gpu.is_planner:
        from helpers import load_package
        x = load_package().Tensor.new(gpu, np.ones((1024, 1024), dtype=np.float32))
        ((x * 2.0) + 1.0).sum(1).materialize()  # the child's kernel goes into the cache
        pytest.skip("plan-only device: nothing runs, nothing is timed")
    import os
    import subprocess
    import sys
    from helpers import ROOT
    script = (
        "import sys, numpy as np\n"
        f"sys.path.insert(0, {os.path.join(ROOT, 'tests')!r})\n"
        "from helpers import load_package\n"
        "w = load_package(); dev = w.Device.new(0)\n"
        "x = w.Tensor.new(dev, np.ones((1024, 1024), dtype=np.float32))\n"
        "y = ((x * 2.0) + 1.0).sum(1)\n"
        "assert np.array_equal(y.to_numpy(), np.full(1024, 3072.0, dtype=np.float32))\n"
        "ks = y.kernels()\n"
        "assert len(ks) == 1 and 500 < ks[0].elapsed_ns < 5_000_000, ks\n"
        "print('timed', ks[0].elapsed_ns)\n"
    )
    for events in ("0", "1"):
        env = dict(os.environ, WKF_TIMER_EVENTS=events)
        out = subprocess.run([sys.executable, "-c", script], env=env, capture_output=True, text=True, timeout=110)
        assert out.returncode == 0 and "timed" in out.stdout, (events, out.stdout, out.stderr[-2000:])
