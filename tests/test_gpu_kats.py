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
