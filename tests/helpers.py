"""Shared by the tests: loading the package (its directory name has a hyphen), the
golden vectors, and running one Tensor-API expression on either implementation."""
import importlib.util
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle.oracle import OTensor, ulp_distance  # noqa: E402  (the checker; tests may import it)

_pkg = None


def _build_if_nothing_is_built():
    """The tests load what is built; only a tree with no built library at all is built first."""
    lib = os.path.join(ROOT, "wgpu-kernal-fusion_amd", "libwkf_hip.so")
    port = os.path.join(ROOT, "oracle", "libwkf_port.so")
    if not os.path.exists(lib) or not os.path.exists(port):
        sys.path.insert(0, ROOT)
        import __graft_entry__
        __graft_entry__.build()


def load_package():
    global _pkg
    if _pkg is None:
        _build_if_nothing_is_built()
        path = os.path.join(ROOT, "wgpu-kernal-fusion_amd", "__init__.py")
        spec = importlib.util.spec_from_file_location("wgpu_kernal_fusion_amd", path)
        mod = importlib.util.module_from_spec(spec)
        sys.modules["wgpu_kernal_fusion_amd"] = mod
        spec.loader.exec_module(mod)
        mod.load()
        _pkg = mod
    return _pkg


def golden_cases():
    with open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")) as f:
        return json.load(f)["cases"]


NP_DTYPE = {"f32": np.float32, "f16": np.float16}


def materialise_input(spec):
    dt = NP_DTYPE[spec["dtype"]]
    if "fill" in spec:
        return np.full(spec["shape"], spec["fill"], dtype=dt)
    return np.asarray(spec["data"], dtype=dt)


def expected_array(case):
    e = case["expected"]
    if isinstance(e, dict):
        return np.full(e["shape"], e["fill"], dtype=np.float64)
    return np.asarray(e, dtype=np.float64)


class OracleAPI:
    """Binds the names a golden `program` may use to the oracle."""
    T = OTensor
    DEV = None
    F32, F16 = np.float32, np.float16

    @staticmethod
    def tensor(arr):
        return OTensor(arr)


class HipAPI:
    """Binds the same names to the HIP path on `device`."""

    def __init__(self, device):
        pkg = load_package()
        self.T, self.DEV, self.F32, self.F16 = pkg.Tensor, device, pkg.F32, pkg.F16
        self._pkg = pkg

    def tensor(self, arr):
        return self._pkg.Tensor.new(self.DEV, arr)


def hip_values(tensor):
    """Values of a HIP tensor as numpy.  On a plan-only device (WKF_TEST_PLAN_ONLY=1: the run that
    fills the on-disk kernel cache before the tree travels to the GPU box) the kernels are generated
    and compiled, nothing is computed, and the test is skipped at this point."""
    if tensor.device.is_planner:
        tensor.materialize()
        import pytest
        pytest.skip("plan-only device: kernels compiled, nothing computed")
    return tensor.to_numpy()


def hip_values_many(tensors):
    """`hip_values` for several tensors: on a plan-only device all of them are compiled before the skip."""
    tensors = list(tensors)
    if tensors and tensors[0].device.is_planner:
        for t in tensors:
            t.materialize()
        import pytest
        pytest.skip("plan-only device: kernels compiled, nothing computed")
    return [t.to_numpy() for t in tensors]


def run_program(api, program, inputs):
    """Evaluates `program` (a Python expression over the Tensor API) and returns a numpy array."""
    env = {"T": api.T, "DEV": api.DEV, "F32": api.F32, "F16": api.F16}
    for name, arr in inputs.items():
        env[name] = api.tensor(arr)
    out = eval(program, {"__builtins__": {"range": range}}, env)  # noqa: S307 (test-only, fixed strings)
    return hip_values(out) if isinstance(api, HipAPI) else out.to_numpy()


def assert_ulp(got, want, max_ulp, what=""):
    assert got.dtype == want.dtype, f"{what}: dtype {got.dtype} vs {want.dtype}"
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    d = ulp_distance(got, want)
    worst = int(d.max()) if d.size else 0
    assert worst <= max_ulp, f"{what}: max ulp distance {worst} > {max_ulp} (at flat index {int(d.argmax())}: got {got.ravel()[d.argmax()]!r}, want {want.ravel()[d.argmax()]!r})"
    return worst
