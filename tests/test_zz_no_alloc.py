"""The allocation-free entry point, wkf_tensor_reduce_into, against the allocating path it is a variant of
(wkf_tensor_reduce + wkf_tensor_materialize): same kernels, so the same bits.  Two calls in a row, the second on a
smaller input, share the device's static scratch array; a reduction folded in ONE launch (no scratch) is covered too."""
import numpy as np
import pytest

from helpers import load_package

pytestmark = pytest.mark.gpu


def _kinds(t):
    return [(k.kind, k.detail) for k in t.kernels()]


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_reduce_into_matches_the_allocating_path(gpu, dtype):
    w = load_package()
    rng = np.random.default_rng(7)
    # (shape, axis, op): few outputs over a long axis -> two launches with f32 partial results in the scratch array;
    # the second of each pair is smaller than the first, so stale partial results of the larger call lie behind it
    cases = [((64, 262144), 1, "sum"), ((32, 65536), 1, "sum"), ((8192, 2048), 0, "max"), ((4096, 512), 0, "sum"),
             ((256, 1024), 1, "min")]
    two_launches = 0
    if gpu.is_planner:  # the run that fills the kernel cache without a GPU: compile every kernel, compute nothing
        for shape, axis, op in cases:
            getattr(w.Tensor.new(gpu, np.zeros(shape, dtype=dtype)), op)(axis).materialize()
        pytest.skip("plan-only device: kernels compiled, nothing computed")
    for shape, axis, op in cases:
        x = rng.standard_normal(shape).astype(dtype)
        tx = w.Tensor.new(gpu, x)
        lazy = getattr(tx, op)(axis)
        want = lazy.to_numpy()            # the allocating path; it also loads the kernels
        launches = _kinds(lazy)
        two_launches += len(launches) == 2
        out_shape = tuple(s for d, s in enumerate(shape) if d != axis)
        for attempt in range(2):          # twice: the second call finds the first call's results in the scratch array
            out = w.Tensor.new(gpu, np.full(out_shape, 7.0, dtype=dtype))
            before, held = gpu.module_stats(), gpu.alloc_stats()
            tx.reduce_into(op, axis, out)
            after = gpu.module_stats()
            assert after["compiled"] == before["compiled"] and after["disk_hits"] == before["disk_hits"]
            # no buffer asked for (neither from the pool nor from hipMalloc), no timer (its events), nothing new alive
            assert gpu.alloc_stats() == held, (held, gpu.alloc_stats())
            got = out.to_numpy()
            assert got.dtype == want.dtype and got.shape == want.shape
            assert np.array_equal(got, want), f"{shape} axis {axis} {op}: differs from the allocating path"
    assert two_launches >= 3, "the cases no longer reach the two-launch reduction that uses the scratch array"


def test_reduce_into_refuses_what_it_cannot_do_without_allocating(gpu):
    w = load_package()
    x = w.Tensor.new(gpu, np.ones((96, 160), dtype=np.float32))
    out = w.Tensor.new(gpu, np.zeros((96,), dtype=np.float32))
    with pytest.raises(w.WkfError, match="shape"):
        x.reduce_into("sum", 1, w.Tensor.new(gpu, np.zeros((95,), dtype=np.float32)))
    with pytest.raises(w.WkfError, match="dtype"):
        x.reduce_into("sum", 1, w.Tensor.new(gpu, np.zeros((96,), dtype=np.float16)))
    with pytest.raises(w.WkfError, match="hold data"):
        (x * 2.0).reduce_into("sum", 1, out)
    with pytest.raises(w.WkfError, match="axis"):
        x.reduce_into("sum", 2, out)
