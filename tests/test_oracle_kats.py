"""Pins the CPU oracle (oracle/oracle.py) before anything is compared against it:
every literal vector of the reference's own tests, then what the mathematics
fixes for the parts those vectors leave open.  Runs without a GPU."""
import itertools

import numpy as np
import pytest

from helpers import OracleAPI, expected_array, golden_cases, materialise_input, run_program
from oracle.oracle import MAX_SEED, MIN_SEED, OTensor, SplitMix64, seeded, ulp_distance

CASES = golden_cases()


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_oracle_matches_reference_vector(case):
    inputs = {k: materialise_input(v) for k, v in case["inputs"].items()}
    got = run_program(OracleAPI, case["program"], inputs).astype(np.float64)
    want = expected_array(case)
    assert got.shape == want.shape, case["ref"]
    if case["tol"] == 0:
        assert np.array_equal(got, want), f"{case['name']} ({case['ref']}): {got} != {want}"
    else:
        assert np.max(np.abs(got - want)) < case["tol"], f"{case['name']} ({case['ref']})"


def test_golden_file_covers_every_reference_test_module():
    refs = {c["ref"].split(":")[0] for c in CASES}
    for module in ["src/element_wise.rs", "src/pair_wise.rs", "src/reduce.rs", "src/matmul.rs", "src/map_layout.rs",
                   "src/resize.rs", "src/slice_assign.rs", "src/tensor.rs", "src/composite/softmax.rs",
                   "src/composite/rms_norm.rs", "src/composite/silu.rs", "src/composite/cat.rs",
                   "src/composite/narrow.rs", "src/composite/unsqueeze.rs", "src/composite/arange.rs",
                   "tests/inplace_clone.rs"]:
        assert module in refs, module


# ---- layout ops against brute-force index maps ------------------------------------------------

def _brute(shape, fn):
    out = np.zeros(shape, dtype=np.float32)
    for idx in itertools.product(*[range(s) for s in shape]):
        out[idx] = fn(idx)
    return out


def test_slice_transpose_broadcast_index_maps():
    base = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4)
    t = OTensor(base)
    s = t.slice([(1, 2), (0, 2), (1, 4)]).to_numpy()
    assert np.array_equal(s, _brute((1, 2, 3), lambda i: base[i[0] + 1, i[1], i[2] + 1]))
    tr = t.transpose(0, 2).to_numpy()
    assert np.array_equal(tr, _brute((4, 3, 2), lambda i: base[i[2], i[1], i[0]]))
    # broadcast inserts the new dimension where the shapes first differ (src/map_layout.rs:72-77)
    m = np.arange(6, dtype=np.float32).reshape(2, 3)
    assert np.array_equal(OTensor(m).broadcast([5, 2, 3]).to_numpy(), _brute((5, 2, 3), lambda i: m[i[1], i[2]]))
    assert np.array_equal(OTensor(m).broadcast([2, 5, 3]).to_numpy(), _brute((2, 5, 3), lambda i: m[i[0], i[2]]))
    assert np.array_equal(OTensor(m).broadcast([2, 3, 5]).to_numpy(), _brute((2, 3, 5), lambda i: m[i[0], i[1]]))
    with pytest.raises(ValueError):
        OTensor(m).broadcast([2, 4, 5])
    # when rows == cols the leading dims match, so a vector lands on dim 0, not dim 1
    v = np.arange(3, dtype=np.float32)
    assert np.array_equal(OTensor(v).broadcast([3, 3]).to_numpy(), _brute((3, 3), lambda i: v[i[0]]))


def test_resize_reshape_slice_assign_cat_index_maps():
    m = np.arange(1, 7, dtype=np.float32).reshape(3, 2)
    r = OTensor(m).resize([4, 5]).to_numpy()
    assert np.array_equal(r, _brute((4, 5), lambda i: m[i] if i[0] < 3 and i[1] < 2 else 0.0))
    crop = OTensor(m).resize([2, 1]).to_numpy()
    assert np.array_equal(crop, m[:2, :1])
    # reshape of a strided view reads the view in its own row-major order
    tr = OTensor(m).transpose(0, 1)
    assert np.array_equal(tr.reshape([6]).to_numpy(), np.array([1, 3, 5, 2, 4, 6], dtype=np.float32))
    base = OTensor(np.zeros((3, 4), dtype=np.float32))
    got = base.slice_assign([(1, 3), (2, 4)], OTensor(np.array([[1, 2], [3, 4]], dtype=np.float32))).to_numpy()
    assert np.array_equal(got, _brute((3, 4), lambda i: [[1, 2], [3, 4]][i[0] - 1][i[1] - 2] if i[0] >= 1 and i[1] >= 2 else 0))
    assert np.array_equal(base.to_numpy(), np.zeros((3, 4), dtype=np.float32))  # the target is not mutated
    c = OTensor.cat([OTensor(m), OTensor(m * 10), OTensor(m * 100)], 0).to_numpy()
    assert np.array_equal(c, np.concatenate([m, m * 10, m * 100], 0))


# ---- arithmetic: per-op rounding, casts, seeds ---------------------------------------------------

def test_every_op_rounds_to_the_tensor_dtype():
    # f16: 2048 + 1 is not representable and rounds to 2048, so the chain gives 0, not 1
    a = OTensor(np.array([2048.0], dtype=np.float16))
    assert ((a + 1.0) - 2048.0).to_numpy()[0] == 0.0
    # f32: 2^24 + 1 rounds back to 2^24
    b = OTensor(np.array([16777216.0], dtype=np.float32))
    assert ((b + 1.0) - 16777216.0).to_numpy()[0] == 0.0
    # the literal itself is rounded to f16 on an f16 tensor: 0.1 -> 0.0999755859375
    c = OTensor(np.array([0.0], dtype=np.float16)) + 0.1
    assert float(c.to_numpy()[0]) == float(np.float16(0.1))


def test_casts_round_to_nearest_even_and_overflow_to_inf():
    x = np.array([65504.0, 65519.0, 65520.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1e-8, -70000.0], dtype=np.float32)
    got = OTensor(x).cast(np.float16).to_numpy()
    want = np.array([65504.0, 65504.0, np.inf, 1.0, 1.0 + 2.0 ** -9, 0.0, -np.inf], dtype=np.float16)
    assert np.array_equal(got, want)
    h = np.array([0.1, 65504.0, 6e-8], dtype=np.float16)
    assert np.array_equal(OTensor(h).cast(np.float32).to_numpy(), h.astype(np.float32))


def test_reduction_closed_forms_and_seeds():
    ones = OTensor(np.ones((7, 1000), dtype=np.float32))
    assert np.array_equal(ones.sum(1).to_numpy(), np.full(7, 1000.0, dtype=np.float32))
    assert np.array_equal(ones.sum(0).to_numpy(), np.full(1000, 7.0, dtype=np.float32))
    assert np.array_equal((ones * 2.0).product(0).to_numpy(), np.full(1000, 128.0, dtype=np.float32))
    g = np.random.default_rng(1).standard_normal((5, 33)).astype(np.float32)
    assert np.array_equal(OTensor(g).max(1).to_numpy(), g.max(1))
    assert np.array_equal(OTensor(g).min(0).to_numpy(), g.min(0))
    # a permutation of the axis does not change a sum beyond rounding, and max/min not at all
    p = np.random.default_rng(2).permutation(33)
    assert np.allclose(OTensor(g).sum(1).to_numpy(), OTensor(g[:, p]).sum(1).to_numpy(), rtol=1e-6)
    assert np.array_equal(OTensor(g).max(1).to_numpy(), OTensor(g[:, p]).max(1).to_numpy())
    # seeds are the f32 literals +-3.40282e+38, not +-inf (src/reduce.rs:640,713)
    neg_inf = OTensor(np.full((2, 3), -np.inf, dtype=np.float32))
    assert np.array_equal(neg_inf.max(1).to_numpy(), np.full(2, MAX_SEED, dtype=np.float32))
    assert np.array_equal((-neg_inf).min(1).to_numpy(), np.full(2, MIN_SEED, dtype=np.float32))
    assert float(MAX_SEED) > -np.finfo(np.float32).max
    # reducing a rank-1 tensor gives rank 0
    assert OTensor(np.arange(4, dtype=np.float32)).sum(0).to_numpy().shape == ()


def test_matmul_identities():
    g = np.random.default_rng(3).standard_normal((9, 17)).astype(np.float32)
    assert np.array_equal(OTensor(g).mat_mul(OTensor(np.eye(17, dtype=np.float32))).to_numpy(), g)
    k = OTensor(np.ones((4, 300), dtype=np.float32)).mat_mul(OTensor(np.ones((300, 5), dtype=np.float32)))
    assert np.array_equal(k.to_numpy(), np.full((4, 5), 300.0, dtype=np.float32))
    # a transposed operand: (A B)^T = B^T A^T
    a = np.random.default_rng(4).standard_normal((6, 8)).astype(np.float32)
    b = np.random.default_rng(5).standard_normal((8, 3)).astype(np.float32)
    ab = OTensor(a).mat_mul(OTensor(b)).to_numpy()
    btat = OTensor(b).transpose(0, 1).mat_mul(OTensor(a).transpose(0, 1)).to_numpy()
    assert np.allclose(ab.T, btat, rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError):
        OTensor(a).mat_mul(OTensor(a))


# ---- composites with no (or a weak) reference vector ----------------------------------------------

def _rope_tables(seq, dim, theta=10000.0):
    inv = theta ** (-np.arange(0, dim, 2, dtype=np.float64) / dim)
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def test_rope_formula_and_invariants():
    heads, seq, dim = 2, 5, 8
    x = np.random.default_rng(6).standard_normal((heads, seq, dim)).astype(np.float32)
    cos, sin = _rope_tables(seq, dim)
    y = OTensor(x).rope(OTensor(cos), OTensor(sin)).to_numpy().astype(np.float64)
    # written out per pair (j, j + d/2): a rotation by angle[pos, j]
    x1, x2 = x[..., : dim // 2].astype(np.float64), x[..., dim // 2:].astype(np.float64)
    c, s = cos.astype(np.float64)[None], sin.astype(np.float64)[None]
    want = np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=-1)
    assert np.allclose(y, want, rtol=1e-6, atol=1e-6)
    assert np.allclose(y[:, 0, :], x[:, 0, :])  # position 0: cos = 1, sin = 0
    n_in = x1 ** 2 + x2 ** 2
    n_out = y[..., : dim // 2] ** 2 + y[..., dim // 2:] ** 2
    assert np.allclose(n_in, n_out, rtol=1e-5)
    # full-width tables and longer tables give the same result
    full_c, full_s = np.concatenate([cos, cos], 1), np.concatenate([sin, sin], 1)
    y2 = OTensor(x).rope(OTensor(full_c), OTensor(full_s)).to_numpy()
    assert np.array_equal(y2.astype(np.float64), y)
    cos9, sin9 = _rope_tables(9, dim)
    assert np.array_equal(OTensor(x).rope(OTensor(cos9), OTensor(sin9)).to_numpy().astype(np.float64), y)


def test_softmax_last_dim_properties():
    x = np.random.default_rng(7).standard_normal((3, 4, 50)).astype(np.float32) * 3
    y = OTensor(x).softmax_last_dim().to_numpy().astype(np.float64)
    assert np.allclose(y.sum(-1), 1.0, atol=1e-6)
    e = np.exp(x.astype(np.float64) - x.max(-1, keepdims=True))
    assert np.allclose(y, e / e.sum(-1, keepdims=True), rtol=1e-6)
    v = x[0, 0]
    assert np.allclose(OTensor(v).softmax().to_numpy(), OTensor(v).softmax_last_dim().to_numpy(), rtol=1e-5)
    big = OTensor(np.array([[1000.0, 1000.0]], dtype=np.float32)).softmax_last_dim().to_numpy()
    assert np.array_equal(big, np.array([[0.5, 0.5]], dtype=np.float32))  # no overflow thanks to the max shift


def test_layer_norm_is_rms_norm_in_f32():
    x = np.random.default_rng(8).standard_normal((6, 10)).astype(np.float32)
    w = np.random.default_rng(9).standard_normal(10).astype(np.float32)
    y = OTensor(x).layer_norm(OTensor(w), 1e-5).to_numpy().astype(np.float64)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-5) * w
    assert np.allclose(y, want, rtol=1e-6, atol=1e-6)
    h = OTensor(x.astype(np.float16)).layer_norm(OTensor(w.astype(np.float16)), 1e-5)
    assert h.to_numpy().dtype == np.float16
    assert np.allclose(h.to_numpy().astype(np.float64), want, rtol=5e-3, atol=5e-3)


def test_silu_closed_form():
    x = np.linspace(-20, 20, 401, dtype=np.float32)
    y = OTensor(x).silu().to_numpy().astype(np.float64)
    assert np.allclose(y, x / (1 + np.exp(-x.astype(np.float64))), rtol=1e-6, atol=1e-9)
    assert OTensor(np.array([0.0], dtype=np.float32)).silu().to_numpy()[0] == 0.0


# ---- the helpers themselves ---------------------------------------------------------------------------

def test_ulp_distance():
    one = np.float32(1.0)
    nxt = np.nextafter(one, np.float32(2.0))
    assert ulp_distance(np.array([one]), np.array([nxt]))[0] == 1
    assert ulp_distance(np.array([np.float32(0.0)]), np.array([np.float32(-0.0)]))[0] == 0
    tiny = np.nextafter(np.float32(0.0), np.float32(1.0))
    assert ulp_distance(np.array([tiny]), np.array([-tiny]))[0] == 2
    assert ulp_distance(np.array([np.float32(np.nan)]), np.array([np.float32(np.nan)]))[0] == 0
    assert ulp_distance(np.array([np.float16(1.0)]), np.array([np.nextafter(np.float16(1.0), np.float16(2.0))]))[0] == 1


def test_seeded_generator_is_deterministic_and_well_distributed():
    a = seeded(1, 0, (1000, 100), "uniform")
    b = seeded(1, 0, (1000, 100), "uniform")
    assert np.array_equal(a, b) and a.dtype == np.float32
    assert not np.array_equal(a, seeded(1, 1, (1000, 100), "uniform"))
    assert -1.0 < a.min() and a.max() < 1.0 and abs(a.mean()) < 0.01
    n = seeded(2, 0, (200000,), "normal")
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1.0) < 0.01
    w = seeded(3, 2, (4096,), "normal", std=0.02)
    assert abs(w.std() - 0.02) < 0.002
    # SplitMix64 first outputs for seed 0 (published test vector of the algorithm)
    g = SplitMix64(0)
    assert [int(v) for v in g.raw(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]


def test_layer_norm_as_the_reference_writes_it_differs_only_on_square_inputs():
    # src/composite/rms_norm.rs:13-14 broadcasts through Tensor::broadcast (first differing dimension,
    # src/map_layout.rs:69-77): RMSNorm for rows != hidden, the weight indexed by ROW for rows == hidden
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 10)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 10).astype(np.float32)
    a = OTensor(x).layer_norm(OTensor(w), 1e-5).to_numpy()
    b = OTensor(x).layer_norm_as_written(OTensor(w), 1e-5).to_numpy()
    assert np.array_equal(a, b)
    sq = rng.standard_normal((10, 10)).astype(np.float32)
    meant = OTensor(sq).layer_norm(OTensor(w), 1e-5).to_numpy()
    written = OTensor(sq).layer_norm_as_written(OTensor(w), 1e-5).to_numpy()
    assert not np.array_equal(meant, written)
    rms = np.sqrt((sq.astype(np.float64) ** 2).mean(1) + 1e-5)
    assert np.allclose(meant, sq / rms[:, None] * w[None, :], rtol=1e-6)
    assert np.allclose(written, sq / rms[:, None] * w[:, None], rtol=1e-6)   # the weight runs down the rows
