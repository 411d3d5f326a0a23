"""Parity of the HIP path against the oracle on seeded inputs: every op, both dtypes,
contiguous and strided operands, every kernel shape the planner can pick, the edge
cases (empty, ragged, rank 0, single element, non-vectorisable sizes), and the
benchmark configurations at full size.

Tolerances (stated where they are used):
  exact ops (+ - * / sqr sqrt abs neg, casts, copies, layout)   bit-exact
  fused element-wise with transcendental ops                       <= 2 ulp
  reductions (sum, product) and what is built on them              1e-5 relative
  max / min                                                        bit-exact
"""
import os

import numpy as np
import pytest

from helpers import HipAPI, OracleAPI, assert_ulp, hip_values, hip_values_many
from oracle.oracle import OTensor, seeded, ulp_distance

pytestmark = pytest.mark.gpu

SHAPES = [(1,), (7,), (4096,), (3, 5), (17, 33), (4, 6, 10), (130, 257), (2, 3, 4, 5)]
EXACT_UNARY = ["sqr", "sqrt", "abs"]
# op -> (lo, hi) of a domain where it is defined
TRANS_UNARY = {"exp": (-20, 20), "exp2": (-20, 20), "log": (1e-3, 100), "log2": (1e-3, 100), "sin": (-50, 50),
               "cos": (-50, 50), "tan": (-1.5, 1.5), "asin": (-1, 1), "acos": (-1, 1), "atan": (-30, 30),
               "sinh": (-8, 8), "cosh": (-8, 8), "tanh": (-6, 6), "asinh": (-100, 100), "acosh": (1, 100),
               "atanh": (-0.99, 0.99)}


def data(shape, lo, hi, dtype, seed):
    rng = np.random.default_rng(seed)
    return rng.uniform(lo, hi, shape).astype(np.float32).astype(dtype)


def both(gpu, fn, *arrays):
    """fn(tensor...) evaluated on the HIP path and on the oracle."""
    api = HipAPI(gpu)
    got = hip_values(fn(*[api.tensor(a) for a in arrays]))
    want = fn(*[OTensor(a) for a in arrays]).to_numpy()
    return got, want


# ---- element-wise ------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_exact_elementwise_ops_are_bit_exact(gpu, shape, dtype):
    x = data(shape, -4, 4, dtype, 1)
    fns = [lambda t: t + 1.5, lambda t: 1.5 + t, lambda t: t - 0.1, lambda t: 0.1 - t, lambda t: t * 3.0,
           lambda t: t / 3.0, lambda t: 3.0 / t, lambda t: -t, lambda t: t.abs(), lambda t: t.sqr(),
           lambda t: t.abs().sqrt(), lambda t: ((t * 0.3) + 7.0) / 1.7 - 2.0]
    api = HipAPI(gpu)
    got = hip_values_many([f(api.tensor(x)) for f in fns])
    for i, f in enumerate(fns):
        assert_ulp(got[i], f(OTensor(x)).to_numpy(), 0, f"fn {i} shape {shape}")


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("op", sorted(TRANS_UNARY), ids=str)
def test_transcendental_ops_within_2_ulp(gpu, op, dtype):
    lo, hi = TRANS_UNARY[op]
    if dtype == np.float16:
        lo, hi = max(lo, -10), min(hi, 10)
    x = data((257, 129), lo, hi, dtype, 2)
    got, want = both(gpu, lambda t: getattr(t, op)(), x)
    assert_ulp(got, want, 2, op)  # <= 2 ulp: the last op of a chain goes through the f32 library


@pytest.mark.parametrize("exact", [False, True], ids=["default-math", "exact-math"])
def test_chains_with_interior_transcendentals(gpu, exact):
    # an op whose value feeds further arithmetic is evaluated with an f64 core, so later ops cannot amplify its error
    x = data((300, 130), -3, 3, np.float32, 3)
    y = data((300, 130), 0.5, 3, np.float32, 4)
    fns = [lambda a, b: ((a * 2.0) + 1.0).sin().exp(),
           lambda a, b: a.silu() * (b + 0.25),
           lambda a, b: (a.exp() + b.cos()) / (1.0 + b.sin().sqr()),
           lambda a, b: (a.tanh() * b.log()).exp() - b.pow(a),
           lambda a, b: (a / b).atan().sinh() + a.cos().cos()]
    api = HipAPI(gpu)
    gpu.set_exact_math(exact)
    try:
        got = hip_values_many([f(api.tensor(x), api.tensor(y)) for f in fns])
    finally:
        gpu.set_exact_math(False)
    for i, f in enumerate(fns):
        # <= 2 ulp in the default mode (only the last op may be off); exact mode: <= 1 ulp
        # (1 only through float64's own libm error in the oracle or the 2^-46 misrounding bound)
        assert_ulp(got[i], f(OTensor(x), OTensor(y)).to_numpy(), 1 if exact else 2, f"chain {i}")


def test_interior_tanh_on_f32_is_rounded_once(gpu):
    # a tanh that feeds further arithmetic on f32 has an f64 core of its own (1 - 2 / (exp(2|x|) + 1), a series near zero):
    # arguments from 1e-30 to beyond saturation, both signs, zeros, infinities and NaN; the product with 1 must be the
    # correctly rounded tanh (the oracle's float64 tanh rounded to f32; one ulp of slack for the oracle's own libm)
    rng = np.random.default_rng(11)
    mags = np.exp(rng.uniform(np.log(1e-30), np.log(30.0), 200000)).astype(np.float32)
    x = np.concatenate([mags, -mags, np.float32([0.0, -0.0, np.inf, -np.inf, np.nan, 2.0 ** -6, 9.0109, 20.0, 1e30]),
                        np.linspace(-0.02, 0.02, 4001, dtype=np.float32)])
    got, want = both(gpu, lambda t: t.tanh() * 1.0, x)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.signbit(got), np.signbit(want))
    assert_ulp(got, want, 1, "interior tanh on f32")
    assert np.mean(got.view(np.uint32) == want.view(np.uint32)) > 0.99999


def test_interior_exp_on_f16_is_correctly_rounded_for_every_argument(gpu):
    # an exp that feeds further arithmetic on an f16 tensor goes through the f32 library and, when that cannot
    # decide the f16 rounding, through the f64 core: checked on all 63488 finite f16 values (subnormals included)
    bits = np.arange(0, 1 << 16, dtype=np.uint16)
    x = bits.view(np.float16)
    x = x[np.isfinite(x)]
    got, want = both(gpu, lambda t: t.exp() * 1.0, x)
    assert_ulp(got, want, 0, "exp on f16")
    got, want = both(gpu, lambda t: t / (1.0 + (-t).exp()), x)  # silu, as the composite builds it
    assert_ulp(got, want, 0, "silu on f16")
    with np.errstate(all="ignore"):
        got, want = both(gpu, lambda t: t.sqrt() * 1.0, x)      # a root that feeds further arithmetic (negative arguments: NaN)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert_ulp(got[~np.isnan(want)], want[~np.isnan(want)], 0, "interior sqrt on f16")


@pytest.mark.parametrize("op", sorted(TRANS_UNARY), ids=str)
def test_interior_transcendentals_on_f16_are_correctly_rounded_for_every_argument(gpu, op):
    # a transcendental op that feeds further arithmetic on an f16 tensor must be the correctly rounded f16 value: the
    # f32 library decides it for most arguments and the f64 routine for the rest; all 63488 finite f16 values
    # (outside the function's domain both sides give NaN)
    bits = np.arange(0, 1 << 16, dtype=np.uint16)
    x = bits.view(np.float16)
    x = x[np.isfinite(x)]
    with np.errstate(all="ignore"):
        got, want = both(gpu, lambda t: getattr(t, op)() * 1.0, x)
    assert_ulp(got, want, 0, f"{op} on f16")


def test_trig_far_arguments_take_the_slow_path(gpu):
    x = np.array([0.0, 1.0, 99999.0, 100001.0, 1e7, -3e9, 1e30, np.inf, np.nan, -0.0] * 13, dtype=np.float32)
    got, want = both(gpu, lambda t: (t.sin() * 2.0) + t.cos() * 0.5, x)
    assert_ulp(got, want, 0, "far sin/cos")  # interior ops: f64 cores, or the f64 library beyond |x| = 1e5


def test_special_values(gpu):
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, -3.4e38, 88.9, -104.0, 1e-38] * 3, dtype=np.float32)
    fns = [lambda t: t.exp() * 1.0, lambda t: t + 1.0, lambda t: t * 0.5, lambda t: t / 3.0, lambda t: t.abs().sqrt(),
           lambda t: t.cast(np.float16) if isinstance(t, OTensor) else t.cast(1)]
    api = HipAPI(gpu)
    got = hip_values_many([f(api.tensor(x)) for f in fns])
    for i, f in enumerate(fns):
        assert_ulp(got[i], f(OTensor(x)).to_numpy(), 0, f"special {i}")  # incl. f32 denormals, which are preserved


@pytest.mark.parametrize("shape", [(5,), (64, 64), (3, 7, 11), (1000, 3)], ids=str)
def test_casts_are_bit_exact(gpu, shape):
    x = data(shape, -70000, 70000, np.float32, 5)
    x.ravel()[:4] = [65504.0, 65520.0, 1e-8, -65519.0][: min(4, x.size)]
    api = HipAPI(gpu)
    a, b, c = hip_values_many([api.tensor(x).cast(1), api.tensor(x.astype(np.float16)).cast(0),
                               (api.tensor(x).cast(1) * 2.0).cast(0) + 1.0])
    with np.errstate(over="ignore"):
        h = x.astype(np.float16)
    assert_ulp(a, h, 0, "f32->f16")
    assert_ulp(b, h.astype(np.float32), 0, "f16->f32")
    assert_ulp(c, ((OTensor(x).cast(np.float16) * 2.0).cast(np.float32) + 1.0).to_numpy(), 0, "cast chain")


# ---- pair-wise, views, in-place ------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", [(6,), (33, 65), (4, 6, 10), (128, 256)], ids=str)
def test_pairwise_ops(gpu, shape, dtype):
    a, b = data(shape, -4, 4, dtype, 6), data(shape, 0.5, 4, dtype, 7)
    api = HipAPI(gpu)
    fns = [lambda p, q: p + q, lambda p, q: p - q, lambda p, q: p * q, lambda p, q: p / q,
           lambda p, q: (p + 1.0) * (q * 2.0) - (p / q), lambda p, q: q.pow(p)]
    got = hip_values_many([f(api.tensor(a), api.tensor(b)) for f in fns])
    for i, f in enumerate(fns):
        assert_ulp(got[i], f(OTensor(a), OTensor(b)).to_numpy(), 2 if i == 5 else 0, f"pair {i}")


def test_strided_and_broadcast_operands(gpu):
    a = data((12, 20, 16), -2, 2, np.float32, 8)
    v = data((16,), -2, 2, np.float32, 9)
    r = data((12, 20), 0.5, 2, np.float32, 10)
    api = HipAPI(gpu)

    def prog(T, a, v, r):
        views = [
            a.slice([(1, 11), (2, 18), (4, 12)]) * 2.0,                       # offset, vectorisable inner dim
            a.slice([(0, 12), (0, 20), (3, 10)]) + 1.0,                       # ragged inner dim: scalar path
            a.transpose(0, 2) - 1.0,                                          # inner stride != 1
            a.transpose(1, 2).slice([(2, 5), (0, 16), (1, 20)]).abs(),
            a * v.broadcast([20, 16]).broadcast([12, 20, 16]),                # bias on the last dim
            a / r.broadcast([12, 20, 16]),                                    # one scalar per row
            (a + v.broadcast([20, 16]).broadcast([12, 20, 16])) * r.broadcast([12, 20, 16]),
            a.slice([(0, 12), (0, 20), (0, 1)]).broadcast([12, 20, 1, 1]) + 0.0,
        ]
        return views

    got = hip_values_many(prog(api.T, api.tensor(a), api.tensor(v), api.tensor(r)))
    want = prog(OTensor, OTensor(a), OTensor(v), OTensor(r))
    for i, (g, w) in enumerate(zip(got, want)):
        assert_ulp(g, w.to_numpy(), 0, f"view {i}")


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_transposed_operands_take_the_tiled_kernel(gpu, dtype):
    # inputs that are unit-stride along another dimension than the output go through a 64 x 64 LDS tile
    api = HipAPI(gpu)
    a = data((300, 523), -2, 2, dtype, 21)
    b = data((523, 300), -2, 2, dtype, 22)
    c = data((5, 130, 200), -2, 2, dtype, 23)
    d = data((200, 5, 130), -2, 2, dtype, 24)

    def progs(ta, tb, tc, td):
        return [ta.transpose(0, 1) + 1.0,                              # ragged edge tiles on both sides
                ta.transpose(0, 1) * tb,                               # one crossed, one straight operand
                (ta.transpose(0, 1) + tb) - ta.transpose(0, 1) * 0.5,  # the crossed operand is read once
                tc.transpose(1, 2) * 2.0,                              # batch dim in front
                tc.transpose(0, 2).transpose(1, 2) + td,               # [200, 5, 130] from [5, 130, 200]
                ta.slice([(3, 290), (10, 500)]).transpose(0, 1) * tb.slice([(10, 500), (3, 290)])]

    got = hip_values_many(progs(api.tensor(a), api.tensor(b), api.tensor(c), api.tensor(d)))
    want = progs(OTensor(a), OTensor(b), OTensor(c), OTensor(d))
    for i, (g, w) in enumerate(zip(got, want)):
        assert np.array_equal(g, w.to_numpy()), f"program {i}"
    if dtype == np.float32:
        far = a.copy()
        far[::7, ::5] *= 1e6  # some arguments beyond the fast trig range
        g = hip_values(api.tensor(far).transpose(0, 1).sin() + api.tensor(b))
        w = (OTensor(far).transpose(0, 1).sin() + OTensor(b)).to_numpy()
        assert_ulp(g, w, 2)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_transposed_operands_with_aligned_shapes(gpu, dtype):
    # the tiled kernel on shapes that are multiples of the vector width, with a per-row scalar operand and sliced views
    api = HipAPI(gpu)
    a = data((304, 520), -2, 2, dtype, 25)
    b = data((520, 304), -2, 2, dtype, 26)
    c = data((3, 136, 264), -2, 2, dtype, 27)
    r = data((520,), 0.5, 2, dtype, 28)

    def progs(ta, tb, tc, tr):
        return [ta.transpose(0, 1) + 1.0,
                ta.transpose(0, 1) * tb - tb,
                (ta.transpose(0, 1) + tb) / tr.broadcast([520, 304]),            # one scalar per output row
                tc.transpose(1, 2) * 2.0,                                        # batch dim in front, partial edge tiles
                ta.slice([(8, 296), (16, 504)]).transpose(0, 1) * tb.slice([(16, 504), (8, 296)]),
                ta.transpose(0, 1).exp() + tb]

    ts = progs(api.tensor(a), api.tensor(b), api.tensor(c), api.tensor(r))
    alone = [hip_values(t) for t in ts]
    # every one of them moves four elements per access on both sides of the tile
    for i, t in enumerate(ts):
        assert any(k.kind == "map" and "tiled" in k.detail and "vec=4" in k.detail for k in t.kernels()), (i, [k.detail for k in t.kernels()])
    got = hip_values_many(progs(api.tensor(a), api.tensor(b), api.tensor(c), api.tensor(r)))
    want = progs(OTensor(a), OTensor(b), OTensor(c), OTensor(r))
    for i, (g, w) in enumerate(zip(got, want)):
        assert_ulp(g, w.to_numpy(), 0, f"program {i}")
        assert np.array_equal(alone[i], g), i


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_large_transposed_operands_take_tiles_of_128(gpu, dtype):
    # with four-element accesses, both extents beyond 128, tiles enough for the chip twice over and room in the LDS for two
    # workgroups per compute unit, the tile is 128 x 128: ragged edges on both sides (3004 = 23 x 128 + 60, 2956 = 23 x 128
    # + 12), a straight second operand, a per-row scalar, a batch in front; two crossed f32 inputs keep 64 x 64 tiles
    api = HipAPI(gpu)
    a = data((3004, 2956), -2, 2, dtype, 31)
    b = data((2956, 3004), -2, 2, dtype, 32)
    c = data((6, 1028, 1156), -2, 2, dtype, 33)
    r = data((2956,), 0.5, 2, dtype, 34)

    def progs(ta, tb, tc, tr):
        return [ta.transpose(0, 1) + 1.0,
                ta.transpose(0, 1) * tb - tb,
                (ta.transpose(0, 1) + tb) / tr.broadcast([3004, 2956]).transpose(0, 1),
                tc.transpose(1, 2) * 2.0,
                ta.transpose(0, 1) * tb.transpose(0, 1).transpose(0, 1) + ta.slice([(4, 3004), (0, 2952)]).transpose(0, 1).resize([2956, 3004])]

    ts = progs(api.tensor(a), api.tensor(b), api.tensor(c), api.tensor(r))
    got = [hip_values(t) for t in ts]
    for i, t in enumerate(ts[:4]):
        assert any(k.kind == "map" and "tiled" in k.detail and "tile=128" in k.detail for k in t.kernels()), (i, [k.detail for k in t.kernels()])
    want = progs(OTensor(a), OTensor(b), OTensor(c), OTensor(r))
    for i, (g, w) in enumerate(zip(got, want)):
        assert_ulp(g, w.to_numpy(), 0, f"program {i}")
    # two crossed f32 inputs: their tiles of 128 would leave one workgroup per compute unit
    two = api.tensor(a).transpose(0, 1) * api.tensor(np.ascontiguousarray(b.T)).transpose(0, 1)
    g2 = hip_values(two)
    assert any("tiled" in k.detail for k in two.kernels())
    assert ("tile=128" in " ".join(k.detail for k in two.kernels())) == (dtype == np.float16)
    assert_ulp(g2, (OTensor(a).transpose(0, 1) * OTensor(np.ascontiguousarray(b.T)).transpose(0, 1)).to_numpy(), 0, "two crossed inputs")


def test_same_results_under_both_fusion_modes(gpu):
    a, b = data((64, 96), -2, 2, np.float32, 11), data((64, 96), 0.5, 2, np.float32, 12)
    api = HipAPI(gpu)

    def progs(a, b):
        return [a.silu() * (b + 1.0), ((a + b) * (a - b)) / (b * b + 1.0), (a.exp() + b).sum(1) * 2.0,
                ((a * b) + a).max(0), (a + b).resize([70, 100]), a.transpose(0, 1).reshape([96 * 64]) + 1.0]

    tree = hip_values_many(progs(api.tensor(a), api.tensor(b)))
    gpu.set_fusion(0)
    try:
        ref = hip_values_many(progs(api.tensor(a), api.tensor(b)))
    finally:
        gpu.set_fusion(1)
    for i, (t, r) in enumerate(zip(tree, ref)):
        if i == 2:
            # exp feeds a sum: fused into the reduce it goes through the f32 library (reduction class,
            # 1e-5 relative), materialised first it goes through the f64 core; the sums agree to rounding
            assert np.allclose(t, r, rtol=1e-6), f"program {i}"
        else:
            assert np.array_equal(t, r), f"program {i}: fusing more must not change a bit"


# ---- reductions ---------------------------------------------------------------------------------------------

RED_SHAPES = [((1,), 0), ((5,), 0), ((4096,), 0), ((3, 2), 0), ((3, 2), 1), ((1, 7), 1), ((7, 1), 1), ((64, 64), 0),
              ((64, 64), 1), ((9, 1000), 1), ((1000, 9), 0), ((3, 100003), 1), ((5, 6, 7), 0), ((5, 6, 7), 1),
              ((5, 6, 7), 2), ((2, 3, 4, 5), 2), ((300, 8192), 1), ((33, 2048), 1), ((16, 4096), 1), ((2, 65536), 1),
              # few outputs over a long axis: folded in two launches; lanes own 4 (f32) / 8 (f16) columns
              ((4096, 160), 0), ((8192, 512), 0), ((4, 262144), 1), ((4100, 36), 0), ((3, 4096, 20), 1), ((4096, 6, 8), 0),
              ((4098, 66), 0)]


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape,axis", RED_SHAPES, ids=[f"{s}-ax{a}" for s, a in RED_SHAPES])
def test_reductions(gpu, shape, axis, dtype):
    x = data(shape, -1, 1, dtype, 13)
    p = data(shape, 0.98, 1.02, dtype, 14)  # products stay in range
    api = HipAPI(gpu)
    got = hip_values_many([api.tensor(x).sum(axis), api.tensor(x).max(axis), api.tensor(x).min(axis),
                           api.tensor(p).product(axis), (api.tensor(x) * 2.0).exp().sum(axis) + 1.0])
    o = OTensor(x)
    assert np.array_equal(got[1], o.max(axis).to_numpy())  # max / min: bit-exact
    assert np.array_equal(got[2], o.min(axis).to_numpy())
    n = shape[axis]
    if dtype == np.float32:
        # 1e-5 relative to the sum of magnitudes (the condition-free form of "1e-5 relative" for signed data)
        scale = np.abs(x.astype(np.float64)).sum(axis)
        assert np.all(np.abs(got[0].astype(np.float64) - x.astype(np.float64).sum(axis)) <= 1e-5 * scale + 1e-30)
        assert np.allclose(got[3], OTensor(p).product(axis).to_numpy(), rtol=1e-5)
        assert np.allclose(got[4], ((o * 2.0).exp().sum(axis) + 1.0).to_numpy(), rtol=1e-5)
    else:
        # f16 tensors: the fold runs in f32 and is rounded to f16 once, so the result is within the f32 fold's 1e-5 of
        # the sum of magnitudes plus one f16 ulp of the oracle's (f64 fold, rounded once) value
        want = o.sum(axis).to_numpy()
        scale = np.abs(x.astype(np.float64)).sum(axis)
        ulp16 = np.spacing(np.abs(want).astype(np.float16)).astype(np.float64)
        assert np.all(np.abs(got[0].astype(np.float64) - want.astype(np.float64)) <= 1e-5 * scale + ulp16)
        # products: the f32 fold of n factors is within n * 2^-24 of the f64 one (1.6e-2 for the longest axis here), and
        # a long product of factors around 1 may end among the f16 subnormals, whose step is 2^-24
        assert np.allclose(got[3].astype(np.float64), OTensor(p).product(axis).to_numpy().astype(np.float64), rtol=2e-2, atol=1.2e-7)
        # the fused prologue and epilogue on f16: every op rounded to f16 as in the oracle; exp's last bit may differ for
        # an element here and there and the fold is f32, so the sum is within two f16 ulps; sums beyond 65504 are inf in both
        want4 = ((o * 2.0).exp().sum(axis) + 1.0).to_numpy()
        assert got[4].dtype == np.float16 and np.array_equal(np.isinf(got[4]), np.isinf(want4))
        assert np.allclose(got[4].astype(np.float64), want4.astype(np.float64), rtol=2e-3)


def test_reductions_of_views_and_rank0(gpu):
    a = data((10, 24, 36), -1, 1, np.float32, 15)
    api = HipAPI(gpu)

    def progs(t):
        return [t.slice([(1, 9), (3, 20), (4, 36)]).sum(2),       # offset honoured (the reference drops it, src/reduce.rs:351-352)
                t.slice([(1, 9), (3, 20), (5, 30)]).sum(2),       # ragged, unaligned rows
                t.transpose(0, 2).sum(2), t.transpose(1, 2).max(1), t.slice([(0, 10), (0, 24), (7, 8)]).sum(1),
                t.sum(2).sum(1).sum(0), t.slice([(2, 3), (5, 6), (0, 36)]).reshape([36]).max(0)]

    got = hip_values_many(progs(api.tensor(a)))
    want = progs(OTensor(a))
    for i, (g, w) in enumerate(zip(got, want)):
        assert g.shape == w.to_numpy().shape
        assert np.allclose(g, w.to_numpy(), rtol=1e-5, atol=1e-6), f"view reduce {i}"
    assert got[5].shape == () and got[6].shape == ()


def test_reductions_of_views_with_many_outer_dimensions(gpu):
    # a 5-D slice leaves four outer dimensions that do not merge: more than the reduce kernels decode, so the view is
    # copied into a dense buffer first (the reference's reduce takes any rank, src/reduce.rs:83-281)
    a = data((6, 6, 6, 6, 6), -1, 1, np.float32, 16)
    api = HipAPI(gpu)
    cut = [(1, 5)] * 5

    def progs(t):
        v = t.slice(cut)
        return [v.sum(4), v.max(0), (v * 2.0).exp().sum(2), v.transpose(0, 4).sum(1)]

    got = hip_values_many(progs(api.tensor(a)))
    want = progs(OTensor(a))
    for i, (g, w) in enumerate(zip(got, want)):
        assert g.shape == w.to_numpy().shape
        assert np.allclose(g, w.to_numpy(), rtol=1e-5, atol=1e-6), f"5-D view reduce {i}"


def test_long_axis_reductions_of_views(gpu):
    api = HipAPI(gpu)
    a = data((4096, 96), -1, 1, np.float32, 16)
    b = data((4, 6, 4096, 9), -1, 1, np.float32, 17)

    def progs(ta, tb):
        return [ta.transpose(0, 1).sum(1),                              # strided axis, unit-stride outputs: sliced in two launches
                (ta.transpose(0, 1) * 0.5).max(1) + 1.0,
                ta.slice([(0, 4096), (8, 72)]).sum(0),
                tb.slice([(0, 3), (0, 5), (0, 4096), (0, 7)]).sum(2),   # three outer dims that do not merge: one launch
                tb.sum(2), tb.transpose(2, 3).min(3)]

    got = hip_values_many(progs(api.tensor(a), api.tensor(b)))
    want = progs(OTensor(a), OTensor(b))
    for i, (g, w) in enumerate(zip(got, want)):
        assert g.shape == w.to_numpy().shape
        # 1e-5 relative to the sum of magnitudes (about 2000 here)
        assert np.allclose(g, w.to_numpy(), rtol=1e-5, atol=1e-3), f"view reduce {i}"
    assert np.array_equal(got[5], want[5].to_numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_tensors_materialised_together(gpu, wkf, dtype):
    # several roots in one pass: sibling row reductions become one kernel; every value is what the tensor gives alone
    x = data((300, 1024), -1, 1, dtype, 41)
    y = data((7, 5, 96), -1, 1, dtype, 42)
    t, u = wkf.Tensor.new(gpu, x), wkf.Tensor.new(gpu, y)
    roots = [t.max(1), (t.clone() - 1.0).exp().sum(1) + 2.0, t.min(1), (t * t).sum(1).sqrt(),
             u.sum(2), u.max(2) * 0.5, u.sum(1), (t * 2.0).exp()]
    if gpu.is_planner:  # the run that only fills the kernel cache: compile both ways, compute nothing
        wkf.materialize_many(roots)
        hip_values_many(roots)
    together = [s.to_numpy() for s in wkf.as_slice_many(roots)]
    assert any(k.kind == "row" and "reductions=" in k.detail for k in roots[0].kernels())
    alone = [r.to_numpy() for r in roots]
    o, v = OTensor(x), OTensor(y)
    want = [o.max(1), (o - 1.0).exp().sum(1) + 2.0, o.min(1), (o * o).sum(1).sqrt(), v.sum(2), v.max(2) * 0.5, v.sum(1), (o * 2.0).exp()]
    rtol = 1e-5 if dtype == np.float32 else 1e-2
    for i, (g, a, w) in enumerate(zip(together, alone, want)):
        w = w.to_numpy()
        assert g.shape == w.shape and g.dtype == w.dtype, i
        if i in (0, 2, 5):
            assert np.array_equal(g, w), f"root {i}: max / min are exact"
        elif i == 7:
            assert_ulp(g, w, 2, f"root {i}")
        else:
            assert np.allclose(g.astype(np.float64), w.astype(np.float64), rtol=rtol, atol=rtol * 50), f"root {i}"
        assert np.allclose(g.astype(np.float64), a.astype(np.float64), rtol=rtol, atol=rtol * 50), f"root {i} vs alone"


def test_reduce_seeds_and_empty_axes(gpu):
    api = HipAPI(gpu)
    ninf = np.full((3, 40), -np.inf, dtype=np.float32)
    empty = np.zeros((4, 0), dtype=np.float32)
    none = np.zeros((0, 4), dtype=np.float32)
    got = hip_values_many([api.tensor(ninf).max(1), api.tensor(-ninf).min(1), api.tensor(empty).sum(1),
                           api.tensor(empty).product(1), api.tensor(empty).max(1), api.tensor(none).sum(1),
                           api.tensor(none) + 1.0])
    assert np.array_equal(got[0], np.full(3, np.float32(-3.40282e38)))  # the seed, not -inf (src/reduce.rs:640)
    assert np.array_equal(got[1], np.full(3, np.float32(3.40282e38)))
    assert np.array_equal(got[2], np.zeros(4, dtype=np.float32))
    assert np.array_equal(got[3], np.ones(4, dtype=np.float32))
    assert np.array_equal(got[4], np.full(4, np.float32(-3.40282e38)))
    assert got[5].shape == (0,) and got[6].shape == (0, 4)


# ---- copies -----------------------------------------------------------------------------------------------------

def test_resize_reshape_slice_assign_cat_are_bit_exact(gpu):
    a = data((9, 14, 6), -5, 5, np.float32, 16)
    b = data((9, 3, 6), -5, 5, np.float32, 17)
    h = data((5, 8), -5, 5, np.float16, 18)
    api = HipAPI(gpu)

    def progs(T, a, b, h):
        return [a.resize([12, 14, 9]), a.resize([4, 20, 6]), a.reshape([9 * 14, 6]), a.transpose(0, 1).reshape([14 * 9 * 6]),
                a.unsqueeze(1), a.unsqueeze(3), a.slice_assign([(0, 9), (4, 7), (0, 6)], b),
                (a * 2.0).slice_assign([(0, 9), (11, 14), (0, 6)], b + 1.0), T.cat([a, b, a], 1), T.cat([b, b], 2),
                T.cat([a.transpose(0, 2), a.transpose(0, 2) * 2.0], 0), h.resize([7, 9]), T.cat([h, h], 1),
                a.slice([(0, 9), (0, 14), (0, 1)]).resize([9, 14, 3])]

    got = hip_values_many(progs(api.T, api.tensor(a), api.tensor(b), api.tensor(h)))
    want = progs(OTensor, OTensor(a), OTensor(b), OTensor(h))
    for i, (g, w) in enumerate(zip(got, want)):
        assert_ulp(g, w.to_numpy(), 0, f"copy {i}")


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_consumers_of_cat_run_per_piece(gpu, dtype):
    # an element-wise consumer of cat([A, B]) never copies the pieces together: one kernel with two stores
    # when the pieces have one shape, two kernels otherwise; cats below broadcasts / narrows are cut the same way
    api = HipAPI(gpu)
    a, a2 = data((7, 4), -2, 2, dtype, 31), data((7, 4), -2, 2, dtype, 32)
    b = data((7, 6), -2, 2, dtype, 33)
    c8, c10 = data((7, 8), -2, 2, dtype, 34), data((7, 10), -2, 2, dtype, 35)
    t = data((5, 4), -2, 2, dtype, 36)
    x = data((3, 5, 8), -2, 2, dtype, 37)

    def progs(T, a, a2, b, c8, c10, t, x):
        table = T.cat([t, t * 2.0], 1).narrow(0, 1, 3)                     # [3, 8], cut at column 4
        xs = x.narrow(1, 1, 3)                                              # [3, 3, 8]
        return [T.cat([a, a2], 1) * c8 + 1.0,                              # equal pieces
                T.cat([a, b], 1) * c10,                                    # unequal pieces
                (T.cat([a.exp(), -a2], 1) - c8) * T.cat([a2, a], 1),       # two cats at the same seam
                T.cat([xs.narrow(2, 4, 4), xs.narrow(2, 0, 4)], 2) * table.broadcast([3, 3, 8]) + xs,
                T.cat([a, a2], 0) + T.cat([a2, a], 0),                     # cut along dim 0
                (T.cat([a, a2], 1) * c8).sum(1)]                           # a reduce consumer takes the ordinary path

    got = hip_values_many(progs(api.T, *[api.tensor(v) for v in (a, a2, b, c8, c10, t, x)]))
    want = progs(OTensor, *[OTensor(v) for v in (a, a2, b, c8, c10, t, x)])
    for i, (g, w) in enumerate(zip(got[:5], want[:5])):
        assert_ulp(g, w.to_numpy(), 2 if i == 2 else 0, f"cat consumer {i}")
    assert np.allclose(got[5].astype(np.float64), want[5].to_numpy().astype(np.float64), rtol=1e-5 if dtype == np.float32 else 1e-2,
                       atol=1e-5 if dtype == np.float32 else 2e-2)


def test_slice_assign_does_not_change_a_tensor_the_caller_holds(gpu, wkf):
    base = np.zeros((4, 4), dtype=np.float32)
    leaf = wkf.Tensor.new(gpu, base)
    patched = leaf.slice_assign([(1, 3), (1, 3)], wkf.Tensor.new(gpu, np.ones((2, 2), dtype=np.float32)))
    got = hip_values(patched)
    assert got.sum() == 4.0
    assert np.array_equal(leaf.to_numpy(), base)


# ---- composites ------------------------------------------------------------------------------------------------------

def rope_tables(seq, dim, theta=10000.0):
    inv = theta ** (-np.arange(0, dim, 2, dtype=np.float64) / dim)
    ang = np.arange(seq, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


@pytest.mark.parametrize("mode", [1, 0], ids=["tree", "reference-rules"])
def test_composites_small(gpu, mode):
    x = data((37, 96), -2, 2, np.float32, 19)
    w = data((96,), 0.5, 1.5, np.float32, 20)
    q = data((3, 17, 32), -2, 2, np.float32, 21)
    sq = data((48, 48), -2, 2, np.float32, 22)
    cos, sin = rope_tables(20, 32)
    api = HipAPI(gpu)

    def progs(x, w, q, sq, cos, sin):
        w48 = w.slice([(0, 48)])
        return [x.silu(), x.layer_norm(w, 1e-5), sq.layer_norm(w48, 1e-5), q.rope(cos, sin), x.softmax_last_dim(),
                q.softmax_last_dim(), x.slice([(0, 1), (0, 96)]).reshape([96]).softmax(),
                x.cast(api.F16 if isinstance(x, api.T) else np.float16).layer_norm(
                    w.cast(api.F16 if isinstance(x, api.T) else np.float16), 1e-5)]

    gpu.set_fusion(mode)
    try:
        got = hip_values_many(progs(*[api.tensor(v) for v in (x, w, q, sq, cos, sin)]))
    finally:
        gpu.set_fusion(1)
    want = [t.to_numpy() for t in progs(*[OTensor(v) for v in (x, w, q, sq, cos, sin)])]
    assert_ulp(got[0], want[0], 0, "silu")  # exp is interior: bit-exact
    for i in (1, 2, 4, 5, 6):
        assert np.allclose(got[i], want[i], rtol=1e-5, atol=1e-7), f"composite {i}"  # reduction class: 1e-5
    assert_ulp(got[3], want[3], 0, "rope")  # mul / add / neg / copies only: bit-exact
    assert np.allclose(got[7].astype(np.float32), want[7].astype(np.float32), rtol=2e-3, atol=2e-3), "f16 rms norm"
    assert np.allclose(got[4].sum(-1), 1.0, atol=1e-5)


@pytest.mark.parametrize("seed", range(24))
def test_composites_on_random_shapes(gpu, seed):
    # row kernels pick lanes per row and vectors per lane from the shape: odd, prime, tiny and long rows, 1-3 leading dims
    rng = np.random.default_rng(500 + seed)
    n = int(rng.choice([1, 2, 3, 7, 8, 30, 64, 100, 128, 255, 384, 1000, 1024, 2040, 4096, 5000, 8192, 12288, 20000]))
    lead = [int(rng.integers(1, 40)) for _ in range(int(rng.integers(1, 4)))]
    while np.prod(lead) * n > (1 << 21):
        lead = lead[:-1] if len(lead) > 1 else [max(1, lead[0] // 2)]
    shape = tuple(lead) + (n,)
    x = data(shape, -3, 3, np.float32, 600 + seed)
    w = data((n,), 0.5, 1.5, np.float32, 700 + seed)
    api = HipAPI(gpu)
    x2 = x.reshape(-1, n)

    def progs(tx, tx2, tw):
        out = [tx.softmax_last_dim(), tx2.layer_norm(tw, 1e-5), tx.silu() * tx, (tx - 1.0).exp().sum(len(shape) - 1),
               tx.max(len(shape) - 1), tx.sum(0)]
        return out

    got = hip_values_many(progs(api.tensor(x), api.tensor(x2), api.tensor(w)))
    want = [t.to_numpy() for t in progs(OTensor(x), OTensor(x2), OTensor(w))]
    assert np.allclose(got[0], want[0], rtol=1e-5, atol=1e-9), f"softmax {shape}"
    assert np.allclose(got[1], want[1], rtol=1e-5, atol=1e-7), f"rms norm {shape}"
    assert_ulp(got[2], want[2], 0, f"silu * x {shape}")  # exp is interior: bit-exact
    assert np.allclose(got[3], want[3], rtol=1e-5), f"sum(exp(x - 1)) {shape}"
    assert np.array_equal(got[4], want[4]), f"max {shape}"
    scale = np.abs(x.astype(np.float64)).sum(0)
    assert np.all(np.abs(got[5].astype(np.float64) - x.astype(np.float64).sum(0)) <= 1e-5 * scale + 1e-30), f"sum(0) {shape}"


RAGGED_ROWS = [(37, 2880, np.float32), (16, 11008, np.float32), (9, 50257, np.float32), (64, 1234, np.float32), (5, 32772, np.float32),
               (3, 65535, np.float32), (2, 65532, np.float32), (40, 1002, np.float32), (7, 77, np.float32), (11, 5, np.float32),
               (33, 2880, np.float16), (8, 11004, np.float16), (6, 50257, np.float16), (50, 1234, np.float16), (2, 131070, np.float16)]


@pytest.mark.parametrize("rows,n,dtype", RAGGED_ROWS, ids=[f"{r}x{n}_{np.dtype(d).name}" for r, n, d in RAGGED_ROWS])
def test_row_kernels_on_rows_that_do_not_split_evenly(gpu, rows, n, dtype):
    # one fused kernel also when the row is not a power-of-two multiple of the vector width: the lanes past the
    # end of the row are masked in their last vector, and odd or unaligned rows take narrower vectors
    x = data((rows, n), -3, 3, dtype, rows * 7 + n)
    w = data((n,), 0.5, 1.5, dtype, n)
    api = HipAPI(gpu)
    tx, tw = api.tensor(x), api.tensor(w)
    ox, ow = OTensor(x), OTensor(w)
    view = [(1, rows), (1, n - 1)]          # rows of the view start one element into the rows of x
    progs = [tx.softmax_last_dim(), tx.slice(view).softmax_last_dim(), tx.slice(view).exp().sum(1)]
    want = [ox.softmax_last_dim().to_numpy(), ox.slice(view).softmax_last_dim().to_numpy(), None]
    if dtype == np.float32:                  # layer_norm is f32 in the reference (src/composite/rms_norm.rs:8-15)
        progs.append(tx.layer_norm(tw, 1e-5))
        want.append(ox.layer_norm(ow, 1e-5).to_numpy())
    got = hip_values_many(progs)
    assert [k.kind for k in progs[0].kernels()] == ["row"], [k.detail for k in progs[0].kernels()]
    rtol = 1e-5 if dtype == np.float32 else 2e-3
    for i in (0, 1, 3):
        if i < len(got) and want[i] is not None:
            assert got[i].shape == want[i].shape
            assert np.allclose(got[i].astype(np.float64), want[i].astype(np.float64), rtol=rtol, atol=1e-7 if dtype == np.float32 else 1e-6), i
    assert np.allclose(got[0].astype(np.float64).sum(1), 1.0, atol=1e-5 if dtype == np.float32 else 2e-2)
    assert np.all(got[0][:, -1] > 0) and np.all(got[1][:, -1] > 0)          # the last element of a row is written
    ref = np.exp(x[1:, 1:n - 1].astype(np.float64))
    if dtype == np.float16:
        ref = ref.astype(np.float16).astype(np.float64)                       # exp is rounded to f16 before the fold
    with np.errstate(over="ignore"):
        total = ref.sum(1).astype(dtype).astype(np.float64)                   # a long f16 row overflows to inf, here as there
    assert np.allclose(got[2].astype(np.float64), total, rtol=1e-5 if dtype == np.float32 else 4e-3)


class row_teams:
    """Row kernels that spread a long row over the registers of several blocks: on (the default) or off for a while."""

    def __init__(self, gpu, on, spin_polls=0):
        self.gpu, self.on, self.spin = gpu, on, spin_polls

    def __enter__(self):
        self.gpu.set_row_teams(self.on, self.spin)

    def __exit__(self, *exc):
        self.gpu.set_row_teams(True, 0)
        return False


LONG_ROWS = [(256, 100003, np.float32), (258, 131076, np.float32), (257, 70000, np.float32), (256, 140002, np.float16),
             (261, 131080, np.float16)]


@pytest.mark.parametrize("teams", [True, False], ids=["teams", "streamed"])
@pytest.mark.parametrize("rows,n,dtype", LONG_ROWS, ids=[f"{r}x{n}_{np.dtype(d).name}" for r, n, d in LONG_ROWS])
def test_rows_longer_than_a_blocks_registers_stay_one_kernel(gpu, rows, n, dtype, teams):
    # Rows beyond 65536 floats do not fit the registers of a block.  They are spread over the registers of a team
    # of blocks that exchange their folds (ONE launch, the row read once); without teams, and with enough rows to
    # occupy the chip, one block per row streams its row once per stage and once more for the result, also in one
    # launch (the reference's reduce takes any length in one kernel, src/reduce.rs:340-350); odd lengths take
    # narrower vectors.
    with row_teams(gpu, teams):
        _long_rows_one_kernel(gpu, rows, n, dtype, "teams of" if teams else "streamed")


def _long_rows_one_kernel(gpu, rows, n, dtype, mark):
    x = data((rows, n), -3, 3, dtype, rows * 11 + n)
    w = data((n,), 0.5, 1.5, dtype, n + 1)
    api = HipAPI(gpu)
    tx, tw = api.tensor(x), api.tensor(w)
    ox, ow = OTensor(x), OTensor(w)
    progs = [tx.softmax_last_dim()]
    want = [ox.softmax_last_dim().to_numpy()]
    if dtype == np.float32:
        progs.append(tx.layer_norm(tw, 1e-5))
        want.append(ox.layer_norm(ow, 1e-5).to_numpy())
    got = hip_values_many(progs)
    for p in progs:
        assert [k.kind for k in p.kernels()] == ["row"] and mark in p.kernels()[0].detail, [k.detail for k in p.kernels()]
    rtol = 1e-5 if dtype == np.float32 else 2e-3
    for i in range(len(got)):
        assert got[i].shape == want[i].shape
        assert np.allclose(got[i].astype(np.float64), want[i].astype(np.float64), rtol=rtol, atol=1e-9 if dtype == np.float32 else 1e-7), i
    assert np.allclose(got[0].astype(np.float64).sum(1), 1.0, atol=1e-5 if dtype == np.float32 else 5e-2)
    assert np.array_equal(np.argmax(got[0], 1), np.argmax(x, 1))
    # both reductions of the rows in one pass (materialize_many): also one streamed kernel, the same values as alone
    if dtype == np.float32:
        pair = [tx.max(1), (tx.clone() - 1.0).exp().sum(1)]
        m, se = hip_values_many(pair)
        assert np.array_equal(m, x.max(1))
        ref = np.exp((x - np.float32(1.0)).astype(np.float64)).astype(np.float32).astype(np.float64).sum(1)
        assert np.allclose(se, ref, rtol=1e-5)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("rows,n", [(5, 100003), (64, 65540), (1, 1 << 20), (100, 70000), (127, 65600), (3, 70001)])
@pytest.mark.parametrize("teams", [True, False], ids=["teams", "split"])
def test_few_long_rows_are_split_into_parts(gpu, rows, n, dtype, teams):
    # with only a few rows a block per row would leave most compute units idle: every row is cut into parts with a
    # block each.  In a team the parts stay in the blocks' registers and the blocks exchange their folds (one
    # launch); without teams every stage becomes one launch that leaves its parts' values to the next (softmax: the
    # online pair of max and sum, then the result = two launches; layer_norm: three).  The reference's reduce takes
    # any length in one kernel (src/reduce.rs:340-350).
    with row_teams(gpu, teams):
        _few_long_rows(gpu, rows, n, dtype, teams)


def _few_long_rows(gpu, rows, n, dtype, teams):
    if dtype == np.float16:
        # as many bytes as the f32 case, so that the rows are too long for a block's registers, but no more
        # than about 390 000 elements: beyond that sum(exp(x - max)) of these inputs overflows f16
        n = min(2 * n, 1 << 18)
    x = data((rows, n), -3, 3, dtype, rows * 13 + n)
    w = data((n,), 0.5, 1.5, dtype, n + 2)
    api = HipAPI(gpu)
    tx, tw = api.tensor(x), api.tensor(w)
    ox, ow = OTensor(x), OTensor(w)
    progs = [tx.softmax_last_dim()]
    want = [ox.softmax_last_dim().to_numpy()]
    launches = [2]
    if dtype == np.float32:
        progs.append(tx.layer_norm(tw, 1e-5))
        want.append(ox.layer_norm(ow, 1e-5).to_numpy())
        launches.append(2)
    got = hip_values_many(progs)
    for i, (p, count) in enumerate(zip(progs, launches)):
        ks = p.kernels()
        # (layer_norm holds two operands per lane, so its teams are twice as large: beyond 256 parts it stays split)
        team = teams and (i == 0 or "teams of" in ks[0].detail)
        assert [k.kind for k in ks] == ["row"] * (1 if team else count), [(k.kind, k.detail) for k in ks]
        assert all(("teams of" if team else "rows split in") in k.detail for k in ks), [k.detail for k in ks]
    rtol = 1e-5 if dtype == np.float32 else 2e-3
    for i in range(len(got)):
        assert got[i].shape == want[i].shape
        assert np.allclose(got[i].astype(np.float64), want[i].astype(np.float64), rtol=rtol, atol=1e-9 if dtype == np.float32 else 1e-7), i
    assert np.allclose(got[0].astype(np.float64).sum(1), 1.0, atol=1e-5 if dtype == np.float32 else 5e-2)
    assert np.array_equal(np.argmax(got[0], 1), np.argmax(x, 1))


@pytest.mark.parametrize("teams", [True, False], ids=["teams", "split"])
def test_split_rows_of_a_view_and_with_stages_that_do_not_pair(gpu, teams):
    with row_teams(gpu, teams):
        _rows_of_a_view_and_stages_that_do_not_pair(gpu, teams)


def test_a_team_that_gives_up_waiting_is_computed_again_without_teams(gpu, wkf):
    # The blocks of a team wait for each other's values a bounded number of polls.  Here part 0 of every row stays
    # silent (a kernel variant of its own, the top bit of the bound) and the bound is tiny, so the lanes that wait
    # for it give up and every block still runs to its end.  The read-back notices, computes the tensor again
    # without teams and hands out that result; the device counts it, and the next computation is a team kernel again.
    x = data((4, 100000), -3, 3, np.float32, 21)
    w = data((100000,), 0.5, 1.5, np.float32, 22)
    api = HipAPI(gpu)
    want = OTensor(x).softmax_last_dim().to_numpy()
    before = gpu.row_team_fallbacks()
    if gpu.is_planner:  # compile every kernel of this test (teams, their silent variants, the passes without teams), then skip
        for spin in (0, (1 << 31) | 64):
            for on in (True, False):
                with row_teams(gpu, on, spin):
                    api.tensor(x).softmax_last_dim().materialize()
                    wkf.materialize_many([api.tensor(x).softmax_last_dim(), api.tensor(x).layer_norm(api.tensor(w), 1e-5)])
        hip_values(api.tensor(x).softmax_last_dim())
    with row_teams(gpu, True, (1 << 31) | 64):
        t = api.tensor(x).softmax_last_dim()
        got = hip_values(t)
        assert gpu.row_team_fallbacks() == before + 1
        assert all("teams of" not in k.detail for k in t.kernels()) and len(t.kernels()) == 2, [k.detail for k in t.kernels()]
        assert np.allclose(got, want, rtol=1e-5, atol=1e-9)
        # two tensors read back together: one second pass for both
        ta, tb = api.tensor(x).softmax_last_dim(), api.tensor(x).layer_norm(api.tensor(w), 1e-5)
        ga, gb = [sl.to_numpy() for sl in wkf.as_slice_many([ta, tb])]
        assert gpu.row_team_fallbacks() == before + 2
        assert np.allclose(ga, want, rtol=1e-5, atol=1e-9)
        assert np.allclose(gb, OTensor(x).layer_norm(OTensor(w), 1e-5).to_numpy(), rtol=1e-5, atol=1e-9)
        # a give-up that nobody reads back (materialize only) does not leak into the next read-back
        api.tensor(x).softmax_last_dim().materialize()
    t = api.tensor(x).softmax_last_dim()
    got = hip_values(t)
    assert gpu.row_team_fallbacks() == before + 2
    assert "teams of" in t.kernels()[0].detail and len(t.kernels()) == 1
    assert np.allclose(got, want, rtol=1e-5, atol=1e-9)


def _rows_of_a_view_and_stages_that_do_not_pair(gpu, teams):
    # the operand is a column block of a wider matrix (row stride != row length)
    big = data((6, 3 * 100000), -2, 2, np.float32, 5)
    api = HipAPI(gpu)
    w = data((100000,), 0.5, 1.5, np.float32, 6)
    t = api.tensor(big).slice([(0, 6), (100000, 200000)]).layer_norm(api.tensor(w), 1e-5)
    got = hip_values(t)
    want = OTensor(big).slice([(0, 6), (100000, 200000)]).layer_norm(OTensor(w), 1e-5).to_numpy()
    mark = "teams of" if teams else "rows split in"
    assert len(t.kernels()) == (1 if teams else 2) and all(mark in k.detail for k in t.kernels()), [k.detail for k in t.kernels()]
    assert np.allclose(got, want, rtol=1e-5, atol=1e-7)
    # softmax of 2x: the maximum is not of the operand itself, so max and sum stay passes of their own (three launches)
    x = data((9, 90000), -3, 3, np.float32, 8)
    t = (api.tensor(x) * 0.5).softmax_last_dim()
    got = hip_values(t)
    want = (OTensor(x) * 0.5).softmax_last_dim().to_numpy()
    ks = t.kernels()
    assert len(ks) == (1 if teams else 3), [k.detail for k in ks]
    assert all(mark in k.detail and "in one pass" not in k.detail and "in one exchange" not in k.detail for k in ks), [k.detail for k in ks]
    assert np.allclose(got, want, rtol=1e-5, atol=1e-9)


def test_few_long_rows_of_stored_reductions_fold_across_the_grid(gpu):
    # reductions that are stored (no result rows) of a few long rows keep the kernels that fold across the whole grid
    x = data((5, 100003), -3, 3, np.float32, 77)
    api = HipAPI(gpu)
    t = api.tensor(x)
    pair = [t.max(1), (t.clone() - 1.0).exp().sum(1)]
    m, se = hip_values_many(pair)
    assert np.array_equal(m, x.max(1))
    ref = np.exp((x - np.float32(1.0)).astype(np.float64)).astype(np.float32).astype(np.float64).sum(1)
    assert np.allclose(se, ref, rtol=1e-5)


# ---- the benchmark configurations at full size ------------------------------------------------------------------------------

def test_config1_fused_unary_chain_full_size(gpu):
    x = seeded(1, 0, (4096, 4096), "uniform")
    got, want = both(gpu, lambda t: ((t * 2.0) + 1.0).sin().exp(), x)
    assert_ulp(got, want, 2, "config 1")  # <= 2 ulp (measured: <= 1)


def test_config2_row_reductions_full_size(gpu):
    x = seeded(2, 0, (8192, 8192), "normal")
    api = HipAPI(gpu)
    t = api.tensor(x)
    m, s = hip_values_many([t.max(1), (t.clone() - 1.0).exp().sum(1)])
    assert np.array_equal(m, x.max(1))  # bit-exact
    want = np.exp((x - np.float32(1.0)).astype(np.float64)).astype(np.float32).astype(np.float64).sum(1)
    assert np.max(np.abs(s - want) / want) < 1e-5  # 1e-5 relative


def test_config3_swiglu_gate_full_size(gpu):
    a = seeded(3, 0, (32, 1024, 4096), "uniform")
    b = seeded(3, 1, (32, 1024, 4096), "uniform")
    bias = seeded(3, 2, (4096,), "normal", std=0.02)
    api = HipAPI(gpu)
    ta, tb, tbias = api.tensor(a), api.tensor(b), api.tensor(bias)
    bias3 = tbias.broadcast([1024, 4096]).broadcast([32, 1024, 4096])
    out = ta.silu() * (tb + bias3)
    got = hip_values(out)
    # the oracle on every one of the 32 slabs, slab by slab:
    obias = OTensor(np.broadcast_to(bias, (1024, 4096)))
    for sl in range(32):
        oa, ob = OTensor(a[sl]), OTensor(b[sl])
        want = (oa.silu() * (ob + obias)).to_numpy()
        assert_ulp(got[sl], want, 2, f"config 3 slab {sl}")  # <= 2 ulp (measured: 0)
    # the reference's own 3-kernel decomposition gives the same bits at full size
    gpu.set_fusion(0)
    try:
        ref_rules = out.to_numpy()
    finally:
        gpu.set_fusion(1)
    assert np.array_equal(got, ref_rules)


def test_config4_llama_composites_full_size(gpu):
    api = HipAPI(gpu)
    x = seeded(4, 0, (2048, 4096), "normal")
    w = seeded(4, 1, (4096,), "normal", mean=1.0, std=0.02)
    q = seeded(4, 2, (32, 2048, 128), "normal")
    cos, sin = rope_tables(2048, 128)
    scores = seeded(4, 3, (32, 2048, 2048), "normal")
    ts = api.tensor(scores)
    got = hip_values_many([api.tensor(x).layer_norm(api.tensor(w), 1e-5), api.tensor(q).rope(api.tensor(cos), api.tensor(sin)),
                           ts.softmax_last_dim()])
    want_norm = OTensor(x).layer_norm(OTensor(w), 1e-5).to_numpy()
    assert np.allclose(got[0], want_norm, rtol=1e-5, atol=1e-7)  # 1e-5 relative
    want_rope = OTensor(q).rope(OTensor(cos), OTensor(sin)).to_numpy()
    assert_ulp(got[1], want_rope, 0, "rope")
    sm = got[2]
    # the oracle on 128 rows of every head (every 16th row, starting at a different row per head): 4096 rows in all
    for h in range(32):
        rows = np.arange(h % 16, 2048, 16)
        want = OTensor(scores[h, rows]).softmax_last_dim().to_numpy()
        assert np.allclose(sm[h, rows], want, rtol=1e-5, atol=1e-10), f"softmax head {h}"
    assert np.allclose(sm.sum(-1, dtype=np.float64), 1.0, atol=1e-5)  # every one of the 65536 rows
    assert np.array_equal(np.argmax(sm, -1), np.argmax(scores, -1))


# ---- mat_mul ---------------------------------------------------------------------------------------------------------------
# Oracle: the textbook product accumulated in float64 (what the reference's own test compares with,
# src/matmul.rs:268-318).  Tolerances: 1e-3 relative for f32, 1e-2 for f16, measured both as
# ||C - C_ref||_F / ||C_ref||_F and as max|C - C_ref| / max|C_ref|.

def gemm_check(got, a, b, tol):
    want = a.astype(np.float64) @ b.astype(np.float64)
    g = got.astype(np.float64)
    assert g.shape == want.shape
    denom_f = np.linalg.norm(want) or 1.0
    denom_m = np.abs(want).max() or 1.0
    assert np.linalg.norm(g - want) / denom_f <= tol, "Frobenius"
    assert np.abs(g - want).max() / denom_m <= tol, "max-abs"
    # ... and element by element on (up to) 64 rows: |error| <= tol * sum_k |a_ik| |b_kj|, the bound that a small element
    # next to large ones cannot hide behind (the norms above are dominated by the large ones)
    m = want.shape[0]
    rows = np.arange(m) if m <= 64 else np.random.default_rng(m * 31 + want.shape[1]).choice(m, 64, replace=False)
    bound = tol * (np.abs(a[rows].astype(np.float64)) @ np.abs(b.astype(np.float64)))
    worst = np.abs(g[rows] - want[rows]) - bound
    assert np.all(worst <= 1e-30), f"element-wise bound exceeded by {worst.max():.3e}"


GEMM_SHAPES = [(1, 1, 1), (2, 2, 1), (3, 5, 7), (17, 33, 65), (64, 64, 64), (100, 200, 50), (255, 257, 63),
               (256, 256, 64), (256, 256, 32), (512, 256, 128), (256, 512, 320), (768, 512, 96), (256, 256, 1000),
               # ragged shapes on the MFMA kernels (edge tiles): rows 16-byte aligned, nothing a multiple of the tile
               (100, 200, 56), (300, 264, 72), (257, 520, 1000), (1000, 40, 328), (16, 1024, 24), (700, 8, 512),
               (513, 776, 200),
               # a handful of rows (decode): the bandwidth kernel, K cut into slices, then a reduce over the slices
               # few tiles over a long K: K is cut into slices across the grid (f32 partial sums + a reduce)
               (300, 264, 2048), (128, 1032, 4096), (512, 512, 8192), (256, 256, 2048), (40, 512, 1096),
               (1, 1024, 512), (5, 2048, 300), (16, 520, 1000), (8, 264, 4096), (2, 96, 8192), (3, 4104, 77),
               # ... and against a narrow B (rows of at most 2 KiB): the lanes of a block share consecutive rows of B
               (1, 128, 2048), (4, 1000, 515), (3, 8, 70000), (1, 64, 1100), (2, 1024, 64),
               # rows of B off the 16-byte grid (N odd): a transposed copy of B keeps a large product on the MFMA kernels
               (300, 1001, 512), (512, 1002, 256), (17, 1003, 4096), (1, 5001, 4096),
               # K off the vector grid: zero-padded copies of A and B keep a large product on the MFMA kernels
               (300, 1000, 515), (512, 512, 1001), (300, 1001, 515),
               # 5 to 32 rows against a row-major B: the MFMA decode kernel (LDS transpose reads), K in slices
               (32, 4096, 512), (17, 264, 1000), (8, 1000, 4096), (31, 72, 2048), (5, 4104, 136), (24, 8, 8200), (32, 1028, 700),
               # 128 x 128 tiles (products that would not fill the chip with 256 x 256 ones): full, ragged, K in slices
               (128, 128, 64), (129, 136, 64), (384, 640, 192), (200, 1000, 520), (511, 136, 2048), (33, 4096, 1024),
               # full tiles that leave a partly filled last round on 256 compute units (272, 300 and 257 tiles): the
               # tiles of that round run as two halves of 128 rows each (f16 and f32)
               (4096, 4352, 512), (2560, 7680, 1024), (256, 65792, 2048),
               # the same with ragged edges (272 and 288 tiles): a last tile row that ends inside its upper half (the lower
               # half tiles do nothing), one that ends inside its lower half, ragged columns, a K that is no multiple of 64
               (3900, 4360, 136), (4000, 4104, 72), (4090, 4352, 200),
               # 1024 full tiles over K = 64 and K = 128: the kernel that keeps a tile's whole K in the LDS
               (8192, 8192, 64), (4096, 16384, 128)]


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-3), (np.float16, 1e-2)], ids=["f32", "f16"])
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES, ids=[f"{m}x{n}x{k}" for m, n, k in GEMM_SHAPES])
def test_mat_mul(gpu, m, n, k, dtype, tol):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k)
    a = rng.standard_normal((m, k)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    api = HipAPI(gpu)
    got = hip_values(api.tensor(a).mat_mul(api.tensor(b)))
    assert got.dtype == dtype
    gemm_check(got, a, b, tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("m,n,k,bt", [(1, 128, 1024, False), (2, 64, 3000, False), (1, 4096, 520, False), (1, 300, 4096, True),
                                      (8, 100, 8192, True), (3, 1000, 264, True), (40, 264, 512, False), (300, 264, 136, True)],
                         ids=lambda v: str(v))
@pytest.mark.parametrize("side", ["a", "b"])
def test_mat_mul_with_an_infinite_operand_has_no_stray_nan(gpu, m, n, k, bt, dtype, side):
    # Kernels pad with zeros past the end of K, of a slice of K or of a tile, and zero times an infinite operand
    # would be NaN: with positive operands and +inf in the last (and the first) position along K of A, or of B, every
    # product is +inf.
    rng = np.random.default_rng(m * 31 + n * 7 + k)
    a = rng.uniform(0.5, 1.0, (m, k)).astype(dtype)
    b = rng.uniform(0.5, 1.0, (n, k) if bt else (k, n)).astype(dtype)
    if side == "a":
        a[:, k - 1] = np.inf
        a[0, 0] = np.inf
    elif bt:
        b[:, k - 1] = np.inf
        b[n - 1, 0] = np.inf
    else:
        b[k - 1, :] = np.inf
        b[0, n - 1] = np.inf
    api = HipAPI(gpu)
    tb = api.tensor(b)
    got = hip_values(api.tensor(a).mat_mul(tb.transpose(0, 1) if bt else tb))
    assert got.shape == (m, n) and np.all(np.isposinf(got)), (np.isnan(got).sum(), np.isfinite(got).sum())


BT_SHAPES = [(256, 512, 128), (300, 264, 2048), (100, 136, 72), (513, 260, 328), (1, 1024, 512), (7, 520, 1000),
             (32, 264, 4096), (2, 4100, 96), (20, 100, 64), (3, 5, 7), (33, 2048, 1024), (300, 1000, 515),
             (4096, 4352, 512),
             # up to 16 rows of f32 against a transposed weight run on the vector ALUs: edge columns, a K that ends inside
             # a step, a slice of K longer than one step
             (12, 520, 1000), (16, 4100, 264), (9, 100, 4100), (8, 33, 8192), (1, 11008, 4096),
             # f16: up to 4 rows; rows of A that fit the LDS whole take one launch with 2, 4 or 8 rows of W a wave
             (3, 1000, 520), (4, 4100, 136), (2, 100, 4104), (1, 33, 8200), (4, 20000, 64), (2, 6000, 12296),
             # 5 to 16 rows against at least 256 groups of 32 rows of W: the eight waves of a block share K (edge rows
             # of W, a K that leaves some waves without work, a K that ends inside a step)
             (8, 8200, 1024), (16, 9000, 520), (5, 8192, 4104), (12, 10000, 8192)]


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-3), (np.float16, 1e-2)], ids=["f32", "f16"])
@pytest.mark.parametrize("m,n,k", BT_SHAPES, ids=[f"{m}x{n}x{k}" for m, n, k in BT_SHAPES])
def test_mat_mul_with_a_transposed_weight(gpu, m, n, k, dtype, tol):
    # x * W^T with W [N, K] dense (the linear-layer form): read as it lies by the MFMA kernels, streamed once at
    # decode sizes (M <= 32), copied first only when its rows are unaligned or the problem is tiny
    rng = np.random.default_rng(m * 7919 + n * 104729 + k)
    a = rng.standard_normal((m, k)).astype(dtype)
    w = rng.standard_normal((n, k)).astype(dtype)
    api = HipAPI(gpu)
    got = hip_values(api.tensor(a).mat_mul(api.tensor(w).transpose(0, 1)))
    assert got.dtype == dtype
    gemm_check(got, a, np.ascontiguousarray(w.T), tol)


def test_a_few_rows_against_a_very_wide_weight_keep_their_slice_of_a_small(gpu):
    # [16 x K] x W[65536 x K]^T in f32 (a vocabulary projection): the columns alone fill the chip, so K is cut only
    # as far as the block's slice of A demands, and that slice is static LDS, [16][chunk_max] floats: it is bounded
    # by 64 KiB (chunk_max 1024 here), not only by 2048 elements a row.
    m, n, k = 16, 65536, 1536
    rng = np.random.default_rng(99)
    a = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((n, k)).astype(np.float32)
    api = HipAPI(gpu)
    t = api.tensor(a).mat_mul(api.tensor(w).transpose(0, 1))
    got = hip_values(t)
    first = t.kernels()[0]
    assert "|skinny_bt|valu|m16|c1024" in first.signature and "slices=2" in first.detail, (first.signature, first.detail)
    gemm_check(got, a, np.ascontiguousarray(w.T), 1e-3)


FLEX_CONFIGS = ["2,3,4,1", "2,3,4,3", "2,3,3,2", "2,2,2,1", "2,2,2,4", "1,3,4,1", "1,3,4,2", "1,4,4,1", "1,2,5,2", "1,2,5,4", "2,4,3,1", "2,4,2,2"]


@pytest.mark.parametrize("config", FLEX_CONFIGS)
def test_every_tile_of_the_flexible_f16_kernel(wkf, config, monkeypatch):
    # The f16 kernel that loads its operands straight into the LDS takes tiles of 64 NI x 64 NJ, a ring of LDS stages and K
    # slices chosen per shape.  Here every configuration the planner may choose (and two more) is forced on a device of its
    # own (the override is read when a device is created): ragged M and N, a single K step, fewer steps than stages, B
    # as it lies and transposed, and a batch; all against the f64 product.
    monkeypatch.setenv("WKF_GEMM_FLEX", config)
    planner_run = os.environ.get("WKF_TEST_PLAN_ONLY") == "1"
    dev = wkf.Device.planner() if planner_run else wkf.Device.new(0)
    try:
        slices = int(config.split(",")[3])
        rng = np.random.default_rng(sum(int(v) * 7 ** i for i, v in enumerate(config.split(","))))
        cases = [(300, 1000, 512, False, ()), (77, 200, 64, False, ()), (512, 776, 1024, True, ()), (129, 136, 128, False, ()),
                 (64, 192, 2048, True, ()), (200, 264, 256, False, (3,))]
        for m, n, k, bt, lead in cases:
            a = rng.standard_normal(lead + (m, k)).astype(np.float16)
            b = rng.standard_normal(lead + ((n, k) if bt else (k, n))).astype(np.float16)
            ta, tb = wkf.Tensor.new(dev, a), wkf.Tensor.new(dev, b)
            r = len(lead) + 2
            t = ta.mat_mul(tb.transpose(r - 2, r - 1) if bt else tb)
            if planner_run:
                t.materialize()
                continue
            got = t.to_numpy()
            first = t.kernels()[0]
            assert "operands loaded straight into the LDS" in first.detail and f"{64 * int(config[0])}x{64 * int(config[2])} tiles" in first.detail, first.detail
            if slices > 1 and not lead and k // slices >= 64:
                assert "slices=" in first.detail and len(t.kernels()) == 2
            bm = np.swapaxes(b, -1, -2) if bt else b
            if lead:
                for z in range(lead[0]):
                    gemm_check(got[z], a[z], np.ascontiguousarray(bm[z]), 1e-2)
            else:
                gemm_check(got, a, np.ascontiguousarray(bm), 1e-2)
    finally:
        dev.close()
    if planner_run:
        pytest.skip("plan-only device: kernels compiled, nothing computed")


# (batch dimensions, m, n, k, B given as a transposed view): attention-like products, ragged ones, tiny ones
BATCH_SHAPES = [((4,), 256, 256, 64, False), ((3,), 100, 72, 40, False), ((2, 3), 17, 33, 65, False), ((5,), 3, 5, 7, False),
                ((8,), 512, 512, 128, True), ((8,), 512, 128, 512, False), ((2, 2), 300, 264, 72, True), ((6,), 1, 384, 128, True),
                ((3,), 20, 100, 64, True), ((1,), 256, 512, 128, False), ((70,), 64, 64, 32, False),
                # decode-sized products per matrix: the bandwidth kernels, K in slices, one fold for the batch
                ((32,), 1, 2048, 128, True), ((32,), 1, 128, 2048, False), ((4,), 8, 520, 1000, False), ((3, 2), 20, 264, 4096, True),
                ((3,), 300, 1001, 128, False),
                # a batch of one with a long K: few tiles, so K is cut into slices (256 x 256 and 128 x 128 tiles); the
                # leading dimensions of size 1 must survive the fold of the slices
                ((1,), 256, 256, 4096, False), ((1, 1), 256, 512, 2048, True), ((1,), 128, 384, 4096, False),
                ((1, 1), 100, 136, 1024, False), ((1,), 100, 102, 2048, True), ((1,), 120, 100, 1024, True),
                # one column of 128-wide tiles over a long K (attention probabilities against values): every workgroup
                # starts its walk over K at a different tile and wraps around; K with a partial last tile, B^T, edge columns
                ((2,), 2048, 128, 2048, False), ((4,), 640, 100, 1096, False), ((3,), 384, 128, 2048, True), ((2, 2), 130, 72, 520, False)]
# many full tiles over K = 64 or 128: one workgroup per compute unit walks the tiles of the whole batch
BATCH_SHAPES += [((3,), 4, 72, 300, False), ((64,), 1, 64, 1024, False)]  # decode rows against a narrow B
BATCH_SHAPES += [((5,), 2, 300, 264, True), ((40,), 1, 1000, 72, True), ((2, 3), 4, 260, 4096, True)]  # decode rows on the vector ALUs
BATCH_SHAPES += [((16,), 2048, 2048, 128, True), ((4,), 4096, 4096, 64, False), ((2, 2), 4096, 4096, 128, False), ((13,), 2304, 2304, 64, True), ((1030,), 256, 256, 128, False),
                 ((16,), 2048, 2048, 192, True), ((17,), 2048, 2048, 256, False), ((5,), 4096, 3840, 192, False)]
WHOLE_K = {((4,), 4096, 4096, 64, False), ((13,), 2304, 2304, 64, True)}
# many full tiles over K = 128 to 256: a tile's stores leave under the next tile's MFMAs (a tile count that is no multiple
# of 8 or of the compute units, every K, B as it lies and transposed)
STREAMED = {((16,), 2048, 2048, 128, True), ((2, 2), 4096, 4096, 128, False), ((1030,), 256, 256, 128, False), ((16,), 2048, 2048, 192, True),
            ((17,), 2048, 2048, 256, False), ((5,), 4096, 3840, 192, False)}
ROTATED = {((2,), 2048, 128, 2048, False), ((4,), 640, 100, 1096, False), ((3,), 384, 128, 2048, True), ((2, 2), 130, 72, 520, False),
           ((8,), 512, 128, 512, False)}


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-3), (np.float16, 1e-2)], ids=["f32", "f16"])
@pytest.mark.parametrize("lead,m,n,k,bt", BATCH_SHAPES, ids=[f"{'x'.join(map(str, l))}_{m}x{n}x{k}{'_bt' if t else ''}" for l, m, n, k, t in BATCH_SHAPES])
def test_batched_mat_mul(gpu, lead, m, n, k, bt, dtype, tol):
    # [..., M, K] x [..., K, N]: every matrix of the batch against its own float64 product; one launch for the batch
    rng = np.random.default_rng(sum(lead) * 31 + m * 1000003 + n * 1009 + k)
    a = rng.standard_normal(lead + (m, k)).astype(dtype)
    b = rng.standard_normal(lead + ((n, k) if bt else (k, n))).astype(dtype)
    api = HipAPI(gpu)
    tb = api.tensor(b)
    R = len(lead) + 2
    prod = api.tensor(a).mat_mul(tb.transpose(R - 2, R - 1) if bt else tb)
    dense_b = np.swapaxes(b, -1, -2) if bt else b
    first = tuple(0 for _ in lead)
    one = api.tensor(a[first]).mat_mul(api.tensor(np.ascontiguousarray(dense_b[first])))
    # the product as an operand of a following pair-wise op: its recorded shape and its buffer's must agree
    chained = prod + prod
    got, alone, twice = hip_values_many([prod, one, chained])
    assert got.dtype == dtype and got.shape == lead + (m, n)
    assert twice.shape == lead + (m, n) and np.array_equal(twice, got + got)
    for idx in np.ndindex(*lead):
        gemm_check(got[idx], a[idx], np.ascontiguousarray(dense_b[idx]), tol)
    assert len([kk for kk in prod.kernels() if kk.kind == "gemm"]) == 1
    # and the same numbers as one product at a time (bit for bit when both take the same kernel with the same K slices)
    gemm_of = lambda t: [kk for kk in t.kernels() if kk.kind == "gemm"][0].detail  # noqa: E731
    if (lead, m, n, k, bt) in WHOLE_K and dtype == np.float16:
        assert "whole K in LDS" in gemm_of(prod), gemm_of(prod)
    if (lead, m, n, k, bt) in STREAMED and dtype == np.float16:
        assert "stores under the next tile" in gemm_of(prod), gemm_of(prod)
    if (lead, m, n, k, bt) in ROTATED and dtype == np.float16:
        assert "K start rotated" in gemm_of(prod), gemm_of(prod)
    if not bt and "skinny" not in prod.kernels()[0].detail and "slices" not in gemm_of(one):
        assert np.array_equal(alone, got[first])
    else:
        gemm_check(alone, a[first], np.ascontiguousarray(dense_b[first]), tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_mat_mul_identities_and_views(gpu, dtype):
    rng = np.random.default_rng(23)
    a = rng.standard_normal((256, 512)).astype(dtype)
    eye = np.eye(512, dtype=dtype)
    small = rng.integers(-3, 4, (256, 64)).astype(dtype)
    small_b = rng.integers(-3, 4, (64, 256)).astype(dtype)
    api = HipAPI(gpu)
    ta = api.tensor(a)
    got = hip_values_many([ta.mat_mul(api.tensor(eye)),                         # A I = A, exactly
                           api.tensor(small).mat_mul(api.tensor(small_b)),     # small integers: exact in f16 and f32
                           ta.transpose(0, 1).mat_mul(ta),                     # a strided operand is made dense first
                           (ta * 2.0).mat_mul(api.tensor(eye) + 0.0) - 1.0,    # element-wise work around it does not fuse into it
                           api.tensor(np.ones((4, 300), dtype=dtype)).mat_mul(api.tensor(np.ones((300, 5), dtype=dtype)))])
    assert np.array_equal(got[0], a)
    assert np.array_equal(got[1].astype(np.float64), small.astype(np.float64) @ small_b.astype(np.float64))
    gemm_check(got[2], a.T, a, 1e-3 if dtype == np.float32 else 1e-2)
    assert np.array_equal(got[3], ((OTensor(a) * 2.0) - 1.0).to_numpy())
    assert np.array_equal(got[4], np.full((4, 5), 300.0, dtype=dtype))


@pytest.mark.parametrize("name,m,n,k,dtype,tol", [("f32-4096", 4096, 4096, 4096, np.float32, 1e-3),
                                                  ("f16-4096", 4096, 4096, 4096, np.float16, 1e-2),
                                                  ("f16-llama-mlp", 2048, 11008, 4096, np.float16, 1e-2)],
                         ids=["f32-4096", "f16-4096", "f16-llama-mlp"])
def test_config5_gemm_full_size(gpu, name, m, n, k, dtype, tol):
    a = seeded(5, 0, (m, k), "normal", dtype=dtype, std=0.02)
    b = seeded(5, 1, (k, n), "normal", dtype=dtype, std=0.02)
    api = HipAPI(gpu)
    prod = api.tensor(a).mat_mul(api.tensor(b))
    got = hip_values(prod)
    gemm_check(got, a, b, tol)
    if name == "f16-llama-mlp":  # 344 tiles on 256 compute units
        assert "last round: 88 tiles as 176 halves" in prod.kernels()[0].detail, prod.kernels()[0].detail


# ---- maps over f16 as table lookups ------------------------------------------------------------------------------------

def test_a_costly_map_over_one_f16_tensor_runs_as_a_table_lookup(gpu):
    # An element-wise kernel over ONE dense f16 tensor with an f16 result is a function of 16 bits.  From a size on (the
    # device setting; lowered here) a costly chain is computed once for all 65536 bit patterns by the ordinary kernel
    # and the data goes through a lookup in the LDS.  The input holds every bit pattern (NaNs, infinities, denormals,
    # both zeros) and a ragged tail; the result must be the ordinary kernel's, bit for bit, and the oracle's.
    n = 3 * 65536 + 5
    bits = np.concatenate([np.arange(65536, dtype=np.uint16), np.random.default_rng(3).integers(0, 65536, n - 65536).astype(np.uint16)])
    x = bits.view(np.float16)
    api = HipAPI(gpu)

    def chains(t):
        return [((t * 2.0) + 1.0).sin().exp(), t.silu(), (t.tanh() * 0.5 + 0.5).sqrt(), (t * t + 1.0).log().cos() / 3.0]

    if gpu.is_planner:  # compile every kernel of this test, with and without tables, then skip
        for least in (1 << 17, 0):
            gpu.set_map_table(least)
            try:
                tx = api.tensor(x)
                for p in chains(tx) + [((tx * 3.0) + 1.0).sin().exp(), ((tx.narrow(0, 8, 2 * 65536) * 2.0) + 1.0).sin().exp(),
                                       ((tx.narrow(0, 3, 2 * 65536) * 2.0) + 1.0).sin().exp(), tx * 2.0 + 1.0, tx.sin().exp() + api.tensor(x)]:
                    p.materialize()
            finally:
                gpu.set_map_table(1 << 25)
        hip_values(api.tensor(x) * 2.0)
    gpu.set_map_table(1 << 17)
    try:
        tx = api.tensor(x)
        progs = chains(tx)
        looked_up = [hip_values(p) for p in progs]
        for p in progs:
            details = [k.detail for k in p.kernels()]
            assert "table lookup" in details[-1], details
        # a second tensor, other constants: its own table; the same program again: the cached one (one launch)
        again = ((tx * 2.0) + 1.0).sin().exp()
        assert np.array_equal(hip_values(again).view(np.uint16), looked_up[0].view(np.uint16))
        assert len(again.kernels()) == 1 and "table lookup" in again.kernels()[0].detail
        other = ((tx * 3.0) + 1.0).sin().exp()
        got_other = hip_values(other)
        assert len(other.kernels()) == 2
        # views: a dense slice that starts 16-byte aligned qualifies, a strided one and one off the grid do not
        part = api.tensor(x).narrow(0, 8, 2 * 65536)
        assert "table lookup" in [k.detail for k in ((part * 2.0) + 1.0).sin().exp().materialize().kernels()][-1]
        # (one off the 16-byte grid goes through the general map kernel, which then looks the whole chain up as well)
        off = api.tensor(x).narrow(0, 3, 2 * 65536)
        off_chain = ((off * 2.0) + 1.0).sin().exp()
        assert np.array_equal(hip_values(off_chain).view(np.uint16), looked_up[0][3:3 + 2 * 65536].view(np.uint16))
        assert "vec=1" in off_chain.kernels()[-1].detail and "table lookup" in off_chain.kernels()[-1].detail
        assert np.array_equal(hip_values(((part * 2.0) + 1.0).sin().exp()).view(np.uint16), looked_up[0][8:8 + 2 * 65536].view(np.uint16))
        # a cheap chain stays an ordinary kernel
        assert "table lookup" not in (tx * 2.0 + 1.0).materialize().kernels()[0].detail
    finally:
        gpu.set_map_table(1 << 25)
    gpu.set_map_table(0)
    try:
        plain = [hip_values(p) for p in chains(api.tensor(x))]
        plain_other = hip_values(((api.tensor(x) * 3.0) + 1.0).sin().exp())
    finally:
        gpu.set_map_table(1 << 25)
    for a, b in zip(looked_up, plain):
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    assert np.array_equal(got_other.view(np.uint16), plain_other.view(np.uint16))
    with np.errstate(all="ignore"):
        o = OTensor(x)
        want = ((o * 2.0) + 1.0).sin().exp().to_numpy()
    finite = np.isfinite(want)
    assert np.array_equal(np.isnan(looked_up[0]), np.isnan(want))
    assert np.array_equal(looked_up[0][finite].view(np.uint16), want[finite].view(np.uint16))


def test_a_costly_value_of_one_f16_operand_inside_a_larger_map_is_looked_up(gpu):
    # silu(a) inside silu(a) * (b + bias), tanh(a) inside a * tanh(a) + b: a value that depends on ONE f16 operand is a
    # function of 16 bits whatever else the kernel does.  The planner cuts the costliest such value out of the fused
    # program, fills a table with it (the cut program run over all 65536 bit patterns, its last op evaluated as the
    # interior op it was) and the kernel, 1024 lanes per compute unit around the table in the LDS, looks it up.  Results
    # must equal the ordinary kernel's bit for bit and the oracle's.
    rows, cols = 260, 1032   # ragged: the last chunk of 1024 work items is partly filled
    a = data((rows, cols), -6, 6, np.float16, 501)
    a.reshape(-1)[:65536] = np.arange(65536, dtype=np.uint16).view(np.float16)   # every bit pattern, NaNs included
    b = data((rows, cols), -2, 2, np.float16, 502)
    bias = data((cols,), -1, 1, np.float16, 503)
    c32 = data((rows, cols), -2, 2, np.float32, 504)
    wide = data((rows, 2 * cols), -2, 2, np.float16, 505)
    api = HipAPI(gpu)

    def graphs(T, ta, tb, tbias, tc, twide):
        strided = twide.slice([(0, rows), (8, 8 + cols)])
        return {
            "silu(a)*(b+bias)": ta.silu() * (tb + tbias.broadcast([rows, cols])),
            "tanh(a)*b": ta.tanh() * tb,
            "a*tanh(a)+b": ta * ta.tanh() + tb,
            "sin(a)*b+cos(a)": ta.sin() * tb + ta.cos(),                      # two values of one operand: one is looked up
            "exp(a/2)+strided": (ta / 2.0).exp() + strided,                   # a strided second operand
            "tanh(a) as f32 * c": ta.tanh().cast(0) * tc,            # the value is f16, the kernel's result f32
            "log(1+a*a)-b*3": ((ta * ta) + 1.0).log() - (tb * 3.0),           # a pair-wise op inside the value
        }

    def run(least):
        gpu.set_map_table(least)
        try:
            g = graphs(api, api.tensor(a), api.tensor(b), api.tensor(bias), api.tensor(c32), api.tensor(wide))
            vals = {k: hip_values(t) for k, t in g.items()}
            return vals, {k: [kk.detail for kk in t.kernels()] for k, t in g.items()}
        finally:
            gpu.set_map_table(1 << 25)

    if gpu.is_planner:  # compile every kernel of this test, with and without tables, then skip
        for least in (1 << 17, 0):
            gpu.set_map_table(least)
            try:
                for t in graphs(api, api.tensor(a), api.tensor(b), api.tensor(bias), api.tensor(c32), api.tensor(wide)).values():
                    t.materialize()
            finally:
                gpu.set_map_table(1 << 25)
    got, details = run(1 << 17)
    for k, d in details.items():
        assert "table lookup" in d[-1], (k, d)
    want, plain = run(0)
    for k, d in plain.items():
        assert "table lookup" not in d[-1], (k, d)
    for k in got:
        assert got[k].dtype == want[k].dtype and np.array_equal(got[k].view(np.uint16 if got[k].dtype == np.float16 else np.uint32),
                                                                  want[k].view(np.uint16 if got[k].dtype == np.float16 else np.uint32)), k
    with np.errstate(all="ignore"):
        oa, ob, obias = OTensor(a), OTensor(b), OTensor(bias)
        ref = (oa.silu() * (ob + obias.broadcast([rows, cols]))).to_numpy()
        ref2 = (oa * oa.tanh() + ob).to_numpy()
    for r, g in ((ref, got["silu(a)*(b+bias)"]), (ref2, got["a*tanh(a)+b"])):
        finite = np.isfinite(r)
        assert np.array_equal(np.isnan(g), np.isnan(r))
        assert np.array_equal(g[finite].view(np.uint16), r[finite].view(np.uint16))


def test_random_f16_maps_agree_with_and_without_tables(gpu):
    # Random fused maps over three f16 operands (unary, literal, pair-wise ops, casts to f32 and back, values used more
    # than once): whatever value the planner cuts out into a table, the kernel must give the bits of the ordinary kernel.
    rows, cols = 300, 520
    rng0 = np.random.default_rng(900)
    hosts = [data((rows, cols), -4, 4, np.float16, 901 + i) for i in range(3)]
    hosts[0].reshape(-1)[:65536] = np.arange(65536, dtype=np.uint16).view(np.float16)
    hosts[1].reshape(-1)[:65536] = rng0.permutation(65536).astype(np.uint16).view(np.float16)
    unary = ["exp", "sin", "cos", "tanh", "abs", "sqrt", "log", "atan", "sinh", "sqr"]
    api = HipAPI(gpu)

    def build(seed, leaves):
        rng = np.random.default_rng(seed)
        vals = list(leaves)           # (tensor, is_f16)
        for _ in range(int(rng.integers(4, 10))):
            kind = rng.integers(0, 10)
            t, h = vals[int(rng.integers(0, len(vals)))]
            if kind < 4:
                nv = (getattr(t, unary[int(rng.integers(0, len(unary)))])(), h)
            elif kind < 6:
                c = float(np.float16(rng.uniform(-2, 2)))
                nv = ([t + c, t * c, c - t, t / (abs(c) + 0.5)][int(rng.integers(0, 4))], h)
            elif kind < 9:
                same = [v for v in vals if v[1] == h]
                u = same[int(rng.integers(0, len(same)))][0]
                nv = ([t + u, t - u, t * u, t / u][int(rng.integers(0, 4))], h)
            else:
                nv = (t.cast(0 if h else 1), not h)
            vals.append(nv)
        # the result joins the last value with one of each other operand's, so that several operands come in
        out, h = vals[-1]
        for leaf, lh in leaves[1:]:
            out = out + (leaf if h == lh else leaf.cast(1 if h else 0))
        return out

    def run(least, seeds):
        gpu.set_map_table(least)
        try:
            outs, tabled = [], 0
            for seed in seeds:
                t = build(seed, [(api.tensor(hh), True) for hh in hosts])
                if gpu.is_planner:
                    t.materialize()
                    continue
                outs.append(hip_values(t))
                tabled += any("table lookup" in k.detail for k in t.kernels())
            return outs, tabled
        finally:
            gpu.set_map_table(1 << 25)

    seeds = range(40)
    if gpu.is_planner:
        run(1 << 17, seeds)
        run(0, seeds)
        hip_values(api.tensor(hosts[0]) * 2.0)
    got, tabled = run(1 << 17, seeds)
    want, none = run(0, seeds)
    for seed, (g, w_) in enumerate(zip(got, want)):
        bits = np.uint16 if g.dtype == np.float16 else np.uint32
        assert g.dtype == w_.dtype and np.array_equal(g.view(bits), w_.view(bits)), seed
    assert none == 0 and tabled >= 12, (tabled, none)   # about half of these graphs hold a value worth a table


def test_a_table_lookup_in_place_and_on_a_permuted_tensor(gpu):
    # the operand may be overwritten (an intermediate nobody else holds: a product here), and input and output may share
    # any permutation of dimensions as long as both are dense in it (the transposed product, updated in place)
    a = data((512, 64), -1, 1, np.float16, 77)
    b = data((64, 520), -1, 1, np.float16, 78)
    api = HipAPI(gpu)

    def run():
        ta, tb = api.tensor(a), api.tensor(b)
        straight = (ta.mat_mul(tb) * 2.0 + 1.0).sin().exp()
        turned = (ta.mat_mul(tb).transpose(0, 1) * 2.0 + 1.0).sin().exp()
        vals = hip_values_many([straight, turned])
        return vals, [k.detail for k in straight.kernels()], [k.detail for k in turned.kernels()]

    if gpu.is_planner:
        gpu.set_map_table(0)
        try:
            ta, tb = api.tensor(a), api.tensor(b)
            (ta.mat_mul(tb) * 2.0 + 1.0).sin().exp().materialize()
            (ta.mat_mul(tb).transpose(0, 1) * 2.0 + 1.0).sin().exp().materialize()
        finally:
            gpu.set_map_table(1 << 25)
    gpu.set_map_table(1 << 17)
    try:
        got, d0, d1 = run()
    finally:
        gpu.set_map_table(1 << 25)
    assert "table lookup" in d0[-1] and "in_place" in d0[-1], d0
    assert "table lookup" in d1[-1] and "in_place" in d1[-1], d1
    gpu.set_map_table(0)
    try:
        want, e0, _ = run()
    finally:
        gpu.set_map_table(1 << 25)
    assert "table lookup" not in e0[-1]
    assert got[1].shape == (520, 512)
    for g, w in zip(got, want):
        assert np.array_equal(g.view(np.uint16), w.view(np.uint16))


# ---- the reference's text where it differs in value from what it means ---------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_layer_norm_as_the_reference_text_reads_on_square_inputs(gpu, dtype):
    # src/composite/rms_norm.rs:13-14 broadcasts the weight with Tensor::broadcast (src/map_layout.rs:69-77): on a
    # square input the weight is indexed by row.  Off by default (RMSNorm as meant); with the device's
    # reference-compat flag the library follows the text, in both fusion modes, and non-square inputs do not change.
    sq = data((96, 96), -2, 2, dtype, 31)
    rect = data((64, 96), -2, 2, dtype, 32)
    w = data((96,), 0.5, 1.5, dtype, 33)
    api = HipAPI(gpu)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == np.float32 else dict(rtol=2e-3, atol=1e-3)
    meant = hip_values(api.tensor(sq).layer_norm(api.tensor(w), 1e-5))
    assert np.allclose(meant, OTensor(sq).layer_norm(OTensor(w), 1e-5).to_numpy(), **tol)
    want_sq = OTensor(sq).layer_norm_as_written(OTensor(w), 1e-5).to_numpy()
    want_rect = OTensor(rect).layer_norm(OTensor(w), 1e-5).to_numpy()
    assert not np.allclose(want_sq, meant, **tol)  # the two readings differ on this input
    gpu.set_reference_compat(True)
    try:
        for mode in (1, 0):
            gpu.set_fusion(mode)
            got_sq, got_rect = hip_values_many([api.tensor(sq).layer_norm(api.tensor(w), 1e-5), api.tensor(rect).layer_norm(api.tensor(w), 1e-5)])
            assert np.allclose(got_sq, want_sq, **tol), mode
            assert np.allclose(got_rect, want_rect, **tol), mode
    finally:
        gpu.set_fusion(1)
        gpu.set_reference_compat(False)
    again = hip_values(api.tensor(sq).layer_norm(api.tensor(w), 1e-5))
    assert np.array_equal(again, meant)
