"""Random lazy graphs against the oracle.  The inputs hold small integers (and the constants are small integers
or halves), so every op the generator uses -- + - * by tensors and literals, division by 2, abs, neg, sqr, casts,
views, copies, cat, slice_assign, max / min / sum / product reductions, mat_mul -- is EXACT in f32 and in f16
whatever the order of evaluation: the HIP path must reproduce the oracle bit for bit, in both fusion modes, however
the planner cuts the graph into kernels (fused maps, row kernels, cat-split, tiled maps, two-launch reduces, ...).
The programs are drawn from fixed seeds; a failure prints the program so that it can be replayed."""
import numpy as np
import pytest

from helpers import HipAPI, hip_values
from oracle.oracle import OTensor

pytestmark = pytest.mark.gpu

DIMS = [1, 2, 3, 4, 5, 8, 12, 16, 33, 64, 64, 130, 512, 4096]


class Gen:
    """Builds one random program as a list of steps; `run(api_tensor_factory, T)` replays it on either API."""

    def __init__(self, seed, dtype):
        self.rng = np.random.default_rng(seed)
        self.dtype = dtype
        self.steps = []      # (description, fn(values) -> value)
        self.shapes = []     # shape of every value
        self.bounds = []     # bound on |value|
        self.fbits = []      # values are multiples of 2^-fbits
        self.limit = 2000.0 if dtype == np.float16 else 4.0e6   # |value| * 2^fbits stays below this: exactly representable
        self.leaves = []

    # -- values ---------------------------------------------------------------------------------------
    def leaf(self, shape):
        data = self.rng.integers(-3, 4, size=shape).astype(self.dtype)
        self.leaves.append(data)
        k = len(self.leaves) - 1
        return self.add(f"leaf{k}{tuple(shape)}", lambda v, mk, T, k=k: mk(self.leaves[k]), shape, 3.0)

    def add(self, desc, fn, shape, bound, fb=0):
        if bound * 2.0 ** fb >= self.limit:
            return None  # would not be exactly representable any more
        self.steps.append((desc, fn))
        self.shapes.append(tuple(int(d) for d in shape))
        self.bounds.append(float(bound))
        self.fbits.append(int(fb))
        return len(self.steps) - 1

    def pick(self, pred=lambda i: True):
        c = [i for i in range(len(self.steps)) if pred(i)]
        return int(self.rng.choice(c)) if c else None

    def random_shape(self):
        while True:
            rank = int(self.rng.integers(1, 4))
            shape = tuple(int(self.rng.choice(DIMS)) for _ in range(rank))
            if np.prod(shape) <= (1 << 20):
                return shape

    # -- ops ------------------------------------------------------------------------------------------
    def op_scalar(self):
        i = self.pick()
        kind = int(self.rng.integers(0, 7))
        c = float(self.rng.integers(1, 4))
        b, f, sh = self.bounds[i], self.fbits[i], self.shapes[i]
        if kind == 0:
            return self.add(f"v{i}+{c}", lambda v, mk, T: v[i] + c, sh, b + c, f)
        if kind == 1:
            return self.add(f"{c}-v{i}", lambda v, mk, T: c - v[i], sh, b + c, f)
        if kind == 2:
            return self.add(f"v{i}*{c}", lambda v, mk, T: v[i] * c, sh, b * c, f)
        if kind == 3:
            return self.add(f"v{i}/2", lambda v, mk, T: v[i] / 2.0, sh, b, f + 1)
        if kind == 4:
            return self.add(f"abs(v{i})", lambda v, mk, T: v[i].abs(), sh, b, f)
        if kind == 5:
            return self.add(f"sqr(v{i})", lambda v, mk, T: v[i].sqr(), sh, b * b, 2 * f)
        return self.add(f"-v{i}", lambda v, mk, T: -v[i], sh, b, f)

    def op_pair(self):
        i = self.pick()
        j = self.pick(lambda k: self.shapes[k] == self.shapes[i])
        kind = int(self.rng.integers(0, 3))
        bi, bj, fi, fj = self.bounds[i], self.bounds[j], self.fbits[i], self.fbits[j]
        if kind == 2:
            return self.add(f"v{i}*v{j}", lambda v, mk, T: v[i] * v[j], self.shapes[i], bi * bj, fi + fj)
        if kind == 0:
            return self.add(f"v{i}+v{j}", lambda v, mk, T: v[i] + v[j], self.shapes[i], bi + bj, max(fi, fj))
        return self.add(f"v{i}-v{j}", lambda v, mk, T: v[i] - v[j], self.shapes[i], bi + bj, max(fi, fj))

    def op_view(self):
        i = self.pick(lambda k: len(self.shapes[k]) >= 1)
        s = self.shapes[i]
        kind = int(self.rng.integers(0, 6))
        if kind == 0 and len(s) >= 2:
            a, b = sorted(self.rng.choice(len(s), 2, replace=False).tolist())
            ns = list(s)
            ns[a], ns[b] = ns[b], ns[a]
            return self.add(f"v{i}.T({a},{b})", lambda v, mk, T: v[i].transpose(a, b), ns, self.bounds[i], self.fbits[i])
        if kind == 1:
            ranges = []
            for d in s:
                lo = int(self.rng.integers(0, d))
                hi = int(self.rng.integers(lo + 1, d + 1))
                ranges.append((lo, hi))
            ns = [hi - lo for lo, hi in ranges]
            return self.add(f"v{i}.slice({ranges})", lambda v, mk, T: v[i].slice(ranges), ns, self.bounds[i], self.fbits[i])
        if kind == 2 and len(s) <= 2:
            new = int(self.rng.choice([2, 3, 5, 16]))
            pos = int(self.rng.integers(0, len(s) + 1))
            ns = list(s)
            ns.insert(pos, new)
            # Tensor::broadcast puts the new dim where the shapes first differ: only unambiguous targets are drawn
            first_diff = 0
            while first_diff < len(s) and s[first_diff] == ns[first_diff]:
                first_diff += 1
            if first_diff != pos:
                return None
            return self.add(f"v{i}.broadcast({ns})", lambda v, mk, T: v[i].broadcast(ns), ns, self.bounds[i], self.fbits[i])
        if kind == 3:
            axis = int(self.rng.integers(0, len(s)))
            start = int(self.rng.integers(0, s[axis]))
            length = int(self.rng.integers(1, s[axis] - start + 1))
            ns = list(s)
            ns[axis] = length
            return self.add(f"v{i}.narrow({axis},{start},{length})", lambda v, mk, T: v[i].narrow(axis, start, length), ns, self.bounds[i], self.fbits[i])
        if kind == 4 and len(s) <= 2:
            axis = int(self.rng.integers(0, len(s) + 1))
            ns = list(s)
            ns.insert(axis, 1)
            return self.add(f"v{i}.unsqueeze({axis})", lambda v, mk, T: v[i].unsqueeze(axis), ns, self.bounds[i], self.fbits[i])
        n = int(np.prod(s))
        divs = [d for d in (1, 2, 3, 4, 5, 8, 16) if n % d == 0]
        d = int(self.rng.choice(divs))
        ns = [d, n // d]
        return self.add(f"v{i}.reshape({ns})", lambda v, mk, T: v[i].reshape(ns), ns, self.bounds[i], self.fbits[i])

    def op_copy(self):
        i = self.pick(lambda k: len(self.shapes[k]) >= 1)
        s = self.shapes[i]
        kind = int(self.rng.integers(0, 3))
        if kind == 0:
            ns = [int(max(1, d + self.rng.integers(-2, 3))) for d in s]
            return self.add(f"v{i}.resize({ns})", lambda v, mk, T: v[i].resize(ns), ns, self.bounds[i], self.fbits[i])
        if kind == 1:
            axis = int(self.rng.integers(0, len(s)))
            j = self.pick(lambda k: len(self.shapes[k]) == len(s) and all(a == b or d == axis for d, (a, b) in enumerate(zip(self.shapes[k], s))))
            ns = list(s)
            ns[axis] = s[axis] + self.shapes[j][axis]
            return self.add(f"cat(v{i},v{j};{axis})", lambda v, mk, T: T.cat([v[i], v[j]], axis), ns, max(self.bounds[i], self.bounds[j]), max(self.fbits[i], self.fbits[j]))
        ranges = []
        for d in s:
            lo = int(self.rng.integers(0, d))
            hi = int(self.rng.integers(lo + 1, d + 1))
            ranges.append((lo, hi))
        vs = tuple(hi - lo for lo, hi in ranges)
        j = self.pick(lambda k: self.shapes[k] == vs)
        if j is None:
            return None
        return self.add(f"v{i}.slice_assign({ranges},v{j})", lambda v, mk, T: v[i].slice_assign(ranges, v[j]), s, max(self.bounds[i], self.bounds[j]), max(self.fbits[i], self.fbits[j]))

    def op_reduce(self):
        i = self.pick(lambda k: len(self.shapes[k]) >= 1)
        s = self.shapes[i]
        axis = int(self.rng.integers(0, len(s)))
        ns = [d for k, d in enumerate(s) if k != axis]
        kind = int(self.rng.integers(0, 4))
        b, f = self.bounds[i], self.fbits[i]
        if kind == 0:
            return self.add(f"v{i}.sum({axis})", lambda v, mk, T: v[i].sum(axis), ns, b * s[axis], f)
        if kind == 1:
            return self.add(f"v{i}.max({axis})", lambda v, mk, T: v[i].max(axis), ns, b, f)
        if kind == 2:
            return self.add(f"v{i}.min({axis})", lambda v, mk, T: v[i].min(axis), ns, b, f)
        if s[axis] <= 4:
            return self.add(f"v{i}.product({axis})", lambda v, mk, T: v[i].product(axis), ns, max(1.0, b) ** s[axis], f * s[axis])
        return None

    def op_rows(self):
        """A last-axis reduction used again on the same rows (the softmax / RMSNorm shape of graph)."""
        i = self.pick(lambda k: len(self.shapes[k]) >= 1 and self.shapes[k][-1] >= 2)
        if i is None:
            return None
        s = self.shapes[i]
        last = len(s) - 1
        kind = int(self.rng.integers(0, 3))
        b, f = self.bounds[i], self.fbits[i]
        if kind == 0:
            return self.add(f"v{i}-rowmax(v{i})", lambda v, mk, T: v[i] - v[i].max(last).broadcast(list(s)), s, 2 * b, f)
        if kind == 1:
            return self.add(f"v{i}*rowmin(v{i})", lambda v, mk, T: v[i] * v[i].min(last).broadcast(list(s)), s, b * b, 2 * f)
        return self.add(f"v{i}+rowsum(v{i})", lambda v, mk, T: v[i] + v[i].sum(last).broadcast(list(s)), s, b * (s[last] + 1), f)

    def op_matmul(self):
        i = self.pick(lambda k: len(self.shapes[k]) == 2)
        if i is None:
            return None
        m, k = self.shapes[i]
        j = self.pick(lambda q: len(self.shapes[q]) == 2 and self.shapes[q][0] == k)
        if j is None:
            return None
        return self.add(f"v{i}@v{j}", lambda v, mk, T: v[i].mat_mul(v[j]), (m, self.shapes[j][1]),
                        self.bounds[i] * self.bounds[j] * k, self.fbits[i] + self.fbits[j])

    def build(self, nops):
        for _ in range(int(self.rng.integers(2, 4))):
            self.leaf(self.random_shape())
        self.leaf(self.shapes[0])  # a partner of the first leaf's shape, so that pair-wise ops always find one
        ops = [self.op_scalar, self.op_scalar, self.op_pair, self.op_pair, self.op_view, self.op_view, self.op_copy,
               self.op_reduce, self.op_reduce, self.op_matmul, self.op_rows]
        made = guard = 0
        while made < nops and guard < 20 * nops:
            guard += 1
            if ops[int(self.rng.integers(0, len(ops)))]() is not None:
                made += 1
        return self

    def describe(self):
        return "; ".join(f"v{k}={d}" for k, (d, _) in enumerate(self.steps))

    def run_all(self, make_tensor, T, upto):
        vals = []
        for desc, fn in self.steps[: upto + 1]:
            vals.append(fn(vals, make_tensor, T))
        return vals

    def run(self, make_tensor, T, upto):
        return self.run_all(make_tensor, T, upto)[upto]


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("seed", range(100))
def test_random_graphs_are_bit_exact_in_both_fusion_modes(gpu, wkf, seed, dtype):
    g = Gen(1000 * seed + (7 if dtype == np.float16 else 0), dtype).build(14)
    api = HipAPI(gpu)
    roots = list(range(len(g.steps)))[-4:]
    if gpu.is_planner:  # the run that only fills the kernel cache: plan everything this test launches, compute nothing
        for root in roots:
            for mode in (wkf.FUSION_TREE, wkf.FUSION_REFERENCE):
                gpu.set_fusion(mode)
                try:
                    g.run(api.tensor, api.T, root).materialize()
                finally:
                    gpu.set_fusion(wkf.FUSION_TREE)
    for root in roots:
        want = g.run(lambda a: OTensor(a), OTensor, root).to_numpy()
        for mode in (wkf.FUSION_TREE, wkf.FUSION_REFERENCE):
            gpu.set_fusion(mode)
            try:
                got = hip_values(g.run(api.tensor, api.T, root))
            finally:
                gpu.set_fusion(wkf.FUSION_TREE)
            assert got.shape == want.shape and got.dtype == want.dtype, f"root v{root} mode {mode}: {g.describe()}"
            assert np.array_equal(got, want), f"root v{root} mode {mode} differs from the oracle: {g.describe()}"
    # the same roots as ONE graph materialised in one pass (shared sub-graphs once, sibling reductions together)
    vals = g.run_all(api.tensor, api.T, roots[-1])
    wants = g.run_all(lambda a: OTensor(a), OTensor, roots[-1])
    if gpu.is_planner:
        wkf.materialize_many([vals[r] for r in roots])
        pytest.skip("plan-only device: kernels compiled, nothing computed")
    for r, sl in zip(roots, wkf.as_slice_many([vals[r] for r in roots])):
        assert np.array_equal(sl.to_numpy(), wants[r].to_numpy()), f"root v{r} of the joint pass differs: {g.describe()}"
