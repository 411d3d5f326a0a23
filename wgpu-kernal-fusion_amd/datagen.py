"""Deterministic synthetic inputs for the benchmark configurations: a SplitMix64 stream per
tensor, U(-1, 1) from the top 24 bits, N(mean, std) by Box-Muller.  Shared by bench.py and
the tests so that the GPU path and the checker see identical bytes."""
import numpy as np


class SplitMix64:
    """Deterministic input generator shared by the GPU path and the oracle."""

    def __init__(self, seed):
        self.state = np.uint64(seed)

    def raw(self, n):
        with np.errstate(over="ignore"):
            idx = np.arange(1, n + 1, dtype=np.uint64)
            z = self.state + idx * np.uint64(0x9E3779B97F4A7C15)
            self.state = self.state + np.uint64(n) * np.uint64(0x9E3779B97F4A7C15)
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            return z ^ (z >> np.uint64(31))

    def uniform(self, n, lo=-1.0, hi=1.0):
        u = (self.raw(n) >> np.uint64(40)).astype(np.float64) + 0.5  # 24 bits, never 0 or 1
        return lo + (hi - lo) * (u * 2.0 ** -24)

    def normal(self, n, mean=0.0, std=1.0):
        m = (n + 1) // 2
        u1 = self.uniform(m, 0.0, 1.0)
        u2 = self.uniform(m, 0.0, 1.0)
        r = np.sqrt(-2.0 * np.log(u1))
        z = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:n]
        return mean + std * z


def seeded(config_index, tensor_index, shape, dist, dtype=np.float32, **kw):
    """Input tensor `tensor_index` of benchmark config `config_index` (seed = 0x5EED0000 + 16*config + tensor)."""
    g = SplitMix64(0x5EED0000 + config_index * 16 + tensor_index)
    n = int(np.prod(shape, dtype=np.int64))
    v = g.uniform(n, **kw) if dist == "uniform" else g.normal(n, **kw)
    return v.astype(np.float32).astype(dtype).reshape(shape)
