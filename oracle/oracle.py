"""CPU oracle for the lazy-tensor hot path.  TEST INFRASTRUCTURE ONLY.

This is the checker the HIP path is compared against.  Only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import
it; the product (the `wgpu-kernal-fusion_amd` package and its library) never
does.

What it restates.  The reference crate evaluates its ops in WGSL on whatever
GPU driver wgpu finds, so its arithmetic for transcendental functions is not
in the repository (wgpu / naga 24.0.0, git fork `FL33TW00D/wgpu` at
9c0628039c61, `Cargo.lock:1780-1782`).  What IS fixed by the reference is
 * which ops exist and what each one means (`src/element_wise.rs:197-1471`,
   `src/pair_wise.rs:205-528`, `src/reduce.rs:433-815`),
 * that every fused op is a separately typed function, so each intermediate is
   rounded to the tensor dtype (`src/kernel.rs:540-553`, `src/element_wise.rs:64-79`),
 * the layout algebra (`src/layout.rs:33-94`, `src/map_layout.rs:42-98`),
 * the copies (`src/resize.rs:43-145`, `src/slice_assign.rs:49-80`) and
 * how the composites are built from the primitives (`src/composite/*.rs`).
`OTensor` restates exactly that, eagerly, with numpy: every op is computed in
float64 and rounded (round-to-nearest-even) to the tensor dtype before the next
op sees it.  For + - * / sqr sqrt abs neg and casts this IS the IEEE result; for
transcendental functions it is the correctly rounded value up to float64's own
libm error (about 2^-29 of an f32 ulp).

How it is pinned (tests/test_oracle_kats.py): every literal test vector the
reference's own tests hold for this path (tests/golden/reference_kats.json, each
entry citing file:line), closed forms (sum of ones, A @ I, norm preservation of
rope pairs ...), and brute-force index maps for the layout ops.  Functions with
no reference vector at all: `rope` (the reference has no test for it) and
`softmax_last_dim` (not in the reference); they are pinned by the mathematics
only (parity unpinned at the last bit) and say so in their docstrings.
`layer_norm` names its broadcast dimensions (RMSNorm as meant); the reference's
text misplaces the weight on square inputs, which `layer_norm_as_written`
restates and the tests pin.
"""
from __future__ import annotations

import numpy as np

F32, F16 = np.float32, np.float16

# seeds of max / min, src/reduce.rs:640,713 (f32 literals -3.40282e+38 / 3.40282e+38)
MAX_SEED = np.float32(-3.40282e38)
MIN_SEED = np.float32(3.40282e38)

_UNARY64 = {
    "exp": np.exp, "exp2": np.exp2, "log": np.log, "log2": np.log2, "sqr": lambda v: v * v, "sqrt": np.sqrt,
    "sin": np.sin, "cos": np.cos, "tan": np.tan, "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan,
    "sinh": np.sinh, "cosh": np.cosh, "tanh": np.tanh, "asinh": np.arcsinh, "acosh": np.arccosh,
    "atanh": np.arctanh, "abs": np.abs, "neg": lambda v: -v,
}


def _round(v64, dtype):
    with np.errstate(over="ignore", invalid="ignore"):
        return np.asarray(v64, dtype=np.float64).astype(dtype)


class OTensor:
    """Eager mirror of `Tensor<R, D>` (src/tensor.rs:418-644): same method names, numpy inside."""

    def __init__(self, data, dtype=None):
        arr = np.asarray(data)
        if dtype is None:
            dtype = F16 if arr.dtype == np.float16 else F32
        self.a = np.array(arr, dtype=dtype)  # logical values, own copy

    # -- static info ------------------------------------------------------
    def shape(self):
        return tuple(self.a.shape)

    def rank(self):
        return self.a.ndim

    def datatype(self):
        return 1 if self.a.dtype == np.float16 else 0

    def to_numpy(self):
        return np.array(self.a)

    def clone(self):
        return OTensor(self.a)

    def _like(self, v64):
        return OTensor(_round(v64, self.a.dtype), self.a.dtype)

    def _c(self, c):
        # the literal is an f32; on an f16 tensor it is converted to f16 first (src/element_wise.rs:197-210)
        return np.float64(np.float32(c).astype(self.a.dtype))

    def _x(self):
        return self.a.astype(np.float64)

    # -- tensor (op) literal, src/element_wise.rs:197-675 --------------------
    def __add__(self, o):
        return self._pair(o, np.add) if isinstance(o, OTensor) else self._like(self._x() + self._c(o))

    __radd__ = __add__

    def __sub__(self, o):
        return self._pair(o, np.subtract) if isinstance(o, OTensor) else self._like(self._x() - self._c(o))

    def __rsub__(self, o):
        return self._like(self._c(o) - self._x())

    def __mul__(self, o):
        return self._pair(o, np.multiply) if isinstance(o, OTensor) else self._like(self._x() * self._c(o))

    __rmul__ = __mul__

    def __truediv__(self, o):
        with np.errstate(divide="ignore", invalid="ignore"):
            return self._pair(o, np.divide) if isinstance(o, OTensor) else self._like(self._x() / self._c(o))

    def __rtruediv__(self, o):
        with np.errstate(divide="ignore", invalid="ignore"):
            return self._like(self._c(o) / self._x())

    def __neg__(self):
        return self._like(-self._x())

    # -- pair-wise, src/pair_wise.rs:205-528 -----------------------------------
    def _pair(self, o, fn):
        if self.a.shape != o.a.shape:
            raise ValueError("pair-wise op: operand shapes differ")  # src/pair_wise.rs:92
        if self.a.dtype != o.a.dtype:
            raise ValueError("pair-wise op: operand dtypes differ")
        with np.errstate(all="ignore"):
            return self._like(fn(self._x(), o._x()))

    def pow(self, o):
        return self._pair(o, np.power)

    # -- cast, src/element_wise.rs:1408-1471 -----------------------------------
    def cast(self, dtype):
        np_dt = F16 if dtype in (1, F16) else F32
        with np.errstate(over="ignore"):
            return OTensor(self.a.astype(np_dt), np_dt)  # f32 -> f16: RNE, overflow -> inf; f16 -> f32 exact

    # -- reductions, src/reduce.rs:433-815 --------------------------------------
    def _reduce(self, kind, dim):
        if not 0 <= dim < self.a.ndim:
            raise ValueError("reduce: axis out of range")
        x = self._x()
        if kind == "sum":
            r = x.sum(axis=dim)
        elif kind == "product":
            r = x.prod(axis=dim)
        elif kind == "max":
            r = np.maximum(np.float64(MAX_SEED), x.max(axis=dim, initial=-np.inf))
        else:
            r = np.minimum(np.float64(MIN_SEED), x.min(axis=dim, initial=np.inf))
        return self._like(r)

    def sum(self, dim):
        return self._reduce("sum", dim)

    def max(self, dim):
        return self._reduce("max", dim)

    def min(self, dim):
        return self._reduce("min", dim)

    def product(self, dim):
        return self._reduce("product", dim)

    # -- matmul: the textbook product the reference's own test checks against
    # (ndarray `dot`, src/matmul.rs:268-318); accumulated in float64, rounded once.
    def mat_mul(self, o):
        # rank 2 in the reference; equal leading dimensions are a batch of independent products (this library's extension)
        if self.a.ndim < 2 or o.a.ndim != self.a.ndim or self.a.shape[:-2] != o.a.shape[:-2]:
            raise ValueError("mat_mul: operands must have the same rank (2 or more) and the same batch dimensions")
        if self.a.shape[-1] != o.a.shape[-2]:
            raise ValueError("mat_mul: inner dimensions differ")  # src/matmul.rs:194
        return self._like(self._x() @ o._x())

    # -- views, src/map_layout.rs:42-98 -------------------------------------------
    def slice(self, ranges):
        idx = tuple(slice(r.start, r.stop) if isinstance(r, range) else slice(r[0], r[1]) for r in ranges)
        if len(idx) != self.a.ndim:
            raise ValueError("slice: one range per dimension is required")
        return OTensor(self.a[idx], self.a.dtype)

    def transpose(self, first_axis, second_axis):
        return OTensor(np.swapaxes(self.a, first_axis, second_axis), self.a.dtype)

    def broadcast(self, out_shape):
        s = self.a.shape
        out_shape = tuple(out_shape)
        if len(out_shape) != len(s) + 1:
            raise ValueError("broadcast: the output rank must be the input rank + 1")
        new_dim = 0
        while new_dim < len(s) and s[new_dim] == out_shape[new_dim]:
            new_dim += 1  # first position where the shapes differ, src/map_layout.rs:72-77
        if tuple(s[new_dim:]) != tuple(out_shape[new_dim + 1:]):
            raise ValueError("broadcast: shapes do not line up")
        return OTensor(np.broadcast_to(np.expand_dims(self.a, new_dim), out_shape), self.a.dtype)

    def narrow(self, axis, start, length):
        if axis >= self.a.ndim or start + length > self.a.shape[axis]:
            raise ValueError("narrow: out of range")  # src/composite/narrow.rs:6-7
        idx = [slice(None)] * self.a.ndim
        idx[axis] = slice(start, start + length)
        return OTensor(self.a[tuple(idx)], self.a.dtype)

    # -- copies, src/resize.rs:121-145 ---------------------------------------------
    def resize(self, new_shape):
        if len(new_shape) != self.a.ndim:
            raise ValueError("resize: rank must not change")
        out = np.zeros(tuple(new_shape), dtype=self.a.dtype)  # wgpu zero-initialises new buffers
        corner = tuple(slice(0, min(a, b)) for a, b in zip(self.a.shape, new_shape))
        out[corner] = self.a[corner]
        return OTensor(out, self.a.dtype)

    def reshape(self, new_shape):
        if int(np.prod(new_shape, dtype=np.int64)) != self.a.size:
            raise ValueError("reshape: element counts differ")  # src/resize.rs:132-135
        return OTensor(np.ascontiguousarray(self.a).reshape(tuple(new_shape)), self.a.dtype)

    def unsqueeze(self, axis):
        return OTensor(np.expand_dims(self.a, axis), self.a.dtype)  # src/composite/unsqueeze.rs:3-16

    def slice_assign(self, ranges, value):
        idx = tuple(slice(r.start, r.stop) if isinstance(r, range) else slice(r[0], r[1]) for r in ranges)
        out = np.array(self.a)
        if out[idx].shape != value.a.shape:
            raise ValueError("slice_assign: the value's shape does not match the slice")  # src/slice_assign.rs:69
        out[idx] = value.a
        return OTensor(out, self.a.dtype)

    @staticmethod
    def cat(tensors, dim):
        tensors = list(tensors)
        if dim >= tensors[0].a.ndim:
            raise ValueError("cat: dim out of range")
        return OTensor(np.concatenate([t.a for t in tensors], axis=dim), tensors[0].a.dtype)  # src/composite/cat.rs:3-41

    @staticmethod
    def arange(device, start, end, dtype=F32):
        return OTensor.arange_step(device, start, end, 1.0, dtype)

    @staticmethod
    def arange_step(device, start, end, step, dtype=F32):
        # host loop with the running value kept in the tensor dtype, src/composite/arange.rs:8-22
        dt = F16 if dtype in (1, F16) else F32
        cur, end, step = dt(start), dt(end), dt(step)
        vals = []
        if step >= 0:
            while cur < end:
                vals.append(cur)
                cur = dt(cur + step)
        else:
            while cur > end:
                vals.append(cur)
                cur = dt(cur + step)
        return OTensor(np.array(vals, dtype=dt), dt)

    # -- composites, src/composite/*.rs (each is the same composition of primitives) ----
    def silu(self):
        return self / (1.0 + (-self).exp())  # src/composite/silu.rs:4-7

    def layer_norm(self, weight, eps):
        # RMSNorm computed in f32, src/composite/rms_norm.rs:8-15
        hidden = self.a.shape[-1]
        f32_self = self.cast(F32)
        norm_x = (f32_self.sqr().sum(1)) / float(hidden)
        rms = (norm_x + eps).sqrt()
        x_normed = f32_self / OTensor(np.broadcast_to(rms.a[:, None], self.a.shape), F32)
        w = OTensor(np.broadcast_to(weight.a[None, :], self.a.shape), weight.a.dtype)
        return x_normed.cast(self.a.dtype) * w

    def layer_norm_as_written(self, weight, eps):
        """`layer_norm` exactly as the reference's text reads (src/composite/rms_norm.rs:8-15): both broadcasts go
        through `Tensor::broadcast`, which inserts the new dimension at the FIRST position where the shapes differ
        (src/map_layout.rs:69-77).  For rows != hidden that is RMSNorm; for a square input (rows == hidden) the
        weight's shape [hidden] matches the output's first dimension, the new dimension lands at position 1, and the
        weight ends up indexed by ROW.  `layer_norm` above names its dimensions and is what the HIP path computes;
        this form exists to pin the difference (tests/test_oracle_kats.py)."""
        hidden = self.a.shape[-1]
        f32_self = self.cast(F32)
        norm_x = (f32_self.sqr().sum(1)) / float(hidden)
        x_normed = f32_self / (norm_x + eps).sqrt().broadcast(self.a.shape)
        return x_normed.cast(self.a.dtype) * weight.broadcast(self.a.shape)

    def rope(self, cos, sin):
        """y = x*cos + rotate_half(x)*sin, rotate_half(x) = cat(-x2, x1) on the last dim
        (src/composite/rope.rs:5-22).  No reference test vector exists: pinned by the
        formula, by position 0 being the identity and by |(y_j, y_{j+d/2})| = |(x_j, x_{j+d/2})|."""
        heads, seq, dim = self.a.shape
        if cos.a.shape[1] * 2 == dim:
            cos = OTensor.cat([cos, cos], 1)
            sin = OTensor.cat([sin, sin], 1)
        cos, sin = cos.narrow(0, 0, seq), sin.narrow(0, 0, seq)
        x1 = self.narrow(2, 0, dim // 2)
        x2 = self.narrow(2, dim // 2, dim - dim // 2)
        rotated = OTensor.cat([-x2, x1], 2)
        cb = OTensor(np.broadcast_to(cos.a[None], self.a.shape), self.a.dtype)
        sb = OTensor(np.broadcast_to(sin.a[None], self.a.shape), self.a.dtype)
        return self * cb + rotated * sb

    def softmax(self):
        e = self.exp()  # rank 1, no max subtraction: src/composite/softmax.rs:4-10
        s = e.sum(0)
        return e / OTensor(np.broadcast_to(s.a, e.a.shape), e.a.dtype)

    def softmax_last_dim(self):
        """Max-subtracted softmax over the last dim from the primitives max, sub, exp, sum, div.
        Not in the reference (rank-1 `softmax` only): pinned by rows summing to 1 and by
        agreement with `softmax` on rank-1 data up to the max shift."""
        last = self.a.ndim - 1
        m = self.max(last)
        mb = OTensor(np.broadcast_to(np.expand_dims(m.a, last), self.a.shape), self.a.dtype)
        e = (self - mb).exp()
        s = e.sum(last)
        sb = OTensor(np.broadcast_to(np.expand_dims(s.a, last), self.a.shape), self.a.dtype)
        return e / sb


def _add_unary(name):
    def method(self):
        with np.errstate(all="ignore"):
            return self._like(_UNARY64[name](self._x()))

    method.__name__ = name
    setattr(OTensor, name, method)


for _n in _UNARY64:
    if _n != "neg":
        _add_unary(_n)


# ---- helpers shared by the tests ------------------------------------------------

def ulp_distance(a, b):
    """Distance in units of the last place between two arrays of the same float dtype:
    difference of the monotone integer images; +0 == -0; NaN matches NaN."""
    a, b = np.asarray(a), np.asarray(b)
    assert a.dtype == b.dtype and a.shape == b.shape, (a.dtype, b.dtype, a.shape, b.shape)
    if a.dtype == np.float32:
        ia, ib, mask = a.view(np.int32).astype(np.int64), b.view(np.int32).astype(np.int64), 0x7FFFFFFF
    else:
        ia, ib, mask = a.view(np.int16).astype(np.int64), b.view(np.int16).astype(np.int64), 0x7FFF
    ia = np.where(ia < 0, -(ia & mask), ia)
    ib = np.where(ib < 0, -(ib & mask), ib)
    d = np.abs(ia - ib)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, d)


def _load_datagen():
    # the seeded input generator lives with the product (bench.py uses it too); re-exported here for the tests
    import importlib.util
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "wgpu-kernal-fusion_amd", "datagen.py")
    spec = importlib.util.spec_from_file_location("wkf_datagen", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


_dg = _load_datagen()
SplitMix64, seeded = _dg.SplitMix64, _dg.seeded
