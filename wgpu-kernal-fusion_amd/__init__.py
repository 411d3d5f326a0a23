"""ctypes binding of libwkf_hip.so, shaped like the reference crate's public API.

The library's host side (lazy graph, fusion pass, HIP kernel generator) is C++
behind a C ABI (include/wkf_hip.h, include/wkf_tensor.h).  This module is a thin
mirror of the reference's `Device` / `Tensor` / `TensorSlice` surface
(src/lib.rs:1-11 of the reference) over that ABI, so that tests and benchmarks
read like the reference's own: `((x * 2.0) + 1.0).sin().exp().as_slice()`.

There is no CPU fallback: without the built library, or without a gfx950 GPU,
construction fails.  `Device.planner()` gives a device that generates and
compiles kernels but cannot run them (host-side tests only).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_float, c_int, c_size_t, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwkf_hip.so")

F32, F16 = 0, 1
ERR_HIP, ERR_HIPRTC, ERR_INVALID_ARG, ERR_OOM, ERR_NO_DEVICE, ERR_UNSUPPORTED = 1, 2, 3, 4, 5, 6
FUSION_REFERENCE, FUSION_TREE = 0, 1

OP_ADD_CONST, OP_SUB_CONST, OP_CONST_SUB, OP_MUL_CONST, OP_DIV_CONST, OP_CONST_DIV = range(6)
_UNARY = ["exp", "exp2", "log", "log2", "sqr", "sqrt", "sin", "cos", "tan", "asin", "acos", "atan", "sinh",
          "cosh", "tanh", "asinh", "acosh", "atanh", "abs", "neg"]
UNARY_OPS = {name: 16 + i for i, name in enumerate(_UNARY)}
BINARY_OPS = {"add": 64, "sub": 65, "mul": 66, "div": 67, "pow": 68}
REDUCE_OPS = {"sum": 0, "max": 1, "min": 2, "product": 3}

# Every symbol the two headers declare; `load()` checks that the library exports all of them.
EXPORTS = [
    "wkf_device_create", "wkf_device_create_planner", "wkf_device_destroy", "wkf_device_is_planner",
    "wkf_device_props", "wkf_device_sync", "wkf_device_trim", "wkf_buffer_alloc", "wkf_buffer_retain",
    "wkf_buffer_release", "wkf_buffer_refcount", "wkf_buffer_size", "wkf_buffer_ptr", "wkf_buffer_upload",
    "wkf_buffer_download", "wkf_buffer_copy", "wkf_module_get", "wkf_module_find", "wkf_module_stats", "wkf_device_alloc_stats", "wkf_launch",
    "wkf_timer_create", "wkf_timer_destroy", "wkf_timer_begin", "wkf_timer_end", "wkf_timer_elapsed_ns",
    "wkf_last_error",
    "wkf_device_set_fusion", "wkf_device_get_fusion", "wkf_device_set_exact_math", "wkf_device_set_row_teams", "wkf_device_row_team_fallbacks", "wkf_device_set_map_table", "wkf_device_set_reference_compat", "wkf_device_set_timing", "wkf_tensor_new", "wkf_tensor_clone", "wkf_tensor_free",
    "wkf_tensor_rank", "wkf_tensor_shape", "wkf_tensor_dtype", "wkf_tensor_scalar_op", "wkf_tensor_unary_op",
    "wkf_tensor_cast", "wkf_tensor_binary_op", "wkf_tensor_reduce", "wkf_tensor_reduce_into", "wkf_tensor_mat_mul", "wkf_tensor_slice",
    "wkf_tensor_transpose", "wkf_tensor_broadcast", "wkf_tensor_narrow", "wkf_tensor_resize",
    "wkf_tensor_reshape", "wkf_tensor_unsqueeze", "wkf_tensor_slice_assign", "wkf_tensor_cat", "wkf_tensor_silu",
    "wkf_tensor_layer_norm", "wkf_tensor_rope", "wkf_tensor_softmax", "wkf_tensor_softmax_last_dim",
    "wkf_tensor_arange", "wkf_tensor_materialize", "wkf_tensor_kernel_count", "wkf_tensor_kernel_info",
    "wkf_kernel_source", "wkf_tensor_graphvis", "wkf_tensor_materialize_many", "wkf_tensor_as_slice_many", "wkf_tensor_as_slice", "wkf_slice_free", "wkf_slice_rank", "wkf_slice_dtype",
    "wkf_slice_layout", "wkf_slice_data", "wkf_slice_get",
    "wkf_layout_contiguous", "wkf_layout_is_contiguous", "wkf_layout_slice",
]


class WkfError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"[wkf error {code}] {message}")
        self.code = code


class Props(ctypes.Structure):
    _fields_ = [("ordinal", c_int), ("compute_units", c_int), ("wave_size", c_int),
                ("max_threads_per_block", c_int), ("clock_khz", c_int), ("lds_bytes_per_block", c_size_t),
                ("total_mem_bytes", c_size_t), ("arch", ctypes.c_char * 32)]


_lib = None


def load():
    """Load the in-tree library (never builds it, never falls back)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise WkfError(-1, f"{LIB_PATH} is missing: run wgpu-kernal-fusion_amd/build.sh (or __graft_entry__.build())")
    lib = ctypes.CDLL(LIB_PATH)
    missing = [s for s in EXPORTS if not hasattr(lib, s)]
    if missing:
        raise WkfError(-1, f"{LIB_PATH} does not export: {missing}")
    lib.wkf_last_error.restype = c_char_p
    lib.wkf_slice_data.restype = c_void_p
    lib.wkf_buffer_ptr.restype = c_void_p
    lib.wkf_buffer_size.restype = c_size_t
    for name in EXPORTS:
        fn = getattr(lib, name)
        if fn.restype is c_int and name not in ("wkf_last_error",):
            pass
    # argtypes for the calls that take size_t / float by value (ctypes would pass int otherwise)
    lib.wkf_tensor_scalar_op.argtypes = [c_void_p, c_int, c_float, POINTER(c_void_p)]
    lib.wkf_tensor_unary_op.argtypes = [c_void_p, c_int, POINTER(c_void_p)]
    lib.wkf_tensor_cast.argtypes = [c_void_p, c_int, POINTER(c_void_p)]
    lib.wkf_tensor_binary_op.argtypes = [c_void_p, c_void_p, c_int, POINTER(c_void_p)]
    lib.wkf_tensor_reduce.argtypes = [c_void_p, c_int, c_size_t, POINTER(c_void_p)]
    lib.wkf_tensor_reduce_into.argtypes = [c_void_p, c_int, c_size_t, c_void_p]
    lib.wkf_tensor_mat_mul.argtypes = [c_void_p, c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_new.argtypes = [c_void_p, c_int, c_int, POINTER(c_size_t), c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_clone.argtypes = [c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_free.argtypes = [c_void_p]
    lib.wkf_tensor_free.restype = None
    lib.wkf_tensor_rank.argtypes = [c_void_p]
    lib.wkf_tensor_shape.argtypes = [c_void_p, POINTER(c_size_t)]
    lib.wkf_tensor_dtype.argtypes = [c_void_p]
    lib.wkf_tensor_slice.argtypes = [c_void_p, POINTER(c_size_t), POINTER(c_size_t), POINTER(c_void_p)]
    lib.wkf_tensor_transpose.argtypes = [c_void_p, c_size_t, c_size_t, POINTER(c_void_p)]
    lib.wkf_tensor_broadcast.argtypes = [c_void_p, c_int, POINTER(c_size_t), POINTER(c_void_p)]
    lib.wkf_tensor_narrow.argtypes = [c_void_p, c_size_t, c_size_t, c_size_t, POINTER(c_void_p)]
    lib.wkf_tensor_resize.argtypes = [c_void_p, POINTER(c_size_t), POINTER(c_void_p)]
    lib.wkf_tensor_reshape.argtypes = [c_void_p, c_int, POINTER(c_size_t), POINTER(c_void_p)]
    lib.wkf_tensor_unsqueeze.argtypes = [c_void_p, c_size_t, POINTER(c_void_p)]
    lib.wkf_tensor_slice_assign.argtypes = [c_void_p, POINTER(c_size_t), POINTER(c_size_t), c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_cat.argtypes = [POINTER(c_void_p), c_int, c_size_t, POINTER(c_void_p)]
    lib.wkf_tensor_silu.argtypes = [c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_layer_norm.argtypes = [c_void_p, c_void_p, c_float, POINTER(c_void_p)]
    lib.wkf_tensor_rope.argtypes = [c_void_p, c_void_p, c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_softmax.argtypes = [c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_softmax_last_dim.argtypes = [c_void_p, POINTER(c_void_p)]
    lib.wkf_tensor_arange.argtypes = [c_void_p, c_int, c_float, c_float, c_float, POINTER(c_void_p)]
    lib.wkf_tensor_materialize.argtypes = [c_void_p]
    lib.wkf_tensor_kernel_count.argtypes = [c_void_p]
    lib.wkf_tensor_kernel_info.argtypes = [c_void_p, c_int, POINTER(c_uint64), c_char_p, c_size_t, c_char_p, c_size_t,
                                           c_char_p, c_size_t]
    lib.wkf_kernel_source.argtypes = [c_char_p, c_char_p, c_size_t, POINTER(c_size_t)]
    lib.wkf_tensor_graphvis.argtypes = [c_void_p, c_char_p, c_size_t, POINTER(c_size_t)]
    lib.wkf_tensor_materialize_many.argtypes = [POINTER(c_void_p), c_int]
    lib.wkf_tensor_as_slice_many.argtypes = [POINTER(c_void_p), c_int, POINTER(c_void_p)]
    lib.wkf_tensor_as_slice.argtypes = [c_void_p, POINTER(c_void_p)]
    lib.wkf_slice_free.argtypes = [c_void_p]
    lib.wkf_slice_free.restype = None
    lib.wkf_slice_rank.argtypes = [c_void_p]
    lib.wkf_slice_dtype.argtypes = [c_void_p]
    lib.wkf_slice_layout.argtypes = [c_void_p, POINTER(c_size_t), POINTER(c_size_t), POINTER(c_size_t)]
    lib.wkf_slice_data.argtypes = [c_void_p, POINTER(c_size_t)]
    lib.wkf_layout_contiguous.argtypes = [c_int, POINTER(c_size_t), POINTER(c_size_t)]
    lib.wkf_layout_is_contiguous.argtypes = [c_int, c_size_t, POINTER(c_size_t), POINTER(c_size_t), POINTER(c_int)]
    lib.wkf_layout_slice.argtypes = [c_int, c_size_t, POINTER(c_size_t), POINTER(c_size_t), POINTER(c_size_t),
                                     POINTER(c_size_t), POINTER(c_size_t), POINTER(c_size_t)]
    lib.wkf_slice_get.argtypes = [c_void_p, POINTER(c_size_t), POINTER(c_float)]
    lib.wkf_device_create.argtypes = [c_int, POINTER(c_void_p)]
    lib.wkf_device_create_planner.argtypes = [POINTER(c_void_p)]
    lib.wkf_device_destroy.argtypes = [c_void_p]
    lib.wkf_device_destroy.restype = None
    lib.wkf_device_is_planner.argtypes = [c_void_p]
    lib.wkf_device_props.argtypes = [c_void_p, POINTER(Props)]
    lib.wkf_device_sync.argtypes = [c_void_p]
    lib.wkf_device_trim.argtypes = [c_void_p]
    lib.wkf_device_set_fusion.argtypes = [c_void_p, c_int]
    lib.wkf_device_get_fusion.argtypes = [c_void_p]
    lib.wkf_device_set_exact_math.argtypes = [c_void_p, c_int]
    lib.wkf_device_set_timing.argtypes = [c_void_p, c_int]
    lib.wkf_device_set_row_teams.argtypes = [c_void_p, c_int, ctypes.c_uint32]
    lib.wkf_device_row_team_fallbacks.argtypes = [c_void_p, POINTER(c_uint64)]
    lib.wkf_device_set_map_table.argtypes = [c_void_p, c_uint64]
    lib.wkf_device_set_reference_compat.argtypes = [c_void_p, c_int]
    lib.wkf_module_stats.argtypes = [c_void_p, POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint64)]
    lib.wkf_device_alloc_stats.argtypes = [c_void_p, POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint64)]
    lib.wkf_buffer_alloc.argtypes = [c_void_p, c_size_t, c_int, POINTER(c_void_p)]
    lib.wkf_buffer_release.argtypes = [c_void_p]
    lib.wkf_buffer_release.restype = None
    lib.wkf_buffer_retain.argtypes = [c_void_p]
    lib.wkf_buffer_retain.restype = None
    lib.wkf_buffer_refcount.argtypes = [c_void_p]
    lib.wkf_buffer_size.argtypes = [c_void_p]
    lib.wkf_buffer_ptr.argtypes = [c_void_p]
    lib.wkf_buffer_upload.argtypes = [c_void_p, c_size_t, c_void_p, c_size_t]
    lib.wkf_buffer_download.argtypes = [c_void_p, c_size_t, c_void_p, c_size_t]
    lib.wkf_buffer_copy.argtypes = [c_void_p, c_void_p, c_size_t]
    lib.wkf_module_get.argtypes = [c_void_p, c_char_p, c_char_p, c_char_p, POINTER(c_void_p)]
    lib.wkf_launch.argtypes = [c_void_p, c_void_p, POINTER(ctypes.c_uint32), POINTER(ctypes.c_uint32), ctypes.c_uint32,
                               c_void_p, c_size_t, c_void_p]
    lib.wkf_timer_create.argtypes = [c_void_p, POINTER(c_void_p)]
    lib.wkf_timer_destroy.argtypes = [c_void_p]
    lib.wkf_timer_destroy.restype = None
    lib.wkf_timer_begin.argtypes = [c_void_p]
    lib.wkf_timer_end.argtypes = [c_void_p]
    lib.wkf_timer_elapsed_ns.argtypes = [c_void_p, POINTER(c_uint64)]
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise WkfError(rc, load().wkf_last_error().decode("utf-8", "replace"))


def _sizes(values):
    values = [int(v) for v in values]
    return (c_size_t * max(1, len(values)))(*values)


_NP = {F32: np.float32, F16: np.float16}


class Layout:
    """Layout (src/layout.rs:33-94): offset, shape and strides of a view, in elements."""

    def __init__(self, offset, shape, strides):  # Layout::from_parts, src/layout.rs:50-56
        self._offset, self._shape, self._strides = int(offset), tuple(int(v) for v in shape), tuple(int(v) for v in strides)
        if len(self._shape) != len(self._strides):
            raise ValueError("shape and strides differ in rank")

    from_parts = classmethod(lambda cls, offset, shape, strides: cls(offset, shape, strides))

    @classmethod
    def contiguous(cls, shape):  # src/layout.rs:41-48
        strides = _sizes([0] * len(shape))
        _check(load().wkf_layout_contiguous(len(shape), _sizes(shape), strides))
        return cls(0, shape, [strides[i] for i in range(len(shape))])

    def is_contiguous(self):  # src/layout.rs:58-60
        out = c_int()
        _check(load().wkf_layout_is_contiguous(self.rank(), self._offset, _sizes(self._shape), _sizes(self._strides), byref(out)))
        return bool(out.value)

    def slice(self, ranges):  # src/layout.rs:62-71; ranges = [(begin, end), ...] or Python slices / ranges
        spans = [(r.start, r.stop) if isinstance(r, (slice, range)) else tuple(r) for r in ranges]
        if len(spans) != self.rank():
            raise WkfError(ERR_INVALID_ARG, "slice: one range per dimension is required")
        off, shape = c_size_t(), _sizes([0] * self.rank())
        _check(load().wkf_layout_slice(self.rank(), self._offset, _sizes(self._shape), _sizes(self._strides),
                                       _sizes([b for b, _ in spans]), _sizes([e for _, e in spans]), byref(off), shape))
        return Layout(off.value, [shape[i] for i in range(self.rank())], self._strides)

    def rank(self):
        return len(self._shape)

    def shape(self):
        return self._shape

    def strides(self):
        return self._strides

    def offset(self):
        return self._offset


class Device:
    """`Device::new()` of the reference (src/device.rs:13-32): one GPU, one queue (HIP stream)."""

    def __init__(self, ordinal=0, _planner=False):
        lib = load()
        h = c_void_p()
        if _planner:
            _check(lib.wkf_device_create_planner(byref(h)))
        else:
            _check(lib.wkf_device_create(int(ordinal), byref(h)))
        self._h = h
        self._lib = lib

    @classmethod
    def new(cls, ordinal=0):
        return cls(ordinal)

    @classmethod
    def planner(cls):
        """A device with no GPU behind it: kernels are generated and compiled, never run."""
        return cls(_planner=True)

    @property
    def is_planner(self):
        return bool(self._lib.wkf_device_is_planner(self._h))

    def props(self):
        p = Props()
        _check(self._lib.wkf_device_props(self._h, byref(p)))
        return p

    def sync(self):
        _check(self._lib.wkf_device_sync(self._h))

    def trim(self):
        _check(self._lib.wkf_device_trim(self._h))

    def set_fusion(self, mode):
        _check(self._lib.wkf_device_set_fusion(self._h, int(mode)))

    def fusion(self):
        return self._lib.wkf_device_get_fusion(self._h)

    def set_timing(self, enabled):
        _check(self._lib.wkf_device_set_timing(self._h, 1 if enabled else 0))

    def set_exact_math(self, exact):
        _check(self._lib.wkf_device_set_exact_math(self._h, 1 if exact else 0))

    def set_row_teams(self, enabled, spin_polls=0):
        """Rows held in the registers of several workgroups that wait for each other (one launch, one read); see
        wkf_device_set_row_teams.  spin_polls = 0 keeps the default bound of the wait."""
        _check(self._lib.wkf_device_set_row_teams(self._h, 1 if enabled else 0, int(spin_polls)))

    def set_reference_compat(self, enabled):
        """Composites follow the reference's text where it differs in value from what it means (layer_norm on square
        inputs: the weight indexed by row); see wkf_device_set_reference_compat."""
        _check(self._lib.wkf_device_set_reference_compat(self._h, 1 if enabled else 0))

    def set_map_table(self, min_elements):
        """Fewest elements for which a costly map over one dense f16 tensor runs as a table lookup (0: never); see
        wkf_device_set_map_table."""
        _check(self._lib.wkf_device_set_map_table(self._h, int(min_elements)))

    def row_team_fallbacks(self):
        """Read-backs that were computed a second time, without teams, because a team kernel gave up waiting."""
        n = c_uint64()
        _check(self._lib.wkf_device_row_team_fallbacks(self._h, byref(n)))
        return n.value

    def module_stats(self):
        a, b, c = c_uint64(), c_uint64(), c_uint64()
        _check(self._lib.wkf_module_stats(self._h, byref(a), byref(b), byref(c)))
        return {"compiled": a.value, "disk_hits": b.value, "mem_hits": c.value}

    def alloc_stats(self):
        a, b, c, d = c_uint64(), c_uint64(), c_uint64(), c_uint64()
        _check(self._lib.wkf_device_alloc_stats(self._h, byref(a), byref(b), byref(c), byref(d)))
        return {"buffer_allocs": a.value, "device_mallocs": b.value, "timers": c.value, "live_buffers": d.value}

    def close(self):
        if self._h:
            self._lib.wkf_device_destroy(self._h)
            self._h = None


class KernelTiming:
    """One entry of `Tensor::all_timing_information()` (QueryResults, src/query.rs:19-47)."""

    def __init__(self, kind, signature, detail, elapsed_ns):
        self.kind, self.signature, self.detail, self.elapsed_ns = kind, signature, detail, elapsed_ns

    def elapsed(self):
        return self.elapsed_ns * 1e-9

    def __repr__(self):
        return f"KernelTiming({self.kind}, {self.elapsed_ns} ns, {self.detail})"


class TensorSlice:
    """Host copy of a materialised tensor: the whole buffer plus its layout
    (TensorSlice, src/tensor.rs:669-855).  Index with a tuple; `to_numpy()` decodes the view."""

    def __init__(self, handle):
        lib = load()
        self._lib, self._h = lib, handle
        rank = lib.wkf_slice_rank(handle)
        off = c_size_t()
        shape, strides = _sizes([0] * rank), _sizes([0] * rank)
        _check(lib.wkf_slice_layout(handle, byref(off), shape, strides))
        self.offset = off.value
        self.shape = tuple(shape[i] for i in range(rank))
        self.strides = tuple(strides[i] for i in range(rank))
        self.dtype = lib.wkf_slice_dtype(handle)
        nbytes = c_size_t()
        ptr = lib.wkf_slice_data(handle, byref(nbytes))
        raw = (ctypes.c_ubyte * nbytes.value).from_address(ptr)
        self.buffer = np.frombuffer(raw, dtype=_NP[self.dtype]).copy()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.wkf_slice_free(self._h)
            self._h = None

    def get(self, index):
        """`TensorSlice::get`: None when an index is out of range (src/tensor.rs:827-846)."""
        if len(index) != len(self.shape):
            raise IndexError("wrong number of indices")
        out = c_float()
        rc = self._lib.wkf_slice_get(self._h, _sizes(index), byref(out))
        return None if rc != 0 else out.value

    def __getitem__(self, index):
        if not isinstance(index, (tuple, list)):
            index = (index,)
        v = self.get(index)
        if v is None:
            raise IndexError(f"index {index} out of range for shape {self.shape}")
        return v

    def to_numpy(self):
        itemsize = self.buffer.itemsize
        view = np.lib.stride_tricks.as_strided(self.buffer[self.offset:], shape=self.shape,
                                               strides=tuple(s * itemsize for s in self.strides), writeable=False)
        return np.array(view)

    def __eq__(self, other):
        if not isinstance(other, TensorSlice):
            return NotImplemented
        return self.shape == other.shape and np.array_equal(self.to_numpy(), other.to_numpy())

    def __repr__(self):
        return f"TensorSlice({self.to_numpy()!r})"


class Tensor:
    """Lazy tensor handle: every method only records a node (src/tensor.rs:418-644)."""

    def __init__(self, device, handle):
        self.device, self._h, self._lib = device, handle, load()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.wkf_tensor_free(self._h)
            self._h = None

    # -- construction -----------------------------------------------------
    @classmethod
    def new(cls, device, data, dtype=None):
        """`Tensor::new(&device, &data)`; ragged input raises like the reference panics."""
        if dtype is None:
            dtype = F16 if getattr(data, "dtype", None) == np.float16 else F32
        arr = np.ascontiguousarray(np.asarray(data, dtype=_NP[dtype]))
        h = c_void_p()
        _check(load().wkf_tensor_new(device._h, dtype, arr.ndim, _sizes(arr.shape), arr.ctypes.data_as(c_void_p), byref(h)))
        return cls(device, h)

    @classmethod
    def arange(cls, device, start, end, dtype=F32):
        return cls.arange_step(device, start, end, 1.0, dtype)

    @classmethod
    def arange_step(cls, device, start, end, step, dtype=F32):
        h = c_void_p()
        _check(load().wkf_tensor_arange(device._h, dtype, float(start), float(end), float(step), byref(h)))
        return cls(device, h)

    @classmethod
    def cat(cls, tensors, dim):
        tensors = list(tensors)
        arr = (c_void_p * len(tensors))(*[t._h for t in tensors])
        h = c_void_p()
        _check(load().wkf_tensor_cat(arr, len(tensors), int(dim), byref(h)))
        return cls(tensors[0].device, h)

    def clone(self):
        h = c_void_p()
        _check(self._lib.wkf_tensor_clone(self._h, byref(h)))
        return Tensor(self.device, h)

    # -- static info --------------------------------------------------------
    def rank(self):
        return self._lib.wkf_tensor_rank(self._h)

    def shape(self):
        r = self.rank()
        out = _sizes([0] * r)
        _check(self._lib.wkf_tensor_shape(self._h, out))
        return tuple(out[i] for i in range(r))

    def datatype(self):
        return self._lib.wkf_tensor_dtype(self._h)

    # -- element-wise ---------------------------------------------------------
    def _new(self, h):
        return Tensor(self.device, h)

    def _scalar(self, op, c):
        h = c_void_p()
        _check(self._lib.wkf_tensor_scalar_op(self._h, op, float(c), byref(h)))
        return self._new(h)

    def _unary(self, name):
        h = c_void_p()
        _check(self._lib.wkf_tensor_unary_op(self._h, UNARY_OPS[name], byref(h)))
        return self._new(h)

    def _binary(self, other, name):
        h = c_void_p()
        _check(self._lib.wkf_tensor_binary_op(self._h, other._h, BINARY_OPS[name], byref(h)))
        return self._new(h)

    def __add__(self, o):
        return self._binary(o, "add") if isinstance(o, Tensor) else self._scalar(OP_ADD_CONST, o)

    def __radd__(self, o):
        return self._scalar(OP_ADD_CONST, o)

    def __sub__(self, o):
        return self._binary(o, "sub") if isinstance(o, Tensor) else self._scalar(OP_SUB_CONST, o)

    def __rsub__(self, o):
        return self._scalar(OP_CONST_SUB, o)

    def __mul__(self, o):
        return self._binary(o, "mul") if isinstance(o, Tensor) else self._scalar(OP_MUL_CONST, o)

    def __rmul__(self, o):
        return self._scalar(OP_MUL_CONST, o)

    def __truediv__(self, o):
        return self._binary(o, "div") if isinstance(o, Tensor) else self._scalar(OP_DIV_CONST, o)

    def __rtruediv__(self, o):
        return self._scalar(OP_CONST_DIV, o)

    def __neg__(self):
        return self._unary("neg")

    def pow(self, other):
        return self._binary(other, "pow")

    def cast(self, dtype):
        h = c_void_p()
        _check(self._lib.wkf_tensor_cast(self._h, int(dtype), byref(h)))
        return self._new(h)

    # -- reductions / matmul ----------------------------------------------------
    def _reduce(self, name, dim):
        h = c_void_p()
        _check(self._lib.wkf_tensor_reduce(self._h, REDUCE_OPS[name], int(dim), byref(h)))
        return self._new(h)

    def reduce_into(self, name, dim, out):
        """`self.<name>(dim)` written into `out` (a dense tensor that holds data) without any device allocation:
        wkf_tensor_reduce_into.  Both tensors must be leaves; the kernels must have run once before."""
        _check(self._lib.wkf_tensor_reduce_into(self._h, REDUCE_OPS[name], int(dim), out._h))
        return out

    def sum(self, dim):
        return self._reduce("sum", dim)

    def max(self, dim):
        return self._reduce("max", dim)

    def min(self, dim):
        return self._reduce("min", dim)

    def product(self, dim):
        return self._reduce("product", dim)

    def mat_mul(self, other):
        h = c_void_p()
        _check(self._lib.wkf_tensor_mat_mul(self._h, other._h, byref(h)))
        return self._new(h)

    # -- layout -------------------------------------------------------------------
    def slice(self, ranges):
        """`tensor.slice([0..2, 0..1])`: ranges are (start, end) pairs or Python ranges."""
        starts = [r.start if isinstance(r, range) else r[0] for r in ranges]
        ends = [r.stop if isinstance(r, range) else r[1] for r in ranges]
        if len(starts) != self.rank():
            raise WkfError(3, "slice: one range per dimension is required")
        h = c_void_p()
        _check(self._lib.wkf_tensor_slice(self._h, _sizes(starts), _sizes(ends), byref(h)))
        return self._new(h)

    def transpose(self, first_axis, second_axis):
        h = c_void_p()
        _check(self._lib.wkf_tensor_transpose(self._h, int(first_axis), int(second_axis), byref(h)))
        return self._new(h)

    def broadcast(self, out_shape):
        h = c_void_p()
        _check(self._lib.wkf_tensor_broadcast(self._h, len(out_shape), _sizes(out_shape), byref(h)))
        return self._new(h)

    def narrow(self, axis, start, length):
        h = c_void_p()
        _check(self._lib.wkf_tensor_narrow(self._h, int(axis), int(start), int(length), byref(h)))
        return self._new(h)

    def resize(self, new_shape):
        if len(new_shape) != self.rank():
            raise WkfError(3, "resize: rank must not change")
        h = c_void_p()
        _check(self._lib.wkf_tensor_resize(self._h, _sizes(new_shape), byref(h)))
        return self._new(h)

    def reshape(self, new_shape):
        h = c_void_p()
        _check(self._lib.wkf_tensor_reshape(self._h, len(new_shape), _sizes(new_shape), byref(h)))
        return self._new(h)

    def unsqueeze(self, axis):
        h = c_void_p()
        _check(self._lib.wkf_tensor_unsqueeze(self._h, int(axis), byref(h)))
        return self._new(h)

    def slice_assign(self, ranges, value):
        starts = [r.start if isinstance(r, range) else r[0] for r in ranges]
        ends = [r.stop if isinstance(r, range) else r[1] for r in ranges]
        if len(starts) != self.rank():
            raise WkfError(3, "slice_assign: one range per dimension is required")
        h = c_void_p()
        _check(self._lib.wkf_tensor_slice_assign(self._h, _sizes(starts), _sizes(ends), value._h, byref(h)))
        return self._new(h)

    # -- composites ---------------------------------------------------------------
    def silu(self):
        h = c_void_p()
        _check(self._lib.wkf_tensor_silu(self._h, byref(h)))
        return self._new(h)

    def layer_norm(self, weight, eps):
        h = c_void_p()
        _check(self._lib.wkf_tensor_layer_norm(self._h, weight._h, float(eps), byref(h)))
        return self._new(h)

    def rope(self, cos, sin):
        h = c_void_p()
        _check(self._lib.wkf_tensor_rope(self._h, cos._h, sin._h, byref(h)))
        return self._new(h)

    def softmax(self):
        h = c_void_p()
        _check(self._lib.wkf_tensor_softmax(self._h, byref(h)))
        return self._new(h)

    def softmax_last_dim(self):
        h = c_void_p()
        _check(self._lib.wkf_tensor_softmax_last_dim(self._h, byref(h)))
        return self._new(h)

    # -- execution ------------------------------------------------------------------
    def materialize(self):
        """Run the graph under this tensor; the result stays on the device."""
        _check(self._lib.wkf_tensor_materialize(self._h))
        return self

    def as_slice(self):
        """`tensor.as_slice().await`: materialise and download (src/tensor.rs:533-554)."""
        h = c_void_p()
        _check(self._lib.wkf_tensor_as_slice(self._h, byref(h)))
        return TensorSlice(h)

    def to_numpy(self):
        return self.as_slice().to_numpy()

    def graphvis(self):
        """Tensor::graphvis (src/tensor.rs:641-643 of the reference): the lazy graph below this tensor as DOT text."""
        need = c_size_t()
        _check(self._lib.wkf_tensor_graphvis(self._h, None, 0, byref(need)))
        buf = ctypes.create_string_buffer(need.value)
        _check(self._lib.wkf_tensor_graphvis(self._h, buf, need.value, byref(need)))
        return buf.value.decode()

    def kernels(self):
        """Kernels launched by the last materialize / as_slice, with GPU times."""
        out = []
        for i in range(self._lib.wkf_tensor_kernel_count(self._h)):
            ns = c_uint64()
            kind = ctypes.create_string_buffer(32)
            sig = ctypes.create_string_buffer(4096)
            detail = ctypes.create_string_buffer(256)
            _check(self._lib.wkf_tensor_kernel_info(self._h, i, byref(ns), kind, 32, sig, 4096, detail, 256))
            out.append(KernelTiming(kind.value.decode(), sig.value.decode(), detail.value.decode(), ns.value))
        return out

    def all_timing_information(self):
        """`Tensor::all_timing_information` (src/tensor.rs:556-558): re-materialises, then reports."""
        self.materialize()
        return self.kernels()


def materialize_many(tensors):
    """Materialise several tensors in one pass (shared work once, sibling row reductions in one kernel).
    The launches are recorded on tensors[0]."""
    lib = load()
    arr = (c_void_p * len(tensors))(*[t._h for t in tensors])
    _check(lib.wkf_tensor_materialize_many(arr, len(tensors)))


def as_slice_many(tensors):
    """`as_slice` for several tensors in one pass over their joint graph; returns one TensorSlice each."""
    lib = load()
    arr = (c_void_p * len(tensors))(*[t._h for t in tensors])
    out = (c_void_p * len(tensors))()
    _check(lib.wkf_tensor_as_slice_many(arr, len(tensors), out))
    return [TensorSlice(c_void_p(h)) for h in out]


def kernel_source(signature):
    """Generated HIP source of a kernel signature this process has seen."""
    lib = load()
    need = c_size_t()
    _check(lib.wkf_kernel_source(signature.encode(), None, 0, byref(need)))
    buf = ctypes.create_string_buffer(need.value)
    _check(lib.wkf_kernel_source(signature.encode(), buf, need.value, byref(need)))
    return buf.value.decode()


for _name in _UNARY:
    if _name != "neg":
        setattr(Tensor, _name, (lambda n: lambda self: self._unary(n))(_name))
