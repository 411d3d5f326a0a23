"""ctypes wrapper of oracle/libwkf_port.so (the CPU port that bench.py times as
`cpu_baseline`).  Test / baseline infrastructure only; see port.c."""
import ctypes
import os
from ctypes import POINTER, c_float, c_size_t

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwkf_port.so")
_lib = None
_F = POINTER(c_float)


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(LIB_PATH)
        lib.port_threads.restype = ctypes.c_int
        lib.port_c1.argtypes = [_F, _F, c_size_t]
        lib.port_row_max.argtypes = [_F, _F, c_size_t, c_size_t]
        lib.port_row_sum_exp_sub.argtypes = [_F, _F, c_size_t, c_size_t, c_float]
        lib.port_c3.argtypes = [_F, _F, _F, _F, _F, c_size_t, c_size_t]
        lib.port_rmsnorm.argtypes = [_F, _F, c_float, _F, _F, c_size_t, c_size_t]
        lib.port_rope.argtypes = [_F, _F, _F, _F, _F, c_size_t, c_size_t, c_size_t]
        lib.port_softmax_rows.argtypes = [_F, _F, _F, _F, c_size_t, c_size_t]
        lib.port_gemm_f32.argtypes = [_F, _F, _F, c_size_t, c_size_t, c_size_t]
        _lib = lib
    return _lib


def _p(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_F)


def threads():
    return load().port_threads()


def c1(x, out=None):
    out = np.empty_like(x) if out is None else out
    load().port_c1(_p(x), _p(out), x.size)
    return out


def row_max(x, out=None):
    out = np.empty(x.shape[0], dtype=np.float32) if out is None else out
    load().port_row_max(_p(x), _p(out), x.shape[0], x.shape[1])
    return out


def row_sum_exp_sub(x, c0=1.0, out=None):
    out = np.empty(x.shape[0], dtype=np.float32) if out is None else out
    load().port_row_sum_exp_sub(_p(x), _p(out), x.shape[0], x.shape[1], c0)
    return out


def c3(a, b, bias, t1=None, t2=None):
    t1 = np.empty_like(a) if t1 is None else t1
    t2 = np.empty_like(a) if t2 is None else t2
    inner = a.shape[-1]
    load().port_c3(_p(a), _p(b), _p(bias), _p(t1), _p(t2), a.size // inner, inner)
    return t1


def rmsnorm(x, w, eps):
    rms = np.empty(x.shape[0], dtype=np.float32)
    out = np.empty_like(x)
    load().port_rmsnorm(_p(x), _p(w), eps, _p(rms), _p(out), x.shape[0], x.shape[1])
    return out


def rope(x, cos_full, sin_full):
    rot, out = np.empty_like(x), np.empty_like(x)
    load().port_rope(_p(x), _p(cos_full), _p(sin_full), _p(rot), _p(out), *x.shape)
    return out


def softmax_rows(x):
    rows, cols = x.size // x.shape[-1], x.shape[-1]
    mx, sm = np.empty(rows, dtype=np.float32), np.empty(rows, dtype=np.float32)
    out = np.empty_like(x)
    load().port_softmax_rows(_p(x), _p(mx), _p(sm), _p(out), rows, cols)
    return out


def gemm_f32(a, b):
    c = np.empty((a.shape[0], b.shape[1]), dtype=np.float32)
    load().port_gemm_f32(_p(a), _p(b), _p(c), a.shape[0], b.shape[1], a.shape[1])
    return c
