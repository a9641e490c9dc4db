"""ctypes binding of oracle/liboracle.so (the C oracle).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    so = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        L = C.CDLL(build())
        u8p, f32p, u16p, i32p, f64p = (C.POINTER(t) for t in (C.c_uint8, C.c_float, C.c_uint16, C.c_int32, C.c_double))
        L.orc_h2f.restype = C.c_float
        L.orc_h2f.argtypes = [C.c_uint16]
        L.orc_f2h.restype = C.c_uint16
        L.orc_f2h.argtypes = [C.c_float]
        L.orc_f2bf.restype = C.c_uint16
        L.orc_f2bf.argtypes = [C.c_float]
        L.orc_bf2f.restype = C.c_float
        L.orc_bf2f.argtypes = [C.c_uint16]
        L.orc_h2f_n.argtypes = [u16p, f32p, C.c_int64]
        L.orc_f2h_n.argtypes = [f32p, u16p, C.c_int64]
        L.orc_type_sizes.argtypes = [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.orc_row_bytes.restype = C.c_int64
        L.orc_row_bytes.argtypes = [C.c_int, C.c_int64]
        L.orc_dequant.argtypes = [C.c_int, u8p, C.c_int64, f32p]
        L.orc_dense_vecmat.argtypes = [f64p, f64p, C.c_int, C.c_int, f64p]
        L.orc_dense_matmul.argtypes = [f64p, f64p, C.c_int, C.c_int, C.c_int, f64p]
        L.orc_matvec_q.argtypes = [C.c_int, u8p, C.c_int, C.c_int, f32p, f32p]
        L.orc_matvec_q_reference_algorithm.argtypes = [C.c_int, u8p, C.c_int, C.c_int, f32p, f32p]
        L.orc_gemm_q.argtypes = [C.c_int, u8p, C.c_int, C.c_int, u16p, C.c_int, f32p]
        L.orc_attn_decode.argtypes = [f32p, u16p, u16p, i32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_double, f32p]
        L.orc_rmsnorm.argtypes = [f32p, f32p, C.c_int, C.c_double, f32p]
        L.orc_rope.argtypes = [f32p, C.c_int, C.c_int, C.c_int, C.c_double]
        L.orc_swiglu.argtypes = [f32p, f32p, C.c_int, f32p]
        L.orc_argmax.argtypes = [f32p, C.c_int]
        L.orc_set_num_threads.argtypes = [C.c_int]
        _LIB = L
    return _LIB


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def _u8(raw):
    a = np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw
    return np.ascontiguousarray(a).reshape(-1).view(np.uint8)


def _check(rc, what):
    if rc != 0:
        raise ValueError(f"{what} failed with code {rc}")


def type_sizes(t):
    be, bb = C.c_int(), C.c_int()
    _check(lib().orc_type_sizes(t, C.byref(be), C.byref(bb)), "orc_type_sizes")
    return be.value, bb.value


def row_bytes(t, k):
    return int(lib().orc_row_bytes(t, k))


def h2f(bits):
    b = np.ascontiguousarray(bits, dtype=np.uint16).reshape(-1)
    out = np.empty(b.size, dtype=np.float32)
    lib().orc_h2f_n(_p(b, C.c_uint16), _p(out, C.c_float), b.size)
    return out.reshape(np.shape(bits))


def f2h(x):
    f = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    out = np.empty(f.size, dtype=np.uint16)
    lib().orc_f2h_n(_p(f, C.c_float), _p(out, C.c_uint16), f.size)
    return out.reshape(np.shape(x))


def dequant(t, raw, n_elems=None):
    w = _u8(raw)
    if n_elems is None:
        be, bb = type_sizes(t)
        n_elems = w.size // bb * be
    out = np.empty(n_elems, dtype=np.float32)
    _check(lib().orc_dequant(t, _p(w, C.c_uint8), n_elems, _p(out, C.c_float)), "orc_dequant")
    return out


def matvec_q(t, raw, n, k, x, reference_algorithm=False):
    w = _u8(raw)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(n, dtype=np.float32)
    fn = lib().orc_matvec_q_reference_algorithm if reference_algorithm else lib().orc_matvec_q
    _check(fn(t, _p(w, C.c_uint8), n, k, _p(x, C.c_float), _p(y, C.c_float)), "orc_matvec_q")
    return y


def gemm_q(t, raw, n, k, a_bf16, m):
    w = _u8(raw)
    a = np.ascontiguousarray(a_bf16, dtype=np.uint16)
    c = np.empty((m, n), dtype=np.float32)
    _check(lib().orc_gemm_q(t, _p(w, C.c_uint8), n, k, _p(a, C.c_uint16), m, _p(c, C.c_float)), "orc_gemm_q")
    return c


def dense_vecmat(x, b):
    x = np.ascontiguousarray(x, dtype=np.float64)
    b = np.ascontiguousarray(b, dtype=np.float64)
    y = np.empty(b.shape[1])
    lib().orc_dense_vecmat(_p(x, C.c_double), _p(b, C.c_double), b.shape[0], b.shape[1], _p(y, C.c_double))
    return y


def dense_matmul(a, b):
    a = np.ascontiguousarray(a, dtype=np.float64)
    b = np.ascontiguousarray(b, dtype=np.float64)
    c = np.empty((a.shape[0], b.shape[1]))
    lib().orc_dense_matmul(_p(a, C.c_double), _p(b, C.c_double), a.shape[0], a.shape[1], b.shape[1], _p(c, C.c_double))
    return c


def attn_decode(q, k_bits, v_bits, n_ctx, scale):
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k_bits, dtype=np.uint16)
    v = np.ascontiguousarray(v_bits, dtype=np.uint16)
    n = np.ascontiguousarray(n_ctx, dtype=np.int32)
    s, h, d = q.shape
    out = np.empty_like(q)
    lib().orc_attn_decode(_p(q, C.c_float), _p(k, C.c_uint16), _p(v, C.c_uint16), _p(n, C.c_int32), s, h, d,
                          k.shape[1], float(scale), _p(out, C.c_float))
    return out


def rmsnorm(x, w, eps=1e-5):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    y = np.empty_like(x)
    lib().orc_rmsnorm(_p(x, C.c_float), _p(w, C.c_float), x.size, eps, _p(y, C.c_float))
    return y


def rope(x, pos, base=10000.0):
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    lib().orc_rope(_p(y, C.c_float), y.shape[-2], y.shape[-1], pos, base)
    return y


def swiglu(g, u):
    g = np.ascontiguousarray(g, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    o = np.empty_like(g)
    lib().orc_swiglu(_p(g, C.c_float), _p(u, C.c_float), g.size, _p(o, C.c_float))
    return o


def argmax(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    return int(lib().orc_argmax(_p(x, C.c_float), x.size))


def set_num_threads(n):
    lib().orc_set_num_threads(int(n))


def num_threads():
    return int(lib().orc_num_threads())
