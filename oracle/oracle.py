"""Python loader of the CPU oracle (oracle/prad_oracle.cpp).

TEST INFRASTRUCTURE ONLY.  Only tests, the smoke check and the benchmark's cpu_baseline leg may
import this module; the product package never does.  Every function takes and returns numpy
arrays and calls the C++ restatement of the reference's algorithm.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build():
    """Compiles liboracle.so with the Makefile next to this file (always recompiles)."""
    subprocess.run(["make", "-B", "-C", _HERE, "liboracle.so"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.oracle_u01.restype = ctypes.c_double
        _lib.oracle_u01.argtypes = [ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64]
        for sfx in ("f64", "f32"):
            getattr(_lib, "oracle_time_matmul_fwdbwd_" + sfx).restype = ctypes.c_double
            getattr(_lib, "oracle_time_matmul_fwdbwd_" + sfx).argtypes = [
                ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
        _lib.oracle_cce_fwd_f64.restype = ctypes.c_double
        _lib.oracle_cce_fwd_f32.restype = ctypes.c_float
        _lib.oracle_mse_fwd_f64.restype = ctypes.c_double
        _lib.oracle_mse_fwd_f32.restype = ctypes.c_float
    return _lib


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return "f64", ctypes.c_double
    if dtype == np.float32:
        return "f32", ctypes.c_float
    raise TypeError("oracle supports float64 and float32")


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _fn(name, dtype):
    return getattr(load(), "oracle_%s_%s" % (name, _sfx(dtype)[0]))


def hardware_threads():
    return int(load().oracle_hardware_threads())


def matmul_fwd(A, B, threads=1, tiled8=False):
    dt = A.dtype
    A, B = _c(A, dt), _c(B, dt)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    C = np.empty((M, N), dt)
    _fn("matmul_fwd_tiled8" if tiled8 else "matmul_fwd", dt)(_p(A), _p(B), _p(C), M, K, N, threads)
    return C


def matmul_bwd(dC, A, B, threads=1):
    dt = A.dtype
    dC, A, B = _c(dC, dt), _c(A, dt), _c(B, dt)
    M, K = A.shape
    N = B.shape[1]
    dA, dB = np.empty((M, K), dt), np.empty((K, N), dt)
    _fn("matmul_bwd", dt)(_p(dC), _p(A), _p(B), _p(dA), _p(dB), M, K, N, threads)
    return dA, dB


def matmul_sum_fwd(A, B, threads=1):
    dt = A.dtype
    A, B = _c(A, dt), _c(B, dt)
    M, K = A.shape
    P, K2, N = B.shape
    assert K == K2
    out = np.empty((1, P), dt)
    _fn("matmul_sum_fwd", dt)(_p(A), _p(B), _p(out), M, K, N, P, threads)
    return out


def matmul_sum_bwd(A, B, dOut):
    dt = A.dtype
    A, B, dOut = _c(A, dt), _c(B, dt), _c(dOut, dt)
    M, K = A.shape
    P, _, N = B.shape
    assert N == M, "the reference adds transpose(B[q]) to a matrix shaped like A"
    dA, dB = np.empty((M, K), dt), np.empty((P, K, M), dt)
    _fn("matmul_sum_bwd", dt)(_p(A), _p(B), _p(dOut), _p(dA), _p(dB), M, K, N, P)
    return dA, dB


def _unary(name, x, *scalars):
    dt = x.dtype
    x = _c(x, dt)
    y = np.empty_like(x)
    ct = _sfx(dt)[1]
    _fn(name, dt)(_p(x), _p(y), ctypes.c_int64(x.size), *[ct(s) for s in scalars])
    return y


def _binary(name, a, b, *scalars):
    dt = a.dtype
    a, b = _c(a, dt), _c(b, dt)
    y = np.empty_like(a)
    ct = _sfx(dt)[1]
    _fn(name, dt)(_p(a), _p(b), _p(y), ctypes.c_int64(a.size), *[ct(s) for s in scalars])
    return y


def leakyrelu_fwd(x, alpha):
    return _unary("leakyrelu_fwd", x, alpha)


def leakyrelu_bwd(x, dy, alpha):
    return _binary("leakyrelu_bwd", x, dy, alpha)


def sigmoid_fwd(x):
    return _unary("sigmoid_fwd", x)


def sigmoid_bwd(y, dy):
    return _binary("sigmoid_bwd", y, dy)


def tanh_fwd(x):
    return _unary("tanh_fwd", x)


def tanh_bwd(y, dy):
    return _binary("tanh_bwd", y, dy)


def gelu_fwd(x):
    return _unary("gelu_fwd", x)


def gelu_bwd(x, dy):
    return _binary("gelu_bwd", x, dy)


def hadamard_fwd(a, b):
    return _binary("hadamard_fwd", a, b)


def hadamard_bwd(a, b, dy):
    dt = a.dtype
    a, b, dy = _c(a, dt), _c(b, dt), _c(dy, dt)
    da, db = np.empty_like(a), np.empty_like(a)
    _fn("hadamard_bwd", dt)(_p(a), _p(b), _p(dy), _p(da), _p(db), ctypes.c_int64(a.size))
    return da, db


def accumulate(dest, grad):
    dt = dest.dtype
    out = np.array(dest, dtype=dt, order="C", copy=True)
    grad = _c(grad, dt)
    _fn("accumulate", dt)(_p(out), _p(grad), ctypes.c_int64(out.size))
    return out


def clip(g, clip_value, min_value):
    dt = g.dtype
    out = np.array(g, dtype=dt, order="C", copy=True)
    ct = _sfx(dt)[1]
    _fn("clip", dt)(_p(out), ctypes.c_int64(out.size), ct(clip_value), ct(min_value))
    return out


def adam(w, m, v, g, lr, beta1, beta2, eps, t, reverse=False):
    dt = w.dtype
    w, m, v = (np.array(x, dtype=dt, order="C", copy=True) for x in (w, m, v))
    g = _c(g, dt)
    ct = _sfx(dt)[1]
    _fn("adam_reverse" if reverse else "adam", dt)(_p(w), _p(m), _p(v), _p(g), ctypes.c_int64(w.size), ct(lr), ct(beta1),
                                                   ct(beta2), ct(eps), ct(t))
    return w, m, v


def add_broadcast_fwd(x, b):
    dt = x.dtype
    x, b = _c(x, dt), _c(b, dt).reshape(-1)
    y = np.empty_like(x)
    _fn("add_broadcast_fwd", dt)(_p(x), _p(b), _p(y), x.shape[0], x.shape[1])
    return y


def add_broadcast_bwd_bias(dy):
    dt = dy.dtype
    dy = _c(dy, dt)
    db = np.empty((1, dy.shape[1]), dt)
    _fn("add_broadcast_bwd_bias", dt)(_p(dy), _p(db), dy.shape[0], dy.shape[1])
    return db


def softmax_fwd(x):
    dt = x.dtype
    x = _c(x, dt)
    y = np.empty_like(x)
    _fn("softmax_fwd", dt)(_p(x), _p(y), x.shape[0], x.shape[1])
    return y


def softmax_bwd(y, dy):
    dt = y.dtype
    y, dy = _c(y, dt), _c(dy, dt)
    dx = np.empty_like(y)
    _fn("softmax_bwd", dt)(_p(y), _p(dy), _p(dx), y.shape[0], y.shape[1])
    return dx


def cce_fwd(p, t):
    dt = p.dtype
    p, t = _c(p, dt), _c(t, dt)
    return float(_fn("cce_fwd", dt)(_p(p), _p(t), p.shape[0], p.shape[1]))


def cce_bwd(p, t):
    dt = p.dtype
    p, t = _c(p, dt), _c(t, dt)
    dp = np.empty_like(p)
    _fn("cce_bwd", dt)(_p(p), _p(t), _p(dp), p.shape[0], p.shape[1])
    return dp


def mse_fwd(y, t):
    dt = y.dtype
    y, t = _c(y, dt), _c(t, dt)
    return float(_fn("mse_fwd", dt)(_p(y), _p(t), y.shape[0], y.shape[1]))


def mse_bwd(y, t):
    dt = y.dtype
    y, t = _c(y, dt), _c(t, dt)
    dy = np.empty_like(y)
    _fn("mse_bwd", dt)(_p(y), _p(t), _p(dy), y.shape[0], y.shape[1])
    return dy


def matrix_add(a, b):
    return _binary("matrix_add", a, b)


def matrix_add_three(a, b, c):
    dt = a.dtype
    a, b, c = _c(a, dt), _c(b, dt), _c(c, dt)
    y = np.empty_like(a)
    _fn("matrix_add_three", dt)(_p(a), _p(b), _p(c), _p(y), ctypes.c_int64(a.size))
    return y


def matrix_transpose(x):
    dt = x.dtype
    x = _c(x, dt)
    y = np.empty((x.shape[1], x.shape[0]), dt)
    _fn("matrix_transpose", dt)(_p(x), _p(y), x.shape[0], x.shape[1])
    return y


def layernorm_fwd(x):
    """Returns (y, mean, stddev); mean and stddev have one entry per row."""
    dt = x.dtype
    x = _c(x, dt)
    y = np.empty_like(x)
    mean, std = np.empty(x.shape[0], dt), np.empty(x.shape[0], dt)
    _fn("layernorm_fwd", dt)(_p(x), _p(y), _p(mean), _p(std), x.shape[0], x.shape[1])
    return y, mean, std


def layernorm_bwd(x, mean, stddev, dy):
    dt = x.dtype
    x, mean, stddev, dy = _c(x, dt), _c(mean, dt), _c(stddev, dt), _c(dy, dt)
    dx = np.empty_like(x)
    _fn("layernorm_bwd", dt)(_p(x), _p(mean), _p(stddev), _p(dy), _p(dx), x.shape[0], x.shape[1])
    return dx


def amplified_sigmoid_fwd(x):
    return _unary("amplified_sigmoid_fwd", x)


def amplified_sigmoid_bwd(x, dy):
    return _binary("amplified_sigmoid_bwd", x, dy)


def time_matmul_fwdbwd(n, dtype=np.float64, threads=1, iters=1):
    """Seconds for `iters` forward+backward passes of an n x n x n product on jagged rows."""
    chk = ctypes.c_double()
    return float(_fn("time_matmul_fwdbwd", dtype)(n, threads, iters, ctypes.byref(chk)))


def u01(seed, tensor, idx):
    return float(load().oracle_u01(seed, tensor, idx))
