"""ctypes front end of the CPU oracle (oracle/oracle.c).

TEST INFRASTRUCTURE ONLY.  The oracle is the checker the HIP kernels are
compared with.  Nothing in the product package may import this module; the
tests, the smoke check and the CPU-baseline leg of the benchmark do.

The reference (donglinz/kernel_optimization) is CUDA-only and holds no CPU
implementation for softmax or LayerNorm and only a commented-out GEMM loop
(nn_operators/gemm/main.cu:162-167), so there is no oracle/_ref build.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i64 = ctypes.c_int64


def build(force=False):
    """Compile oracle.c with gcc (make -C oracle)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_max_threads.restype = ctypes.c_int
        L.oracle_set_threads.argtypes = [ctypes.c_int]
        L.oracle_softmax_f32.argtypes = [_f32p, _f32p, _i64, _i64, _i32p, _i64]
        L.oracle_layernorm_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _i64, _i64,
                                           ctypes.c_double, ctypes.c_int]
        L.oracle_layernorm_welford_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _i64,
                                                   _i64, ctypes.c_float, ctypes.c_int, ctypes.c_int,
                                                   ctypes.c_int]
        L.oracle_sgemm_f32.argtypes = [_i64, _i64, _i64, ctypes.c_double, _f32p, _f32p,
                                       ctypes.c_double, _f32p, _f32p, _f64p]
        L.oracle_gemm_16.argtypes = [_i64, _i64, _i64, ctypes.c_double, _u16p, _u16p, ctypes.c_int,
                                     ctypes.c_double, _u16p, _u16p, ctypes.c_int, _f64p, _f64p]
        L.oracle_gemm_16_bias_act.argtypes = [_i64, _i64, _i64, ctypes.c_double, _u16p, _u16p, ctypes.c_int,
                                              ctypes.c_double, _u16p, _u16p, ctypes.c_int, _u16p, ctypes.c_int,
                                              _f64p, _f64p]
        L.oracle_softmax_16.argtypes = [_u16p, _u16p, _f64p, _i64, _i64, _i32p, _i64, ctypes.c_int]
        L.oracle_layernorm_16.argtypes = [_u16p, _u16p, _f64p, _f32p, _f32p, _u16p, _u16p, _i64, _i64,
                                          ctypes.c_double, ctypes.c_int, ctypes.c_int]
        for name in ("oracle_f16_to_f64", "oracle_bf16_to_f64"):
            getattr(L, name).argtypes = [_u16p, _f64p, _i64]
        for name in ("oracle_f64_to_f16", "oracle_f64_to_bf16"):
            getattr(L, name).argtypes = [_f64p, _u16p, _i64]
        _lib = L
    return _lib


def _ptr(a, ty):
    return None if a is None else a.ctypes.data_as(ty)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def max_threads():
    return lib().oracle_max_threads()


def set_threads(n):
    lib().oracle_set_threads(int(n))


def softmax(x, valid_len=None, rows_per_seq=0):
    """Row softmax of a [rows, cols] float32 array; optional padding mask."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    out = np.empty_like(x)
    vl = _c(valid_len, np.int32)
    rc = lib().oracle_softmax_f32(_ptr(x, _f32p), _ptr(out, _f32p), rows, cols, _ptr(vl, _i32p),
                                  int(rows_per_seq))
    if rc:
        raise ValueError("oracle_softmax_f32: bad arguments")
    return out


def layernorm(x, gamma=None, beta=None, eps=1e-5, unbiased=False):
    """Returns (y, mean, rstd) of a [rows, cols] float32 array (two-pass, double)."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    y = np.empty_like(x)
    mean = np.empty(rows, np.float32)
    rstd = np.empty(rows, np.float32)
    g, b = _c(gamma, np.float32), _c(beta, np.float32)
    rc = lib().oracle_layernorm_f32(_ptr(x, _f32p), _ptr(y, _f32p), _ptr(mean, _f32p),
                                    _ptr(rstd, _f32p), _ptr(g, _f32p), _ptr(b, _f32p), rows, cols,
                                    float(eps), int(bool(unbiased)))
    if rc:
        raise ValueError("oracle_layernorm_f32: bad arguments")
    return y, mean, rstd


def layernorm_welford(x, gamma=None, beta=None, eps=1e-5, unbiased=False, lanes=32, vec_len=4):
    """Float-only Welford/Chan restatement with the reference's lane structure."""
    x = _c(x, np.float32)
    rows, cols = x.shape
    y = np.empty_like(x)
    mean = np.empty(rows, np.float32)
    rstd = np.empty(rows, np.float32)
    g, b = _c(gamma, np.float32), _c(beta, np.float32)
    rc = lib().oracle_layernorm_welford_f32(_ptr(x, _f32p), _ptr(y, _f32p), _ptr(mean, _f32p),
                                            _ptr(rstd, _f32p), _ptr(g, _f32p), _ptr(b, _f32p), rows,
                                            cols, float(eps), int(bool(unbiased)), int(lanes),
                                            int(vec_len))
    if rc:
        raise ValueError("oracle_layernorm_welford_f32: bad arguments")
    return y, mean, rstd


def softmax16(x_bits, valid_len=None, rows_per_seq=0, bf16=False):
    """Row softmax on 16-bit storage (uint16 bit patterns [rows, cols]).  Returns (y_bits, y_float64)."""
    x_bits = _c(x_bits, np.uint16)
    rows, cols = x_bits.shape
    out = np.empty_like(x_bits)
    out64 = np.empty(x_bits.shape, np.float64)
    vl = _c(valid_len, np.int32)
    rc = lib().oracle_softmax_16(_ptr(x_bits, _u16p), _ptr(out, _u16p), _ptr(out64, _f64p), rows, cols,
                                 _ptr(vl, _i32p), int(rows_per_seq), int(bool(bf16)))
    if rc:
        raise ValueError("oracle_softmax_16: bad arguments")
    return out, out64


def layernorm16(x_bits, gamma_bits=None, beta_bits=None, eps=1e-5, unbiased=False, bf16=False):
    """LayerNorm on 16-bit storage.  Returns (y_bits, y_float64, mean float32, rstd float32)."""
    x_bits = _c(x_bits, np.uint16)
    rows, cols = x_bits.shape
    out = np.empty_like(x_bits)
    out64 = np.empty(x_bits.shape, np.float64)
    mean = np.empty(rows, np.float32)
    rstd = np.empty(rows, np.float32)
    g, b = _c(gamma_bits, np.uint16), _c(beta_bits, np.uint16)
    rc = lib().oracle_layernorm_16(_ptr(x_bits, _u16p), _ptr(out, _u16p), _ptr(out64, _f64p), _ptr(mean, _f32p),
                                   _ptr(rstd, _f32p), _ptr(g, _u16p), _ptr(b, _u16p), rows, cols, float(eps),
                                   int(bool(unbiased)), int(bool(bf16)))
    if rc:
        raise ValueError("oracle_layernorm_16: bad arguments")
    return out, out64, mean, rstd


def sgemm(A, B, C=None, alpha=1.0, beta=0.0, want_absprod=False):
    """D = alpha*A@B + beta*C, fp32 in/out, double accumulate.  Row-major."""
    A, B, C = _c(A, np.float32), _c(B, np.float32), _c(C, np.float32)
    m, k = A.shape
    k2, n = B.shape
    assert k == k2
    D = np.empty((m, n), np.float32)
    ap = np.empty((m, n), np.float64) if want_absprod else None
    rc = lib().oracle_sgemm_f32(m, n, k, float(alpha), _ptr(A, _f32p), _ptr(B, _f32p), float(beta),
                                _ptr(C, _f32p), _ptr(D, _f32p), _ptr(ap, _f64p))
    if rc:
        raise ValueError("oracle_sgemm_f32: bad arguments")
    return (D, ap) if want_absprod else D


ACT_NONE, ACT_GELU_ERF, ACT_GELU_TANH = 0, 1, 2


def gemm16(A_bits, B_bits, m, n, k, b_col_major=True, C_bits=None, alpha=1.0, beta=0.0,
           bf16=False, bias_bits=None, act=ACT_NONE):
    """16-bit-input GEMM.  A_bits [m,k], B_bits [n,k] (col-major B) or [k,n]; uint16 bit patterns.

    Returns (D_bits uint16 [m,n], d64 float64 [m,n], absprod float64 [m,n])."""
    A_bits, B_bits, C_bits = _c(A_bits, np.uint16), _c(B_bits, np.uint16), _c(C_bits, np.uint16)
    assert A_bits.size == m * k and B_bits.size == n * k
    D = np.empty((m, n), np.uint16)
    d64 = np.empty((m, n), np.float64)
    ap = np.empty((m, n), np.float64)
    bias_bits = _c(bias_bits, np.uint16)
    assert bias_bits is None or bias_bits.size == n
    rc = lib().oracle_gemm_16_bias_act(m, n, k, float(alpha), _ptr(A_bits, _u16p), _ptr(B_bits, _u16p),
                                       int(bool(b_col_major)), float(beta), _ptr(C_bits, _u16p),
                                       _ptr(bias_bits, _u16p), int(act), _ptr(D, _u16p), int(bool(bf16)),
                                       _ptr(d64, _f64p), _ptr(ap, _f64p))
    if rc:
        raise ValueError("oracle_gemm_16_bias_act: bad arguments")
    return D, d64, ap


def f16_to_f64(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float64)
    lib().oracle_f16_to_f64(_ptr(bits, _u16p), _ptr(out, _f64p), bits.size)
    return out


def f64_to_f16(x):
    x = _c(x, np.float64)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f64_to_f16(_ptr(x, _f64p), _ptr(out, _u16p), x.size)
    return out


def bf16_to_f64(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float64)
    lib().oracle_bf16_to_f64(_ptr(bits, _u16p), _ptr(out, _f64p), bits.size)
    return out


def f64_to_bf16(x):
    x = _c(x, np.float64)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f64_to_bf16(_ptr(x, _f64p), _ptr(out, _u16p), x.size)
    return out
