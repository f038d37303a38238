"""GPU parity on seeded random shapes under the AUTO policy: row counts and row lengths drawn log-uniformly, odd
lengths included, so that every dispatch path (lane groups of 1 to 64, workgroup kernels, re-reading, element-wise,
pieces of a few long rows) is reached by shapes nobody picked by hand.  Against the oracle at the usual gates."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs
from tolerances import (assert_layernorm16_close, assert_layernorm_close, assert_softmax16_close,
                        assert_softmax_close)

pytestmark = pytest.mark.gpu


def _shapes(seed, count, max_elems=6_000_000):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        rows = int(np.exp(rng.uniform(0, np.log(20000))))
        cols = int(np.exp(rng.uniform(0, np.log(300000))))
        if rows * cols <= max_elems:
            out.append((rows, cols))
    return out


def _bits(x, bf16):
    x = np.asarray(x, np.float32)
    return inputs.f32_to_bf16_bits(x).reshape(x.shape) if bf16 else x.astype(np.float16).view(np.uint16)


def _to64(bits, bf16):
    return oracle.bf16_to_f64(bits) if bf16 else oracle.f16_to_f64(bits)


@pytest.mark.parametrize("rows,cols", _shapes(1, 40))
def test_softmax_random_shapes(ko, rows, cols):
    x = inputs.normal_f32((rows, cols), rows + cols, 0.0, 4.0)
    assert_softmax_close(ko.softmax_host(x), oracle.softmax(x))
    rps = 1 + rows % 3
    vl = np.random.default_rng(rows).integers(0, cols + 1, (rows + rps - 1) // rps).astype(np.int32)
    assert_softmax_close(ko.softmax_host(x, vl, rps), oracle.softmax(x, vl, rps))


@pytest.mark.parametrize("rows,cols", _shapes(2, 40))
def test_layernorm_random_shapes(ko, rows, cols):
    if cols < 2:
        cols = 2  # one column has no variance to speak of with the unbiased divisor
    x = inputs.normal_f32((rows, cols), rows + cols, 0.5, 2.0)
    g = inputs.normal_f32((cols,), 3, 1.0, 0.1)
    b = inputs.normal_f32((cols,), 4, 0.0, 0.1)
    unbiased = bool(rows % 2)
    assert_layernorm_close(ko.layernorm_host(x, g, b, 1e-5, unbiased), oracle.layernorm(x, g, b, 1e-5, unbiased))
    assert_layernorm_close(ko.layernorm_host(x), oracle.layernorm(x))


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,cols", _shapes(3, 16))
def test_rows16_random_shapes(ko, rows, cols, bf16):
    dt = ko.BF16 if bf16 else ko.F16
    cols = max(cols, 2)
    xb = _bits(inputs.normal_f32((rows, cols), rows + cols, 0.0, 3.0), bf16)
    _, ref64 = oracle.softmax16(xb, bf16=bf16)
    assert_softmax16_close(_to64(ko.softmax16_host(xb, dtype=dt), bf16), ref64, bf16)
    gb = _bits(inputs.normal_f32((cols,), 5, 1.0, 0.1), bf16)
    _, ref64, rmean, rrstd = oracle.layernorm16(xb, gb, None, 1e-5, False, bf16)
    y, mean, rstd = ko.layernorm16_host(xb, gb, None, 1e-5, False, dtype=dt)
    assert_layernorm16_close((_to64(y, bf16), mean, rstd), (ref64, rmean, rrstd), bf16)


def _gemm_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        m = int(np.exp(rng.uniform(0, np.log(6000))))
        n = int(np.exp(rng.uniform(0, np.log(6000))))
        k = 8 * int(np.exp(rng.uniform(0, np.log(1024))))
        if m * n <= 6_000_000 and (m + n) * k <= 12_000_000:
            out.append((m, n, k))
    return out


@pytest.mark.parametrize("m,n,k", _gemm_shapes(4, 30))
def test_gemm16_random_shapes_are_exact_on_small_integers(ko, m, n, k):
    """Random M, N and K (a multiple of 8), both layouts of B, binary16 and bfloat16 by turns, with C and a bias:
    small integers, so the whole output equals the exact result rounded once."""
    bf16 = bool((m + n) % 2)
    b_col_major = bool(k // 8 % 2)
    rng = np.random.default_rng(m * 7 + n)
    f16 = lambda x: oracle.f64_to_bf16(x) if bf16 else oracle.f64_to_f16(x)
    A = rng.integers(-2, 3, (m, k)).astype(np.float64)
    B = rng.integers(-2, 3, (n, k)).astype(np.float64)
    C = rng.integers(-8, 9, (m, n)).astype(np.float64)
    bias = rng.integers(-8, 9, (n,)).astype(np.float64)
    exact = A @ B.T
    Bm = B if b_col_major else np.ascontiguousarray(B.T)
    kw = dict(b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR, dtype=ko.BF16 if bf16 else ko.F16)
    np.testing.assert_array_equal(ko.gemm16_host(f16(A), f16(Bm), m, n, k, **kw), f16(exact))
    got = ko.gemm16_host(f16(A), f16(Bm), m, n, k, C_bits=f16(C), alpha=1.0, beta=-1.0, bias_bits=f16(bias), **kw)
    np.testing.assert_array_equal(got, f16(exact - C + bias))


@pytest.mark.parametrize("m,n,k", _gemm_shapes(5, 30))
def test_sgemm_random_shapes_are_exact_on_small_integers(ko, m, n, k):
    k = max(1, k // 8 * (1 + m % 8) // 1) if m % 3 else k + m % 5   # not only multiples of 8
    rng = np.random.default_rng(m * 11 + n)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    C = rng.integers(-8, 9, (m, n)).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_array_equal(ko.sgemm_host(A, B), ref)
    np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C)
