"""Pins the GEMM oracles: the reference's own identity known-answer inputs
(nn_operators/gemm/main.cu:217-235), exact integer cases, numpy float64 matmul, and the
half / bfloat16 conversions against numpy's."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs


def test_sgemm_identity_kat():
    n = 128
    A = (np.arange(n * n) // 1024).astype(np.float32).reshape(n, n)  # A[idx] = idx / 1024 (integer division)
    np.testing.assert_array_equal(oracle.sgemm(A, np.eye(n, dtype=np.float32)), A)


def test_sgemm_all_ones_and_integers():
    np.testing.assert_array_equal(oracle.sgemm(np.ones((8, 100), np.float32), np.ones((100, 12), np.float32)),
                                  np.full((8, 12), 100, np.float32))
    rng = np.random.default_rng(0)
    A = rng.integers(-4, 5, (33, 1024)).astype(np.float32)
    B = rng.integers(-4, 5, (1024, 20)).astype(np.float32)
    np.testing.assert_array_equal(oracle.sgemm(A, B), A.astype(np.float64) @ B.astype(np.float64))


def test_sgemm_matches_float64_matmul_and_layout():
    A = inputs.uniform_f32((37, 53), 1)
    B = inputs.uniform_f32((53, 29), 2)  # non-square: a transposed operand or swapped index would fail
    C = inputs.normal_f32((37, 29), 3)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    D, ap = oracle.sgemm(A, B, want_absprod=True)
    np.testing.assert_array_equal(D, ref.astype(np.float32))
    np.testing.assert_allclose(ap, np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64), rtol=1e-14)
    np.testing.assert_array_equal(oracle.sgemm(A, B, C, 1.0, 1.0), (ref + C).astype(np.float32))  # D = acc + C
    np.testing.assert_allclose(oracle.sgemm(A, B, C, 0.5, -2.0), 0.5 * ref - 2.0 * C, rtol=1e-6, atol=1e-6)
    np.testing.assert_array_equal(oracle.sgemm(A, B, None, 1.0, 5.0), ref.astype(np.float32))  # C null: beta ignored


def test_f16_conversions_match_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float64)
    got = oracle.f16_to_f64(bits)
    finite = np.isfinite(vals)
    np.testing.assert_array_equal(got[finite], vals[finite])
    assert np.all(np.isnan(got[np.isnan(vals)]))
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.normal(0, 10, 20000), rng.normal(0, 1e-6, 20000), rng.uniform(-70000, 70000, 20000),
                        vals[finite], (vals[finite][:-1] + vals[finite][1:]) / 2])  # includes exact ties
    x = x[np.isfinite(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(oracle.f64_to_f16(x), want)


def test_bf16_conversions():
    rng = np.random.default_rng(2)
    x32 = rng.normal(0, 5, 50000).astype(np.float32)
    bits = inputs.f32_to_bf16_bits(x32)
    np.testing.assert_array_equal(oracle.f64_to_bf16(x32.astype(np.float64)), bits)
    np.testing.assert_array_equal(oracle.bf16_to_f64(bits), inputs.bf16_bits_to_f32(bits).astype(np.float64))


@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("bf16", [False, True])
def test_gemm16_matches_float64_matmul(b_col_major, bf16):
    m, n, k = 19, 23, 40
    if bf16:
        A = inputs.uniform_bf16_bits((m, k), 1)
        Bt = inputs.uniform_bf16_bits((n, k), 2)
        a64, b64 = oracle.bf16_to_f64(A), oracle.bf16_to_f64(Bt)
    else:
        A = inputs.uniform_f16((m, k), 1).view(np.uint16)
        Bt = inputs.uniform_f16((n, k), 2).view(np.uint16)
        a64, b64 = oracle.f16_to_f64(A), oracle.f16_to_f64(Bt)
    B = Bt if b_col_major else np.ascontiguousarray(Bt.T)
    D, d64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, bf16=bf16)
    ref = a64 @ b64.T
    np.testing.assert_allclose(d64, ref, rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(ap, np.abs(a64) @ np.abs(b64).T, rtol=1e-13)
    back = oracle.bf16_to_f64(D) if bf16 else oracle.f16_to_f64(D)
    np.testing.assert_allclose(back, ref, rtol=2.0 ** -8 if bf16 else 2.0 ** -11, atol=2.0 ** -24)


def test_gemm16_identity_kat_and_epilogue():
    n = 64
    A = (np.arange(n * n) // 1024).astype(np.float16)
    I = np.eye(n, dtype=np.float16)
    D, _, _ = oracle.gemm16(A.view(np.uint16), I.view(np.uint16), n, n, n, b_col_major=False)
    np.testing.assert_array_equal(D.view(np.float16), A.reshape(n, n))
    C = inputs.uniform_f16((n, n), 4, -2.0, 2.0)
    D, d64, _ = oracle.gemm16(A.view(np.uint16), I.view(np.uint16), n, n, n, C_bits=C.view(np.uint16), alpha=1.0, beta=1.0)
    np.testing.assert_array_equal(d64, A.reshape(n, n).astype(np.float64) + C.astype(np.float64))
