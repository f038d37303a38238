"""Pins the 16-bit-storage softmax and LayerNorm oracles: exact widening of the inputs, the same
double arithmetic as the fp32 oracles, one rounding to the storage type."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs


def _bits(x, bf16):
    x = np.asarray(x, np.float32)
    return inputs.f32_to_bf16_bits(x).reshape(x.shape) if bf16 else x.astype(np.float16).view(np.uint16)


def _widen(bits, bf16):
    return inputs.bf16_bits_to_f32(bits).astype(np.float64).reshape(bits.shape) if bf16 \
        else bits.view(np.float16).astype(np.float64)


def _round(x64, bf16):
    return oracle.f64_to_bf16(x64) if bf16 else oracle.f64_to_f16(x64)


@pytest.mark.parametrize("bf16", [False, True])
def test_softmax16_matches_float64_and_fp32_oracle(bf16):
    xb = _bits(inputs.normal_f32((9, 136), 5, 0.0, 4.0), bf16)
    yb, y64 = oracle.softmax16(xb, bf16=bf16)
    x = _widen(xb, bf16)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    ref = e / e.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(y64, ref, rtol=1e-14, atol=0)
    np.testing.assert_array_equal(yb, _round(y64, bf16))          # one rounding of the double result
    y32 = oracle.softmax(x.astype(np.float32))                    # the inputs are exact in fp32
    np.testing.assert_allclose(y32, y64, rtol=2.0 ** -24, atol=1e-45)
    if not bf16:                                                  # numpy's own binary16 rounding
        np.testing.assert_array_equal(yb, ref.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("bf16", [False, True])
def test_softmax16_closed_forms_and_mask(bf16):
    const = _bits(np.full((3, 64), 2.5, np.float32), bf16)
    yb, _ = oracle.softmax16(const, bf16=bf16)
    np.testing.assert_array_equal(_widen(yb, bf16), np.full((3, 64), 1.0 / 64))     # 2^-6 is exact in both types
    xb = _bits(inputs.normal_f32((4, 64), 6, 0.0, 3.0), bf16)
    lens = np.array([0, 40], np.int32)
    yb, y64 = oracle.softmax16(xb, lens, 2, bf16=bf16)
    np.testing.assert_array_equal(_widen(yb[:2], bf16), np.full((2, 64), 1.0 / 64))  # fully masked -> uniform
    assert np.all(y64[2:, 40:] == 0.0) and np.all(yb[2:, 40:] == 0)                   # padded columns: exact zero
    inner, _ = oracle.softmax16(np.ascontiguousarray(xb[2:, :40]), bf16=bf16)
    np.testing.assert_array_equal(yb[2:, :40], inner)                                 # valid part = softmax of the slice
    big = _bits(np.array([[60000.0, -60000.0, 0.0, 59000.0] * 2], np.float32), bf16)
    _, y64 = oracle.softmax16(big, bf16=bf16)
    assert np.all(np.isfinite(y64)) and abs(y64.sum() - 1.0) < 1e-12                  # max subtraction


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("unbiased", [False, True])
def test_layernorm16_matches_float64(bf16, unbiased):
    xb = _bits(inputs.normal_f32((7, 264), 8, 0.5, 2.0), bf16)
    gb = _bits(inputs.normal_f32((264,), 9, 1.0, 0.1), bf16)
    bb = _bits(inputs.normal_f32((264,), 10, 0.0, 0.1), bf16)
    eps = 1e-5
    yb, y64, mean, rstd = oracle.layernorm16(xb, gb, bb, eps, unbiased, bf16)
    x, g, b = _widen(xb, bf16), _widen(gb, bf16), _widen(bb, bf16)
    m = x.mean(axis=1)
    r = 1.0 / np.sqrt(x.var(axis=1, ddof=1 if unbiased else 0) + eps)
    ref = (x - m[:, None]) * r[:, None] * g + b
    np.testing.assert_allclose(y64, ref, rtol=1e-12, atol=1e-13)
    np.testing.assert_array_equal(yb, _round(y64, bf16))
    np.testing.assert_allclose(mean, m, rtol=2.0 ** -23)
    np.testing.assert_allclose(rstd, r, rtol=2.0 ** -23)
    y32, m32, r32 = oracle.layernorm(x.astype(np.float32), g.astype(np.float32), b.astype(np.float32), eps, unbiased)
    np.testing.assert_allclose(y32, y64, rtol=2.0 ** -23, atol=1e-7)                 # same arithmetic as the fp32 oracle
    np.testing.assert_array_equal(m32, mean)
    np.testing.assert_array_equal(r32, rstd)


@pytest.mark.parametrize("bf16", [False, True])
def test_layernorm16_closed_forms(bf16):
    cols = 64
    bb = _bits(inputs.uniform_f32((cols,), 11), bf16)
    xb = _bits(np.full((2, cols), 3.0, np.float32), bf16)
    yb, _, mean, rstd = oracle.layernorm16(xb, None, bb, 1e-4, False, bf16)
    np.testing.assert_array_equal(yb, np.broadcast_to(bb, (2, cols)))               # constant row -> y = beta
    np.testing.assert_array_equal(mean, np.float32(3.0))
    np.testing.assert_allclose(rstd, 100.0, rtol=1e-6)
    ramp = _bits(np.arange(cols, dtype=np.float32)[None, :], bf16)                   # 0..63 exact in both types
    _, y64, mean, rstd = oracle.layernorm16(ramp, None, None, 0.0, False, bf16)
    np.testing.assert_allclose(mean, (cols - 1) / 2.0)
    np.testing.assert_allclose(rstd, 1.0 / np.sqrt((cols * cols - 1) / 12.0), rtol=1e-6)
    np.testing.assert_allclose(y64[0, 0], -(cols - 1) / 2.0 / np.sqrt((cols * cols - 1) / 12.0), rtol=1e-12)
