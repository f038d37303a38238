"""Parity gates between the HIP kernels and the CPU oracle (the tolerances are part of the tests).

softmax   |d| <= 1e-6  and  |d| <= 1e-5 * |ref| wherever |ref| >= FLT_MIN
LayerNorm |dy| <= 1e-5 * max(|ref|, 1);  rstd: |d| <= 1e-5 * |ref|;
          mean: |d| <= 1e-5 * max(|ref mean|, ref std) with ref std = 1/ref rstd.  The mean is a sum with
          cancellation: its fp32 partial sums are of the size of the row's spread, so an error relative to
          |mean| alone is out of reach of any fp32 reduction when |mean| << std (partial sums of size
          std*sqrt(n) carry an ulp of about 1e-7*std each)
SGEMM     |d| <= 2 K 2^-24 * sum_k |a_ik||b_kj|   (any summation order), plus the reference's own
          gate |d| <= 1e-3 (nn_operators/gemm/main.cu:169-170) where the test says so
GEMM16    |d| <= 2^-11 |ref| + K 2^-24 sum_k |a_ik||b_kj| + 2^-24   (one rounding to 16 bits + fp32 sums);
          bfloat16 output: 2^-8 |ref| instead of 2^-11 |ref|
"""
import numpy as np

FLT_MIN = np.finfo(np.float32).tiny


def assert_softmax_close(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape
    assert np.all(np.isfinite(got)), "non-finite softmax output"
    d = np.abs(got - ref)
    assert d.max() <= 1e-6, "softmax abs err %.3e > 1e-6" % d.max()
    sel = ref >= FLT_MIN
    rel = d[sel] / ref[sel]
    assert rel.size == 0 or rel.max() <= 1e-5, "softmax rel err %.3e > 1e-5" % rel.max()
    return d.max(), (rel.max() if rel.size else 0.0)


def assert_layernorm_close(got, ref):
    (y, mean, rstd), (ry, rmean, rrstd) = got, ref
    y, ry = np.asarray(y, np.float64), np.asarray(ry, np.float64)
    assert np.all(np.isfinite(y))
    dy = np.abs(y - ry) / np.maximum(np.abs(ry), 1.0)
    assert dy.max() <= 1e-5, "layernorm y err %.3e > 1e-5" % dy.max()
    if mean is not None:
        mean, rmean = np.asarray(mean, np.float64), np.asarray(rmean, np.float64)
        scale = np.maximum(np.abs(rmean), 1.0 / np.asarray(rrstd, np.float64))
        dm = np.abs(mean - rmean) / scale
        assert dm.max() <= 1e-5, "layernorm mean err %.3e > 1e-5" % dm.max()
    if rstd is not None:
        rstd, rrstd = np.asarray(rstd, np.float64), np.asarray(rrstd, np.float64)
        dr = np.abs(rstd - rrstd) / np.abs(rrstd)
        assert dr.max() <= 1e-5, "layernorm rstd err %.3e > 1e-5" % dr.max()
    return dy.max()


def assert_sgemm_close(got, ref, absprod, k, reference_gate=False):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert np.all(np.isfinite(got))
    d = np.abs(got - ref)
    bound = 2.0 * k * 2.0 ** -24 * absprod + 1e-30
    worst = (d / bound).max()
    assert worst <= 1.0, "sgemm err exceeds 2K*2^-24*|A||B| by factor %.3f" % worst
    if reference_gate:
        assert d.max() <= 1e-3, "sgemm abs err %.3e > 1e-3" % d.max()
    return d.max(), worst


def assert_gemm16_close(got_f64, ref_f64, absprod, k, bf16=False):
    got, ref = np.asarray(got_f64, np.float64), np.asarray(ref_f64, np.float64)
    assert np.all(np.isfinite(got))
    d = np.abs(got - ref)
    ulp = 2.0 ** -8 if bf16 else 2.0 ** -11
    bound = ulp * np.abs(ref) + k * 2.0 ** -24 * absprod + 2.0 ** -24
    worst = (d / bound).max()
    assert worst <= 1.0, "gemm16 err exceeds bound by factor %.3f" % worst
    return d.max(), worst


# 16-bit storage (binary16 / bfloat16 in and out, fp32 arithmetic): the fp32 gates above plus one
# rounding to the storage type - half an ulp, i.e. 2^-11 |ref| (binary16; 2^-25 absolute in its
# subnormal range) or 2^-8 |ref| (bfloat16).
def _round16_bound(ref, bf16):
    return (2.0 ** -8 if bf16 else 2.0 ** -11) * np.abs(ref) + (0.0 if bf16 else 2.0 ** -25)


def assert_softmax16_close(got64, ref64, bf16=False):
    got, ref = np.asarray(got64, np.float64), np.asarray(ref64, np.float64)
    assert got.shape == ref.shape and np.all(np.isfinite(got))
    d = np.abs(got - ref)
    bound = _round16_bound(ref, bf16) + np.minimum(1e-6, 1e-5 * np.abs(ref)) + 1e-45
    worst = (d / bound).max()
    assert worst <= 1.0, "softmax16 err exceeds rounding + fp32 gate by factor %.3f" % worst
    return worst


def assert_layernorm16_close(got, ref, bf16=False):
    (y, mean, rstd), (ry64, rmean, rrstd) = got, ref
    y, ry = np.asarray(y, np.float64), np.asarray(ry64, np.float64)
    assert np.all(np.isfinite(y))
    bound = _round16_bound(ry, bf16) + 1e-5 * np.maximum(np.abs(ry), 1.0)
    worst = (np.abs(y - ry) / bound).max()
    assert worst <= 1.0, "layernorm16 y err exceeds rounding + fp32 gate by factor %.3f" % worst
    mean, rmean = np.asarray(mean, np.float64), np.asarray(rmean, np.float64)
    rstd, rrstd = np.asarray(rstd, np.float64), np.asarray(rrstd, np.float64)
    scale = np.maximum(np.abs(rmean), 1.0 / rrstd)
    assert (np.abs(mean - rmean) / scale).max() <= 1e-5
    assert (np.abs(rstd - rrstd) / rrstd).max() <= 1e-5
    return worst
