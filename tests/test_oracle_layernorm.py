"""Pins the LayerNorm oracle (two-pass double) and the float Welford restatement
(nn_operators/layernorm/layernorm.h:13-47 with the merge fixed) without the reference."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs


def test_constant_row():
    cols = 768
    g = inputs.normal_f32((cols,), 1, 1.0, 0.1)
    b = inputs.normal_f32((cols,), 2, 0.0, 0.1)
    y, m, r = oracle.layernorm(np.full((2, cols), 3.5, np.float32), g, b, eps=1e-5)
    np.testing.assert_array_equal(y, np.broadcast_to(b, y.shape))
    np.testing.assert_array_equal(m, [3.5, 3.5])
    np.testing.assert_allclose(r, 1 / np.sqrt(1e-5), rtol=1e-7)


def test_arithmetic_progression_closed_form():
    for cols in (4, 128, 768):
        x = np.arange(cols, dtype=np.float32)[None]
        y, m, r = oracle.layernorm(x, eps=0.0)
        var = (cols * cols - 1) / 12.0
        np.testing.assert_allclose(m, (cols - 1) / 2, rtol=1e-7)
        np.testing.assert_allclose(r, 1 / np.sqrt(var), rtol=1e-7)
        np.testing.assert_allclose(y[0], (np.arange(cols) - (cols - 1) / 2) / np.sqrt(var), rtol=1e-6, atol=1e-7)
        _, _, ru = oracle.layernorm(x, eps=0.0, unbiased=True)
        np.testing.assert_allclose(ru, 1 / np.sqrt(var * cols / (cols - 1)), rtol=1e-7)  # Bessel


def test_output_moments():
    x = inputs.normal_f32((64, 768), 5, 0.5, 2.0)
    y, m, r = oracle.layernorm(x, eps=1e-5)
    y64 = y.astype(np.float64)
    assert np.abs(y64.mean(1)).max() < 1e-6
    var = x.astype(np.float64).var(1)
    np.testing.assert_allclose(y64.var(1), var / (var + 1e-5), rtol=1e-5)
    np.testing.assert_allclose(m, x.astype(np.float64).mean(1), rtol=1e-6)
    np.testing.assert_allclose(r, 1 / np.sqrt(var + 1e-5), rtol=1e-6)


def test_affine_is_applied_after_normalisation():
    x = inputs.normal_f32((8, 128), 7, 0.5, 2.0)
    g = inputs.normal_f32((128,), 8, 1.0, 0.1)
    b = inputs.normal_f32((128,), 9, 0.0, 0.1)
    y0, _, _ = oracle.layernorm(x)
    y1, _, _ = oracle.layernorm(x, g, b)
    np.testing.assert_allclose(y1, y0.astype(np.float64) * g + b, rtol=3e-7, atol=1e-7)
    yg, _, _ = oracle.layernorm(x, gamma=g)
    np.testing.assert_allclose(yg, y0.astype(np.float64) * g, rtol=3e-7, atol=1e-7)


def test_library_third_opinion():
    torch = pytest.importorskip("torch")
    x = inputs.normal_f32((128, 768), 11, 0.5, 2.0)
    g = inputs.normal_f32((768,), 12, 1.0, 0.1)
    b = inputs.normal_f32((768,), 13, 0.0, 0.1)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (768,), torch.from_numpy(g).double(),
                                         torch.from_numpy(b).double(), eps=1e-5).numpy()
    y, _, _ = oracle.layernorm(x, g, b, eps=1e-5)
    np.testing.assert_allclose(y, ref, rtol=2e-7, atol=2e-7)


def test_offset_stability():
    """x = 1e4 + N(0,1): a naive fp32 E[x^2] - E[x]^2 loses everything; the oracle (double two-pass) and
    the float Welford restatement must agree with an exact-rational style computation."""
    x = (1.0e4 + inputs.normal_f64(4 * 768, 3, 0.0, 1.0)).astype(np.float32).reshape(4, 768)
    y, m, r = oracle.layernorm(x)
    x64 = x.astype(np.float64)
    d = x64 - x64.mean(1, keepdims=True)
    np.testing.assert_allclose(r, 1 / np.sqrt((d * d).mean(1) + 1e-5), rtol=1e-7)
    # The float restatement keeps the reference's unshifted fp32 triplets: every partial mean is rounded
    # to an ulp of 1e4 (about 5e-4 of the spread), which costs a few 1e-5 of the variance.
    yw, mw, rw = oracle.layernorm_welford(x, lanes=64, vec_len=4)
    np.testing.assert_allclose(rw, r, rtol=2e-4)
    assert np.abs(rw / r - 1).max() > 2e-6  # ... and the loss is real: the HIP kernels shift the row first
    np.testing.assert_allclose(mw, m, rtol=1e-6)
    naive_var = (x * x).mean(1, dtype=np.float32) - x.mean(1, dtype=np.float32) ** 2
    assert np.abs(naive_var - (d * d).mean(1)).max() > 0.1  # the failure mode the Welford form avoids


@pytest.mark.parametrize("lanes,vec_len,cols", [(32, 4, 768), (64, 4, 768), (16, 4, 128), (64, 4, 260), (8, 1, 36),
                                               (32, 4, 4)])
def test_welford_merge_algebra(lanes, vec_len, cols):
    """Streaming update + Chan merge (layernorm.h:13-23, :36-47) == two-pass, for even and ragged
    lane loads (lanes with no elements merge as the identity)."""
    x = inputs.normal_f32((16, cols), 17 + cols, 0.5, 2.0)
    for unbiased in (False, True):
        y, m, r = oracle.layernorm(x, unbiased=unbiased)
        yw, mw, rw = oracle.layernorm_welford(x, unbiased=unbiased, lanes=lanes, vec_len=vec_len)
        np.testing.assert_allclose(mw, m, rtol=2e-6, atol=2e-7)
        np.testing.assert_allclose(rw, r, rtol=5e-6)
        np.testing.assert_allclose(yw, y, rtol=1e-5, atol=1e-5)


def test_welford_equal_count_closed_form():
    """Two halves with equal counts: mean = (ma+mb)/2, M2 = M2a + M2b + (mb-ma)^2 * n/2."""
    x = inputs.normal_f64(512, 23, 0.5, 2.0)
    a, b = x[:256], x[256:]
    ma, mb = a.mean(), b.mean()
    m2 = ((a - ma) ** 2).sum() + ((b - mb) ** 2).sum() + (mb - ma) ** 2 * 256 / 2
    np.testing.assert_allclose(m2, ((x - x.mean()) ** 2).sum(), rtol=1e-12)
    _, mo, ro = oracle.layernorm(x.astype(np.float32)[None], eps=0.0)
    x32 = x.astype(np.float32).astype(np.float64)
    np.testing.assert_allclose(ro, 1 / np.sqrt(x32.var()), rtol=1e-7)


def test_reference_bug_is_not_reproduced():
    """Dividing M2 by count-1 inside every merge (layernorm.h:48) does not give a variance; the oracle's
    rstd is the true one, far from what that recurrence yields."""
    x = inputs.normal_f32((1, 768), 29, 0.5, 2.0)
    _, _, r = oracle.layernorm(x, eps=0.0, unbiased=True)
    np.testing.assert_allclose(r, 1 / x.astype(np.float64).std(ddof=1), rtol=1e-7)


def test_special_values_leave_a_row_without_statistics():
    """A NaN or an infinity in a row: y, mean and rstd of that row are NaN (the sum of squared deviations is
    inf - inf); other rows are untouched."""
    import special_values as sv
    cols = 40
    base = inputs.normal_f32((5, cols), 78, 0.5, 2.0)
    x, classes = sv.build(sv.LAYERNORM_ROWS, cols, base)
    g = inputs.normal_f32((cols,), 79, 1.0, 0.1)
    b = inputs.normal_f32((cols,), 80, 0.0, 0.1)
    y, mean, rstd = oracle.layernorm(x, g, b)
    ok = sv.check_rows(y, y, classes, "oracle layernorm y")
    sv.check_rows(mean, mean, classes, "oracle layernorm mean")
    sv.check_rows(rstd, rstd, classes, "oracle layernorm rstd")
    clean = np.array([base[i % 5] for i in range(x.shape[0])], np.float32)
    yc, mc, rc = oracle.layernorm(clean, g, b)
    np.testing.assert_array_equal(y[ok], yc[ok])
    np.testing.assert_array_equal(mean[ok], mc[ok])
    np.testing.assert_array_equal(rstd[ok], rc[ok])
