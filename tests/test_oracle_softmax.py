"""Pins the softmax oracle without the reference (which holds no vectors and no CPU softmax):
closed forms, invariants, brute force in extended precision and a library routine."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs


def brute_softmax(x):
    """Textbook definition in long double, no max subtraction needed at these magnitudes."""
    x = np.asarray(x, np.longdouble)
    e = np.exp(x)
    return (e / e.sum(axis=-1, keepdims=True)).astype(np.float64)


def test_constant_rows_are_uniform():
    for cols in (4, 128, 512):
        y = oracle.softmax(np.full((3, cols), -7.25, np.float32))
        np.testing.assert_array_equal(y, np.full((3, cols), 1.0 / cols, np.float32))


def test_brute_force_small_rows():
    rng = np.random.default_rng(0)
    x = rng.normal(0, 4, (64, 12)).astype(np.float32)
    np.testing.assert_allclose(oracle.softmax(x), brute_softmax(x), rtol=2e-7, atol=0)


def test_two_element_closed_form():
    # softmax([a, b]) = [1/(1+e^(b-a)), 1/(1+e^(a-b))]; padded to the vector width with -inf-like columns
    a, b = 1.5, -0.75
    x = np.array([[a, b, -1e30, -1e30]], np.float32)
    y = oracle.softmax(x)[0]
    np.testing.assert_allclose(y[:2], [1 / (1 + np.exp(b - a)), 1 / (1 + np.exp(a - b))], rtol=1e-7)
    assert y[2] == 0 and y[3] == 0


def test_shift_invariance_and_normalisation():
    x = inputs.normal_f32((32, 128), 3, 0.0, 4.0)
    xq = np.round(x * 64) / 64
    np.testing.assert_array_equal(oracle.softmax(xq), oracle.softmax(xq + np.float32(32)))
    y = oracle.softmax(x)
    assert np.abs(y.sum(1, dtype=np.float64) - 1).max() < 128 * 2.0 ** -24
    order = np.argsort(x, axis=1)
    assert np.all(np.diff(np.take_along_axis(y, order, 1), axis=1) >= 0)  # order preserved


def test_max_subtraction_large_magnitudes():
    """exp(x) alone overflows fp32 here; the reference's x + max (functors.h:168) would too."""
    x = np.array([[88.0, 90.0, -90.0, 89.0], [1e4, 1e4, 0.0, -1e4]], np.float32)
    y = oracle.softmax(x)
    assert np.all(np.isfinite(y))
    np.testing.assert_allclose(y[0], brute_softmax(x[0] - 90.0), rtol=1e-7, atol=1e-45)  # 4e-79 underflows fp32
    np.testing.assert_allclose(y[1], [0.5, 0.5, 0, 0])


def test_one_hot_dominance():
    x = np.zeros((1, 128), np.float32)
    x[0, 17] = 100.0
    y = oracle.softmax(x)
    assert y[0, 17] == 1.0 and y[0].argmax() == 17 and np.all(y[0, :17] < 1e-40)


def test_library_third_opinion():
    torch = pytest.importorskip("torch")
    x = inputs.normal_f32((256, 128), 9, 0.0, 4.0)
    ref = torch.softmax(torch.from_numpy(x).double(), dim=-1).numpy()
    np.testing.assert_allclose(oracle.softmax(x), ref, rtol=1.5e-7, atol=1e-45)


def test_mask_semantics():
    rows_per_seq, cols = 3, 16
    vl = np.array([5, 16, 0, 1], np.int32)
    x = inputs.normal_f32((rows_per_seq * 4, cols), 1, 0.0, 4.0)
    y = oracle.softmax(x, valid_len=vl, rows_per_seq=rows_per_seq)
    # "set to -10000" == softmax of the row with the padded entries replaced
    xm = x.copy()
    for s, L in enumerate(vl):
        xm[s * rows_per_seq:(s + 1) * rows_per_seq, L:] = inputs.MASK_VALUE
    np.testing.assert_array_equal(y, oracle.softmax(xm))
    # "add -10000" gives the same bits (exp of <= -9900 is exactly 0 in fp32 next to an O(1) sum)
    xa = x.copy()
    for s, L in enumerate(vl):
        xa[s * rows_per_seq:(s + 1) * rows_per_seq, L:] += np.float32(inputs.MASK_VALUE)
    ya = oracle.softmax(xa)
    np.testing.assert_array_equal(y[:6], ya[:6])
    # valid part == unmasked softmax of the valid slice; padded part exactly 0
    np.testing.assert_allclose(y[0, :5], brute_softmax(x[0, :5]), rtol=2e-7)
    assert np.all(y[:3, 5:] == 0)
    # fully masked row -> uniform, never NaN; equal valid values -> 1/L
    np.testing.assert_array_equal(y[6:9], np.full((3, cols), 1.0 / cols, np.float32))
    xe = np.full((1, cols), 2.0, np.float32)
    ye = oracle.softmax(xe, valid_len=np.array([4], np.int32), rows_per_seq=1)
    np.testing.assert_array_equal(ye[0], [0.25] * 4 + [0.0] * 12)
    # ragged last sequence and out-of-range lengths are clamped
    y2 = oracle.softmax(x[:10], valid_len=np.array([5, 16, 0, 99], np.int32), rows_per_seq=3)
    np.testing.assert_array_equal(y2[:9], y[:9])
    np.testing.assert_array_equal(y2[9], oracle.softmax(x[9:10])[0])


def test_bad_arguments():
    with pytest.raises(ValueError):
        oracle.softmax(np.zeros((2, 4), np.float32), valid_len=np.array([1], np.int32), rows_per_seq=0)


def test_special_values_follow_the_reference_arithmetic():
    """NaN and +inf poison their row (exp(x - max) is NaN), -inf elements get probability 0, a row of -inf is
    0/0 = NaN, a row of -FLT_MAX is uniform (softmax.h:33: the running maximum starts at -FLT_MAX)."""
    import special_values as sv
    cols = 24
    base = inputs.normal_f32((5, cols), 77, 0.0, 4.0)
    x, classes = sv.build(sv.SOFTMAX_ROWS, cols, base)
    y = oracle.softmax(x)
    ok = sv.check_rows(y, y, classes, "oracle softmax")
    names = [n for n, _, _ in sv.SOFTMAX_ROWS]
    # ordinary rows: equal to a float64 numpy softmax over the finite part, exact zeros at -inf
    for i in np.nonzero(ok)[0]:
        r = x[i].astype(np.float64)
        if names[i] == "minus_flt_max_all":
            np.testing.assert_array_equal(y[i], np.float32(1.0 / cols))
            continue
        fin = np.isfinite(r)
        e = np.exp(r[fin] - r[fin].max())
        np.testing.assert_allclose(y[i][fin], e / e.sum(), rtol=1e-6)
        np.testing.assert_array_equal(y[i][~fin], 0.0)
    # a masked row ignores what lies in the padding, special values included
    xm = base[:1].copy()
    xm[0, 10:] = [np.nan, np.inf, -np.inf] + [np.nan] * (cols - 13)
    ym = oracle.softmax(xm, np.array([10], np.int32), 1)
    np.testing.assert_array_equal(ym, oracle.softmax(base[:1], np.array([10], np.int32), 1))
