"""GPU parity for a few long rows (rows for at most a quarter of the compute units, or half of them when rows are 1 MB
and longer): under the AUTO policy such a row is cut into pieces that run as workgroups of their own, in two launches that hand the
pieces' partial results over through the stream's workspace.  Against the oracle at the usual gates - with masks,
special values, 16-bit storage, in place - and the same bits from call to call."""
import numpy as np
import pytest

import oracle
import special_values as sv
from kernel_optimization_amd import inputs
from tolerances import (assert_layernorm16_close, assert_layernorm_close, assert_softmax16_close,
                        assert_softmax_close)

pytestmark = pytest.mark.gpu

# rows of 256 KB and more for up to 64 rows, of 1 MB and more for up to 128 (what the library cuts into pieces), and
# two shapes just outside (65 rows, rows just under 256 KB) that stay with one workgroup per row
SHAPES = [(1, 65536), (1, 1000000), (3, 131072), (64, 128256), (128, 262148), (16, 262148), (2, 70000), (100, 300000),
          (65, 128256), (4, 65532)]


def _bits(x, bf16):
    x = np.asarray(x, np.float32)
    with np.errstate(over="ignore"):
        return inputs.f32_to_bf16_bits(x).reshape(x.shape) if bf16 else x.astype(np.float16).view(np.uint16)


def _to64(bits, bf16):
    return oracle.bf16_to_f64(bits) if bf16 else oracle.f16_to_f64(bits)


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_softmax_few_long_rows(ko, rows, cols):
    x = inputs.normal_f32((rows, cols), 800 + rows, 0.0, 4.0)
    ref = oracle.softmax(x)
    got = ko.softmax_host(x)
    assert_softmax_close(got, ref)
    np.testing.assert_array_equal(ko.softmax_host(x), got)               # the same bits from call to call
    assert_softmax_close(ko.softmax_host(x, in_place=True), ref)
    np.testing.assert_allclose(got, ko.softmax_host(x, policy=3), rtol=1e-5, atol=1e-7)   # the one-workgroup-per-row kernel
    rps = 2
    vl = np.random.default_rng(cols).integers(0, cols + 1, (rows + rps - 1) // rps).astype(np.int32)
    assert_softmax_close(ko.softmax_host(x, vl, rps), oracle.softmax(x, vl, rps))


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,cols", [(1, 131072), (5, 256000), (64, 140000), (100, 530000)])
def test_softmax16_few_long_rows(ko, rows, cols, bf16):
    dt = ko.BF16 if bf16 else ko.F16
    xb = _bits(inputs.normal_f32((rows, cols), 810 + rows, 0.0, 4.0), bf16)
    _, ref64 = oracle.softmax16(xb, bf16=bf16)
    assert_softmax16_close(_to64(ko.softmax16_host(xb, dtype=dt), bf16), ref64, bf16)


def test_softmax_few_long_rows_special_values(ko):
    cols = 70000
    base = inputs.normal_f32((5, cols), 820, 0.0, 4.0)
    x, classes = sv.build(sv.SOFTMAX_ROWS, cols, base, repeat=2)
    ref = oracle.softmax(x)
    got = ko.softmax_host(x)
    ok = sv.check_rows(got, ref, classes, "softmax few rows")
    assert_softmax_close(got[ok], ref[ok])


@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_layernorm_few_long_rows(ko, rows, cols, affine):
    x = inputs.normal_f32((rows, cols), 830 + rows, 0.5, 2.0)
    g = inputs.normal_f32((cols,), 831, 1.0, 0.1) if affine else None
    b = inputs.normal_f32((cols,), 832, 0.0, 0.1) if affine else None
    ref = oracle.layernorm(x, g, b, 1e-5, True)
    got = ko.layernorm_host(x, g, b, 1e-5, True)
    assert_layernorm_close(got, ref)
    again = ko.layernorm_host(x, g, b, 1e-5, True)
    for a1, a2 in zip(got, again):
        np.testing.assert_array_equal(a1, a2)                               # the same bits from call to call
    assert_layernorm_close(ko.layernorm_host(x, g, b, 1e-5, True, in_place=True), ref)
    # a large common offset: the statistics are taken of x - x0 in every piece
    x2 = (x + 1.0e4).astype(np.float32)
    assert_layernorm_close(ko.layernorm_host(x2, g, b), oracle.layernorm(x2, g, b))


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,cols", [(1, 131072), (5, 256000), (64, 140000), (100, 530000)])
def test_layernorm16_few_long_rows(ko, rows, cols, bf16):
    dt = ko.BF16 if bf16 else ko.F16
    xb = _bits(inputs.normal_f32((rows, cols), 840 + rows, 0.5, 2.0), bf16)
    gb = _bits(inputs.normal_f32((cols,), 841, 1.0, 0.1), bf16)
    bb = _bits(inputs.normal_f32((cols,), 842, 0.0, 0.1), bf16)
    _, ref64, rmean, rrstd = oracle.layernorm16(xb, gb, bb, 1e-5, False, bf16)
    y, mean, rstd = ko.layernorm16_host(xb, gb, bb, 1e-5, False, dtype=dt)
    assert_layernorm16_close((_to64(y, bf16), mean, rstd), (ref64, rmean, rrstd), bf16)


def test_layernorm_few_long_rows_special_values(ko):
    cols = 70000
    base = inputs.normal_f32((5, cols), 850, 0.5, 2.0)
    x, classes = sv.build(sv.LAYERNORM_ROWS, cols, base, repeat=2)
    ref = oracle.layernorm(x)
    got = ko.layernorm_host(x)
    ok = None
    for name, a, r in zip(("y", "mean", "rstd"), got, ref):
        ok = sv.check_rows(a, r, classes, "layernorm few rows %s" % name)
    assert_layernorm_close(tuple(a[ok] for a in got), tuple(r[ok] for r in ref))
