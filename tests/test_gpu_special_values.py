"""GPU parity on rows that hold NaN and infinities: the kernels (through the C ABI) and the oracle agree on
which rows are NaN, and ordinary rows next to them keep their usual tolerance.  The expected behaviour is what
the reference's arithmetic gives (expf of NaN or of inf - inf, nn_operators/softmax/softmax.h:46; the Welford
update on an infinity, nn_operators/layernorm/layernorm.h:16-22)."""
import numpy as np
import pytest

import oracle
import special_values as sv
from kernel_optimization_amd import inputs
from tolerances import (assert_layernorm16_close, assert_layernorm_close, assert_softmax16_close,
                        assert_softmax_close)

pytestmark = pytest.mark.gpu


def _bits(x, bf16):
    x = np.asarray(x, np.float32)
    with np.errstate(over="ignore"):
        return inputs.f32_to_bf16_bits(x).reshape(x.shape) if bf16 else x.astype(np.float16).view(np.uint16)


def _to64(bits, bf16):
    return oracle.bf16_to_f64(bits) if bf16 else oracle.f16_to_f64(bits)


# policy, cols: WARP at several lane mappings (ragged 260 and 1000 leave empty vector slots), BLOCK, re-read
SOFTMAX_SHAPES = [(1, 128), (1, 512), (1, 260), (1, 1000), (1, 2048), (2, 128), (2, 4096), (2, 5000), (2, 40960),
                  (3, 128), (3, 5000), (3, 40000), (0, 768), (2, 131072)]


@pytest.mark.parametrize("policy,cols", SOFTMAX_SHAPES)
def test_softmax_special_values(ko, policy, cols):
    base = inputs.normal_f32((5, cols), 500 + cols, 0.0, 4.0)
    x, classes = sv.build(sv.SOFTMAX_ROWS, cols, base, repeat=6)  # 72 rows: several waves / workgroups
    ref = oracle.softmax(x)
    got = ko.softmax_host(x, policy=policy)
    ok = sv.check_rows(got, ref, classes, "softmax policy %d cols %d" % (policy, cols))
    assert_softmax_close(got[ok], ref[ok])
    # in place as well
    got = ko.softmax_host(x, policy=policy, in_place=True)
    ok = sv.check_rows(got, ref, classes, "softmax in place")
    assert_softmax_close(got[ok], ref[ok])


@pytest.mark.parametrize("policy", [1, 2, 3])
def test_masked_softmax_ignores_special_values_in_the_padding(ko, policy):
    cols, rps = 512, 4
    base = inputs.normal_f32((5, cols), 900, 0.0, 4.0)
    x, classes = sv.build(sv.SOFTMAX_ROWS, cols, base, repeat=2)
    rows = x.shape[0]
    vl = np.array([cols, 300, 64, 1, 0, 511], np.int32)[: rows // rps]
    x2 = x.copy()
    for r in range(rows):
        x2[r, vl[r // rps]:] = [np.nan, np.inf, -np.inf, 1e30][r % 4]  # garbage where the mask applies
    ref = oracle.softmax(x2, vl, rps)
    ref_clean = oracle.softmax(x, vl, rps)
    np.testing.assert_array_equal(np.isnan(ref), np.isnan(ref_clean))
    got = ko.softmax_host(x2, vl, rps, policy=policy)
    nan_rows = np.all(np.isnan(ref), axis=1)
    assert np.array_equal(np.any(np.isnan(ref), axis=1), nan_rows)
    assert np.all(np.isnan(got[nan_rows])) and not np.any(np.isnan(got[~nan_rows]))
    assert_softmax_close(got[~nan_rows], ref[~nan_rows])


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("policy,cols", [(1, 128), (1, 1000), (1, 4096), (2, 8192), (2, 5000), (3, 40000)])
def test_softmax16_special_values(ko, policy, cols, bf16):
    base = inputs.normal_f32((5, cols), 600 + cols, 0.0, 4.0)
    x, classes = sv.build(sv.SOFTMAX_ROWS, cols, base, repeat=3)
    xb = _bits(x, bf16)  # -FLT_MAX becomes -inf in binary16: that row is then all -inf, i.e. NaN
    x16 = _to64(xb, bf16)
    classes = np.where(np.all(np.isneginf(x16), axis=1), "nan", classes)
    _, ref64 = oracle.softmax16(xb, bf16=bf16)
    got = _to64(ko.softmax16_host(xb, dtype=ko.BF16 if bf16 else ko.F16, policy=policy), bf16)
    ok = sv.check_rows(got, ref64, classes, "softmax16 policy %d cols %d" % (policy, cols))
    assert_softmax16_close(got[ok], ref64[ok], bf16)


@pytest.mark.parametrize("policy,cols", [(1, 128), (1, 768), (1, 260), (1, 1000), (1, 2048), (2, 768), (2, 4096),
                                         (2, 5000), (2, 40960), (3, 768), (3, 5000), (3, 40000), (0, 1024),
                                         (2, 131072)])
@pytest.mark.parametrize("affine", [True, False])
def test_layernorm_special_values(ko, policy, cols, affine):
    base = inputs.normal_f32((5, cols), 700 + cols, 0.5, 2.0)
    x, classes = sv.build(sv.LAYERNORM_ROWS, cols, base, repeat=6)
    g = inputs.normal_f32((cols,), 701, 1.0, 0.1) if affine else None
    b = inputs.normal_f32((cols,), 702, 0.0, 0.1) if affine else None
    ref = oracle.layernorm(x, g, b)
    got = ko.layernorm_host(x, g, b, policy=policy)
    ok = None
    for name, a, r in zip(("y", "mean", "rstd"), got, ref):
        ok = sv.check_rows(a, r, classes, "layernorm %s policy %d cols %d" % (name, policy, cols))
    assert_layernorm_close(tuple(a[ok] for a in got), tuple(r[ok] for r in ref))


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("policy,cols", [(1, 768), (1, 1000), (2, 8192), (3, 40000)])
def test_layernorm16_special_values(ko, policy, cols, bf16):
    base = inputs.normal_f32((5, cols), 800 + cols, 0.5, 2.0)
    x, classes = sv.build(sv.LAYERNORM_ROWS, cols, base, repeat=3)
    xb = _bits(x, bf16)
    gb = _bits(inputs.normal_f32((cols,), 801, 1.0, 0.1), bf16)
    bb = _bits(inputs.normal_f32((cols,), 802, 0.0, 0.1), bf16)
    _, ref64, rmean, rrstd = oracle.layernorm16(xb, gb, bb, bf16=bf16)
    y, mean, rstd = ko.layernorm16_host(xb, gb, bb, dtype=ko.BF16 if bf16 else ko.F16, policy=policy)
    y64 = _to64(y, bf16)
    ok = sv.check_rows(y64, ref64, classes, "layernorm16 y")
    sv.check_rows(mean, rmean, classes, "layernorm16 mean")
    sv.check_rows(rstd, rrstd, classes, "layernorm16 rstd")
    assert_layernorm16_close((y64[ok], mean[ok], rstd[ok]), (ref64[ok], rmean[ok], rrstd[ok]), bf16)
