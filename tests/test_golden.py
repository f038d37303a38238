"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU part: the seeded generators reproduce the stored inputs bit for bit, and the oracle reproduces the stored
outputs (to one unit in the last place: libm's exp may differ between machines).
GPU part: the HIP kernels, called through the C ABI, meet the parity gates against the stored outputs.
"""
import json
import os

import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs
from tolerances import assert_gemm16_close, assert_layernorm_close, assert_sgemm_close, assert_softmax_close

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
with open(os.path.join(GOLDEN, "manifest.json")) as _f:
    MANIFEST = json.load(_f)


def _load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _cases(op):
    return sorted(k for k, v in MANIFEST.items() if v["op"] == op)


def _to64(bits, bf16):
    return oracle.bf16_to_f64(bits) if bf16 else oracle.f16_to_f64(bits)


def test_manifest_matches_files():
    for name, meta in MANIFEST.items():
        data = _load(name)
        assert sorted(data) == sorted(meta["arrays"])
        for k, (dtype, shape) in meta["arrays"].items():
            assert str(data[k].dtype) == dtype and list(data[k].shape) == shape


# ------------------------------------------------------------------ CPU: generators and oracle

@pytest.mark.parametrize("name", _cases("softmax"))
def test_oracle_softmax_golden(name):
    meta, d = MANIFEST[name], _load(name)
    np.testing.assert_array_equal(inputs.normal_f32(d["x"].shape, meta["seed"], meta["mean"], meta["std"]), d["x"])
    got = oracle.softmax(d["x"], d.get("valid_len"), meta["rows_per_seq"])
    np.testing.assert_array_max_ulp(got, d["y"], maxulp=1)


@pytest.mark.parametrize("name", _cases("layernorm"))
def test_oracle_layernorm_golden(name):
    meta, d = MANIFEST[name], _load(name)
    np.testing.assert_array_equal(inputs.normal_f32(d["x"].shape, meta["seed"], meta["mean"], meta["std"]), d["x"])
    y, mean, rstd = oracle.layernorm(d["x"], d.get("gamma"), d.get("beta"), meta["eps"], meta["unbiased"])
    np.testing.assert_array_max_ulp(y, d["y"], maxulp=1)
    np.testing.assert_array_max_ulp(mean, d["mean"], maxulp=1)
    np.testing.assert_array_max_ulp(rstd, d["rstd"], maxulp=1)
    # the float-only Welford restatement (the kernels' algorithm) meets the kernels' gate on the same vectors
    assert_layernorm_close(oracle.layernorm_welford(d["x"], d.get("gamma"), d.get("beta"), meta["eps"], meta["unbiased"]),
                           (d["y"], d["mean"], d["rstd"]))


@pytest.mark.parametrize("name", _cases("sgemm"))
def test_oracle_sgemm_golden(name):
    meta, d = MANIFEST[name], _load(name)
    np.testing.assert_array_equal(inputs.uniform_f32(d["A"].shape, meta["seeds"][0]), d["A"])
    np.testing.assert_array_equal(inputs.uniform_f32(d["B"].shape, meta["seeds"][1]), d["B"])
    np.testing.assert_array_equal(oracle.sgemm(d["A"], d["B"], d.get("C"), meta["alpha"], meta["beta"]), d["D"])


@pytest.mark.parametrize("name", _cases("gemm16"))
def test_oracle_gemm16_golden(name):
    meta, d = MANIFEST[name], _load(name)
    D, _, _ = oracle.gemm16(d["A"], d["B"], meta["m"], meta["n"], meta["k"], b_col_major=meta["b_col_major"],
                            bf16=meta["bf16"])
    np.testing.assert_array_equal(D, d["D"])


# ------------------------------------------------------------------ GPU: kernels against the stored outputs

@pytest.mark.gpu
@pytest.mark.parametrize("name", _cases("softmax"))
def test_gpu_softmax_golden(ko, name):
    meta, d = MANIFEST[name], _load(name)
    got = ko.softmax_host(d["x"], d.get("valid_len"), meta["rows_per_seq"])
    assert_softmax_close(got, d["y"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", _cases("layernorm"))
def test_gpu_layernorm_golden(ko, name):
    meta, d = MANIFEST[name], _load(name)
    got = ko.layernorm_host(d["x"], d.get("gamma"), d.get("beta"), meta["eps"], unbiased=meta["unbiased"])
    assert_layernorm_close(got, (d["y"], d["mean"], d["rstd"]))


@pytest.mark.gpu
@pytest.mark.parametrize("name", _cases("sgemm"))
def test_gpu_sgemm_golden(ko, name):
    meta, d = MANIFEST[name], _load(name)
    _, ap = oracle.sgemm(d["A"], d["B"], want_absprod=True)
    if "C" in d:
        ap = ap + np.abs(d["C"].astype(np.float64))
    got = ko.sgemm_host(d["A"], d["B"], d.get("C"), meta["alpha"], meta["beta"])
    assert_sgemm_close(got, d["D"], ap, meta["k"], reference_gate=True)


@pytest.mark.gpu
@pytest.mark.parametrize("name", _cases("gemm16"))
def test_gpu_gemm16_golden(ko, name):
    meta, d = MANIFEST[name], _load(name)
    m, n, k, bf16 = meta["m"], meta["n"], meta["k"], meta["bf16"]
    _, ref64, ap = oracle.gemm16(d["A"], d["B"], m, n, k, b_col_major=meta["b_col_major"], bf16=bf16)
    got = ko.gemm16_host(d["A"], d["B"], m, n, k, b_layout=ko.COL_MAJOR if meta["b_col_major"] else ko.ROW_MAJOR,
                         dtype=ko.BF16 if bf16 else ko.F16)
    # gate against the stored 16-bit outputs (their exact values) with the usual bound
    assert_gemm16_close(_to64(got, bf16), _to64(d["D"], bf16), ap, k, bf16=bf16)
    assert np.abs(_to64(d["D"], bf16) - ref64).max() <= (2.0 ** -8 if bf16 else 2.0 ** -11) * np.abs(ref64).max()
