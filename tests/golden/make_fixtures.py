"""Writes the small golden fixtures of this directory (run once, here on the CPU; the .npz files are committed).

The reference holds no recorded outputs for its operators (its only known answers are the identity
GEMM inputs of nn_operators/gemm/main.cu:219-233, which the tests build directly), so the vectors are
made from this build's own oracle on seeded inputs.  Before a case is written its expected outputs are
checked against an independent formulation in numpy float64 (library exp / mean / var / matmul instead
of the oracle's loops); a disagreement beyond the stated bound aborts the run.

Each case is one ``<name>.npz`` (inputs and expected outputs, loadable with allow_pickle=False) plus an
entry in ``manifest.json`` with the seeds, shapes and the parity gate that applies.

    python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from kernel_optimization_amd import inputs  # noqa: E402

MANIFEST = {}


def _save(name, meta, **arrays):
    np.savez(os.path.join(HERE, name + ".npz"), **arrays)
    MANIFEST[name] = dict(meta, arrays={k: [str(v.dtype), list(v.shape)] for k, v in arrays.items()})


def _np_softmax(x, valid_len=None, rows_per_seq=0):
    x = x.astype(np.float64)
    if valid_len is not None:
        seq = np.arange(x.shape[0]) // rows_per_seq
        x = np.where(np.arange(x.shape[1])[None, :] >= valid_len[seq][:, None], inputs.MASK_VALUE, x)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def softmax_cases():
    for name, rows, cols, seed, lens, rps in (
            ("softmax_4x128", 4, 128, 101, None, 0),
            ("softmax_3x36", 3, 36, 102, None, 0),
            ("softmax_masked_6x512", 6, 512, 103, np.array([64, 300, 512], np.int32), 2),
            ("softmax_masked_4x128_len0", 4, 128, 104, np.array([0, 5], np.int32), 2)):
        x = inputs.normal_f32((rows, cols), seed, 0.0, 4.0)
        y = oracle.softmax(x, lens, rps)
        ref = _np_softmax(x, lens, rps)
        assert np.abs(y - ref).max() <= 2.0 ** -24, name  # one fp32 rounding of a value <= 1
        arrays = dict(x=x, y=y)
        if lens is not None:
            arrays["valid_len"] = lens
        _save(name, dict(op="softmax", seed=seed, mean=0.0, std=4.0, rows_per_seq=rps,
                         gate="abs 1e-6 and rel 1e-5"), **arrays)


def layernorm_cases():
    for name, rows, cols, seed, unbiased, affine in (
            ("layernorm_4x768_population", 4, 768, 201, False, True),
            ("layernorm_4x768_unbiased", 4, 768, 201, True, True),
            ("layernorm_5x100_plain", 5, 100, 202, False, False)):
        x = inputs.normal_f32((rows, cols), seed, 0.5, 2.0)
        g = inputs.normal_f32((cols,), seed + 1, 1.0, 0.1) if affine else None
        b = inputs.normal_f32((cols,), seed + 2, 0.0, 0.1) if affine else None
        eps = 1e-5
        y, mean, rstd = oracle.layernorm(x, g, b, eps, unbiased)
        x64 = x.astype(np.float64)
        m64 = x64.mean(axis=1)
        v64 = x64.var(axis=1, ddof=1 if unbiased else 0)
        r64 = 1.0 / np.sqrt(v64 + np.float64(np.float32(eps)))
        y64 = (x64 - m64[:, None]) * r64[:, None]
        if affine:
            y64 = y64 * g.astype(np.float64) + b.astype(np.float64)
        assert np.abs(mean - m64).max() <= 2.0 ** -23 * np.abs(m64).max(), name
        assert (np.abs(rstd - r64) / r64).max() <= 2.0 ** -23, name
        assert (np.abs(y - y64) / np.maximum(np.abs(y64), 1.0)).max() <= 2.0 ** -22, name
        arrays = dict(x=x, y=y, mean=mean, rstd=rstd)
        if affine:
            arrays.update(gamma=g, beta=b)
        _save(name, dict(op="layernorm", seed=seed, mean=0.5, std=2.0, eps=eps, unbiased=bool(unbiased),
                         gate="y 1e-5*max(|ref|,1); mean 1e-5*max(|mean|,std); rstd 1e-5 rel"), **arrays)


def gemm_cases():
    m, n, k = 64, 48, 72
    A = inputs.uniform_f32((m, k), 301)
    B = inputs.uniform_f32((k, n), 302)
    C = inputs.uniform_f32((m, n), 303)
    for name, c, alpha, beta in (("sgemm_64x48x72", None, 1.0, 0.0), ("sgemm_64x48x72_plus_c", C, 1.0, 1.0)):
        D = oracle.sgemm(A, B, c, alpha, beta)
        ref = alpha * (A.astype(np.float64) @ B.astype(np.float64)) + (beta * c.astype(np.float64) if c is not None else 0)
        assert (np.abs(D - ref) <= 2.0 ** -23 * np.abs(ref) + 1e-12).all(), name  # one fp32 rounding
        arrays = dict(A=A, B=B, D=D)
        if c is not None:
            arrays["C"] = c
        _save(name, dict(op="sgemm", seeds=[301, 302, 303], m=m, n=n, k=k, alpha=alpha, beta=beta,
                         gate="2*K*2^-24*|A||B|"), **arrays)
    for name, bf16, col in (("gemm_f16_64x48x72_colmajor_b", False, True), ("gemm_f16_64x48x72_rowmajor_b", False, False),
                            ("gemm_bf16_64x48x72_colmajor_b", True, True)):
        gen = inputs.uniform_bf16_bits if bf16 else (lambda s, sd: inputs.uniform_f16(s, sd).view(np.uint16))
        Ab = gen((m, k), 311)
        Bb = gen((n, k) if col else (k, n), 312)
        Db, d64, _ = oracle.gemm16(Ab, Bb, m, n, k, b_col_major=col, bf16=bf16)
        to64 = (lambda b: inputs.bf16_bits_to_f32(b).astype(np.float64)) if bf16 else (lambda b: b.view(np.float16).astype(np.float64))
        Bm = to64(Bb).T if col else to64(Bb)
        ref = to64(Ab) @ Bm
        assert np.abs(d64 - ref).max() <= 1e-12, name
        assert (np.abs(to64(Db) - ref) <= (2.0 ** -8 if bf16 else 2.0 ** -11) * np.abs(ref) + 2.0 ** -24).all(), name
        _save(name, dict(op="gemm16", seeds=[311, 312], m=m, n=n, k=k, bf16=bf16, b_col_major=col,
                         gate="2^-11|ref| (bf16: 2^-8) + K*2^-24*|A||B| + 2^-24"), A=Ab, B=Bb, D=Db)


if __name__ == "__main__":
    softmax_cases()
    layernorm_cases()
    gemm_cases()
    with open(os.path.join(HERE, "manifest.json"), "w") as f:
        json.dump(MANIFEST, f, indent=1, sort_keys=True)
    print("wrote %d cases" % len(MANIFEST))
