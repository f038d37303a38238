"""GPU parity: ko_softmax_16 and ko_layernorm_16 (binary16 / bfloat16 storage, fp32 arithmetic) through the
C ABI against the 16-bit-storage oracle on identical inputs."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs
from tolerances import assert_layernorm16_close, assert_softmax16_close

pytestmark = pytest.mark.gpu


def _bits(x, bf16):
    x = np.asarray(x, np.float32)
    return inputs.f32_to_bf16_bits(x).reshape(x.shape) if bf16 else x.astype(np.float16).view(np.uint16)


def _to64(bits, bf16):
    return oracle.bf16_to_f64(bits) if bf16 else oracle.f16_to_f64(bits)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,cols", [(4, 128), (1000, 128), (7, 8), (33, 40), (64, 512), (129, 768), (5, 4096),
                                       (77, 1000), (3, 264), (9, 2048)])
def test_softmax16_matches_oracle(ko, rows, cols, bf16):
    xb = _bits(inputs.normal_f32((rows, cols), 50 + rows + cols, 0.0, 4.0), bf16)
    _, ref64 = oracle.softmax16(xb, bf16=bf16)
    got = ko.softmax16_host(xb, dtype=ko.BF16 if bf16 else ko.F16)
    assert_softmax16_close(_to64(got, bf16), ref64, bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("lpr", [8, 16, 32, 64])
def test_softmax16_every_lane_mapping(ko, lpr, bf16):
    xb = _bits(inputs.normal_f32((515, 512), 60 + lpr, 0.0, 4.0), bf16)
    _, ref64 = oracle.softmax16(xb, bf16=bf16)
    ko.set_tuning("softmax.lanes_per_row", lpr)
    try:
        got = ko.softmax16_host(xb, dtype=ko.BF16 if bf16 else ko.F16)
    finally:
        ko.set_tuning("softmax.lanes_per_row", 0)
    assert_softmax16_close(_to64(got, bf16), ref64, bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("policy,rows,cols", [(2, 37, 128), (2, 19, 1024), (2, 5, 16384), (2, 3, 65536), (2, 11, 5000),
                                              (2, 2, 81920), (2, 2, 98304), (0, 2, 98304),
                                              (3, 37, 128), (3, 4, 40000), (3, 2, 262144), (0, 3, 8192), (0, 2, 131072),
                                              (2, 2, 131072), (2, 2, 172032), (0, 2, 172040)])
def test_softmax16_block_policies(ko, policy, rows, cols, bf16):
    xb = _bits(inputs.normal_f32((rows, cols), 70 + cols, 0.0, 4.0), bf16)
    _, ref64 = oracle.softmax16(xb, bf16=bf16)
    got = ko.softmax16_host(xb, dtype=ko.BF16 if bf16 else ko.F16, policy=policy)
    assert_softmax16_close(_to64(got, bf16), ref64, bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("policy", [0, 1, 2, 3])
def test_masked_softmax16(ko, policy, bf16):
    """The masked configuration's shape in small (512 columns, lengths in [64, 512]) plus the edge lengths 0, 1,
    one short of a vector boundary, and the full row; a ragged last sequence."""
    rps = 40
    lens = np.array([64, 300, 512, 0, 1, 255, 257, 511], np.int32)
    rows = rps * len(lens) - 7
    xb = _bits(inputs.normal_f32((rows, 512), 80, 0.0, 4.0), bf16)
    yb_ref, ref64 = oracle.softmax16(xb, lens, rps, bf16=bf16)
    got = ko.softmax16_host(xb, lens, rps, dtype=ko.BF16 if bf16 else ko.F16, policy=policy)
    assert_softmax16_close(_to64(got, bf16), ref64, bf16)
    seq = np.arange(rows) // rps
    padded = np.arange(512)[None, :] >= np.maximum(lens[seq], 1)[:, None]
    full_mask = (lens[seq] == 0)[:, None]
    assert np.all(got[padded & ~full_mask] == 0)          # exact zeros in the padding


@pytest.mark.parametrize("bf16", [False, True])
def test_softmax16_in_place_and_errors(ko, bf16):
    dt = ko.BF16 if bf16 else ko.F16
    xb = _bits(inputs.normal_f32((50, 256), 90, 0.0, 4.0), bf16)
    _, ref64 = oracle.softmax16(xb, bf16=bf16)
    assert_softmax16_close(_to64(ko.softmax16_host(xb, dtype=dt, in_place=True), bf16), ref64, bf16)
    d = ko.DeviceBuffer(4096)
    assert ko.lib().ko_softmax_16(d.ptr, d.ptr, 2, 12, None, 0, dt, 0, None) == ko.KO_OK  # any row length
    assert ko.lib().ko_softmax_16(d.ptr, d.ptr, 2, (1 << 30) + 8, None, 0, dt, 0, None) == ko.KO_ERR_UNSUPPORTED_SHAPE
    assert ko.lib().ko_softmax_16(d.ptr, d.ptr, 2, 16, None, 0, 7, 0, None) == ko.KO_ERR_INVALID_ARGUMENT
    assert ko.lib().ko_softmax_16(d.ptr, d.ptr, 2, 8192, None, 0, dt, 1, None) == ko.KO_ERR_UNSUPPORTED_SHAPE
    assert ko.lib().ko_softmax_16(None, d.ptr, 2, 16, None, 0, dt, 0, None) == ko.KO_ERR_INVALID_ARGUMENT
    assert ko.lib().ko_softmax_16(d.ptr, d.ptr, 0, 16, None, 0, dt, 0, None) == ko.KO_OK


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("unbiased", [False, True])
@pytest.mark.parametrize("rows,cols", [(4, 768), (1000, 128), (7, 8), (33, 40), (129, 1024), (5, 4096), (77, 1000),
                                       (16, 3072)])
def test_layernorm16_matches_oracle(ko, rows, cols, unbiased, bf16):
    if unbiased and cols < 2:
        pytest.skip("needs two columns")
    xb = _bits(inputs.normal_f32((rows, cols), 100 + rows + cols, 0.5, 2.0), bf16)
    gb = _bits(inputs.normal_f32((cols,), 101, 1.0, 0.1), bf16)
    bb = _bits(inputs.normal_f32((cols,), 102, 0.0, 0.1), bf16)
    _, ref64, rmean, rrstd = oracle.layernorm16(xb, gb, bb, 1e-5, unbiased, bf16)
    y, mean, rstd = ko.layernorm16_host(xb, gb, bb, 1e-5, unbiased, dtype=ko.BF16 if bf16 else ko.F16)
    assert_layernorm16_close((_to64(y, bf16), mean, rstd), (ref64, rmean, rrstd), bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("policy,rows,cols", [(2, 37, 128), (2, 19, 1024), (2, 5, 16384), (2, 3, 32768),
                                              (2, 2, 65536), (2, 2, 81920), (0, 2, 81920),
                                              (3, 37, 128), (3, 4, 40000), (0, 3, 8192), (0, 2, 65536), (0, 2, 131072),
                                              (2, 2, 98304), (2, 2, 139264), (2, 2, 139272), (2, 1, 300000)])
def test_layernorm16_block_policies(ko, policy, rows, cols, bf16):
    xb = _bits(inputs.normal_f32((rows, cols), 110 + cols, 0.5, 2.0), bf16)
    gb = _bits(inputs.normal_f32((cols,), 111, 1.0, 0.1), bf16)
    _, ref64, rmean, rrstd = oracle.layernorm16(xb, gb, None, 1e-5, False, bf16)
    y, mean, rstd = ko.layernorm16_host(xb, gb, None, 1e-5, False, dtype=ko.BF16 if bf16 else ko.F16, policy=policy)
    assert_layernorm16_close((_to64(y, bf16), mean, rstd), (ref64, rmean, rrstd), bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,cols", [(7, 4104), (5, 5120), (9, 8192), (3, 12296), (4, 16384)])
def test_layernorm16_rows_of_a_few_vectors_per_thread(ko, rows, cols, bf16):
    """16-bit storage through the one-shot BLOCK kernel (513 to 2048 vectors of eight values), one and two rows per
    workgroup, with and without gamma and beta, and through the walking grid."""
    dt = ko.BF16 if bf16 else ko.F16
    xb = _bits(inputs.normal_f32((rows, cols), 130 + cols, 0.5, 2.0), bf16)
    gb = _bits(inputs.normal_f32((cols,), 131, 1.0, 0.1), bf16)
    bb = _bits(inputs.normal_f32((cols,), 132, 0.0, 0.1), bf16)
    try:
        for g_, b_ in ((gb, bb), (None, None)):
            _, ref64, rmean, rrstd = oracle.layernorm16(xb, g_, b_, 1e-5, False, bf16)
            for block_rows in (0, 1, 2, -1):
                ko.set_tuning("layernorm.block_rows", block_rows)
                y, mean, rstd = ko.layernorm16_host(xb, g_, b_, 1e-5, False, dtype=dt, policy=2)
                assert_layernorm16_close((_to64(y, bf16), mean, rstd), (ref64, rmean, rrstd), bf16)
    finally:
        ko.set_tuning("layernorm.block_rows", 0)


@pytest.mark.parametrize("bf16", [False, True])
def test_layernorm16_plain_in_place_and_errors(ko, bf16):
    dt = ko.BF16 if bf16 else ko.F16
    xb = _bits(inputs.normal_f32((60, 768), 120, 0.5, 2.0), bf16)
    _, ref64, rmean, rrstd = oracle.layernorm16(xb, None, None, 1e-5, False, bf16)
    y, mean, rstd = ko.layernorm16_host(xb, None, None, 1e-5, False, dtype=dt, in_place=True)
    assert_layernorm16_close((_to64(y, bf16), mean, rstd), (ref64, rmean, rrstd), bf16)
    d = ko.DeviceBuffer(4096)
    L = ko.lib()
    assert L.ko_layernorm_16(d.ptr, d.ptr, None, None, None, None, 2, 12, 1e-5, 0, dt, 0, None) == ko.KO_OK  # any row length
    assert L.ko_layernorm_16(d.ptr, d.ptr, None, None, None, None, 2, (1 << 30) + 8, 1e-5, 0, dt, 0, None) == ko.KO_ERR_UNSUPPORTED_SHAPE
    assert L.ko_layernorm_16(d.ptr, d.ptr, None, None, None, None, 2, 16, 1e-5, 0, 9, 0, None) == ko.KO_ERR_INVALID_ARGUMENT
    assert L.ko_layernorm_16(d.ptr, d.ptr, None, None, None, None, 0, 16, 1e-5, 0, dt, 0, None) == ko.KO_OK


@pytest.mark.parametrize("bf16", [False, True])
def test_rows16_large(ko, bf16):
    """BERT-sized shapes on 16-bit storage: softmax [12 * 512 * 8, 512] masked, LayerNorm [16384, 768]; sampled
    rows against the oracle."""
    dt = ko.BF16 if bf16 else ko.F16
    rows, cols, rps = 49152, 512, 6144
    lens = inputs.valid_lengths(rows // rps, 130)
    xb = _bits(inputs.normal_f32((rows, cols), 131, 0.0, 4.0), bf16)
    got = ko.softmax16_host(xb, lens, rps, dtype=dt)
    idx = np.sort(np.random.default_rng(5).choice(rows, 512, replace=False))
    seq_lens = lens[idx // rps]
    _, ref64 = oracle.softmax16(xb[idx], seq_lens, 1, bf16=bf16)
    assert_softmax16_close(_to64(got[idx], bf16), ref64, bf16)
    rows, cols = 16384, 768
    xb = _bits(inputs.normal_f32((rows, cols), 132, 0.5, 2.0), bf16)
    gb = _bits(inputs.normal_f32((cols,), 133, 1.0, 0.1), bf16)
    bb = _bits(inputs.normal_f32((cols,), 134, 0.0, 0.1), bf16)
    y, mean, rstd = ko.layernorm16_host(xb, gb, bb, 1e-5, False, dtype=dt)
    _, ref64, rmean, rrstd = oracle.layernorm16(xb, gb, bb, 1e-5, False, bf16)
    assert_layernorm16_close((_to64(y, bf16), mean, rstd), (ref64, rmean, rrstd), bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("cols", [8, 16, 24, 32, 48, 64, 128])
def test_softmax16_rows_of_a_few_vectors(ko, cols, bf16):
    for rows in (1, 63, 64, 65, 5000):
        xb = _bits(inputs.normal_f32((rows, cols), 950 + rows + cols, 0.0, 4.0), bf16)
        _, ref64 = oracle.softmax16(xb, bf16=bf16)
        assert_softmax16_close(_to64(ko.softmax16_host(xb, dtype=ko.BF16 if bf16 else ko.F16), bf16), ref64, bf16)
