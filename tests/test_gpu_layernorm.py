"""GPU parity: ko_layernorm_f32 (through the C ABI) against the CPU oracle on identical seeded inputs."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs
from tolerances import assert_layernorm_close

pytestmark = pytest.mark.gpu


def _case(rows, cols, seed, affine=True):
    x = inputs.normal_f32((rows, cols), seed, 0.5, 2.0)
    g = inputs.normal_f32((cols,), seed + 1, 1.0, 0.1) if affine else None
    b = inputs.normal_f32((cols,), seed + 2, 0.0, 0.1) if affine else None
    return x, g, b


@pytest.mark.parametrize("rows,cols", [(4, 768), (1024, 768), (1001, 768), (7, 4), (33, 36), (64, 512),
                                       (129, 128), (5, 2048), (77, 1000), (3, 260), (50, 1024)])
@pytest.mark.parametrize("unbiased", [False, True])
def test_layernorm_matches_oracle(ko, rows, cols, unbiased):
    x, g, b = _case(rows, cols, 100 + rows + cols)
    got = ko.layernorm_host(x, g, b, eps=1e-5, unbiased=unbiased)
    assert_layernorm_close(got, oracle.layernorm(x, g, b, eps=1e-5, unbiased=unbiased))


@pytest.mark.parametrize("lpr", [8, 16, 32, 64])
@pytest.mark.parametrize("cols", [128, 768, 1024, 200])
def test_layernorm_every_lane_mapping(ko, lpr, cols):
    """Every group width, on row lengths that fill the lanes evenly (equal-count merge: 128 with 8/16/32 lanes,
    768 and 1024 with 64) and on ones that do not (general merge with ragged per-lane counts)."""
    x, g, b = _case(517, cols, 31 + lpr)
    ref = oracle.layernorm(x, g, b)
    ko.set_tuning("layernorm.lanes_per_row", lpr)
    try:
        for unbiased in (False, True):
            assert_layernorm_close(ko.layernorm_host(x, g, b, unbiased=unbiased), oracle.layernorm(x, g, b, unbiased=unbiased))
    finally:
        ko.set_tuning("layernorm.lanes_per_row", 0)


@pytest.mark.parametrize("policy,rows,cols", [
    (2, 37, 768), (2, 19, 1024), (2, 9, 4096), (2, 5, 8192), (2, 3, 32768), (2, 11, 5000),
    (2, 3, 40960), (2, 2, 49152), (2, 3, 65536), (2, 2, 81920), (2, 2, 70004), (2, 5000, 2052),
    (3, 5000, 2052), (3, 37, 768), (3, 19, 1024), (3, 4, 40000), (3, 2, 131072), (0, 3, 4096), (0, 2, 65536), (0, 2, 81920),
    (0, 2, 81924),
    # past the registers of a workgroup: nine vectors per thread in LDS, what lies beyond streamed twice
    (2, 3, 81924), (2, 2, 98304), (2, 3, 118784), (2, 2, 118788), (2, 3, 131072), (0, 2, 131072), (2, 2, 200004), (0, 1, 400000)])
def test_layernorm_block_policies(ko, policy, rows, cols):
    x, g, b = _case(rows, cols, 900 + cols)
    assert_layernorm_close(ko.layernorm_host(x, g, b, policy=policy), oracle.layernorm(x, g, b))


@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("rows,cols", [(7, 2052), (33, 2560), (9, 3072), (5, 4096), (11, 5000), (3, 6148), (6, 7168), (4, 8192)])
def test_layernorm_rows_of_a_few_vectors_per_thread(ko, rows, cols, affine):
    """2052 to 8192 columns through the default dispatch and through each form it chooses between: the one-shot
    kernel with one and with two rows per workgroup (odd row counts leave the last workgroup a single row; row
    lengths that do not fill the last vector of every thread; gamma and beta present or absent) and the walking
    grid.  Every form against the oracle, in place as well."""
    x, g, b = _case(rows, cols, 1300 + cols)
    if not affine:
        g = b = None
    ref = oracle.layernorm(x, g, b)
    try:
        for block_rows in (0, 1, 2, -1):
            ko.set_tuning("layernorm.block_rows", block_rows)
            for policy in (0, 2):
                assert_layernorm_close(ko.layernorm_host(x, g, b, policy=policy), ref)
            assert_layernorm_close(ko.layernorm_host(x, g, b, policy=2, in_place=True), ref)
            assert_layernorm_close(ko.layernorm_host(x, g, b, unbiased=True, policy=2), oracle.layernorm(x, g, b, unbiased=True))
    finally:
        ko.set_tuning("layernorm.block_rows", 0)


def test_layernorm_optional_arguments(ko):
    """gamma, beta, mean and rstd are independently optional (the reference runs with affine off,
    nn_operators/layernorm/main.cu:22)."""
    x, g, b = _case(40, 768, 5)
    ry, rm, rr = oracle.layernorm(x, None, None, eps=1e-4)
    y = ko.layernorm_host(x, eps=1e-4, want_stats=False)
    assert_layernorm_close((y, None, None), (ry, rm, rr))
    assert_layernorm_close(ko.layernorm_host(x, gamma=g), oracle.layernorm(x, gamma=g))
    assert_layernorm_close(ko.layernorm_host(x, beta=b), oracle.layernorm(x, beta=b))
    assert_layernorm_close(ko.layernorm_host(x, g, b, in_place=True), oracle.layernorm(x, g, b))
    ko.layernorm(None, None, 0, 768)  # zero rows


def test_layernorm_properties(ko):
    cols = 768
    b = inputs.normal_f32((cols,), 1, 0.0, 0.1)
    g = inputs.normal_f32((cols,), 2, 1.0, 0.1)
    # constant row: y = beta, mean = c, rstd = 1/sqrt(eps)
    x = np.full((3, cols), 2.5, np.float32)
    y, m, r = ko.layernorm_host(x, g, b, eps=1e-5)
    np.testing.assert_array_equal(y, np.broadcast_to(b, y.shape))
    np.testing.assert_array_equal(m, np.full(3, 2.5, np.float32))
    np.testing.assert_allclose(r, 1 / np.sqrt(1e-5), rtol=1e-6)
    # arithmetic progression 0..C-1: mean (C-1)/2, population variance (C^2-1)/12
    x = np.tile(np.arange(cols, dtype=np.float32), (2, 1))
    y, m, r = ko.layernorm_host(x, eps=0.0)
    np.testing.assert_allclose(m, (cols - 1) / 2, rtol=1e-6)
    np.testing.assert_allclose(r, 1 / np.sqrt((cols * cols - 1) / 12), rtol=1e-6)
    _, _, ru = ko.layernorm_host(x, eps=0.0, unbiased=True)
    np.testing.assert_allclose(ru, 1 / np.sqrt((cols * cols - 1) / 12 * cols / (cols - 1)), rtol=1e-6)
    # large offset: Welford does not cancel (a naive E[x^2]-E[x]^2 in fp32 would)
    x = (1.0e4 + inputs.normal_f64(8 * cols, 3, 0.0, 1.0)).astype(np.float32).reshape(8, cols)
    assert_layernorm_close(ko.layernorm_host(x), oracle.layernorm(x))


def test_layernorm_errors(ko):
    buf = ko.DeviceBuffer(1 << 16)
    with pytest.raises(ko.KoError) as e:
        ko.layernorm(buf, buf, 4, (1 << 30) + 4)
    assert e.value.status == ko.KO_ERR_UNSUPPORTED_SHAPE
    with pytest.raises(ko.KoError) as e:
        ko.layernorm(buf, None, 4, 768)
    assert e.value.status == ko.KO_ERR_INVALID_ARGUMENT
    with pytest.raises(ko.KoError) as e:
        ko.layernorm(buf, buf, 1, 4096, policy=1)
    assert e.value.status == ko.KO_ERR_UNSUPPORTED_SHAPE


def test_layernorm_full_size_cfg2(ko):
    """[16384,768] with gamma/beta, filled on the device; whole output against the oracle run on the
    bytes the kernel read."""
    rows, cols = 16384, 768
    n = rows * cols
    dx, dy = ko.DeviceBuffer(n * 4), ko.DeviceBuffer(n * 4)
    dg, db = ko.DeviceBuffer(cols * 4), ko.DeviceBuffer(cols * 4)
    dm, dr = ko.DeviceBuffer(rows * 4), ko.DeviceBuffer(rows * 4)
    ko.fill_normal_f32(dx, n, inputs.tensor_seed(2, 0), 0.5, 2.0)
    ko.fill_normal_f32(dg, cols, inputs.tensor_seed(2, 1), 1.0, 0.1)
    ko.fill_normal_f32(db, cols, inputs.tensor_seed(2, 2), 0.0, 0.1)
    ko.layernorm(dx, dy, rows, cols, dm, dr, dg, db, 1e-5)
    ko.synchronize()
    x = dx.download(np.float32, (rows, cols))
    g, b = dg.download(np.float32, (cols,)), db.download(np.float32, (cols,))
    got = (dy.download(np.float32, (rows, cols)), dm.download(np.float32, (rows,)),
           dr.download(np.float32, (rows,)))
    assert_layernorm_close(got, oracle.layernorm(x, g, b, eps=1e-5))
    hostg = inputs.normal_f32((cols,), inputs.tensor_seed(2, 1), 1.0, 0.1)
    assert np.all(np.abs(hostg - g) <= 2.0 ** -22 * np.maximum(np.abs(hostg), 1.0))


@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("cols", [4, 8, 12, 16, 20, 32, 48, 64])
def test_layernorm_rows_of_a_few_vectors(ko, cols, affine):
    """Rows of one to sixteen vectors: 1, 2 or 4 lanes per row up to four vectors, 16 to 64 rows per wavefront; row
    counts around a wavefront's worth, both variance divisors, in place."""
    g = inputs.normal_f32((cols,), 961, 1.0, 0.1) if affine else None
    b = inputs.normal_f32((cols,), 962, 0.0, 0.1) if affine else None
    for rows in (1, 15, 16, 17, 63, 64, 65, 1000, 100001):
        x = inputs.normal_f32((rows, cols), 960 + rows + cols, 0.5, 2.0)
        assert_layernorm_close(ko.layernorm_host(x, g, b, 1e-5, rows % 2 == 0), oracle.layernorm(x, g, b, 1e-5, rows % 2 == 0))
    x = inputs.normal_f32((777, cols), 963, 0.5, 2.0)
    assert_layernorm_close(ko.layernorm_host(x, g, b, in_place=True), oracle.layernorm(x, g, b))
