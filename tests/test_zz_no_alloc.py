"""ko_sgemm_f32_static_scratch, the SGEMM entry point that allocates nothing, against ko_sgemm_f32 through the C
ABI: the same kernels with the partial products of a K-sliced problem in the library's static device array
instead of an allocated workspace, so the outputs must be the same bits.  Two calls in a row share the array, the
second on a smaller problem (what the first left behind must not reach the second's sum); a problem that is not
sliced takes the same path in both entry points; a slice plan that does not fit the array is refused."""
import numpy as np
import pytest

from kernel_optimization_amd import inputs

pytestmark = pytest.mark.gpu


def _both(ko, m, n, k, seed, with_c):
    A, B = inputs.uniform_f32((m, k), seed), inputs.uniform_f32((k, n), seed + 1)
    C = inputs.normal_f32((m, n), seed + 2) if with_c else None
    dA, dB = ko.DeviceBuffer.from_numpy(A), ko.DeviceBuffer.from_numpy(B)
    dC = None if C is None else ko.DeviceBuffer.from_numpy(C)
    alpha, beta = (0.5, -2.0) if with_c else (1.0, 0.0)
    want, got = ko.DeviceBuffer(m * n * 4), ko.DeviceBuffer(m * n * 4)
    got.upload(np.full(m * n, np.nan, np.float32))
    ko.sgemm(m, n, k, dA, dB, want, dC, alpha, beta)
    ko.sgemm_static_scratch(m, n, k, dA, dB, got, dC, alpha, beta)
    ko.synchronize()
    return A, B, C, alpha, beta, want.download(np.uint32, (m, n)), got.download(np.uint32, (m, n))


def test_static_scratch_sgemm_gives_the_bits_of_the_allocating_entry_point(ko):
    import oracle
    from tolerances import assert_sgemm_close
    # sliced by the cost model (36 tiles of 128 x 128 in seven slices: 16.5 MiB of partial products), then by the
    # few-tiles rule (32 tiles, 8 slices), then a smaller sliced problem with ragged tiles and a ragged last
    # slice, then one that is not sliced at all
    for (m, n, k), with_c in (((768, 768, 4096), True), ((256, 256, 2048), False), ((100, 72, 1300), True),
                              ((512, 384, 256), True)):
        A, B, C, alpha, beta, want, got = _both(ko, m, n, k, 900 + m, with_c)
        np.testing.assert_array_equal(got, want, err_msg=str((m, n, k)))
        ref, ap = oracle.sgemm(A, B, C, alpha, beta, want_absprod=True)
        scale = abs(alpha) * ap + (abs(beta) * np.abs(C) if with_c else 0.0) + 1e-6
        assert_sgemm_close(got.view(np.float32), ref, scale, k)


def test_static_scratch_sgemm_refuses_what_does_not_fit(ko):
    m, n, k = 1024, 1024, 4096  # 16 forced slices of 4 MiB each against an array of 32 MiB
    buf = ko.DeviceBuffer(m * k * 4)
    out = ko.DeviceBuffer(m * n * 4)
    ko.set_tuning("sgemm.k_slices", 16)
    try:
        with pytest.raises(ko.KoError) as e:
            ko.sgemm_static_scratch(m, n, k, buf, buf, out)
        assert e.value.status == ko.KO_ERR_UNSUPPORTED_SHAPE
        assert "static scratch" in str(e.value)
        ko.sgemm(m, n, k, buf, buf, out)  # the allocating entry point runs such a plan unsliced
        ko.synchronize()
    finally:
        ko.set_tuning("sgemm.k_slices", 0)
    with pytest.raises(ko.KoError) as e:
        ko.sgemm_static_scratch(16, 16, 16, None, buf, out)
    assert e.value.status == ko.KO_ERR_INVALID_ARGUMENT
