"""GPU parity: ko_sgemm_f32 and ko_gemm_f16f32acc (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest

import oracle
from kernel_optimization_amd import inputs
from tolerances import assert_gemm16_close, assert_sgemm_close

pytestmark = pytest.mark.gpu

SGEMM_VARIANTS = [0, 13, 16, 21, 33, 35, 36, 37, 40, 41]
SGEMM_PIPELINED = [13, 16, 21, 33, 35, 36, 37, 40, 41]  # two K tiles per loop trip; 33 on: direct-to-LDS
GEMM16_VARIANTS = [0, 3, 6, 9, 10, 11, 12, 13, 30, 50, 52, 53, 54]


@pytest.fixture
def sgemm_variant(ko, request):
    ko.set_tuning("sgemm.variant", request.param)
    yield request.param
    ko.set_tuning("sgemm.variant", 0)


@pytest.fixture
def gemm16_variant(ko, request):
    ko.set_tuning("gemm16.variant", request.param)
    yield request.param
    ko.set_tuning("gemm16.variant", 0)


# ------------------------------------------------------------------------------------ SGEMM

@pytest.mark.parametrize("sgemm_variant", SGEMM_VARIANTS, indirect=True)
@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (128, 256, 96), (200, 136, 40), (1, 4, 4), (65, 129, 33),
                                   (37, 50, 7), (128, 256, 128), (256, 128, 384), (200, 136, 264), (130, 260, 128),
                                   (61, 68, 520)])
def test_sgemm_matches_oracle(ko, sgemm_variant, m, n, k):
    A = inputs.uniform_f32((m, k), 11 + m)
    B = inputs.uniform_f32((k, n), 13 + n)
    ref, ap = oracle.sgemm(A, B, want_absprod=True)
    assert_sgemm_close(ko.sgemm_host(A, B), ref, ap, k)


@pytest.mark.parametrize("sgemm_variant", SGEMM_PIPELINED, indirect=True)
@pytest.mark.parametrize("m,n,k", [(128, 128, 128), (512, 384, 512), (256, 640, 1152), (1024, 1024, 256), (512, 256, 96),
                                   (300, 520, 392), (1000, 1000, 1000)])
def test_sgemm_pipelined_variants_are_exact_on_small_integers(ko, sgemm_variant, m, n, k):
    """Full tiles and an even number of K tiles put the pipelined kernels (register staging or direct-to-LDS
    loads, two to four LDS stages) on their fast path; with small integers every product and sum is exact, so
    any misplaced element of a tile shows as a wrong integer."""
    rng = np.random.default_rng(1000 * sgemm_variant + m + k)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    np.testing.assert_array_equal(ko.sgemm_host(A, B), A.astype(np.float64) @ B.astype(np.float64))
    C = rng.integers(-8, 9, (m, n)).astype(np.float32)
    np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0),
                                  2.0 * (A.astype(np.float64) @ B.astype(np.float64)) - C)


@pytest.mark.parametrize("m,n,k", [(2176, 2048, 512), (2100, 2050, 520), (4224, 2048, 512)])
def test_sgemm_uneven_last_round_goes_out_as_two_launches(ko, m, n, k):
    """A few more 128 x 128 tiles than a whole number of rounds on 256 compute units: the tile rows of the full
    rounds and the rows below them are separate launches with different tilings.  Small integers make every
    sum exact, so a row computed twice, skipped or offset shows as a wrong integer; with the split switched
    off the same call gives the same matrix."""
    rng = np.random.default_rng(m + n + k)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    C = rng.integers(-8, 9, (m, n)).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_array_equal(ko.sgemm_host(A, B), ref)
    np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C)
    ko.set_tuning("sgemm.split_rows", 1)
    try:
        np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C)
    finally:
        ko.set_tuning("sgemm.split_rows", 0)


@pytest.fixture
def sgemm_k_slices(ko):
    """Sets the slice count (0: by shape, 1: never, n: n slices) and puts the default back afterwards."""
    yield lambda value: ko.set_tuning("sgemm.k_slices", value)
    ko.set_tuning("sgemm.k_slices", 0)


@pytest.mark.parametrize("m,n,k", [(256, 256, 2048), (128, 64, 4096), (100, 200, 3000), (33, 68, 1300), (512, 512, 8192),
                                   (64, 64, 516), (1, 4, 16384), (320, 192, 1024),
                                   # operand rows off 16-byte boundaries (four-byte loads) and an M x N that is no multiple of 4
                                   (282, 31, 13104), (48, 107, 7144), (100, 201, 3001), (16, 1001, 4008), (339, 670, 6784)])
def test_sgemm_deep_k_on_few_tiles_is_cut_into_slices(ko, sgemm_k_slices, m, n, k):
    """Few output tiles and a deep K: the default dispatch cuts K into slices that run as workgroups of one
    launch and sums their partial products in a second kernel.  Small integers make every product and sum
    exact, so a slice that starts at the wrong k, overlaps its neighbour, pads with anything but zeros or
    lands at the wrong place of the partial products shows as a wrong integer.  The unsliced path and forced
    slice counts (ragged last slices among them) must give the same matrix."""
    rng = np.random.default_rng(m + n + k)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    C = rng.integers(-8, 9, (m, n)).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    for slices in (0, 1, 2, 3, 7):
        sgemm_k_slices(slices)
        np.testing.assert_array_equal(ko.sgemm_host(A, B), ref, err_msg=f"k_slices={slices}")
        np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C, err_msg=f"k_slices={slices}")


@pytest.mark.parametrize("m,n,k", [(768, 768, 4096), (1280, 1280, 4096), (700, 836, 2052), (1536, 640, 8192)])
def test_sgemm_rounds_that_do_not_fill_the_chip_are_sliced(ko, sgemm_k_slices, m, n, k):
    """More tiles than half the compute units but rounds that leave many of them idle, and a deep K: the
    planner's cost model picks a tiling and a slice count (128 x 128 tiles in seven slices for the first shape).
    Exact on small integers, whichever plan it takes, and equal to the unsliced result."""
    rng = np.random.default_rng(m + n + k)
    A = rng.integers(-3, 4, (m, k)).astype(np.float32)
    B = rng.integers(-3, 4, (k, n)).astype(np.float32)
    C = rng.integers(-8, 9, (m, n)).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    for slices in (0, 1):
        sgemm_k_slices(slices)
        np.testing.assert_array_equal(ko.sgemm_host(A, B), ref, err_msg=f"k_slices={slices}")
        np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C, err_msg=f"k_slices={slices}")
    for variant in (36, 40, 35, 41):  # forced plans on every tiling the planner can choose
        ko.set_tuning("sgemm.slice_variant", variant)
        try:
            for slices in (3, 7):
                sgemm_k_slices(slices)
                np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C,
                                              err_msg=f"variant={variant} k_slices={slices}")
        finally:
            ko.set_tuning("sgemm.slice_variant", 0)


def test_sgemm_random_deep_shapes_are_exact_on_small_integers(ko):
    """Random shapes with K of 2048 and more, through the default dispatch: whatever the planner decides (whole,
    few-tiles slices, or a tiling and slice count from its cost model), small integers must come out exact."""
    rng = np.random.default_rng(23)
    for _ in range(10):
        m, n = int(rng.integers(20, 400)) * 4, int(rng.integers(20, 400)) * 4
        k = int(rng.integers(512, 1500)) * 4
        A = rng.integers(-3, 4, (m, k)).astype(np.float32)
        B = rng.integers(-3, 4, (k, n)).astype(np.float32)
        C = rng.integers(-8, 9, (m, n)).astype(np.float32)
        ref = A.astype(np.float64) @ B.astype(np.float64)
        np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C, err_msg=str((m, n, k)))


def test_sgemm_k_slices_against_oracle_and_repeatable(ko, sgemm_k_slices):
    """Uniform inputs through the sliced path: within the fp32 summation bound of the oracle, bit-identical
    from call to call (the partial products are summed in slice order, not in order of arrival), and the
    epilogue (alpha, beta, C) is applied once, to the sum."""
    m, n, k = 256, 256, 2048
    A, B = inputs.uniform_f32((m, k), 21), inputs.uniform_f32((k, n), 22)
    C = inputs.normal_f32((m, n), 23)
    ref, ap = oracle.sgemm(A, B, want_absprod=True)
    first = ko.sgemm_host(A, B)
    assert_sgemm_close(first, ref, ap, k)
    for _ in range(3):
        np.testing.assert_array_equal(ko.sgemm_host(A, B), first)
    ref2, ap2 = oracle.sgemm(A, B, C, 0.5, -2.0, want_absprod=True)
    assert_sgemm_close(ko.sgemm_host(A, B, C, 0.5, -2.0), ref2, 0.5 * ap2 + 2.0 * np.abs(C) + 1e-6, k)
    # C and D the same buffer (D = alpha A B + beta D): the summing kernel reads C where it writes D
    dA, dB, dD = ko.DeviceBuffer.from_numpy(A), ko.DeviceBuffer.from_numpy(B), ko.DeviceBuffer.from_numpy(C)
    ko.sgemm(m, n, k, dA, dB, dD, dD, 0.5, -2.0)
    ko.synchronize()
    assert_sgemm_close(dD.download(np.float32, (m, n)), ref2, 0.5 * ap2 + 2.0 * np.abs(C) + 1e-6, k)
    sgemm_k_slices(1)
    assert_sgemm_close(ko.sgemm_host(A, B), ref, ap, k)


def test_sgemm_cfg3_full(ko):
    """1024^3, U(-1,1), alpha=1, beta=0, C null: the whole output against the oracle, with the
    reference's own abs <= 1e-3 gate (nn_operators/gemm/main.cu:169-170) as well."""
    c = inputs.make_inputs(3)
    ref, ap = oracle.sgemm(c["A"], c["B"], want_absprod=True)
    assert_sgemm_close(ko.sgemm_host(c["A"], c["B"]), ref, ap, 1024, reference_gate=True)


def test_sgemm_epilogue(ko):
    """D = acc + C (the reference's epilogue with C given, simt_gemm.h:325-354) and alpha/beta."""
    m, n, k = 96, 160, 72
    A, B = inputs.uniform_f32((m, k), 1), inputs.uniform_f32((k, n), 2)
    C = inputs.normal_f32((m, n), 3)
    for alpha, beta in ((1.0, 1.0), (0.5, -2.0), (2.0, 0.0)):
        ref, ap = oracle.sgemm(A, B, C, alpha, beta, want_absprod=True)
        bound_scale = abs(alpha) * ap + abs(beta) * np.abs(C)
        assert_sgemm_close(ko.sgemm_host(A, B, C, alpha, beta), ref, bound_scale + 1e-6, k)


def test_sgemm_exact_cases(ko):
    """Identity known-answer test of the reference (A[idx] = idx/1024, B = I, gemm/main.cu:219,226),
    all-ones -> exactly K, and small integers -> bit-exact for any summation order."""
    n = 256
    A = (np.arange(n * n) // 1024).astype(np.float32).reshape(n, n)
    np.testing.assert_array_equal(ko.sgemm_host(A, np.eye(n, dtype=np.float32)), A)
    np.testing.assert_array_equal(ko.sgemm_host(np.ones((64, 512), np.float32), np.ones((512, 128), np.float32)),
                                  np.full((64, 128), 512, np.float32))
    rng = np.random.default_rng(5)
    Ai = rng.integers(-4, 5, (130, 1024)).astype(np.float32)
    Bi = rng.integers(-4, 5, (1024, 72)).astype(np.float32)
    np.testing.assert_array_equal(ko.sgemm_host(Ai, Bi), (Ai.astype(np.float64) @ Bi.astype(np.float64)))


def test_sgemm_errors(ko):
    buf = ko.DeviceBuffer(1 << 16)
    with pytest.raises(ko.KoError) as e:
        ko.sgemm(16, 16, 16, None, buf, buf)
    assert e.value.status == ko.KO_ERR_INVALID_ARGUMENT
    with pytest.raises(ko.KoError) as e:
        ko.sgemm(-1, 16, 16, buf, buf, buf)
    assert e.value.status == ko.KO_ERR_INVALID_ARGUMENT
    ko.sgemm(0, 16, 16, buf, buf, buf)  # empty problem


# ----------------------------------------------------------------------------------- GEMM16

def _bits16(shape, seed, bf16):
    if bf16:
        return inputs.uniform_bf16_bits(shape, seed)
    return inputs.uniform_f16(shape, seed).view(np.uint16)


def _to_f64(bits, bf16):
    return oracle.bf16_to_f64(bits) if bf16 else oracle.f16_to_f64(bits)


@pytest.mark.parametrize("gemm16_variant", GEMM16_VARIANTS, indirect=True)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (300, 520, 72), (33, 36, 8), (128, 384, 768), (512, 768, 192),
                                   (384, 512, 256)])
def test_gemm16_matches_oracle(ko, gemm16_variant, bf16, b_col_major, m, n, k):
    if gemm16_variant == 30 and not b_col_major:
        pytest.skip("the compiler-scheduled direct-to-LDS kernel takes column-major B")
    if gemm16_variant >= 30 and (m % (128 if gemm16_variant == 54 else 256) or n % 256 or k % 64):
        pytest.skip("the direct-to-LDS kernels take full tiles only")
    if gemm16_variant >= 50 and k % 128:
        pytest.skip("the pinned kernel takes an even number of K tiles")
    A = _bits16((m, k), 21 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 23 + n, bf16)
    _, ref64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, bf16=bf16)
    got = ko.gemm16_host(A, B, m, n, k, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR,
                         dtype=ko.BF16 if bf16 else ko.F16)
    assert_gemm16_close(_to_f64(got, bf16), ref64, ap, k, bf16=bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("m,n,k", [(512, 768, 128), (2048, 1024, 256), (16384, 3072, 768), (4096, 4096, 200)])
def test_gemm16_row_major_b_gives_the_same_bits(ko, m, n, k, bf16):
    """B handed over as [K][N] (the reference's layout, tensor_core_gemm.h) or as its transpose [N][K]: the same
    products are accumulated in the same order by the same instruction, so D must agree bit for bit - through the
    register pipeline (small and ragged-K shapes) and through the pinned direct-to-LDS kernel (the big ones)."""
    dt = ko.BF16 if bf16 else ko.F16
    dA, dBc, dBr = ko.DeviceBuffer(m * k * 2), ko.DeviceBuffer(n * k * 2), ko.DeviceBuffer(n * k * 2)
    ko.fill_uniform_16(dA, m * k, 81, dtype=dt)
    ko.fill_uniform_16(dBc, n * k, 82, dtype=dt)
    ko.synchronize()
    b_col = dBc.download(np.uint16, (n, k))
    dBr.upload(np.ascontiguousarray(b_col.T))
    outs = []
    for buf, layout in ((dBc, ko.COL_MAJOR), (dBr, ko.ROW_MAJOR)):
        dD = ko.DeviceBuffer(m * n * 2)
        ko.gemm16(m, n, k, dA, buf, dD, b_layout=layout, dtype=dt)
        ko.synchronize()
        outs.append(dD.download(np.uint16, (m, n)))
    np.testing.assert_array_equal(outs[0], outs[1])


@pytest.mark.parametrize("m,n,k", [(8192, 4096, 192), (2048, 1024, 64), (16384, 3072, 768)])
def test_gemm16_variants_agree_bitwise(ko, m, n, k):
    """Every tiling accumulates in the same K order with the same matrix instruction, so all variants
    must give the same bits; the persistent variants walk several tiles per workgroup here (and an odd
    number of K tiles, which flips the LDS stage parity from tile to tile).  Sampled rows also go
    against the oracle."""
    dA, dB = ko.DeviceBuffer(m * k * 2), ko.DeviceBuffer(n * k * 2)
    ko.fill_uniform_16(dA, m * k, 77)
    ko.fill_uniform_16(dB, n * k, 78)
    outs = {}
    try:
        for v in GEMM16_VARIANTS[1:]:
            if v >= 50 and k % 128:
                continue
            ko.set_tuning("gemm16.variant", v)
            dD = ko.DeviceBuffer(m * n * 2)
            ko.gemm16(m, n, k, dA, dB, dD)
            ko.synchronize()
            outs[v] = dD.download(np.uint16, (m, n))
    finally:
        ko.set_tuning("gemm16.variant", 0)
    base = outs[3]
    for v, d in outs.items():
        np.testing.assert_array_equal(d, base, err_msg="variant %d differs from variant 3" % v)
    idx = np.sort(np.random.default_rng(3).choice(m, 48, replace=False))
    A = dA.download(np.uint16, (m, k))[idx]
    B = dB.download(np.uint16, (n, k))
    _, ref64, ap = oracle.gemm16(A, B, len(idx), n, k)
    assert_gemm16_close(oracle.f16_to_f64(base[idx]), ref64, ap, k)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(4096, 2048, 760), (2048, 4096, 200), (4352, 2304, 136), (2048, 4096, 1032)])
def test_gemm16_k_off_the_k_tile_is_padded_with_zeros(ko, m, n, k, b_col_major, bf16):
    """K a multiple of 8 but not of 128 on shapes of full 256 x 256 tiles: the pinned kernel pads K with zeros
    up to the next pair of K tiles (lanes whose chunk or row lies past K fetch a zero chunk).  A zero that is
    missing, a chunk fetched from the next row instead, or padding applied to the wrong K tile changes the
    sums: the whole output must equal the register pipeline's (variant 9, which bounds-checks K) bit for bit,
    and sampled rows must agree with the oracle."""
    A = _bits16((m, k), 61, bf16)
    B = _bits16((n, k), 62, bf16)
    Bdev = B if b_col_major else np.ascontiguousarray(B.T)
    kw = dict(dtype=ko.BF16 if bf16 else ko.F16, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR)
    got = ko.gemm16_host(A, Bdev, m, n, k, **kw)
    ko.set_tuning("gemm16.variant", 9)
    try:
        want = ko.gemm16_host(A, Bdev, m, n, k, **kw)
    finally:
        ko.set_tuning("gemm16.variant", 0)
    np.testing.assert_array_equal(got, want)
    idx = np.sort(np.random.default_rng(5).choice(m, 48, replace=False))
    _, ref64, ap = oracle.gemm16(A[idx], B, len(idx), n, k, bf16=bf16)
    assert_gemm16_close(_to_f64(got[idx], bf16), ref64, ap, k, bf16=bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("k", [320, 384])
def test_gemm16_default_path_big(ko, bf16, k):
    """Large enough for the default dispatch to take a persistent direct-to-LDS kernel (512 tiles of
    256 x 256: several tiles per workgroup), both 16-bit types.  k = 320 is an odd number of K tiles
    (compiler-scheduled kernel), k = 384 an even one (pinned kernel)."""
    m, n = 8192, 4096
    A = _bits16((m, k), 31, bf16)
    B = _bits16((n, k), 32, bf16)
    got = ko.gemm16_host(A, B, m, n, k, dtype=ko.BF16 if bf16 else ko.F16)
    idx = np.sort(np.random.default_rng(4).choice(m, 64, replace=False))
    _, ref64, ap = oracle.gemm16(A[idx], B, len(idx), n, k, bf16=bf16)
    assert_gemm16_close(_to_f64(got[idx], bf16), ref64, ap, k, bf16=bf16)


@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n", [(4096, 3072), (2048, 4096), (3072, 2816), (2048, 2048), (1024, 1536), (4352, 4096),
                                 (4136, 2048)])
def test_gemm16_default_path_partly_filled_chip(ko, m, n, b_col_major):
    """Between half a chip's and a chip's worth of 256 x 256 tiles (192, 128 and 132 of them): the default dispatch
    still takes the pinned kernel, with fewer workgroups than compute units and, for 132 tiles, a grid that is not a
    multiple of eight.  Fewer still (64 and 24 big tiles): the 128 x 64 and 64 x 64 tilings of the register
    pipeline.  272 tiles: sixteen workgroups walk two tiles, the others one.  Sampled rows against the oracle, both
    layouts of B."""
    k = 256
    A = _bits16((m, k), 35, False)
    B = _bits16((n, k) if b_col_major else (k, n), 36, False)
    got = ko.gemm16_host(A, B, m, n, k, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR)
    idx = np.random.default_rng(5).choice(m, 64, replace=False)
    # 272 tiles go out as two launches (tile rows 0..15, then the last 256 rows): both sides of the cut
    # 4136 rows: the 4096 rows of full tiles on the pinned kernel, the last 40 as a launch of their own
    idx = np.unique(np.concatenate([idx, [0, m - 257, m - 256, m - 255, m - 1, m // 256 * 256 - 1,
                                          min(m // 256 * 256, m - 1)]]))
    _, ref64, ap = oracle.gemm16(A[idx], B, len(idx), n, k, b_col_major=b_col_major)
    assert_gemm16_close(_to_f64(got[idx], False), ref64, ap, k)


def test_gemm16_odd_n(ko):
    """n not a multiple of 4: the element-wise store path."""
    m, n, k = 70, 45, 40
    A, B = _bits16((m, k), 1, False), _bits16((n, k), 2, False)
    _, ref64, ap = oracle.gemm16(A, B, m, n, k)
    assert_gemm16_close(_to_f64(ko.gemm16_host(A, B, m, n, k), False), ref64, ap, k)


def test_gemm16_epilogue(ko):
    m, n, k = 160, 192, 64
    A, B = _bits16((m, k), 4, False), _bits16((n, k), 5, False)
    C = inputs.uniform_f16((m, n), 6, -2.0, 2.0).view(np.uint16)
    for alpha, beta in ((1.0, 1.0), (0.5, -1.5)):
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, C_bits=C, alpha=alpha, beta=beta)
        got = ko.gemm16_host(A, B, m, n, k, C_bits=C, alpha=alpha, beta=beta)
        scale = abs(alpha) * ap + abs(beta) * np.abs(oracle.f16_to_f64(C))
        assert_gemm16_close(_to_f64(got, False), ref64, scale, k)


def test_gemm16_exact_cases(ko):
    """Reference known-answer inputs (A[idx] = idx/1024, B = I, C = 0; gemm/main.cu:219,226,233) and
    small integers (every partial sum < 2^11 is exact in fp32 and in binary16)."""
    n = 256
    A = (np.arange(n * n) // 1024).astype(np.float16)
    I = np.eye(n, dtype=np.float16)
    for layout in (ko.COL_MAJOR, ko.ROW_MAJOR):
        got = ko.gemm16_host(A.view(np.uint16), I.view(np.uint16), n, n, n, b_layout=layout)
        np.testing.assert_array_equal(got.view(np.float16), A.reshape(n, n))
    rng = np.random.default_rng(9)
    Ai = rng.integers(-2, 3, (96, 128)).astype(np.float16)
    Bi = rng.integers(-2, 3, (200, 128)).astype(np.float16)  # [n][k]
    got = ko.gemm16_host(Ai.view(np.uint16), Bi.view(np.uint16), 96, 200, 128).view(np.float16)
    np.testing.assert_array_equal(got.astype(np.float64), Ai.astype(np.float64) @ Bi.astype(np.float64).T)


def _cfg4_rows(m, tile=256):
    """Rows of D compared with the oracle: two at random inside every 256-row tile row of the kernel's walk, both
    sides of every tile-row boundary, and the first and last two rows - every tile of the output is covered
    (each sampled row is checked over all of its columns)."""
    rng = np.random.default_rng(1)
    inside = [t * tile + rng.choice(np.arange(1, tile - 1), 2, replace=False) for t in range(m // tile)]
    edges = [[t * tile - 1, t * tile] for t in range(1, m // tile)]
    return np.unique(np.concatenate(inside + edges + [[0, 1, m - 2, m - 1]]))


def test_gemm16_cfg4_sampled(ko):
    """BERT FFN up-projection at full size (16384 x 3072 x 768, fp16, column-major B), operands filled on
    the device: rows from every tile row of D (see _cfg4_rows) against the oracle on the bytes the kernel read,
    and linearity over the whole output (D(2A) == 2 D(A) bit for bit wherever the result is a normal fp16
    number: scaling by 2 is exact in fp16 and fp32)."""
    m, n, k = 16384, 3072, 768
    dA, dB, dD = ko.DeviceBuffer(m * k * 2), ko.DeviceBuffer(n * k * 2), ko.DeviceBuffer(m * n * 2)
    ko.fill_uniform_16(dA, m * k, inputs.tensor_seed(4, 0))
    ko.fill_uniform_16(dB, n * k, inputs.tensor_seed(4, 1))
    ko.gemm16(m, n, k, dA, dB, dD)
    ko.synchronize()
    A = dA.download(np.uint16, (m, k))
    B = dB.download(np.uint16, (n, k))
    D = dD.download(np.uint16, (m, n))
    hostA = inputs.uniform_f16((8, k), inputs.tensor_seed(4, 0)).view(np.uint16)
    np.testing.assert_array_equal(hostA, A[:8])  # device fill == host generator, bit for bit
    idx = _cfg4_rows(m)
    assert len(idx) >= 2 * (m // 256) + 2 * (m // 256 - 1)
    _, ref64, ap = oracle.gemm16(A[idx], B, len(idx), n, k)
    assert_gemm16_close(oracle.f16_to_f64(D[idx]), ref64, ap, k)
    assert np.all(np.isfinite(D.view(np.float16)))
    dA2 = ko.DeviceBuffer.from_numpy((A.view(np.float16) * np.float16(2)).view(np.uint16))
    dD2 = ko.DeviceBuffer(m * n * 2)
    ko.gemm16(m, n, k, dA2, dB, dD2)
    ko.synchronize()
    D2 = dD2.download(np.uint16, (m, n)).view(np.float16)
    want = D.view(np.float16) * np.float16(2)
    normal = np.abs(want) >= 2.0 ** -13  # subnormal results round on a fixed grid, so scaling is exact only above it
    np.testing.assert_array_equal(D2[normal], want[normal])
    assert np.abs(D2[~normal].astype(np.float64) - want[~normal].astype(np.float64)).max(initial=0.0) <= 2.0 ** -23


def _vendor_lib():
    import ctypes
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "kernel_optimization_amd", "lib",
                        "libko_vendor.so")
    if not os.path.exists(path):
        pytest.skip("libko_vendor.so (hipBLASLt comparison harness) is not built")
    V = ctypes.CDLL(path)
    i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    V.kov_gemm16.argtypes = [i64, i64, i64, vp, vp, ci, vp, ci, ci, ci, ctypes.POINTER(ctypes.c_float),
                             ctypes.POINTER(ci)]
    V.kov_sgemm.argtypes = [i64, i64, i64, vp, vp, vp, ci, ci, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ci)]
    return V


@pytest.mark.parametrize("b_col_major", [True, False])
def test_gemm16_cfg4_agrees_with_hipblaslt(ko, b_col_major):
    """The vendor library on the same device buffers, the role cublasHgemm plays in the reference's driver
    (nn_operators/gemm/main.cu:314-318): the whole 16384 x 3072 output.  Both accumulate in fp32 and round once,
    so they may differ by the last bit where the K order differs: every element within one fp16 ulp, and all but
    a thousandth of them identical (on the library version this was written against: all of them)."""
    import ctypes
    V = _vendor_lib()
    m, n, k = 16384, 3072, 768
    dA, dB = ko.DeviceBuffer(m * k * 2), ko.DeviceBuffer(n * k * 2)
    dD, dV = ko.DeviceBuffer(m * n * 2), ko.DeviceBuffer(m * n * 2)
    ko.fill_uniform_16(dA, m * k, inputs.tensor_seed(4, 0))
    ko.fill_uniform_16(dB, n * k, inputs.tensor_seed(4, 1))
    ko.gemm16(m, n, k, dA, dB, dD, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR)
    ko.synchronize()
    us, na = ctypes.c_float(), ctypes.c_int()
    rc = V.kov_gemm16(m, n, k, dA.ptr, dB.ptr, 1 if b_col_major else 0, dV.ptr, 0, 4, 3, ctypes.byref(us), ctypes.byref(na))
    assert rc == 0, "hipBLASLt found no algorithm"
    got = dD.download(np.uint16, (m, n)).view(np.float16).astype(np.float32)
    ref = dV.download(np.uint16, (m, n)).view(np.float16).astype(np.float32)
    ulp = np.maximum(np.spacing(np.abs(ref).astype(np.float16)).astype(np.float32), np.float32(2.0 ** -24))
    assert np.all(np.abs(got - ref) <= ulp), "differs from hipBLASLt by more than one fp16 ulp"
    assert np.mean(got != ref) <= 1e-3, "%.4f of the elements differ from hipBLASLt" % np.mean(got != ref)


def test_sgemm_cfg3_agrees_with_hipblaslt(ko):
    """fp32 1024^3 against the vendor library with the reference's own gate: abs <= 1e-3
    (nn_operators/gemm/main.cu:169-170)."""
    import ctypes
    V = _vendor_lib()
    n = 1024
    dA, dB, dD, dV = (ko.DeviceBuffer(n * n * 4) for _ in range(4))
    ko.fill_uniform_f32(dA, n * n, inputs.tensor_seed(3, 0))
    ko.fill_uniform_f32(dB, n * n, inputs.tensor_seed(3, 1))
    ko.sgemm(n, n, n, dA, dB, dD)
    ko.synchronize()
    us, na = ctypes.c_float(), ctypes.c_int()
    assert V.kov_sgemm(n, n, n, dA.ptr, dB.ptr, dV.ptr, 4, 3, ctypes.byref(us), ctypes.byref(na)) == 0
    d = np.abs(dD.download(np.float32, (n, n)) - dV.download(np.float32, (n, n)))
    assert d.max() <= 1e-3, "differs from hipBLASLt by %.3e" % d.max()


def test_gemm16_errors(ko):
    buf = ko.DeviceBuffer(1 << 16)
    with pytest.raises(ko.KoError) as e:
        ko.gemm16(16, 16, 12, buf, buf, buf)  # k % 8 != 0
    assert e.value.status == ko.KO_ERR_UNSUPPORTED_SHAPE
    with pytest.raises(ko.KoError) as e:
        ko.gemm16(16, 16, 16, buf, buf, buf, dtype=7)
    assert e.value.status == ko.KO_ERR_INVALID_ARGUMENT
    with pytest.raises(ko.KoError) as e:
        ko.gemm16(16, 16, 16, buf, None, buf)
    assert e.value.status == ko.KO_ERR_INVALID_ARGUMENT


# ------------------------------------------------------------------------------------ fused epilogue

def assert_gemm16_act_close(got_f64, ref_f64, absprod, k, bf16=False):
    """act(alpha A B + beta C + bias): the activations used here have slope <= 1.13, and their fp32
    evaluation (erff / exp) adds a few units in the last place of the result."""
    got, ref = np.asarray(got_f64, np.float64), np.asarray(ref_f64, np.float64)
    assert np.all(np.isfinite(got))
    ulp = 2.0 ** -8 if bf16 else 2.0 ** -11
    bound = ulp * np.abs(ref) + 1.13 * (k * 2.0 ** -24 * absprod + 2.0 ** -22) + 4 * 2.0 ** -24 * np.abs(ref) + 2.0 ** -24
    worst = (np.abs(got - ref) / bound).max()
    assert worst <= 1.0, "gemm16 epilogue err exceeds bound by factor %.3f" % worst


@pytest.mark.parametrize("act", [0, 1, 2])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (300, 520, 72), (33, 36, 8), (70, 45, 40)])
def test_gemm16_bias_activation(ko, act, bf16, b_col_major, m, n, k):
    A = _bits16((m, k), 41 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 43 + n, bf16)
    C = _bits16((m, n), 45, bf16)
    bias = _bits16((n,), 47, bf16)
    for c_bits, beta, use_bias in ((None, 0.0, True), (C, 0.5, True), (C, 1.0, False)):
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, bf16=bf16, C_bits=c_bits, beta=beta,
                                     bias_bits=bias if use_bias else None, act=act)
        ap = ap + 2.0  # |beta C| + |bias| <= 2: their roundings enter like one more product each
        got = ko.gemm16_host(A, B, m, n, k, C_bits=c_bits, beta=beta, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR,
                             dtype=ko.BF16 if bf16 else ko.F16, bias_bits=bias if use_bias else None, act=act)
        assert_gemm16_act_close(_to_f64(got, bf16), ref64, ap, k, bf16=bf16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k,slices", [(512, 512, 8192, 0), (256, 384, 2048, 3), (300, 520, 1096, 2), (768, 768, 4096, 7),
                                          (130, 72, 4104, 5),
                                          # rows of D off 8-byte boundaries, a ragged last group of four columns
                                          (282, 31, 13104, 0), (48, 107, 7144, 0), (130, 75, 4104, 5), (16, 1001, 4008, 0),
                                          (339, 670, 6784, 0), (33, 2, 2048, 3),
                                          # at most 32 rows: 32 x 256 tiles, slices chosen by the planner
                                          (8, 4096, 4096, 0), (1, 512, 8192, 0), (32, 264, 2120, 0), (20, 1000, 2048, 0)])
def test_gemm16_k_slices(ko, m, n, k, slices, b_col_major, bf16):
    """A deep K on few tiles goes out as K slices of the register pipeline (fp32 partial products into the stream's
    workspace) and a kernel that sums them in slice order and applies alpha, beta C, bias and the activation once.
    slices = 0: the planner's own choice; otherwise a forced count (ragged tiles, a last slice that ends inside
    a K tile).  Against the oracle, plain and with the whole epilogue, and bit-stable from call to call."""
    A = _bits16((m, k), 71 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 73 + n, bf16)
    C = _bits16((m, n), 75, bf16)
    bias = _bits16((n,), 77, bf16)
    kw = dict(b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR, dtype=ko.BF16 if bf16 else ko.F16)
    ko.set_tuning("gemm16.k_slices", slices)
    try:
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, bf16=bf16)
        got = ko.gemm16_host(A, B, m, n, k, **kw)
        assert_gemm16_close(_to_f64(got, bf16), ref64, ap, k, bf16=bf16)
        np.testing.assert_array_equal(ko.gemm16_host(A, B, m, n, k, **kw), got)
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, bf16=bf16, C_bits=C, beta=0.5, bias_bits=bias, act=2)
        got = ko.gemm16_host(A, B, m, n, k, C_bits=C, beta=0.5, bias_bits=bias, act=2, **kw)
        assert_gemm16_act_close(_to_f64(got, bf16), ref64, ap + 2.0, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.k_slices", 0)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(1536, 4096, 2048), (1608, 4096, 2048), (2048, 2304, 392)])
def test_gemm16_between_half_and_a_whole_chip_of_128x256_tiles(ko, m, n, k, b_col_major, bf16):
    """Shapes whose 256 x 256 tiles would cover half of the chip or less take 128 x 256 tiles of the pinned kernel
    (192, 192 and 144 of them here; the second shape's last 72 rows go out as a launch of their own, the third
    has a K that ends inside a pair of K tiles).  Sampled rows of every part against the oracle, with the whole
    epilogue, and - in the rows the pinned kernel wrote; the rows below them go out as K slices, which round
    differently - the same bits as the 128 x 128 register pipeline (same K order, same instruction)."""
    A = _bits16((m, k), 91, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 92, bf16)
    C = _bits16((m, n), 93, bf16)
    bias = _bits16((n,), 94, bf16)
    idx = np.unique(np.concatenate([np.random.default_rng(9).choice(m, 40, replace=False), np.arange(m - 8, m)]))
    kw = dict(b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR, dtype=ko.BF16 if bf16 else ko.F16)
    _, ref64, ap = oracle.gemm16(A[idx], B, len(idx), n, k, b_col_major=b_col_major, bf16=bf16, C_bits=C[idx], beta=0.5,
                                 bias_bits=bias, act=2)
    got = ko.gemm16_host(A, B, m, n, k, C_bits=C, beta=0.5, bias_bits=bias, act=2, **kw)
    assert_gemm16_act_close(_to_f64(got[idx], bf16), ref64, ap + 2.0, k, bf16=bf16)
    plain = ko.gemm16_host(A, B, m, n, k, **kw)
    ko.set_tuning("gemm16.variant", 10)
    try:
        top = m // 128 * 128
        np.testing.assert_array_equal(plain[:top], ko.gemm16_host(A, B, m, n, k, **kw)[:top])
    finally:
        ko.set_tuning("gemm16.variant", 0)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
def test_gemm16_parts_cut_off_a_ragged_shape_are_sliced(ko, b_col_major, bf16):
    """2108 x 4232 x 2048: the call is cut into a block of full 256 x 256 tiles, the 60 rows below it and the 136
    columns to its right; the two cut-off parts have few tiles and a deep K and go out as K slices through the
    stream's workspace, one after the other.  Sampled rows of all three parts (every column) against the oracle,
    with the whole epilogue; with slices switched off the parts run whole and must agree to the same bound."""
    m, n, k = 2108, 4232, 2048
    A = _bits16((m, k), 81, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 82, bf16)
    C = _bits16((m, n), 83, bf16)
    bias = _bits16((n,), 84, bf16)
    idx = np.concatenate([np.sort(np.random.default_rng(8).choice(2048, 24, replace=False)), np.arange(2048, m, 5)])
    kw = dict(b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR, dtype=ko.BF16 if bf16 else ko.F16)
    _, ref64, ap = oracle.gemm16(A[idx], B, len(idx), n, k, b_col_major=b_col_major, bf16=bf16, C_bits=C[idx], beta=0.5,
                                 bias_bits=bias, act=2)
    try:
        for slices in (0, 1):
            ko.set_tuning("gemm16.k_slices", slices)
            got = ko.gemm16_host(A, B, m, n, k, C_bits=C, beta=0.5, bias_bits=bias, act=2, **kw)
            assert_gemm16_act_close(_to_f64(got[idx], bf16), ref64, ap + 2.0, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.k_slices", 0)


@pytest.mark.parametrize("variant", [0, 9, 30, 50])
@pytest.mark.parametrize("bf16", [False, True])
def test_gemm16_bias_gelu_big(ko, variant, bf16):
    """The up-projection shape in small (512 tiles of 256 x 256, K = 384): bias + GELU and beta * C through the
    coalesced epilogue of every kernel family; sampled rows against the oracle."""
    m, n, k = 8192, 4096, 384
    A = _bits16((m, k), 51, bf16)
    B = _bits16((n, k), 52, bf16)
    bias = _bits16((n,), 53, bf16)
    C = _bits16((m, n), 54, bf16)
    idx = np.sort(np.random.default_rng(6).choice(m, 48, replace=False))
    ko.set_tuning("gemm16.variant", variant)
    try:
        for act, c_bits, beta in ((1, None, 0.0), (2, C, -0.5), (0, C, 1.0)):
            got = ko.gemm16_host(A, B, m, n, k, C_bits=c_bits, beta=beta, dtype=ko.BF16 if bf16 else ko.F16,
                                 bias_bits=bias, act=act)
            _, ref64, ap = oracle.gemm16(A[idx], B, len(idx), n, k, bf16=bf16, C_bits=None if c_bits is None else c_bits[idx],
                                         beta=beta, bias_bits=bias, act=act)
            assert_gemm16_act_close(_to_f64(got[idx], bf16), ref64, ap + 2.0, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.variant", 0)


def test_gemm16_bias_act_errors(ko):
    d = ko.DeviceBuffer(1 << 16)
    L = ko.lib()
    assert L.ko_gemm_f16f32acc_bias_act(16, 16, 16, 1.0, d.ptr, d.ptr, ko.COL_MAJOR, 0.0, None, None, 7, d.ptr, ko.F16, None) == ko.KO_ERR_INVALID_ARGUMENT
    assert L.ko_gemm_f16f32acc_bias_act(16, 16, 16, 1.0, d.ptr, d.ptr, ko.COL_MAJOR, 0.0, None, d.ptr + 2, 1, d.ptr, ko.F16, None) == ko.KO_ERR_INVALID_ARGUMENT
    assert L.ko_gemm_f16f32acc_bias_act(0, 16, 16, 1.0, d.ptr, d.ptr, ko.COL_MAJOR, 0.0, None, None, 1, d.ptr, ko.F16, None) == ko.KO_OK


def test_sgemm_ragged_shapes_are_exact_on_small_integers(ko):
    """Shapes that fill neither their tiles nor their K tiles, through the default dispatch (edge form of the
    direct-to-LDS kernels where operand rows start on 16-byte boundaries): rows past M and columns past N are
    fetched from clamped addresses and K is padded with zeros, none of which may reach the output.  Small
    integers make every sum exact."""
    rng = np.random.default_rng(7)
    shapes = [(int(rng.integers(1, 3000)), int(rng.integers(1, 750)) * 4, int(rng.integers(1, 500)) * 4) for _ in range(10)]
    shapes += [(2305, 2048, 516), (4100, 2052, 260), (129, 4, 4), (1, 128, 2048), (3000, 36, 1000), (257, 1028, 132)]
    for m, n, k in shapes:
        A = rng.integers(-4, 5, (m, k)).astype(np.float32)
        B = rng.integers(-4, 5, (k, n)).astype(np.float32)
        C = rng.integers(-8, 9, (m, n)).astype(np.float32)
        ref = A.astype(np.float64) @ B.astype(np.float64)
        np.testing.assert_array_equal(ko.sgemm_host(A, B), ref, err_msg=str((m, n, k)))
        np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C, err_msg=str((m, n, k)))


def test_sgemm_rows_off_16_byte_boundaries_are_exact_on_small_integers(ko):
    """N, K or a base pointer that is not a multiple of four floats: operand rows do not start on 16-byte
    boundaries and the direct-to-LDS kernels fill their stages four bytes per lane.  Every lane then fetches one
    element of its own (clamped at M and N, a zero past K), so a wrong element, a missing zero or a swizzle
    applied at the wrong granularity shows as a wrong integer.  The register pipeline (knob sgemm.unaligned = 1)
    must give the same matrix."""
    rng = np.random.default_rng(11)
    shapes = [(int(rng.integers(1, 1500)), int(rng.integers(1, 1500)), int(rng.integers(1, 1500))) for _ in range(10)]
    shapes += [(1023, 1025, 1027), (129, 2, 1), (64, 64, 65), (2500, 2302, 130), (3, 1001, 2050), (2049, 2047, 3000)]
    try:
        for m, n, k in shapes:
            A = rng.integers(-4, 5, (m, k)).astype(np.float32)
            B = rng.integers(-4, 5, (k, n)).astype(np.float32)
            C = rng.integers(-8, 9, (m, n)).astype(np.float32)
            ref = A.astype(np.float64) @ B.astype(np.float64)
            for knob in (0, 1):
                ko.set_tuning("sgemm.unaligned", knob)
                np.testing.assert_array_equal(ko.sgemm_host(A, B), ref, err_msg=str((m, n, k, knob)))
                np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C, err_msg=str((m, n, k, knob)))
    finally:
        ko.set_tuning("sgemm.unaligned", 0)
    # aligned sizes behind base pointers that are one float off a 16-byte boundary
    m, n, k = 200, 136, 264
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    dA, dB, dD = ko.DeviceBuffer(m * k * 4 + 16), ko.DeviceBuffer(k * n * 4 + 16), ko.DeviceBuffer(m * n * 4)
    for offset_a, offset_b in ((4, 0), (0, 4), (12, 8)):
        dA.upload(np.concatenate([np.zeros(offset_a // 4, np.float32), A.ravel(), np.zeros(4 - offset_a // 4, np.float32)]))
        dB.upload(np.concatenate([np.zeros(offset_b // 4, np.float32), B.ravel(), np.zeros(4 - offset_b // 4, np.float32)]))
        ko.sgemm(m, n, k, dA.ptr + offset_a, dB.ptr + offset_b, dD)
        ko.synchronize()
        np.testing.assert_array_equal(dD.download(np.float32, (m, n)), A.astype(np.float64) @ B.astype(np.float64))


@pytest.mark.parametrize("sgemm_variant", [33, 35, 36, 37, 41], indirect=True)
def test_sgemm_unaligned_rows_against_oracle(ko, sgemm_variant):
    """Uniform inputs through the four-byte form of every direct-to-LDS tiling, within the fp32 summation bound."""
    m, n, k = 261, 203, 777
    A, B = inputs.uniform_f32((m, k), 31), inputs.uniform_f32((k, n), 32)
    ref, ap = oracle.sgemm(A, B, want_absprod=True)
    assert_sgemm_close(ko.sgemm_host(A, B), ref, ap, k)


@pytest.mark.parametrize("m,n,k", [(4136, 2048, 256), (8000, 2304, 768), (4353, 4096, 128)])
def test_gemm16_ragged_row_counts_whole_output(ko, m, n, k):
    """Row counts that do not fill the last row of 256 x 256 tiles: the full tile rows run on the pinned kernel,
    the rest as a launch of its own (8000 x 2304: two cuts, at the last full round and at the last full tile
    row).  Small integers: the fp32 sums are exact, so the whole output equals the rounded exact product."""
    rng = np.random.default_rng(m + k)
    A = rng.integers(-4, 5, (m, k)).astype(np.float16)
    B = rng.integers(-4, 5, (n, k)).astype(np.float16)
    got = ko.gemm16_host(A.view(np.uint16), B.view(np.uint16), m, n, k).view(np.float16)
    ref = (A.astype(np.float64) @ B.astype(np.float64).T).astype(np.float16)
    np.testing.assert_array_equal(got, ref)


@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(4096, 2200, 256), (4136, 2312, 128), (8192, 1288, 384), (8000, 2312, 768)])
def test_gemm16_ragged_column_counts_whole_output(ko, m, n, k, b_col_major):
    """Column counts (multiples of 8) that do not fill the last column of 256 x 256 tiles, both layouts of B: the full
    tile columns and the remaining ones are separate launches that write column ranges of the same D (row stride
    n), each with its part of B (a row-major B keeps its row stride too), C and the bias.  With 4136 rows the full-tile
    part is cut along the rows as well; 8000 x 2312 x 768 takes the column cut and two row cuts in the left part.
    Small integers: every fp32 sum is exact, so the whole output equals the rounded exact result."""
    rng = np.random.default_rng(n + k)
    A = rng.integers(-4, 5, (m, k)).astype(np.float16)
    B = rng.integers(-4, 5, (n, k)).astype(np.float16)
    C = rng.integers(-8, 9, (m, n)).astype(np.float16)
    bias = rng.integers(-8, 9, (n,)).astype(np.float16)
    exact = A.astype(np.float64) @ B.astype(np.float64).T
    Bm = B if b_col_major else np.ascontiguousarray(B.T)
    layout = ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR
    got = ko.gemm16_host(A.view(np.uint16), Bm.view(np.uint16), m, n, k, b_layout=layout).view(np.float16)
    np.testing.assert_array_equal(got, exact.astype(np.float16))
    got = ko.gemm16_host(A.view(np.uint16), Bm.view(np.uint16), m, n, k, C_bits=C.view(np.uint16), alpha=1.0, beta=2.0,
                         b_layout=layout, bias_bits=bias.view(np.uint16)).view(np.float16)
    np.testing.assert_array_equal(got, (exact + 2.0 * C.astype(np.float64) + bias.astype(np.float64)).astype(np.float16))


@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("m,n,k", [(4096, 2202, 256), (4096, 2203, 128), (4136, 2317, 128), (8192, 1290, 384),
                                   (300, 523, 72), (256, 262, 64), (513, 259, 136)])
def test_gemm16_rows_of_c_and_d_off_16_byte_boundaries_whole_output(ko, m, n, k, b_col_major, bf16):
    """Column counts that are not a multiple of 8 (vocabulary sizes: 30522, 50257): rows of C and D then start on 4- or
    2-byte boundaries.  With a K-contiguous B the full tile columns still run on the pinned kernel and the rest as a
    launch of its own, the coalesced epilogue writing its 16-byte pieces at element alignment; a row-major B (whose
    own rows are off 16-byte boundaries then) keeps the register pipeline.  Small integers, so the whole output
    equals the rounded exact result; D sits in front of a guard area that must come back untouched."""
    rng = np.random.default_rng(n + k)
    f16 = lambda x: oracle.f64_to_bf16(x) if bf16 else oracle.f64_to_f16(x)  # one rounding to the storage type
    A = rng.integers(-4, 5, (m, k)).astype(np.float64)
    B = rng.integers(-4, 5, (n, k)).astype(np.float64)
    C = rng.integers(-8, 9, (m, n)).astype(np.float64)
    bias = rng.integers(-8, 9, (n,)).astype(np.float64)
    exact = A @ B.T
    Bm = B if b_col_major else np.ascontiguousarray(B.T)
    kw = dict(b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR, dtype=ko.BF16 if bf16 else ko.F16)
    dA, dB = ko.DeviceBuffer.from_numpy(f16(A)), ko.DeviceBuffer.from_numpy(f16(Bm))
    dC, dbias = ko.DeviceBuffer.from_numpy(f16(C)), ko.DeviceBuffer.from_numpy(f16(bias))
    guard = 64
    dD = ko.DeviceBuffer((m * n + guard) * 2)
    for c, beta, b in ((None, 0.0, None), (dC, 2.0, dbias)):
        dD.upload(np.full(m * n + guard, 0x7e7e, np.uint16))
        ko.gemm16(m, n, k, dA, dB, dD, c, 1.0, beta, bias=b, **kw)
        ko.synchronize()
        out = dD.download(np.uint16, (m * n + guard,))
        want = exact if c is None else exact + 2.0 * C + bias
        np.testing.assert_array_equal(out[:m * n].reshape(m, n), f16(want))
        assert np.all(out[m * n:] == 0x7e7e)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("m,n,k", [(2048, 1024, 8), (1024, 2048, 40), (4096, 4096, 32), (1300, 2100, 24)])
def test_gemm16_shallow_k_whole_output(ko, m, n, k, bf16):
    """K below one K tile (a rank-8 to rank-40 update): the edge form of the register pipeline pads K with zeros, and
    its tiles that lie inside the matrix take the coalesced epilogue (1300 x 2100 has both kinds of tile).  Small
    integers: the whole output, with C and a bias, equals the rounded exact result."""
    rng = np.random.default_rng(m + k)
    f16 = lambda x: oracle.f64_to_bf16(x) if bf16 else oracle.f64_to_f16(x)
    A = rng.integers(-4, 5, (m, k)).astype(np.float64)
    B = rng.integers(-4, 5, (n, k)).astype(np.float64)
    C = rng.integers(-8, 9, (m, n)).astype(np.float64)
    bias = rng.integers(-8, 9, (n,)).astype(np.float64)
    exact = A @ B.T
    kw = dict(dtype=ko.BF16 if bf16 else ko.F16)
    got = ko.gemm16_host(f16(A), f16(B), m, n, k, **kw)
    np.testing.assert_array_equal(got, f16(exact))
    got = ko.gemm16_host(f16(A), f16(B), m, n, k, C_bits=f16(C), alpha=1.0, beta=-1.0, bias_bits=f16(bias), **kw)
    np.testing.assert_array_equal(got, f16(exact - C + bias))


@pytest.mark.parametrize("m,n,k", [(2048, 2304, 8), (4096, 1024, 32), (2100, 2500, 20),
                                   # many small tiles that make no full round of big ones, K up to 256
                                   (9523, 344, 32), (9523, 343, 200), (597, 7992, 128), (597, 7990, 256), (3000, 1500, 72)])
def test_sgemm_shallow_k_is_exact_on_small_integers(ko, m, n, k):
    """A K of one 32-deep K tile or less on enough 128 x 128 tiles to fill the chip goes to the register pipeline
    (one K tile instead of a padded pair); a K of up to 256 on many small tiles to 128 x 128 tiles or the 64 x 64
    register pipeline instead of the three-stage direct-to-LDS kernels.  Small integers: exact, with alpha, beta
    and C."""
    rng = np.random.default_rng(m + k)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    C = rng.integers(-8, 9, (m, n)).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_array_equal(ko.sgemm_host(A, B), ref)
    np.testing.assert_array_equal(ko.sgemm_host(A, B, C, 2.0, -1.0), 2.0 * ref - C)


@pytest.mark.parametrize("m,n", [(64, 64), (37, 50), (1, 3), (300, 1027)])
def test_sgemm_empty_product(ko, m, n):
    """k == 0: the reference's kernel runs no K tile and its epilogue leaves D = C, or zero without a C
    (simt_gemm.h:325-354).  Here D = beta * C in one launch; A and B are not touched and may be null."""
    C = inputs.normal_f32((m, n), 5 + m)
    dC, dD = ko.DeviceBuffer.from_numpy(C), ko.DeviceBuffer(m * n * 4)
    for c, alpha, beta, want in ((dC, 1.0, 1.0, C), (dC, 3.0, -0.5, np.float32(-0.5) * C), (dC, 1.0, 0.0, np.zeros_like(C)),
                                 (None, 2.0, 1.0, np.zeros_like(C))):
        dD.upload(np.full(m * n, np.nan, np.float32))
        ko.sgemm(m, n, 0, None, None, dD, c, alpha, beta)
        ko.sgemm_static_scratch(m, n, 0, None, None, dD, c, alpha, beta)
        ko.synchronize()
        np.testing.assert_array_equal(dD.download(np.float32, (m, n)), want)
    ko.sgemm(m, n, 0, None, None, dC, dC, 1.0, 2.0)  # in place
    ko.synchronize()
    np.testing.assert_array_equal(dC.download(np.float32, (m, n)), np.float32(2.0) * C)
    with pytest.raises(ko.KoError):
        ko.sgemm(m, n, 0, None, None, None)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("m,n", [(64, 64), (37, 50), (5, 3), (130, 1032)])
def test_gemm16_empty_product(ko, bf16, m, n):
    """k == 0 on the 16-bit entries: D = activation(beta * C + bias), evaluated in fp32 and rounded once - the
    oracle's epilogue on an accumulator of zero."""
    import oracle
    dt = ko.BF16 if bf16 else ko.F16
    if bf16:
        C, bias = inputs.uniform_bf16_bits((m, n), 7 + m, -2.0, 2.0), inputs.uniform_bf16_bits((n,), 8 + m, -1.0, 1.0)
    else:
        C = inputs.uniform_f16((m, n), 7 + m, -2.0, 2.0).view(np.uint16)
        bias = inputs.uniform_f16((n,), 8 + m, -1.0, 1.0).view(np.uint16)
    c64, b64 = _to_f64(C, bf16), _to_f64(bias, bf16)
    dC, dB, dD = ko.DeviceBuffer.from_numpy(C), ko.DeviceBuffer.from_numpy(bias), ko.DeviceBuffer(m * n * 2)
    for use_c, beta, use_bias, act in ((True, 1.0, False, ko.ACT_NONE), (True, -0.5, True, ko.ACT_NONE),
                                       (False, 0.0, False, ko.ACT_NONE), (True, 1.5, True, ko.ACT_GELU_ERF),
                                       (False, 0.0, True, ko.ACT_GELU_TANH)):
        dD.upload(np.full(m * n, 0x7e00, np.uint16))
        ko.gemm16(m, n, 0, None, None, dD, C=dC if use_c else None, alpha=2.0, beta=beta, dtype=dt,
                  bias=dB if use_bias else None, act=act)
        ko.synchronize()
        got = _to_f64(dD.download(np.uint16, (m, n)), bf16)
        pre = (np.float32(beta) * c64.astype(np.float32) if use_c else np.zeros((m, n), np.float32)).astype(np.float64)
        if use_bias:
            pre = (pre.astype(np.float32) + b64.astype(np.float32)[None, :]).astype(np.float64)
        if act == ko.ACT_GELU_ERF:
            from scipy.special import erf
            want = 0.5 * pre * (1.0 + erf(pre / np.sqrt(2.0)))
        elif act == ko.ACT_GELU_TANH:
            want = 0.5 * pre * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (pre + 0.044715 * pre ** 3)))
        else:
            want = pre
        ulp = 2.0 ** -8 if bf16 else 2.0 ** -11
        assert np.all(np.abs(got - want) <= ulp * np.abs(want) + (1e-5 if act else 1e-6)), (use_c, beta, use_bias, act)
        if act == ko.ACT_NONE and not use_bias:  # one rounding of an exactly representable product chain: exact
            exact = pre if use_c else np.zeros((m, n))
            assert np.all(np.abs(got - exact) <= ulp * np.abs(exact))


def test_sgemm_forced_slices_keep_a_kernel_that_takes_them(ko):
    """A slice count forced through the knob with the tiling left to the shape: 1024 x 2048 x 512 in two slices is a
    shallow K on many small tiles, the shape class of the register pipeline, which takes no slices - the sliced
    launch has to go to the direct-to-LDS kernel of the same tile instead of being refused."""
    m, n, k = 1024, 2048, 512
    rng = np.random.default_rng(5)
    A = rng.integers(-4, 5, (m, k)).astype(np.float32)
    B = rng.integers(-4, 5, (k, n)).astype(np.float32)
    dA, dB, dD = ko.DeviceBuffer.from_numpy(A), ko.DeviceBuffer.from_numpy(B), ko.DeviceBuffer(m * n * 4)
    for slices in (2, 4):
        ko.set_tuning("sgemm.k_slices", slices)
        try:
            assert ko.gemm_plan(m, n, k)[0] == slices
            dD.upload(np.full(m * n, np.nan, np.float32))
            ko.sgemm(m, n, k, dA, dB, dD)
            ko.synchronize()
        finally:
            ko.set_tuning("sgemm.k_slices", 0)
        np.testing.assert_array_equal(dD.download(np.float32, (m, n)), A.astype(np.float64) @ B.astype(np.float64))


@pytest.mark.parametrize("variant", [60, 61])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(8, 256, 128), (136, 512, 256), (264, 256, 200), (1000, 768, 384), (3000, 512, 1032),
                                   (1, 256, 128), (257, 256, 136), (1001, 512, 392), (2047, 256, 1024)])
def test_gemm16_pinned_kernel_takes_any_row_count(ko, variant, bf16, b_col_major, m, n, k):
    """The pinned kernel with a last row of tiles that reaches past M (any M): its loads of rows at or past M
    fetch row M - 1 instead and its epilogue leaves those rows of the tile alone.  Against the oracle,
    on 256 x 256 and 128 x 256 tiles, both layouts of B, K that is and is not whole K tiles, with C and beta, and with a
    guard area behind D that must come back untouched."""
    dt = ko.BF16 if bf16 else ko.F16
    A = _bits16((m, k), 31 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 33 + n, bf16)
    C = _bits16((m, n), 35 + k, bf16)
    layout = ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR
    guard = 4096
    dA, dB, dC = ko.DeviceBuffer.from_numpy(A), ko.DeviceBuffer.from_numpy(B), ko.DeviceBuffer.from_numpy(C)
    dD = ko.DeviceBuffer((m * n + guard) * 2)
    ko.set_tuning("gemm16.variant", variant)
    try:
        for use_c in (False, True):
            dD.upload(np.full(m * n + guard, 0x7b7b, np.uint16))
            ko.gemm16(m, n, k, dA, dB, dD, C=dC if use_c else None, alpha=0.5 if use_c else 1.0,
                      beta=-1.5 if use_c else 0.0, b_layout=layout, dtype=dt)
            ko.synchronize()
            out = dD.download(np.uint16, (m * n + guard,))
            assert np.all(out[m * n:] == 0x7b7b), "rows past M were written"
            if use_c:
                _, ref64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, C_bits=C, alpha=0.5, beta=-1.5, bf16=bf16)
                ap = 0.5 * ap + 1.5 * np.abs(_to_f64(C, bf16))
            else:
                _, ref64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, bf16=bf16)
            assert_gemm16_close(_to_f64(out[:m * n].reshape(m, n), bf16), ref64, ap, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.variant", 0)


@pytest.mark.parametrize("m,n,k", [(3000, 3072, 768), (6000, 1024, 1024), (1240, 2304, 3072), (16000, 3072, 768),
                                   (4093, 3072, 768), (8191, 1024, 1024), (5001, 2304, 776), (19500, 1024, 1032)])
def test_gemm16_ragged_rows_through_the_default_dispatch_are_exact(ko, m, n, k):
    """Row counts that are not multiples of the tile height (of 8 or not), on the shapes the dispatch sends to the pinned
    kernel as they are (256 x 256 tiles, and 128 x 256 tiles): small integers make every sum exact, so any row fetched
    from the wrong place or stored where it does not belong shows.  19500 x 1024: 308 tiles on 256 compute units - the
    52 below the full round are cut off and go to the ring kernel's 128 x 128 tiles."""
    rng = np.random.default_rng(m + k)
    A = rng.integers(-3, 4, (m, k)).astype(np.float16)
    B = rng.integers(-3, 4, (n, k)).astype(np.float16)
    bias = rng.integers(-8, 9, (n,)).astype(np.float16)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    assert np.abs(want).max() < 2048 - 8  # exactly representable in binary16
    got = ko.gemm16_host(A.view(np.uint16), B.view(np.uint16), m, n, k)
    np.testing.assert_array_equal(got.view(np.float16).astype(np.float64), want)
    got = ko.gemm16_host(A.view(np.uint16), B.view(np.uint16), m, n, k, bias_bits=bias.view(np.uint16))
    np.testing.assert_array_equal(got.view(np.float16).astype(np.float64), want + bias.astype(np.float64)[None, :])


# K split over the waves of a workgroup (few output tiles, column-major B): 70 = 64 x 64 tiles over 4 waves,
# 71 = 32 x 64 over 4, 72 = 32 x 32 over 8, 73 = 32 x 64 over 6
WAVE_K_VARIANTS = [70, 71, 72, 73]


@pytest.mark.parametrize("variant", WAVE_K_VARIANTS)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(1, 1, 8), (33, 36, 8), (64, 64, 64), (100, 200, 1032), (31, 67, 136), (130, 75, 4104),
                                   (256, 256, 2048), (65, 129, 72), (96, 128, 448), (8, 520, 1544), (70, 8, 264),
                                   (40, 328, 200)])
def test_gemm16_wave_k_variants_match_oracle(ko, variant, bf16, b_col_major, m, n, k):
    """Every wave of a workgroup multiplies its own K tiles (w, w + WAVES, ...) of the workgroup's one output tile and
    the partial tiles are added in wave order: against the oracle, plain and with the whole epilogue (beta C, bias,
    activation), bit-stable from call to call - ragged M and N, row lengths of D off 8 bytes, a K that ends inside
    a K tile, fewer K tiles than waves, more K tiles than one round of the waves' two stages.  B as [N][K], or as
    [K][N] when N is a multiple of 8 (rows of whole 16-byte chunks)."""
    if not b_col_major and n % 8:
        pytest.skip("a row-major B off 16-byte rows does not go to these kernels")
    A = _bits16((m, k), 91 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 93 + n, bf16)
    C = _bits16((m, n), 95, bf16)
    bias = _bits16((n,), 97, bf16)
    kw = dict(dtype=ko.BF16 if bf16 else ko.F16, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR)
    ko.set_tuning("gemm16.variant", variant)
    try:
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major)
        got = ko.gemm16_host(A, B, m, n, k, **kw)
        assert_gemm16_close(_to_f64(got, bf16), ref64, ap, k, bf16=bf16)
        np.testing.assert_array_equal(ko.gemm16_host(A, B, m, n, k, **kw), got)
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major, C_bits=C, beta=0.5, bias_bits=bias, act=2)
        got = ko.gemm16_host(A, B, m, n, k, C_bits=C, beta=0.5, bias_bits=bias, act=2, **kw)
        assert_gemm16_act_close(_to_f64(got, bf16), ref64, ap + 2.0, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.variant", 0)


@pytest.mark.parametrize("variant", WAVE_K_VARIANTS)
def test_gemm16_wave_k_variants_are_exact_on_small_integers(ko, variant):
    """Entries in -2 .. 2: every partial sum is an integer below 2^11, exact in fp32 and in binary16, so the result
    does not depend on the order of the sum - a K tile left out, taken twice or taken by the wrong wave shows as a
    wrong integer.  K off the K tile and off the waves' round, M and N off the tiles."""
    rng = np.random.default_rng(variant)
    ko.set_tuning("gemm16.variant", variant)
    try:
        for m, n, k in ((96, 200, 128), (70, 90, 456), (33, 64, 1992), (128, 32, 72), (257, 100, 328), (100, 328, 520)):
            Ai = rng.integers(-2, 3, (m, k)).astype(np.float16)
            Bi = rng.integers(-2, 3, (n, k)).astype(np.float16)  # [n][k]
            scale = 64.0 / k if k > 64 else 1.0  # keeps |sum| below 2^11: thin out the non-zeros of A
            Ai[rng.random((m, k)) > scale] = 0
            want = Ai.astype(np.float64) @ Bi.astype(np.float64).T
            got = ko.gemm16_host(Ai.view(np.uint16), Bi.view(np.uint16), m, n, k).view(np.float16)
            np.testing.assert_array_equal(got.astype(np.float64), want, err_msg="%dx%dx%d" % (m, n, k))
            if n % 8 == 0:  # the same product with B handed over as [K][N]
                got = ko.gemm16_host(Ai.view(np.uint16), np.ascontiguousarray(Bi.T).view(np.uint16), m, n, k,
                                     b_layout=ko.ROW_MAJOR).view(np.float16)
                np.testing.assert_array_equal(got.astype(np.float64), want, err_msg="%dx%dx%d, B row-major" % (m, n, k))
    finally:
        ko.set_tuning("gemm16.variant", 0)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("m,n,k,tile", [(100, 1024, 1024, 32032), (512, 768, 3072, 32064), (1000, 1024, 4096, 64064),
                                        (8, 4096, 4096, 32032), (200, 2304, 768, 32064), (750, 1000, 1032, 64064),
                                        (2040, 704, 2056, 64128), (500, 4000, 1032, 128064), (3000, 1000, 520, 128128),
                                        (8, 16448, 1032, 1032064), (30, 17000, 520, 1032064)])
@pytest.mark.parametrize("b_col_major", [True, False])
def test_gemm16_small_problems_through_the_default_dispatch(ko, m, n, k, tile, bf16, b_col_major):
    """A few hundred to a few thousand rows against a weight matrix: the dispatch sends them to the kernel that
    splits K over the waves of a workgroup or to the one with the deep ring of LDS stages - the plan query says which
    tile - and the whole output agrees with the oracle, plain and with bias + GELU; with those kernels switched off
    (gemm16.wave_k = 1) the older paths give the same result to the same bound."""
    layout = ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR
    if not b_col_major and tile == 64128:
        tile = 128064  # with B as [K][N] the half tile is 128 x 64 whatever the shape
    assert ko.gemm_plan(m, n, k, sixteen_bit=True, b_layout=layout) == (1, 0, tile)
    A = _bits16((m, k), 101 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 103 + n, bf16)
    bias = _bits16((n,), 105, bf16)
    kw = dict(dtype=ko.BF16 if bf16 else ko.F16, b_layout=layout)
    _, ref64, ap = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major)
    _, ref64b, apb = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major, bias_bits=bias, act=1)
    try:
        for off in (0, 1):
            ko.set_tuning("gemm16.wave_k", off)
            got = ko.gemm16_host(A, B, m, n, k, **kw)
            assert_gemm16_close(_to_f64(got, bf16), ref64, ap, k, bf16=bf16)
            got = ko.gemm16_host(A, B, m, n, k, bias_bits=bias, act=1, **kw)
            assert_gemm16_act_close(_to_f64(got, bf16), ref64b, apb + 2.0, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.wave_k", 0)


# a deep ring of LDS stages: 80 = 128 x 128 tiles (4 waves, 4 stages), 81 = 128 x 64, 82 = 64 x 128 (6 stages),
# 83 = 128 x 128 with 8 waves and 5 stages, 84 = 32 x 64 (2 waves, 6 stages: what a problem of at most 32 rows and
# many columns takes)
RING_VARIANTS = [80, 81, 82, 83, 84]


@pytest.mark.parametrize("variant", RING_VARIANTS)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k", [(1, 1, 8), (33, 36, 8), (128, 128, 64), (300, 520, 72), (256, 384, 1032), (130, 75, 4104),
                                   (640, 256, 448), (257, 129, 264), (1000, 256, 328), (96, 1000, 200), (70, 8, 264)])
def test_gemm16_ring_variants_match_oracle(ko, variant, bf16, b_col_major, m, n, k):
    """The waves of a workgroup walk K together through four to six LDS stages, loads three to five K tiles ahead:
    against the oracle, plain and with the whole epilogue, bit-stable from call to call - fewer K tiles than stages,
    a number of K tiles that is no multiple of the stages, a K that ends inside a K tile, ragged M (the coalesced
    epilogue with the rows past M left out) and ragged N (the element-wise one).  B as [N][K], or as [K][N] when N
    is a multiple of 8."""
    if not b_col_major and n % 8:
        pytest.skip("a row-major B off 16-byte rows does not go to these kernels")
    A = _bits16((m, k), 111 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 113 + n, bf16)
    C = _bits16((m, n), 115, bf16)
    bias = _bits16((n,), 117, bf16)
    kw = dict(dtype=ko.BF16 if bf16 else ko.F16, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR)
    ko.set_tuning("gemm16.variant", variant)
    try:
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major)
        got = ko.gemm16_host(A, B, m, n, k, **kw)
        assert_gemm16_close(_to_f64(got, bf16), ref64, ap, k, bf16=bf16)
        np.testing.assert_array_equal(ko.gemm16_host(A, B, m, n, k, **kw), got)
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major, C_bits=C, beta=0.5, bias_bits=bias, act=2)
        got = ko.gemm16_host(A, B, m, n, k, C_bits=C, beta=0.5, bias_bits=bias, act=2, **kw)
        assert_gemm16_act_close(_to_f64(got, bf16), ref64, ap + 2.0, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.variant", 0)


@pytest.mark.parametrize("variant", RING_VARIANTS)
def test_gemm16_ring_variants_are_exact_on_small_integers(ko, variant):
    """Entries in -2 .. 2, sums below 2^11: a K tile left out, taken twice or read before it landed shows as a wrong
    integer.  Also: a guard area behind D stays untouched by the rows past M that the last row of tiles computes."""
    rng = np.random.default_rng(variant)
    ko.set_tuning("gemm16.variant", variant)
    try:
        for m, n, k in ((128, 256, 128), (200, 128, 456), (129, 64, 1992), (384, 384, 72), (1000, 128, 328), (260, 520, 1024)):
            Ai = rng.integers(-2, 3, (m, k)).astype(np.float16)
            Bi = rng.integers(-2, 3, (n, k)).astype(np.float16)  # [n][k]
            Ai[rng.random((m, k)) > (64.0 / k if k > 64 else 1.0)] = 0
            want = Ai.astype(np.float64) @ Bi.astype(np.float64).T
            dA, dB = ko.DeviceBuffer.from_numpy(Ai.view(np.uint16)), ko.DeviceBuffer.from_numpy(Bi.view(np.uint16))
            guard = 4096
            dD = ko.DeviceBuffer.from_numpy(np.full(m * n + guard, 0x7bff, np.uint16))
            ko.gemm16(m, n, k, dA, dB, dD)
            ko.synchronize()
            out = dD.download(np.uint16, (m * n + guard,))
            np.testing.assert_array_equal(out[:m * n].view(np.float16).astype(np.float64).reshape(m, n), want,
                                          err_msg="%dx%dx%d" % (m, n, k))
            assert (out[m * n:] == 0x7bff).all(), "%dx%dx%d: the guard area behind D was written" % (m, n, k)
            if n % 8 == 0:  # the same product with B handed over as [K][N]
                got = ko.gemm16_host(Ai.view(np.uint16), np.ascontiguousarray(Bi.T).view(np.uint16), m, n, k,
                                     b_layout=ko.ROW_MAJOR).view(np.float16)
                np.testing.assert_array_equal(got.astype(np.float64), want, err_msg="%dx%dx%d, B row-major" % (m, n, k))
    finally:
        ko.set_tuning("gemm16.variant", 0)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("b_col_major", [True, False])
@pytest.mark.parametrize("m,n,k,slices", [(256, 256, 256, 2), (300, 512, 648, 2), (1, 256, 1032, 3), (513, 768, 2056, 5),
                                           (1000, 256, 904, 7), (256, 1024, 8, 2)])
def test_gemm16_pinned_kernel_in_k_slices_matches_oracle(ko, bf16, b_col_major, m, n, k, slices):
    """The 256 x 256 tiles of the pinned kernel as pairs (K slice, output tile), fp32 partial products summed by the
    second kernel: against the oracle, plain and with the whole epilogue, bit-stable from call to call - any row count
    (the last row of tiles fetches rows that exist), a K that ends inside the last slice (padded with zeros), slices
    that come out fewer than asked for, more pairs than one per XCD and fewer."""
    A = _bits16((m, k), 211 + m, bf16)
    B = _bits16((n, k) if b_col_major else (k, n), 213 + n, bf16)
    C = _bits16((m, n), 215, bf16)
    bias = _bits16((n,), 217, bf16)
    kw = dict(dtype=ko.BF16 if bf16 else ko.F16, b_layout=ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR)
    ko.set_tuning("gemm16.variant", 62)
    ko.set_tuning("gemm16.k_slices", slices)
    try:
        planned, depth, tile = ko.gemm_plan(m, n, k, sixteen_bit=True, b_layout=kw["b_layout"])
        if k >= 256:
            assert tile == 256 and 2 <= planned <= slices and depth % 128 == 0 and (planned - 1) * depth < k <= planned * depth
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major)
        if k < 256:  # one slice at most: the call says so
            with pytest.raises(ko.KoError):
                ko.gemm16_host(A, B, m, n, k, **kw)
            return
        got = ko.gemm16_host(A, B, m, n, k, **kw)
        assert_gemm16_close(_to_f64(got, bf16), ref64, ap, k, bf16=bf16)
        np.testing.assert_array_equal(ko.gemm16_host(A, B, m, n, k, **kw), got)
        _, ref64, ap = oracle.gemm16(A, B, m, n, k, bf16=bf16, b_col_major=b_col_major, C_bits=C, beta=0.5, bias_bits=bias, act=2)
        got = ko.gemm16_host(A, B, m, n, k, C_bits=C, beta=0.5, bias_bits=bias, act=2, **kw)
        assert_gemm16_act_close(_to_f64(got, bf16), ref64, ap + 2.0, k, bf16=bf16)
    finally:
        ko.set_tuning("gemm16.variant", 0)
        ko.set_tuning("gemm16.k_slices", 0)


def test_gemm16_pinned_kernel_in_k_slices_is_exact_on_small_integers(ko):
    """Entries in -2 .. 2, sums below 2^11: a K tile left out, taken twice, read before it landed or added to the wrong
    slice shows as a wrong integer; a guard area behind D stays as it was.  Pair counts that divide over the 8 XCDs
    (blocked tile order) and that do not, two rounds of pairs per workgroup (257 x 4096 in 15 slices: 480 pairs), both
    layouts of B."""
    rng = np.random.default_rng(62)
    ko.set_tuning("gemm16.variant", 62)
    try:
        for m, n, k, slices in ((512, 1024, 1024, 4), (700, 768, 2432, 7), (2048, 2048, 512, 2), (257, 4096, 1920, 15), (256, 256, 32768, 16),
                                (1500, 3072, 768, 3)):
            ko.set_tuning("gemm16.k_slices", slices)
            Ai = rng.integers(-2, 3, (m, k)).astype(np.float16)
            Bi = rng.integers(-2, 3, (n, k)).astype(np.float16)  # [n][k]
            Ai[rng.random((m, k)) > 64.0 / k] = 0
            want = Ai.astype(np.float64) @ Bi.astype(np.float64).T
            dA, dB = ko.DeviceBuffer.from_numpy(Ai.view(np.uint16)), ko.DeviceBuffer.from_numpy(Bi.view(np.uint16))
            guard = 4096
            dD = ko.DeviceBuffer.from_numpy(np.full(m * n + guard, 0x7bff, np.uint16))
            ko.gemm16(m, n, k, dA, dB, dD)
            ko.synchronize()
            out = dD.download(np.uint16, (m * n + guard,))
            np.testing.assert_array_equal(out[:m * n].view(np.float16).astype(np.float64).reshape(m, n), want,
                                          err_msg="%dx%dx%d in %d slices" % (m, n, k, slices))
            assert (out[m * n:] == 0x7bff).all(), "%dx%dx%d: the guard area behind D was written" % (m, n, k)
            got = ko.gemm16_host(Ai.view(np.uint16), np.ascontiguousarray(Bi.T).view(np.uint16), m, n, k,
                                 b_layout=ko.ROW_MAJOR).view(np.float16)
            np.testing.assert_array_equal(got.astype(np.float64), want, err_msg="%dx%dx%d, B row-major" % (m, n, k))
    finally:
        ko.set_tuning("gemm16.variant", 0)
        ko.set_tuning("gemm16.k_slices", 0)


@pytest.mark.parametrize("m,n,k,b_col_major", [(1000, 1280, 8200, True), (1100, 1024, 8456, False), (520, 2304, 9216, True)])
def test_gemm16_deep_k_on_mid_size_outputs_goes_out_as_pinned_slices(ko, m, n, k, b_col_major):
    """What the default dispatch does with more 128 x 128 tiles than a quarter of the compute units, at most half of them of
    256 x 256 tiles and K beyond 8192: sampled rows (every column) against the oracle, and bit-stable."""
    layout = ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR
    planned, depth, tile = ko.gemm_plan(m, n, k, sixteen_bit=True, b_layout=layout)
    assert tile == 256 and planned >= 2 and depth >= 2048 and depth % 128 == 0
    A = _bits16((m, k), 311, False)
    B = _bits16((n, k) if b_col_major else (k, n), 313, False)
    got = ko.gemm16_host(A, B, m, n, k, b_layout=layout)
    rows = np.unique(np.concatenate([np.arange(0, m, 41), [255, 256, m - 1]]))
    _, ref64, ap = oracle.gemm16(A[rows], B, len(rows), n, k, b_col_major=b_col_major)
    assert_gemm16_close(_to_f64(got[rows], False), ref64, ap, k)
    np.testing.assert_array_equal(ko.gemm16_host(A, B, m, n, k, b_layout=layout), got)


@pytest.mark.parametrize("m,n,k,b_col_major,tile", [(40, 33000, 520, True, 64128), (100, 32776, 2056, True, 128128),
                                                    (60, 32776, 2056, False, 128128)])
def test_gemm16_one_row_of_tiles_against_many_columns(ko, m, n, k, b_col_major, tile):
    """64 or 128 rows against more columns than compute units have 128-wide tiles for: the ring kernel in several
    rounds.  The whole output against the oracle, plain and with bias + GELU, bit-stable."""
    layout = ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR
    assert ko.gemm_plan(m, n, k, sixteen_bit=True, b_layout=layout) == (1, 0, tile)
    A = _bits16((m, k), 401 + m, False)
    B = _bits16((n, k) if b_col_major else (k, n), 403, False)
    bias = _bits16((n,), 405, False)
    _, ref64, ap = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major)
    got = ko.gemm16_host(A, B, m, n, k, b_layout=layout)
    assert_gemm16_close(_to_f64(got, False), ref64, ap, k)
    np.testing.assert_array_equal(ko.gemm16_host(A, B, m, n, k, b_layout=layout), got)
    _, ref64b, apb = oracle.gemm16(A, B, m, n, k, b_col_major=b_col_major, bias_bits=bias, act=1)
    got = ko.gemm16_host(A, B, m, n, k, bias_bits=bias, act=1, b_layout=layout)
    assert_gemm16_act_close(_to_f64(got, False), ref64b, apb + 2.0, k)


@pytest.mark.parametrize("m,n,k,b_col_major,tile", [(657, 7834, 520, True, 0), (640, 7840, 776, False, 0),
                                                    (311, 7983, 8200, True, 128128), (300, 7984, 8456, False, 128128)])
def test_gemm16_ring_kernel_beyond_one_round_and_beyond_k_8192(ko, m, n, k, b_col_major, tile):
    """Up to one and a half rounds of 128 x 128 tiles on a shape that is not whole 256 x 256 tiles (the plan query says 0:
    the choice falls in the later rules of the dispatch), and more than half a round of them at a K beyond 8192:
    sampled rows (every column) against the oracle, and bit-stable."""
    layout = ko.COL_MAJOR if b_col_major else ko.ROW_MAJOR
    assert ko.gemm_plan(m, n, k, sixteen_bit=True, b_layout=layout) == (1, 0, tile)
    A = _bits16((m, k), 501, False)
    B = _bits16((n, k) if b_col_major else (k, n), 503, False)
    got = ko.gemm16_host(A, B, m, n, k, b_layout=layout)
    rows = np.unique(np.concatenate([np.arange(0, m, 29), [127, 128, m - 1]]))
    _, ref64, ap = oracle.gemm16(A[rows], B, len(rows), n, k, b_col_major=b_col_major)
    assert_gemm16_close(_to_f64(got[rows], False), ref64, ap, k)
    np.testing.assert_array_equal(ko.gemm16_host(A, B, m, n, k, b_layout=layout), got)
