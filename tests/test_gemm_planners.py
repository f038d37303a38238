"""The GEMMs' host-side K-slice planners, asked without a GPU.

A plan is arithmetic on the shape and the number of compute units (256 when no device is visible, which is also what
gfx950 has), so its invariants can be checked on the CPU: every slice but the last is a whole number of K tiles, the
slices cover K exactly once, the fp32 partial products fit the workspace (32 MiB of it for the SGEMM, 64 for the 16-bit GEMM), and shapes that fill the chip whole
are left whole.
"""
import itertools

import pytest

import kernel_optimization_amd as ko

WORKSPACE = 32 << 20      # what the SGEMM uses of a stream's workspace
WORKSPACE16 = 64 << 20    # the whole of it
SIZES = [8, 31, 32, 64, 100, 107, 128, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096]
DEPTHS = [64, 512, 767, 768, 1300, 1535, 1536, 2047, 2048, 4096, 8192, 16384, 65536, 262144]


def _check(m, n, k, plan, k_tile, min_k, row_pad=1, workspace=WORKSPACE):
    slices, k_slice, _ = plan
    assert slices >= 1
    if slices == 1:
        return
    assert k >= min_k, (m, n, k, plan)
    assert k_slice > 0 and k_slice % k_tile == 0, (m, n, k, plan)
    assert (slices - 1) * k_slice < k <= slices * k_slice, (m, n, k, plan)   # no empty slice, none missing
    assert slices * m * (-(-n // row_pad) * row_pad) * 4 <= workspace, (m, n, k, plan)


@pytest.mark.parametrize("m,n", list(itertools.product(SIZES, SIZES)))
def test_sgemm_plans_cover_k_once_and_fit_the_workspace(m, n):
    for k in DEPTHS:
        plan = ko.gemm_plan(m, n, k)
        _check(m, n, k, plan, k_tile=128, min_k=768)
        if plan[0] > 1 and plan[2]:
            assert plan[2] in (33, 35, 36, 40), plan       # the direct-to-LDS tilings
            assert plan[2] != 40 or (n % 4 == 0 and k % 4 == 0), plan   # not with four-byte operand loads


@pytest.mark.parametrize("b_layout", [ko.COL_MAJOR, ko.ROW_MAJOR])
@pytest.mark.parametrize("m,n", list(itertools.product(SIZES, SIZES)))
def test_gemm16_plans_cover_k_once_and_fit_the_workspace(m, n, b_layout):
    for k in DEPTHS:
        plan = ko.gemm_plan(m, n, k, sixteen_bit=True, b_layout=b_layout)
        _check(m, n, k, plan, k_tile=64, min_k=1536, row_pad=4, workspace=WORKSPACE16)   # rows of partial products: whole groups of 4
        if plan[0] > 1:
            assert plan[2] in (256, 128, 64, 32)
            if plan[2] == 32:
                assert m <= 32
            if plan[2] == 256:   # the pinned kernel: whole tile columns, K tiles in pairs, at most one pair per compute unit
                assert n % 256 == 0 and k > 8192 and plan[1] % 128 == 0 and plan[1] >= 2048
                assert plan[0] * -(-m // 256) * (n // 256) <= 256 < 4 * -(-m // 128) * -(-n // 128)
            continue
        # one launch: whole, or K split over the waves of workgroups that own one small output tile each - B
        # column-major, or row-major with rows of whole 16-byte chunks; a multiple of 8 deep (as every K the operator
        # takes); at most one such tile per compute unit, and the smallest tile for which that holds
        assert plan[1] == 0 and plan[2] in (0, 32032, 32064, 64064, 64128, 128064, 128128, 1032064)
        if plan[2] == 1032064:   # at most 32 rows against more columns than 64-wide tiles for every compute unit
            assert m <= 32 and -(-n // 64) > 256 and k >= 512 and k % 8 == 0 and (b_layout == ko.COL_MAJOR or n % 8 == 0)
        elif plan[2]:
            tm, tn = divmod(plan[2], 1000)
            # at most one such tile per compute unit - or one row of ring tiles, however many
            assert (-(-m // tm) * -(-n // tn) <= 256 or (m <= tm and plan[2] in (64128, 128128))) and k % 8 == 0
            if plan[2] in (32032, 32064, 64064):   # K over the waves of a workgroup
                assert (b_layout == ko.COL_MAJOR or n % 8 == 0) and 128 <= k <= 8192
                assert plan[2] == 32032 or -(-m // 32) * -(-n // 32) > 256
            else:                                   # a deep ring of LDS stages: when the small tiles are too many
                assert (b_layout == ko.COL_MAJOR or (n % 8 == 0 and plan[2] != 64128)) and 512 <= k <= 16384
                if k > 8192:   # only where two slices do not fit a round and the pinned kernel's slices do not apply
                    assert plan[2] == 128128 and n % 256 != 0 and 2 * -(-m // 128) * -(-n // 128) > 256
                assert -(-m // 64) * -(-n // 64) > 256
                if -(-m // tm) * -(-n // tn) > 256:
                    assert (plan[2] == 64128 and b_layout == ko.COL_MAJOR) or (plan[2] == 128128 and k >= 2048)


def test_measured_decisions_stay_put():
    """Shapes whose plans were chosen from timings: a change of the planner that moves them should be deliberate."""
    assert ko.gemm_plan(256, 256, 2048)[:2] == (8, 256)
    assert ko.gemm_plan(768, 768, 16384)[0] == 7
    assert ko.gemm_plan(1024, 1024, 8192)[0] == 1
    assert ko.gemm_plan(4096, 4096, 4096)[0] == 1
    assert ko.gemm_plan(256, 256, 512)[0] == 1
    assert ko.gemm_plan(768, 768, 16384, sixteen_bit=True) == (5, 3328, 128)
    assert ko.gemm_plan(256, 1024, 16384, sixteen_bit=True) == (8, 2048, 128)
    assert ko.gemm_plan(256, 256, 16384, sixteen_bit=True) == (16, 1024, 64)
    # beyond a quarter of a chip's worth of 128 x 128 tiles and K = 8192: the pinned kernel's tiles in slices
    assert ko.gemm_plan(768, 3072, 16384, sixteen_bit=True) == (7, 2432, 256)
    assert ko.gemm_plan(2048, 4096, 16384, sixteen_bit=True) == (2, 8192, 256)
    assert ko.gemm_plan(2048, 4096, 16384, sixteen_bit=True, b_layout=ko.ROW_MAJOR) == (2, 8192, 256)
    assert ko.gemm_plan(2048, 4096, 8192, sixteen_bit=True)[0] == 1
    assert ko.gemm_plan(1000, 1000, 16384, sixteen_bit=True)[2] == 128    # not whole tile columns
    assert ko.gemm_plan(512, 520, 16384, sixteen_bit=True, b_layout=ko.ROW_MAJOR)[0] > 1
    # few tiles, column-major B, K up to 8192: one launch that splits K over the waves of a workgroup
    assert ko.gemm_plan(512, 512, 8192, sixteen_bit=True) == (1, 0, 32032)
    assert ko.gemm_plan(100, 1024, 1024, sixteen_bit=True) == (1, 0, 32032)
    assert ko.gemm_plan(512, 1024, 4096, sixteen_bit=True) == (1, 0, 32064)
    assert ko.gemm_plan(1000, 1024, 4096, sixteen_bit=True) == (1, 0, 64064)
    # ... up to a K where K slices of the ring kernel's 128 x 128 tiles are faster: at most three quarters of the compute
    # units' worth of workgroups, slices a quarter of K deep or more
    assert ko.gemm_plan(768, 768, 8192, sixteen_bit=True) == (4, 2048, 128)
    assert ko.gemm_plan(1856, 320, 6144, sixteen_bit=True) == (4, 1536, 128)
    assert ko.gemm_plan(1868, 303, 5720, sixteen_bit=True)[0] == 4       # 150 tiles of 64 x 64: sliced from K = 5120 on
    assert ko.gemm_plan(1024, 1024, 5720, sixteen_bit=True) == (1, 0, 64064)   # 256 of them: from 6144 on
    assert ko.gemm_plan(2048, 256, 8192, sixteen_bit=True) == (4, 2048, 128)
    assert ko.gemm_plan(1412, 440, 8952, sixteen_bit=True) == (4, 2240, 128)
    assert ko.gemm_plan(1024, 512, 32768, sixteen_bit=True) == (8, 4096, 128)
    # too many small tiles for that, at most one tile of 128 x 128 (or half of one) per compute unit: the ring kernel
    assert ko.gemm_plan(2048, 768, 3072, sixteen_bit=True) == (1, 0, 64128)
    assert ko.gemm_plan(512, 4096, 4096, sixteen_bit=True) == (1, 0, 128064)
    assert ko.gemm_plan(4096, 1024, 4096, sixteen_bit=True) == (1, 0, 128128)
    assert ko.gemm_plan(6000, 768, 3072, sixteen_bit=True) == (1, 0, 0)
    assert ko.gemm_plan(1000, 1024, 768, sixteen_bit=True) == (1, 0, 0)       # 64 x 64 tiles only from K = 1024 on
    assert ko.gemm_plan(512, 3072, 768, sixteen_bit=True) == (1, 0, 128064)   # more 64 x 64 tiles than compute units
    assert ko.gemm_plan(100, 1024, 1024, sixteen_bit=True, b_layout=ko.ROW_MAJOR) == (1, 0, 32032)
    assert ko.gemm_plan(100, 1028, 1024, sixteen_bit=True, b_layout=ko.ROW_MAJOR) == (1, 0, 0)  # rows of B off 16 bytes
    assert ko.gemm_plan(2048, 2048, 2048, sixteen_bit=True)[0] == 1
    assert ko.gemm_plan(16384, 3072, 768, sixteen_bit=True)[0] == 1
    # a decoding step against a vocabulary: 32 x 64 tiles of the ring kernel, however many rounds
    assert ko.gemm_plan(8, 128256, 4096, sixteen_bit=True) == (1, 0, 1032064)
    assert ko.gemm_plan(32, 32000, 4096, sixteen_bit=True, b_layout=ko.ROW_MAJOR) == (1, 0, 1032064)
    assert ko.gemm_plan(8, 8192, 8192, sixteen_bit=True) == (1, 0, 32032)
    assert ko.gemm_plan(33, 32000, 4096, sixteen_bit=True)[2] != 1032064
    assert ko.gemm_plan(64, 128256, 4096, sixteen_bit=True) == (1, 0, 64128)
    assert ko.gemm_plan(64, 128256, 4096, sixteen_bit=True, b_layout=ko.ROW_MAJOR) == (1, 0, 128128)
    assert ko.gemm_plan(128, 128256, 4096, sixteen_bit=True) == (1, 0, 128128)
    assert ko.gemm_plan(128, 50304, 1024, sixteen_bit=True)[2] == 0
    assert ko.gemm_plan(256, 128256, 4096, sixteen_bit=True)[2] == 0
    # operand rows off 16-byte boundaries are sliced like the others
    assert ko.gemm_plan(282, 31, 13104)[0] > 1
    assert ko.gemm_plan(282, 31, 13104, sixteen_bit=True)[0] > 1


def test_bad_arguments_are_refused():
    with pytest.raises(ko.KoError):
        ko.gemm_plan(0, 16, 16)
    with pytest.raises(ko.KoError):
        ko.gemm_plan(16, 16, -1, sixteen_bit=True)
    with pytest.raises(ko.KoError):
        ko.gemm_plan(1 << 31, 16, 16)
