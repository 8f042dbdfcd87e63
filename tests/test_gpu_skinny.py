"""GPU parity of the skinny kernel (gemm_skinny.hip): a C of 4 ... 32 columns under many rows, or of 4 ... 32 rows over
many columns -- what the reference sends to its 4-column kernels (MM/matMul_sernel.cuh:17-30, dispatched at
MM/matMul.cuh:100-102) and to k18 / k14 / k12 (MM/matMul.cuh:104-106).  Wavefronts stream the long operand from
memory into 4 x 4 x 1 or 16 x 16 x 4 MFMA blocks; integer inputs pin the indexing bit for bit: lines per wavefront, the classes
of k, the K tail, K shared between the wavefronts of a workgroup, both orientations of C."""
import numpy as np
import pytest

from helpers import NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, gpu_matmul_2d, logical_operands, oracle_2d

pytestmark = pytest.mark.gpu

SKINNY = 27


@pytest.fixture(autouse=True)
def _auto_tile(gpu):
    yield
    gpu.force_tile(-1)
    gpu.skinny_form(-1)


def check(gpu, variant, N, M, K, seed, fill=-77.0):
    rng = np.random.default_rng(seed)
    A, B = logical_operands(variant, rng, N, M, K, "int")
    C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=fill)
    R = oracle_2d(variant, A, B)
    what = "%s %d x %d x %d" % (VARIANT_NAMES[variant], N, M, K)
    if not np.array_equal(C, R):
        bad = np.argwhere(C != R)
        raise AssertionError("%s: %d wrong outputs, first at %s (got %s, want %s); rows %s cols %s" % (
            what, len(bad), bad[0], C[tuple(bad[0])], R[tuple(bad[0])], sorted(set(bad[:, 0]))[:12],
            sorted(set(bad[:, 1]))[:12]))
    assert np.count_nonzero(Cp[N:]) == 0 and np.count_nonzero(Cp[:, M:]) == 0, what + ": pads must come out zero"


def test_the_automatic_choice_names_the_kernel(gpu):
    cu = 256
    for (rows, cols) in ((65536, 4), (8192, 8), (256, 4), (4, 65536), (8, 256), (4, 1000)):
        for variant in (NN, T1, T2):
            assert gpu.choose_tile(variant, rows, cols, 1, 1024, cu) == SKINNY
    # 12 or 16 short lines: from 16 lines of the long operand per compute unit on, in every layout
    for variant in (NN, T1, T2):
        for (rows, cols) in ((65536, 16), (4096, 12), (16, 65536), (12, 4096)):
            assert gpu.choose_tile(variant, rows, cols, 1, 1024, cu) == SKINNY
        for (rows, cols) in ((4092, 16), (16, 4000), (256, 12)):
            assert gpu.choose_tile(variant, rows, cols, 1, 1024, cu) != SKINNY
        # 20 ... 32: from 32 lines per compute unit on
        for (rows, cols) in ((8192, 32), (65536, 20), (24, 8192), (28, 100000)):
            assert gpu.choose_tile(variant, rows, cols, 1, 1024, cu) == SKINNY
        for (rows, cols) in ((8188, 32), (32, 4096), (65536, 36), (40, 65536)):
            assert gpu.choose_tile(variant, rows, cols, 1, 1024, cu) != SKINNY
        assert gpu.choose_tile(variant, 2048, 32, 1, 2048, cu) == SKINNY and gpu.choose_tile(variant, 2044, 32, 1, 2048, cu) != SKINNY
        assert gpu.choose_tile(variant, 16, 2048, 1, 4096, cu) == SKINNY and gpu.choose_tile(variant, 16, 2048, 1, 2044, cu) != SKINNY
        assert gpu.choose_tile(variant, 65536, 32, 1, 252, cu) != SKINNY and gpu.choose_tile(variant, 65536, 16, 1, 252, cu) == SKINNY
    # not skinny enough, too short, or a batch / K slices
    for (rows, cols, nz) in ((65536, 36, 1), (252, 4, 1), (4, 252, 1), (8, 8, 1), (16, 252, 1), (65536, 4, 2), (4, 65536, 3)):
        for variant in (NN, T1, T2):
            assert gpu.choose_tile(variant, rows, cols, nz, 1024, cu) != SKINNY


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("form", [-1, 0, 1, 2, 3, 4, 5, 6, 7, 103, 108, 8, 9, 10, 11, 203, 208])
@pytest.mark.parametrize("thin", [1, 2, 3, 4, 5, 7, 8, 9, 12, 13, 16])
def test_thin_columns_bitwise(gpu, variant, thin, form):
    """C of 1 ... 16 columns (stored 4, 8, 12 or 16) under row counts around the 16, 64 and 256 lines a wavefront takes,
    in every form of the kernel: a wavefront per run of lines, K shared between 4 or 16 wavefronts, one or four
    lines per lane."""
    gpu.skinny_form(form)
    if form >= 0:
        gpu.force_tile(SKINNY)      # (a forced form also runs shapes the automatic choice leaves to the tile kernels)
    for (N, K) in ((256, 64), (1000, 1028), (4099, 36), (40000, 100), (20000, 260)):
        check(gpu, variant, N, thin, K, 100 * thin + N + K + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("form", [-1, 0, 1, 2, 3, 4, 5, 6, 7, 103, 108, 8, 9, 10, 11, 203, 208])
@pytest.mark.parametrize("thin", [1, 3, 4, 6, 8, 10, 12, 15, 16])
def test_thin_rows_bitwise(gpu, variant, thin, form):
    gpu.skinny_form(form)
    if form >= 0:
        gpu.force_tile(SKINNY)
    for (M, K) in ((256, 64), (1001, 1028), (4100, 36), (40001, 100), (20000, 260)):
        check(gpu, variant, thin, M, K, 200 * thin + M + K + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("K", [1, 3, 4, 5, 8, 12, 15, 16, 17, 28, 31, 32, 33, 60, 64, 68, 127, 128, 129, 252, 255, 256, 257, 300, 511, 513, 1000])
def test_every_kind_of_k_tail_bitwise(gpu, variant, K):
    """K around the k rows / 32-k panels of a register buffer, the 4-k chunks of a lane, the shares of a K split
    between 4 or 16 wavefronts; in every form."""
    gpu.force_tile(SKINNY)
    for form in (0, 1, 2, 3, 4, 5, 6, 7, 102, 105, 108, 8, 9, 10, 11, 202, 207, 216):
        gpu.skinny_form(form)
        check(gpu, variant, 700, 4, K, 3000 + K + variant)
        check(gpu, variant, 8, 900, K, 4000 + K + variant)
        check(gpu, variant, 530, 16, K, 3500 + K + variant)
        check(gpu, variant, 12, 300, K, 4500 + K + variant)
    gpu.skinny_form(-1)
    gpu.force_tile(-1)
    if K <= 64:
        check(gpu, variant, 70000, 7, K, 5000 + K + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("form", [-1, 8, 9, 10, 11, 204])
@pytest.mark.parametrize("thin", [17, 20, 23, 24, 28, 29, 32])
def test_up_to_32_short_lines_bitwise(gpu, variant, thin, form):
    """Two groups of 16 short lines through the 16 x 16 x 4 blocks, both orientations of C."""
    gpu.force_tile(SKINNY)
    gpu.skinny_form(form)
    for (L, K) in ((256, 64), (1003, 1028), (4099, 36), (20000, 260)):
        check(gpu, variant, L, thin, K, 300 * thin + L + K + variant)
        check(gpu, variant, thin, L + 1, K, 301 * thin + L + K + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("form", [1003, 1004, 1008, 1009, 1999, 2999])
def test_non_temporal_reads_bitwise(gpu, variant, form):
    """The long forms with the long operand read non-temporally (what the automatic choice does from 320 MiB on), forced
    on small shapes."""
    gpu.force_tile(SKINNY)
    gpu.skinny_form(form)
    for thin in (4, 7, 8, 13, 16, 24, 32):
        if thin > 16 and form in (1003, 1004):
            continue
        check(gpu, variant, 5003, thin, 1028, 400 * thin + form + variant)
        check(gpu, variant, thin, 40001, 100, 401 * thin + form + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_long_shapes_against_both_oracles(gpu, variant):
    """Uniform inputs at the benchmark's shapes, scaled down 4 x along the long side, within the FP32 tolerance
    (relative Frobenius error <= 1e-5, elements within 1e-4 * sqrt(K) * max|A| * max|B|); and the same launch
    twice gives the same bits."""
    for (N, M, K) in ((16384, 4, 1024), (2048, 8, 4096), (4, 16384, 1024), (8, 2048, 4096), (16384, 16, 1024), (12, 16384, 1024)):
        rng = np.random.default_rng(N + M + K + variant)
        A, B = logical_operands(variant, rng, N, M, K)
        C, _ = gpu_matmul_2d(gpu, variant, A, B)
        C2, _ = gpu_matmul_2d(gpu, variant, A, B)
        R = oracle_2d(variant, A, B)
        assert_within_tolerance(C, R, K, A, B, "%s %d x %d x %d" % (VARIANT_NAMES[variant], N, M, K))
        assert np.array_equal(C, C2)


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_few_lines_under_a_long_k_cut_across_workgroups(gpu, variant):
    """Fewer runs of lines than compute units: the automatic choice cuts K across workgroups, which meet through
    the stream's workspace and its arrival counters.  Bitwise on integers, the same bits launch after launch
    (the counters are back at zero each time), and a balanced-kernel launch on the same stream in between."""
    for (N, M, K) in ((8, 4096, 4096), (4, 2048, 8192), (2048, 4, 16384), (1000, 8, 3000), (8, 1000, 5000)):
        check(gpu, variant, N, M, K, 600 + N + M + K + variant)
    gpu.force_tile(SKINNY)
    for (N, M, K) in ((16, 4096, 2048), (1000, 12, 3000)):
        check(gpu, variant, N, M, K, 700 + N + M + K + variant)
    gpu.force_tile(-1)
    # 12 ... 32 short lines beside 4096 ... 8191 lines under a K of 2048 or more: the 16 x 16 x 4 blocks' 32-line runs, cut
    for (N, M, K) in ((16, 4100, 2052), (5000, 12, 4096), (8188, 32, 2048), (24, 8000, 2500), (2048, 16, 4100), (8, 3000, 2048), (28, 2100, 3000),
                      (8, 1024, 8192), (4, 512, 16384), (1000, 8, 4100), (260, 4, 9000), (8, 256, 20000), (16, 1024, 8192), (300, 12, 9000)):
        check(gpu, variant, N, M, K, 800 + N + M + K + variant)
    rng = np.random.default_rng(31 + variant)
    A, B = logical_operands(variant, rng, 8, 4096, 4096)
    first, _ = gpu_matmul_2d(gpu, variant, A, B)
    A2, B2 = logical_operands(variant, rng, 1000, 780, 1532, "int")
    for _ in range(20):
        C, _ = gpu_matmul_2d(gpu, variant, A, B)
        assert np.array_equal(C, first)
        C2, _ = gpu_matmul_2d(gpu, variant, A2, B2)             # the balanced kernel: same workspace, same counters
        assert np.array_equal(C2, oracle_2d(variant, A2, B2))
    assert_within_tolerance(first, oracle_2d(variant, A, B), 4096, A, B, "%s 8 x 4096 x 4096" % VARIANT_NAMES[variant])


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_forced_on_another_shape_falls_back(gpu, variant):
    gpu.force_tile(SKINNY)
    check(gpu, variant, 300, 36, 64, 77 + variant)
    check(gpu, variant, 100, 4, 64, 78 + variant)
    check(gpu, variant, 8, 8, 64, 79 + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_agrees_with_the_tile_kernels(gpu, variant):
    """The same integer product through the skinny kernel and through a 64 x 64 tile kernel: equal bits."""
    rng = np.random.default_rng(9 + variant)
    for (N, M, K) in ((5000, 8, 516), (4, 5000, 516)):
        A, B = logical_operands(variant, rng, N, M, K, "int")
        C, _ = gpu_matmul_2d(gpu, variant, A, B)
        gpu.force_tile(1)
        C1, _ = gpu_matmul_2d(gpu, variant, A, B)
        gpu.force_tile(-1)
        assert np.array_equal(C, C1)
