"""GPU parity of the resident-K kernel (gemm_mfma_shortk.hip): batches of ragged products with a K of 89 ... 144,
64 x 64 tiles whose whole K sits in LDS, the rim of C (1 ... 4 rows / columns past a multiple of 64) computed as
strips of 4 x 4 MFMA blocks beside the tiles.  What the reference answers with its padded / texture batch kernels
(BMM/batchMatMul_kernel_padding.cuh:20-42, BMM/batchMatMulT2_kernel_padding.cuh:23-45).  Integer inputs pin the
indexing bit for bit: tile and strip bounds, the K tail, panels, batches shared between workgroups."""
import numpy as np
import pytest

from oracle import oracle
from helpers import NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, gpu_matmul_2d, logical_operands, rel_fro
from test_gpu_batched import make_case, run

pytestmark = pytest.mark.gpu

SHORTK = 26


@pytest.fixture(autouse=True)
def _auto_tile(gpu):
    yield
    gpu.force_tile(-1)


def check(gpu, variant, Batch, N, M, K, seed):
    rng = np.random.default_rng(seed)
    A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "int")
    C = run(gpu, variant, A, B, B4, dims, cshape, fill=-77.0)
    R = oracle.bmm(variant, A, B, B4, *dims)
    what = "%s batch %d of %d x %d x %d" % (VARIANT_NAMES[variant], Batch, N, M, K)
    if not np.array_equal(C, R):
        bad = np.argwhere(C != R)
        raise AssertionError("%s: %d wrong outputs, first at %s (got %s, want %s); batches %s rows %s cols %s" % (
            what, len(bad), bad[0], C[tuple(bad[0])], R[tuple(bad[0])], sorted(set(bad[:, 0]))[:8],
            sorted(set(bad[:, 1]))[:12], sorted(set(bad[:, 2]))[:12]))
    assert np.count_nonzero(C[Batch:]) == 0, what + ": padded batches must come out zero"
    assert np.count_nonzero(C[:, :, M:]) == 0, what + ": padded columns must come out zero"


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("K", [89, 90, 95, 96, 97, 100, 104, 105, 112, 113, 120, 121, 127, 128, 129, 131, 136, 137, 143, 144])
def test_every_k_the_kernel_takes_bitwise(gpu, variant, K):
    """Rows 257 (one rim row) and columns 385 (stored 388: a rim of four) as in the ragged BASELINE batch, over
    the K range of the kernel: the panel the K ends in, the last group's MFMA count, K-inner chunks cut short."""
    gpu.force_tile(SHORTK)
    check(gpu, variant, 5, 257, 385, K, 1000 + K + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("rows", [64, 65, 66, 67, 68, 129, 130, 131, 192, 200, 256, 257, 258, 259, 260, 261, 300])
def test_rows_around_the_tile_multiples_bitwise(gpu, variant, rows):
    """Row counts 0 ... 5 past a multiple of 64 (up to 4: a strip; 5 and more: a partly filled tile row) and in
    the middle of a tile, against a column count with a rim (132) and one without (200)."""
    gpu.force_tile(SHORTK)
    for cols in (129, 200):
        check(gpu, variant, 3, rows, cols, 129, 2000 + rows + cols + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("cols", [64, 65, 69, 126, 128, 129, 131, 133, 192, 193, 250, 385, 386, 387, 388, 389, 512])
def test_columns_around_the_tile_multiples_bitwise(gpu, variant, cols):
    gpu.force_tile(SHORTK)
    for rows in (66, 150):
        check(gpu, variant, 3, rows, cols, 100, 3000 + rows + cols + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_shares_of_the_tiles_bitwise(gpu, variant):
    """Fewer tiles than compute units, one tile each, shares that cross batches, many tiles per workgroup."""
    gpu.force_tile(SHORTK)
    for (Batch, N, M) in ((1, 64, 64), (1, 257, 385), (3, 130, 70), (11, 257, 129), (40, 192, 193), (33, 257, 385),
                          (2, 1000, 777), (130, 65, 65)):
        check(gpu, variant, Batch, N, M, 129, 4000 + Batch + N + M + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("K", [1, 7, 63, 64, 65, 80, 81, 88, 145, 160, 200])
def test_a_k_outside_the_range_takes_another_kernel(gpu, variant, K):
    """Forced on a K it does not take (at most 88, beyond 144) the launch falls back to the tile-per-workgroup
    kernels: same results."""
    gpu.force_tile(SHORTK)
    check(gpu, variant, 3, 257, 385, K, 5000 + K + variant)


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_two_dimensional_products_bitwise(gpu, variant):
    gpu.force_tile(SHORTK)
    rng = np.random.default_rng(60 + variant)
    for (N, M, K) in ((257, 385, 129), (1000, 777, 100), (64, 68, 144), (513, 129, 96)):
        A, B = logical_operands(variant, rng, N, M, K, dist="int")
        C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=9.0)
        assert np.array_equal(C, oracle.matmul(variant, A, B)), (VARIANT_NAMES[variant], N, M, K)
        assert np.count_nonzero(Cp[N:]) == 0 and np.count_nonzero(Cp[:, M:]) == 0


def test_the_ragged_baseline_batch_takes_it_and_stays_within_tolerance(gpu):
    """BASELINE config 5's batch: 33 (36) products of 257 x 129 by 129 x 385, Uniform(-1, 1)."""
    assert gpu.choose_tile(NN, 257, 388, 36, 132, gpu.Cuda.multiProcessorCount(0)) == SHORTK
    rng = np.random.default_rng(5)
    for variant in (NN, T1, T2):
        A, B, dims, cshape, B4 = make_case(variant, rng, 33, 257, 385, 129, "uniform")
        C = run(gpu, variant, A, B, B4, dims, cshape)
        R = oracle.bmm(variant, A, B, B4, *dims)
        assert rel_fro(C, R) <= 1e-5
        assert float(np.abs(C - R).max()) <= 1e-4 * np.sqrt(129.0)
        # the same bits as the tile-per-workgroup kernel on the tiles' part of C (same k order)
        gpu.force_tile(1)
        C1 = run(gpu, variant, A, B, B4, dims, cshape)
        gpu.force_tile(-1)
        assert np.array_equal(C[:, :256, :384].view(np.uint32), C1[:, :256, :384].view(np.uint32))
        assert rel_fro(C, C1) <= 2e-6


def test_what_lies_behind_an_operands_k_stays_out(gpu):
    """B's rows from BK on are the next batch's first rows; A's columns from the chunk after BK on may hold
    anything.  Neither may reach the tiles or the strips."""
    gpu.force_tile(SHORTK)
    rng = np.random.default_rng(14)
    Batch, N, M, K, AK = 4, 257, 388, 129, 144
    A = np.full((Batch, N, AK), np.nan, np.float32)
    A[:, :, :K] = rng.integers(-3, 4, (Batch, N, K))
    A[:, :, K:132] = 0.0
    B = rng.integers(-3, 4, (Batch, K, M)).astype(np.float32)
    Bdev = B.copy()
    C = run(gpu, NN, A, Bdev, Batch, (N, M, K, AK), (Batch, N, M))
    R = np.einsum("bnk,bkm->bnm", A[:, :, :K].astype(np.float64), B.astype(np.float64)).astype(np.float32)
    assert np.array_equal(C, R)
    A2, B2, dims, cshape, B4 = make_case(NN, rng, 4, 257, 385, 129, "int")
    B2[1:, 0, :] = np.inf
    C = run(gpu, NN, A2, B2, B4, dims, cshape)
    assert np.isfinite(C[0]).all() and np.array_equal(C[0], oracle.bmm(NN, A2, B2, B4, *dims)[0])
