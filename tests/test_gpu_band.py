"""GPU parity of the band kernel for products with a short K (at most 64) and a large C: a workgroup keeps a
band of 128 rows of A in LDS, walks along the band's column tiles with the whole K in one LDS stage, and
stores a finished tile while it multiplies the next one (no counterpart in the reference, which runs these
shapes tile by tile, BMM/batchMatMulT2_uernel.cuh:51-173).  Integer inputs pin the indexing bit for bit:
bands and runs of column tiles dealt to workgroups, the two accumulator sets and B buffers taking turns, the
last tile of a workgroup, rows / columns / k beyond the operands."""
import numpy as np
import pytest

from oracle import oracle
from helpers import NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, logical_operands, gpu_matmul_2d
from test_gpu_batched import make_case, run

pytestmark = pytest.mark.gpu
BAND = 24           # bands of 128 rows, tiles of 128 columns
BAND_WIDE = 28      # bands of 64 rows, tiles of 256 columns
BAND_REGS = 29      # the band's rows of A in registers: four wavefronts, two workgroups per compute unit
BANDS = [BAND, BAND_WIDE, BAND_REGS]


@pytest.fixture(autouse=True)
def _auto_tile(gpu):
    yield
    gpu.force_tile(-1)


@pytest.mark.parametrize("band", BANDS)
@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_two_dimensional_shapes_bitwise(gpu, variant, band):
    """One tile; one band with an odd and an even number of tiles; more bands than compute units (a
    workgroup walks several bands: the A buffers take turns); bands cut into runs (few bands, many column
    tiles); rows, columns and K 1..3 past a tile or short of one."""
    rng = np.random.default_rng(8100 + variant)
    gpu.force_tile(band)
    for (N, M, K) in ((4, 4, 4), (128, 128, 64), (128, 384, 64), (128, 512, 60), (100, 1000, 33), (257, 1029, 64),
                      (40000, 260, 64), (33000, 131, 12), (256, 8200, 56), (131, 5000, 61), (1024, 1024, 64),
                      (64, 256, 64), (65, 257, 64), (200, 768, 64), (190, 770, 57)):
        A, B = logical_operands(variant, rng, N, M, K, dist="int")
        C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=91.0)
        R = oracle.matmul_f64(variant, A, B).astype(np.float32)     # small integers: every order is exact
        what = "%s band %s" % (VARIANT_NAMES[variant], (N, M, K))
        assert np.array_equal(C, R), what
        assert np.count_nonzero(Cp[N:, :]) == 0 and np.count_nonzero(Cp[:, M:]) == 0, what


@pytest.mark.parametrize("band", BANDS)
@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_batched_shapes_bitwise(gpu, variant, band):
    rng = np.random.default_rng(8200 + variant)
    gpu.force_tile(band)
    for (Batch, N, M, K) in ((1, 1, 1, 1), (3, 5, 6, 7), (15, 82, 96, 9), (4, 128, 128, 64), (37, 1024, 1024, 64),
                             (33, 257, 385, 61), (6, 300, 1000, 36), (70, 260, 520, 64)):
        A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "int")
        C = run(gpu, variant, A, B, B4, dims, cshape)
        R = oracle.bmm(variant, A, B, B4, *dims)
        what = "%s band batched %s" % (VARIANT_NAMES[variant], (Batch, N, M, K))
        assert np.array_equal(C, R), what
        assert np.count_nonzero(C[Batch:]) == 0 and np.count_nonzero(C[:, :, M:]) == 0, what


@pytest.mark.parametrize("band", BANDS)
@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_a_longer_k_takes_another_kernel(gpu, variant, band):
    # the band kernel holds K in one stage of 64: a forced choice falls back for a longer K
    rng = np.random.default_rng(8300 + variant)
    gpu.force_tile(band)
    A, B = logical_operands(variant, rng, 300, 520, 68, dist="int")
    C, _ = gpu_matmul_2d(gpu, variant, A, B)
    assert np.array_equal(C, oracle.matmul_f64(variant, A, B).astype(np.float32))


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_the_automatic_choice_takes_it_and_stays_within_tolerance(gpu, variant):
    assert gpu.choose_tile(variant, 1024, 1024, 64, 64) == BAND
    rng = np.random.default_rng(8400 + variant)
    Batch, N, M, K = 64, 1024, 1024, 64
    A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "uniform")
    C = run(gpu, variant, A, B, B4, dims, cshape)
    R = oracle.bmm(variant, A, B, B4, *dims)
    assert_within_tolerance(C, R, K, A, B, "%s batch 64 of 1024 x 1024 x 64" % VARIANT_NAMES[variant])
    assert oracle.samePercent_relative(C, R) >= 0.999
