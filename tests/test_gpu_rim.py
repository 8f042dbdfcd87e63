"""GPU parity of the rim path of the 64 x 64 kernels: where C is 1..4 rows and / or columns past a multiple of
64, the tiles cover the part of C that fills them and the launch's first workgroups compute the rim with plain
FMAs (the reference carves such edges down to tiles of 4, MM/matMul.cuh:24-43, and has kernels for a C of 4
columns, MM/matMul_sernel.cuh:17-30).  Integer inputs pin the indexing bit for bit: which rows and columns go
to the rim, jobs of 64 outputs with a ragged last one, the quarters of K, batches, operand padding that does
not exist in memory."""
import numpy as np
import pytest

from oracle import oracle
from helpers import NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, logical_operands, gpu_matmul_2d
from test_gpu_batched import make_case, run

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _auto_tile(gpu):
    yield
    gpu.force_tile(-1)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("tile", [1, 7])
def test_two_dimensional_rims_bitwise(gpu, variant, tile):
    """Rows 1..4 past, columns 4 past (2-D extents are multiples of 4), both, K from 1 to the limit of 256, a
    K that the four quarters do not divide, one tile plus rim, many tiles plus rim."""
    rng = np.random.default_rng(9100 + 10 * variant + tile)
    gpu.force_tile(tile)
    for (N, M, K) in ((65, 65, 8), (66, 68, 1), (67, 64, 3), (68, 132, 37), (129, 257, 129), (257, 385, 129),
                      (260, 196, 256), (513, 1028, 77), (1025, 68, 200), (68, 1025, 200)):
        A, B = logical_operands(variant, rng, N, M, K, dist="int")
        C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=17.0)
        R = oracle.matmul_f64(variant, A, B).astype(np.float32)     # small integers: every order is exact
        what = "%s tile %d shape %s" % (VARIANT_NAMES[variant], tile, (N, M, K))
        assert np.array_equal(C, R), what
        assert np.count_nonzero(Cp[N:, :]) == 0 and np.count_nonzero(Cp[:, M:]) == 0, what


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_batched_rims_bitwise(gpu, variant):
    # unpadded rows (257 = 4 x 64 + 1), columns padded to 388 = 6 x 64 + 4 of which 385 exist in B
    rng = np.random.default_rng(9200 + variant)
    for tile in (-1, 1, 7):
        gpu.force_tile(tile)
        for (Batch, N, M, K) in ((33, 257, 385, 129), (5, 65, 66, 9), (3, 130, 449, 255), (2, 321, 64, 64), (7, 64, 321, 31)):
            A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "int")
            C = run(gpu, variant, A, B, B4, dims, cshape)
            R = oracle.bmm(variant, A, B, B4, *dims)
            what = "%s tile %d batched %s" % (VARIANT_NAMES[variant], tile, (Batch, N, M, K))
            assert np.array_equal(C, R), what
            assert np.count_nonzero(C[Batch:]) == 0 and np.count_nonzero(C[:, :, M:]) == 0, what


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_random_inputs_within_tolerance(gpu, variant):
    rng = np.random.default_rng(9300 + variant)
    Batch, N, M, K = 33, 257, 385, 129          # BASELINE config 5, batched
    A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "uniform")
    C = run(gpu, variant, A, B, B4, dims, cshape)
    R = oracle.bmm(variant, A, B, B4, *dims)
    assert_within_tolerance(C, R, K, A, B, "%s batch 33 of 257 x 385 x 129" % VARIANT_NAMES[variant])
    assert oracle.samePercent_relative(C, R) >= 0.999
