"""GPU parity of batchMatMul / batchMatMulT1 / batchMatMulT2 in the reference's padded
memory layout (unpadded N, BK, CN, BM; padded AK, AN, CM; Batch rounded up to x4 with
all-zero batches)."""
import numpy as np
import pytest

from oracle import oracle
from helpers import NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, rel_fro

pytestmark = pytest.mark.gpu
p4 = lambda v: (v + 3) // 4 * 4


def make_case(variant, rng, Batch, N, M, K, dist):
    """Returns device-layout A, B (Batch already the padded count; trailing batches zero
    when `Batch` is not the logical count), the native dims, logical-real batch count."""
    draw = (lambda s: rng.integers(-3, 4, s).astype(np.float32)) if dist == "int" else \
           (lambda s: rng.uniform(-1, 1, s).astype(np.float32))
    B4 = p4(Batch)
    if variant == NN:
        AK, CM = p4(K), p4(M)
        A = np.zeros((B4, N, AK), np.float32); A[:Batch, :, :K] = draw((Batch, N, K))
        B = np.zeros((B4, K, CM), np.float32); B[:Batch, :, :M] = draw((Batch, K, M))
        dims, cshape = (N, CM, K, AK), (B4, N, CM)
    elif variant == T1:
        AN, CM = p4(N), p4(M)
        A = np.zeros((B4, K, AN), np.float32); A[:Batch, :, :N] = draw((Batch, K, N))
        B = np.zeros((B4, K, CM), np.float32); B[:Batch, :, :M] = draw((Batch, K, M))
        dims, cshape = (N, AN, CM, K), (B4, N, CM)
    else:
        K4, CM = p4(K), p4(M)
        A = np.zeros((B4, N, K4), np.float32); A[:Batch, :, :K] = draw((Batch, N, K))
        B = np.zeros((B4, M, K4), np.float32); B[:Batch, :, :K] = draw((Batch, M, K))
        dims, cshape = (N, CM, M, K4), (B4, N, CM)
    return A, B, dims, cshape, B4


def run(gpu, variant, A, B, B4, dims, cshape, texture=False, fill=55.0):
    BMM = gpu.Cuda_batchMatMul
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC = gpu.DeviceArray(size=int(np.prod(cshape)) + 64)     # guard floats after C
    dC.fill(fill)
    fn = {(NN, False): BMM.batchMatMul, (NN, True): BMM.batchMatMul_texture,
          (T1, False): BMM.batchMatMulT1, (T1, True): BMM.batchMatMulT1,
          (T2, False): BMM.batchMatMulT2, (T2, True): BMM.batchMatMulT2_texture}[(variant, texture)]
    fn([0], 1, dA.address, dB.address, dC.address, B4, *dims)
    gpu.Cuda.streamSynchronize(0)
    full = dC.get()
    n = int(np.prod(cshape))
    assert np.all(full[n:] == fill), "wrote past the end of C"
    for x in (dA, dB, dC):
        x.free()
    return full[:n].reshape(cshape)


SHAPES = [(1, 1, 1, 1), (3, 5, 6, 7), (5, 24, 21, 8), (15, 82, 96, 9), (4, 128, 128, 64),
          (33, 257, 385, 129), (2, 300, 70, 200), (6, 64, 1000, 36), (7, 130, 72, 516)]


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("tile", list(range(-1, 30)) + list(range(256, 266)))
def test_batched_integer_inputs_bitwise(gpu, variant, tile):
    rng = np.random.default_rng(900 + variant * 10 + tile)
    gpu.force_tile(tile)
    try:
        for (Batch, N, M, K) in SHAPES:
            A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "int")
            C = run(gpu, variant, A, B, B4, dims, cshape, texture=(tile % 2 == 0))
            R = oracle.bmm(variant, A, B, B4, *dims)
            assert np.array_equal(C, R), "%s %s" % (VARIANT_NAMES[variant], (Batch, N, M, K))
            assert np.count_nonzero(C[Batch:]) == 0            # padded batches: zero in, zero out
            assert np.count_nonzero(C[:, :, M:]) == 0          # padded columns are exact zeros
    finally:
        gpu.force_tile(-1)


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_batched_random_within_tolerance(gpu, variant):
    rng = np.random.default_rng(31 + variant)
    for (Batch, N, M, K) in SHAPES + [(8, 200, 260, 1024)]:
        A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "uniform")
        C = run(gpu, variant, A, B, B4, dims, cshape)
        R = oracle.bmm(variant, A, B, B4, *dims)
        assert_within_tolerance(C, R, K, A, B, "%s %s" % (VARIANT_NAMES[variant], (Batch, N, M, K)))
        assert oracle.samePercent_relative(C, R) >= 0.999


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_more_tiles_than_resident_workgroups_with_a_partial_last_round(gpu, variant):
    """37 (padded to 40) batches of 1024 x 1024 x 64 are 2560 tiles of 128 x 128 for 1024 resident
    workgroups: two full rounds and a last round of 512 tiles, dealt over the compute units by the
    hardware's workgroup id.  Integer inputs: every tile must come out bit for bit, exactly once."""
    rng = np.random.default_rng(700 + variant)
    Batch, N, M, K = 37, 1024, 1024, 64
    if variant == NN:
        N, M, K = 1024, 1024, 64
    A, B, dims, cshape, B4 = make_case(variant, rng, Batch, N, M, K, "int")
    C = run(gpu, variant, A, B, B4, dims, cshape)
    R = oracle.bmm(variant, A, B, B4, *dims)
    assert np.array_equal(C, R)
    assert np.count_nonzero(C[Batch:]) == 0


def test_reference_batched_sweep(gpu):
    """The reference's batched sweep (N in 1..82, M in 1..96, K in 7..9, batch 5x3,
    Cuda_batchMatMul_test.java:120-123), thinned; the reference demands sp == 1.0 here."""
    rng = np.random.default_rng(99)
    for variant in (NN, T1, T2):
        for K in (7, 8, 9):
            for N in (1, 2, 5, 31, 33, 64, 65, 82):
                for M in (1, 3, 4, 17, 63, 64, 96):
                    A, B, dims, cshape, B4 = make_case(variant, rng, 15, N, M, K, "uniform")
                    C = run(gpu, variant, A, B, B4, dims, cshape)
                    R = oracle.bmm(variant, A, B, B4, *dims)
                    assert rel_fro(C, R) <= 1e-5, (variant, N, M, K)
                    assert oracle.samePercent_relative(C, R, 1e-3) >= 0.999, (variant, N, M, K)


def test_neighbouring_batch_does_not_leak_into_the_k_tail(gpu):
    # BK = 129 is not a multiple of the k tile: rows >= BK of B[b] are the first rows of
    # B[b+1] in memory.  A's zero padding multiplies them in the reference's layout, but a
    # kernel that skipped the row guard would still pick up Inf/NaN from there.
    rng = np.random.default_rng(13)
    Batch, N, M, K = 4, 40, 36, 129
    A, B, dims, cshape, B4 = make_case(NN, rng, Batch, N, M, K, "int")
    B[1:, 0, :] = np.inf          # first row of every following batch
    R = oracle.bmm(NN, A, B, B4, *dims)
    C = run(gpu, NN, A, B, B4, dims, cshape)
    assert np.isfinite(C[0]).all() and np.array_equal(C[0], R[0])


def test_columns_of_a_beyond_the_k_that_exist_are_not_read(gpu):
    # AK may be wider than BK rounded up to 4 (a view into a wider tensor): whatever lies there, NaN included,
    # stays out of the product, as in the reference, whose loop over k stops at BK (BMM/batchMatMul.cuh:15)
    rng = np.random.default_rng(14)
    Batch, N, M, K, AK = 4, 70, 36, 129, 144
    A = np.full((Batch, N, AK), np.nan, np.float32)
    A[:, :, :K] = rng.integers(-3, 4, (Batch, N, K))
    A[:, :, K:132] = 0.0                                  # the rest of the last 16-byte chunk: finite
    B = rng.integers(-3, 4, (Batch, K, M)).astype(np.float32)
    for tile in (-1, 1, 7, 0):
        gpu.force_tile(tile)
        C = run(gpu, NN, A, B, Batch, (N, M, K, AK), (Batch, N, M))
        gpu.force_tile(-1)
        R = np.einsum("bnk,bkm->bnm", A[:, :, :K].astype(np.float64), B.astype(np.float64)).astype(np.float32)
        assert np.array_equal(C, R), tile
