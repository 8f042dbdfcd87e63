"""GPU parity of the 2-D products (matMul, matMulT1, matMulT2) against the CPU oracle,
through the C ABI.  Tolerances (FP32 path): relative Frobenius error <= 1e-5 and
per-element |err| <= 1e-4*sqrt(K)*max|A|*max|B|; integer-valued inputs must match
bit for bit (every summation order is exact there)."""
import numpy as np
import pytest

from oracle import oracle
from helpers import (NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, logical_operands,
                     gpu_matmul_2d, pad2, rel_fro)

pytestmark = pytest.mark.gpu

TILES = {-1: "auto", 0: "128x128", 1: "64x64", 2: "256x64", 3: "64x256", 4: "128x64", 5: "64x128",
         6: "128x128/k32", 7: "64x64/k32", 8: "128x64/k32", 9: "64x128/k32", 10: "64x64/k64",
         11: "64x64/k128", 12: "128x128/k64", 13: "128x64/k64", 14: "64x128/k64",
         # direct global->LDS staging through 4 stage buffers
         15: "dma 128x128", 16: "dma 64x64", 17: "dma 64x64/k32",
         # the balanced kernel: work shared in equal runs of LDS stages (one / two workgroups per compute unit)
         18: "balanced 64x64", 19: "balanced 128x64", 20: "balanced 64x128", 21: "balanced 128x128",
         22: "balanced 64x64 x2", 23: "balanced 128x64 x2",
         # a band of 128 rows of A held in LDS, the whole K (at most 64) in one stage; a longer K falls back
         24: "band 128x128",
         25: "balanced 256x64"}
# + 256: the paired-stage form of the shapes 0..9 (what the automatic choice takes for a long K)
PAIRED = 256
TILES.update({PAIRED + t: TILES[t] + " paired" for t in range(10)})
SHAPES = [(4, 4, 4), (8, 4, 12), (128, 128, 64), (64, 64, 16), (132, 260, 20), (100, 76, 36),
          (257, 129, 385), (512, 512, 512), (1000, 777, 1531), (31, 1023, 77), (1, 1, 1), (3, 2, 5)]


@pytest.fixture(autouse=True)
def _auto_tile(gpu):
    yield
    gpu.force_tile(-1)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("tile", sorted(TILES))
def test_integer_inputs_bitwise(gpu, variant, tile):
    rng = np.random.default_rng(100 + 10 * variant + tile)
    gpu.force_tile(tile)
    for (N, M, K) in SHAPES:
        A, B = logical_operands(variant, rng, N, M, K, dist="int")
        C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=123.0)
        R = oracle.matmul(variant, A, B)
        assert np.array_equal(C, R), "%s tile %s shape %s" % (VARIANT_NAMES[variant], TILES[tile], (N, M, K))
        # padded rows / columns of C are written as exact zeros (C was pre-filled with 123)
        assert np.count_nonzero(Cp[N:, :]) == 0 and np.count_nonzero(Cp[:, M:]) == 0


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("tile,K", [(PAIRED + 0, 112), (PAIRED + 1, 112), (PAIRED + 4, 80), (PAIRED + 5, 176),
                                    (PAIRED + 6, 156), (PAIRED + 7, 156), (PAIRED + 9, 100), (0, 112)])
def test_paired_stages_across_tile_boundaries(gpu, variant, tile, K):
    """More tiles than resident workgroups and an odd number of stages: a workgroup's second tile starts
    on the odd LDS buffer (one single stage, then pairs), the last stage of K is partial for some."""
    rng = np.random.default_rng(4000 + tile + variant)
    N = M = 4224 if tile in (PAIRED, 0) else 3100     # 33 x 33 tiles of 128 x 128; 49 x 49 of 64 x 64
    gpu.force_tile(tile)
    A, B = logical_operands(variant, rng, N, M, K, dist="int")
    C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=123.0)
    R = oracle.matmul_f64(variant, A, B).astype(np.float32)    # small integers: every order is exact
    assert np.array_equal(C, R), "%s tile %s" % (VARIANT_NAMES[variant], TILES[tile])
    assert np.count_nonzero(Cp[N:, :]) == 0 and np.count_nonzero(Cp[:, M:]) == 0


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("dist", ["uniform", "normal"])
def test_random_inputs_within_tolerance(gpu, variant, dist):
    rng = np.random.default_rng(7 + variant)
    for (N, M, K) in SHAPES + [(300, 200, 4096), (64, 2048, 1024)]:
        A, B = logical_operands(variant, rng, N, M, K, dist=dist)
        C, _ = gpu_matmul_2d(gpu, variant, A, B)
        what = "%s %s %s" % (VARIANT_NAMES[variant], dist, (N, M, K))
        assert_within_tolerance(C, oracle.matmul(variant, A, B), K, A, B, what + " vs FP32 oracle")
        assert_within_tolerance(C, oracle.matmul_f64(variant, A, B), K, A, B, what + " vs FP64 oracle")


def test_baseline_config_1_512_cubed(gpu):
    # C = A*B, 512^3, Uniform(-1,1) from the documented seed: the reference's CPU-runnable case
    from dragon_hip import synthetic
    g = synthetic.stream_for(1)
    A = g.uniform((512, 512), -1, 1)
    B = g.uniform((512, 512), -1, 1)
    R = oracle.matmul(NN, A, B)
    assert np.array_equal(R, oracle.multiply_literal(NN, A, B))   # the literal k,i,j loops
    C, _ = gpu_matmul_2d(gpu, NN, A, B)
    rf, me = assert_within_tolerance(C, R, 512, A, B, "config 1")
    assert oracle.samePercent_relative(C, R) >= 0.999               # the reference's own rule


def test_transposed_variants_agree_with_plain_product(gpu):
    rng = np.random.default_rng(5)
    A, B = logical_operands(NN, rng, 200, 333, 515)
    C, _ = gpu_matmul_2d(gpu, NN, A, B)
    C1, _ = gpu_matmul_2d(gpu, T1, A.T.copy(), B)
    C2, _ = gpu_matmul_2d(gpu, T2, A, B.T.copy())
    for X in (C1, C2):
        assert rel_fro(X, C) < 2e-6


def test_power_of_two_scaling_is_bitwise_linear(gpu):
    # scaling an operand by 2 scales every product and partial sum exactly
    rng = np.random.default_rng(6)
    for variant in (NN, T1, T2):
        A, B = logical_operands(variant, rng, 300, 260, 700)
        C, _ = gpu_matmul_2d(gpu, variant, A, B)
        C2, _ = gpu_matmul_2d(gpu, variant, (2 * A).astype(np.float32), B)
        assert np.array_equal(C2, 2 * C)
        Cagain, _ = gpu_matmul_2d(gpu, variant, A, B)
        assert np.array_equal(C, Cagain)          # deterministic


def test_all_stream_handles_accepted_and_left_usable(gpu):
    Cuda = gpu.Cuda
    streams = [Cuda.newStream_Blocking() for _ in range(10)]
    rng = np.random.default_rng(8)
    A, B = logical_operands(NN, rng, 96, 100, 64, dist="int")
    C, _ = gpu_matmul_2d(gpu, NN, A, B, streams=streams)
    assert np.array_equal(C, oracle.matmul(NN, A, B))
    for s in streams:
        Cuda.streamSynchronize(s)
        assert Cuda.streamQuery(s)
        Cuda.deleteStream(s)


def _sweep_values():
    v = set(range(1, 256, 11)) | {2, 3, 4, 5, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 254, 255}
    return sorted(v)


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_reference_correctness_sweep(gpu, variant):
    """The reference's exhaustive sweep (rows, cols in 1..255, K in 128..132 and 512..517,
    Cuda_matMul_test.java:135-141), thinned to every residue class that matters for the
    tiles, with the reference's Uniform[0,1) inputs.  Each case goes through the strided
    upload/download path (set2D/get2D) like eg.tensor()/eg.valueOf() do."""
    Cuda, MM = gpu.Cuda, gpu.Cuda_matMul
    rng = np.random.default_rng(42 + variant)
    cap = 256 * 520
    dA, dB, dC = (gpu.DeviceArray(size=cap) for _ in range(3))
    fn = [MM.matMul, MM.matMulT1, MM.matMulT2][variant]
    p4 = lambda x: (x + 3) // 4 * 4
    vals = _sweep_values()
    ks = [128, 129, 130, 131, 132, 512, 513, 515, 517]
    worst = 0.0
    for K in ks:
        for n in vals:
            ms = vals if n in (1, 64, 129, 255) else vals[::4]
            for m in ms:
                shA = (K, n) if variant == T1 else (n, K)
                shB = (m, K) if variant == T2 else (K, m)
                A = rng.random(shA, dtype=np.float32)
                B = rng.random(shB, dtype=np.float32)
                # tensors of fewer than x4 rows are allocated with zero rows up to x4
                Cuda.memsetAsync(0, dA.address, 0, p4(shA[0]) * p4(shA[1]) * 4)
                Cuda.memsetAsync(0, dB.address, 0, p4(shB[0]) * p4(shB[1]) * 4)
                Cuda.set2D(0, dA.address, A, shA[0], shA[1], p4(shA[1]))
                Cuda.set2D(0, dB.address, B, shB[0], shB[1], p4(shB[1]))
                fn([0], 1, dA.address, dB.address, dC.address, p4(n), p4(m), p4(K))
                C = np.empty((n, m), np.float32)
                Cuda.get2D(0, dC.address, C, n, m, p4(m))
                R = oracle.matmul(variant, A, B)
                worst = max(worst, rel_fro(C, R))
                assert oracle.samePercent_relative(C, R) >= 0.999, (n, m, K)
                assert rel_fro(C, R) <= 1e-5, (n, m, K)
    assert worst <= 1e-5
    for x in (dA, dB, dC):
        x.free()


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_every_row_and_column_count_up_to_255(gpu, variant):
    """The sweep above samples the reference's 1..255 x 1..255 grid; this one walks EVERY row count against four
    column counts and every column count against four row counts (K = 129), so that no residue of the tile,
    block and rim arithmetic goes unvisited."""
    rng = np.random.default_rng(4242 + variant)
    K = 129
    cases = [(n, m) for n in range(1, 256) for m in (1, 64, 130, 255)] + \
            [(n, m) for m in range(1, 256) for n in (3, 65, 128, 254)]
    for (n, m) in cases:
        A, B = logical_operands(variant, rng, n, m, K, dist="int")
        C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=5.0)
        assert np.array_equal(C, oracle.matmul(variant, A, B)), (n, m)
        assert np.count_nonzero(Cp[n:, :]) == 0 and np.count_nonzero(Cp[:, m:]) == 0, (n, m)
