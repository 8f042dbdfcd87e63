"""GPU parity of the balanced kernel for products with few tiles and a long K: persistent workgroups share
the work in equal runs of LDS stages, pieces of shared tiles meet in a per-stream workspace and the
workgroup that arrives last adds them up in run order (no counterpart in the reference, whose answer is the
host's split-K policy, CudaFloat32EngineBase.java:1523-1562).  Integer inputs pin the indexing bit for
bit -- run boundaries inside a tile, pieces, counters that have to be back at zero for the next launch --
and the results must not depend on timing."""
import threading

import numpy as np
import pytest

from oracle import oracle
from helpers import (NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, logical_operands, gpu_matmul_2d, pad2)

pytestmark = pytest.mark.gpu

BALANCED = {18: "64x64", 19: "128x64", 20: "64x128", 21: "128x128", 22: "64x64 x2", 23: "128x64 x2", 25: "256x64"}


@pytest.fixture(autouse=True)
def _auto_tile(gpu):
    yield
    gpu.force_tile(-1)


def device_product(gpu, variant, Ap, Bp, dims, stream=0):
    MM = gpu.Cuda_matMul
    N, M, K = dims
    dA, dB, dC = gpu.DeviceArray(Ap), gpu.DeviceArray(Bp), gpu.DeviceArray(size=N * M)
    dC.fill(-5.0)
    [MM.matMul, MM.matMulT1, MM.matMulT2][variant]([stream], 1, dA.address, dB.address, dC.address, N, M, K)
    gpu.Cuda.streamSynchronize(stream)
    C = dC.get((N, M))
    for x in (dA, dB, dC):
        x.free()
    return C


def padded(variant, A, B):
    Ap, Bp = pad2(A), pad2(B)
    if variant == NN:
        (N, K), M = Ap.shape, Bp.shape[1]
    elif variant == T1:
        (K, N), M = Ap.shape, Bp.shape[1]
    else:
        (N, K), M = Ap.shape, Bp.shape[0]
    return Ap, Bp, (N, M, K)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("tile", sorted(BALANCED))
def test_runs_that_start_and_end_inside_tiles_bitwise(gpu, variant, tile):
    """Shapes chosen for the run arithmetic on 256 units: fewer stages than workgroups (some workgroups idle,
    every stage a piece), one tile for all workgroups, runs of exactly one tile (no piece at all), runs that
    cover several whole tiles between two pieces, a K that ends inside a stage, rows / columns 1..3 past a tile."""
    rng = np.random.default_rng(5000 + 10 * tile + variant)
    gpu.force_tile(tile)
    for (N, M, K) in ((8, 8, 8), (64, 64, 8192), (64, 64, 100), (1024, 1024, 32), (2048, 1024, 96),
                      (1000, 777, 1531), (257, 385, 4100), (129, 66, 2049), (512, 520, 3000)):
        A, B = logical_operands(variant, rng, N, M, K, dist="int")
        C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=77.0)
        R = oracle.matmul_f64(variant, A, B).astype(np.float32)     # small integers: every order is exact
        what = "%s balanced %s shape %s" % (VARIANT_NAMES[variant], BALANCED[tile], (N, M, K))
        assert np.array_equal(C, R), what
        assert np.count_nonzero(Cp[N:, :]) == 0 and np.count_nonzero(Cp[:, M:]) == 0, what


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_the_automatic_choice_takes_it_and_stays_within_tolerance(gpu, variant):
    # the chooser sends these through the balanced kernel (pinned on the CPU in test_c_abi_boundary)
    assert gpu.choose_tile(variant, 1000, 780, 1, 1532) == 18 and gpu.choose_tile(variant, 256, 256, 1, 8192) == 18
    assert gpu.choose_tile(variant, 512, 500, 1, 12000) == 18
    rng = np.random.default_rng(60 + variant)
    for (N, M, K), dist in (((1000, 777, 1531), "uniform"), ((256, 256, 8192), "normal"), ((512, 500, 11999), "normal")):
        A, B = logical_operands(variant, rng, N, M, K, dist=dist)
        C, _ = gpu_matmul_2d(gpu, variant, A, B)
        what = "%s %s %s" % (VARIANT_NAMES[variant], dist, (N, M, K))
        assert_within_tolerance(C, oracle.matmul(variant, A, B), K, A, B, what + " vs FP32 oracle")
        assert_within_tolerance(C, oracle.matmul_f64(variant, A, B), K, A, B, what + " vs FP64 oracle")


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_many_tiles_with_a_long_k_take_the_half_size_tile(gpu, variant):
    """Many 64 x 64 tiles, K >= 4096 and runs that are not whole tiles: the automatic choice is the 128 x 64 / 64 x 128
    balanced tile (fewer bytes staged per FLOP).  Integer inputs: every bit against the exact product."""
    assert gpu.choose_tile(variant, 1000, 780, 1, 4352) in (19, 20) and gpu.choose_tile(variant, 768, 772, 1, 8192) in (19, 20)
    rng = np.random.default_rng(900 + variant)
    for (N, M, K) in ((1000, 777, 4351), (768, 770, 8192)):
        A, B = logical_operands(variant, rng, N, M, K, dist="int")
        C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=3.0)
        R = oracle.matmul_f64(variant, A, B).astype(np.float32)
        assert np.array_equal(C, R), (VARIANT_NAMES[variant], N, M, K)
        assert np.count_nonzero(Cp[N:, :]) == 0 and np.count_nonzero(Cp[:, M:]) == 0


@pytest.mark.parametrize("tile", [22, 23, 18])
def test_every_bit_is_the_same_from_run_to_run(gpu, tile):
    """The pieces of a shared tile are added in run order whichever workgroup arrives last, so rounding
    cannot depend on timing: ten launches on random data, one answer."""
    rng = np.random.default_rng(tile)
    A, B = logical_operands(T1, rng, 1000, 777, 1531, dist="normal")
    Ap, Bp, dims = padded(T1, A, B)
    gpu.force_tile(tile)
    first = device_product(gpu, T1, Ap, Bp, dims)
    for _ in range(9):
        again = device_product(gpu, T1, Ap, Bp, dims)
        assert np.array_equal(first.view(np.uint32), again.view(np.uint32))


def test_two_streams_have_a_workspace_each(gpu):
    """Products issued at the same time on two streams must not meet in one workspace: each stream's
    results equal what the same product gives alone."""
    Cuda, MM = gpu.Cuda, gpu.Cuda_matMul
    rng = np.random.default_rng(11)
    cases = []
    for k, (N, M, K) in enumerate(((1000, 780, 1532), (512, 512, 4096))):
        A = rng.integers(-3, 4, (N, K)).astype(np.float32)
        B = rng.integers(-3, 4, (K, M)).astype(np.float32)
        cases.append((A, B, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32), (N, M, K)))
    streams = [Cuda.newStream_NonBlocking(), Cuda.newStream_NonBlocking()]
    dev = []
    for (A, B, R, (N, M, K)) in cases:
        dev.append((gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(size=N * M)))
    gpu.force_tile(22)
    for rep in range(20):                      # interleaved launches: the two streams' kernels overlap on the device
        for s, (dA, dB, dC), (A, B, R, (N, M, K)) in zip(streams, dev, cases):
            MM.matMul([s], 1, dA.address, dB.address, dC.address, N, M, K)
    for s in streams:
        Cuda.streamSynchronize(s)
    for (dA, dB, dC), (A, B, R, (N, M, K)) in zip(dev, cases):
        assert np.array_equal(dC.get((N, M)), R)
        for x in (dA, dB, dC):
            x.free()
    for s in streams:
        Cuda.deleteStream(s)


@pytest.mark.parametrize("tile", [18, 22, 23])
def test_two_thousand_overlapping_launches_give_one_answer(gpu, tile):
    """A bounded soak of the hand-over of shared tiles' pieces between workgroups, which rests on the order in
    which the hardware makes stores visible rather than on fences: 2000 launches of two products whose tiles
    are shared (1000 x 777 x 1531 and 257 x 385 x 4100), the two on a stream each so that launches overlap on
    the device, twenty in flight at a time, every result compared bit for bit with the first launch's.  Stops
    at the first mismatch."""
    Cuda, MM = gpu.Cuda, gpu.Cuda_matMul
    rng = np.random.default_rng(900 + tile)
    streams = [Cuda.newStream_NonBlocking(), Cuda.newStream_NonBlocking()]
    IN_FLIGHT, ROUNDS = 10, 100
    jobs = []
    for (N, M, K) in ((1000, 777, 1531), (257, 385, 4100)):
        A, B = logical_operands(T1, rng, N, M, K, dist="normal")
        Ap, Bp, dims = padded(T1, A, B)
        jobs.append((gpu.DeviceArray(Ap), gpu.DeviceArray(Bp), [gpu.DeviceArray(size=dims[0] * dims[1]) for _ in range(IN_FLIGHT)], dims))
    gpu.force_tile(tile)
    first = [None, None]
    launches = 0
    try:
        for rnd in range(ROUNDS):
            for i in range(IN_FLIGHT):
                for s, (dA, dB, dCs, (N, M, K)) in zip(streams, jobs):
                    MM.matMulT1([s], 1, dA.address, dB.address, dCs[i].address, N, M, K)
            for s in streams:
                Cuda.streamSynchronize(s)
            for j, (dA, dB, dCs, (N, M, K)) in enumerate(jobs):
                for i in range(IN_FLIGHT):
                    got = dCs[i].get((N, M)).view(np.uint32)
                    launches += 1
                    if first[j] is None:
                        first[j] = got
                    assert np.array_equal(first[j], got), "tile %d, product %d: launch %d differs from the first" % (tile, j, launches)
                    dCs[i].fill(-1.0)
        assert launches == 2 * IN_FLIGHT * ROUNDS
    finally:
        gpu.force_tile(-1)
        for dA, dB, dCs, _ in jobs:
            for x in [dA, dB] + dCs:
                x.free()
        for s in streams:
            Cuda.deleteStream(s)


def test_a_stream_takes_its_workspace_with_it(gpu):
    """The balanced kernel's workspace belongs to the stream that first needed it: a hundred streams made, used
    for a balanced launch and deleted leave the device's free memory where it was (to within one workspace),
    the table of workspaces never fills up, and the hundredth stream still gets the balanced kernel."""
    Cuda, MM = gpu.Cuda, gpu.Cuda_matMul
    rng = np.random.default_rng(4)
    N, M, K = 512, 512, 1024
    A = rng.integers(-3, 4, (N, K)).astype(np.float32)
    B = rng.integers(-3, 4, (K, M)).astype(np.float32)
    R = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(size=N * M)
    gpu.release_workspaces()
    held0, refused0 = gpu.workspace_count(), gpu.workspaces_refused()
    assert held0 == 0
    free0, _ = gpu.mem_get_info()
    gpu.force_tile(21)
    try:
        for i in range(100):
            s = Cuda.newStream_NonBlocking()
            dC.fill(7.0)
            MM.matMul([s], 1, dA.address, dB.address, dC.address, N, M, K)
            Cuda.streamSynchronize(s)
            assert gpu.workspace_count() == 1, "stream %d: the balanced kernel made no workspace" % i
            if i % 33 == 0 or i == 99:
                assert np.array_equal(dC.get((N, M)), R)
            Cuda.deleteStream(s)
            assert gpu.workspace_count() == 0
    finally:
        gpu.force_tile(-1)
    assert gpu.workspaces_refused() == refused0
    free1, _ = gpu.mem_get_info()
    workspace_bytes = 4 * (65536 + 2 * Cuda.multiProcessorCount(0) * 128 * 128)
    assert free0 - free1 <= workspace_bytes, "device memory not given back: %d bytes" % (free0 - free1)
    # streams that are kept: release on request
    s = Cuda.newStream_NonBlocking()
    gpu.force_tile(21)
    MM.matMul([s], 1, dA.address, dB.address, dC.address, N, M, K)
    Cuda.streamSynchronize(s)
    gpu.force_tile(-1)
    assert gpu.workspace_count() == 1 and gpu.release_workspaces() == 1 and gpu.workspace_count() == 0
    gpu.force_tile(21)
    MM.matMul([s], 1, dA.address, dB.address, dC.address, N, M, K)     # and a new one on the next launch
    Cuda.streamSynchronize(s)
    gpu.force_tile(-1)
    assert np.array_equal(dC.get((N, M)), R) and gpu.workspace_count() == 1
    Cuda.deleteStream(s)
    for x in (dA, dB, dC):
        x.free()


def test_host_threads_force_tiles_independently(gpu):
    """The forced tile is a setting of the calling thread: a second thread that forces another shape (or none)
    does not change what this thread's launches run, and its own choice is reported back to it."""
    seen = {}

    def other():
        seen["before"] = gpu.choose_tile(NN, 4096, 4096, 1, 4096)
        gpu.force_tile(3)
        seen["after"] = gpu.choose_tile(NN, 4096, 4096, 1, 4096)

    gpu.force_tile(22)
    th = threading.Thread(target=other)
    th.start()
    th.join()
    assert seen == {"before": 21, "after": 3}
    assert gpu.choose_tile(NN, 4096, 4096, 1, 4096) == 22


def test_batched_products_through_the_balanced_kernel(gpu):
    """Batches are tiles like any other: 5 (padded to 8) batches of 130 x 72 x 516."""
    BMM = gpu.Cuda_batchMatMul
    rng = np.random.default_rng(3)
    Batch, B4, N, M, K = 5, 8, 130, 70, 516
    M4, K4 = 72, 516
    A = np.zeros((B4, N, K4), np.float32)
    B = np.zeros((B4, K, M4), np.float32)
    A[:Batch, :, :K] = rng.integers(-3, 4, (Batch, N, K))
    B[:Batch, :, :M] = rng.integers(-3, 4, (Batch, K, M))
    R = np.einsum("bnk,bkm->bnm", A[:, :, :K].astype(np.float64), B.astype(np.float64)).astype(np.float32)
    for tile in sorted(BALANCED):
        gpu.force_tile(tile)
        dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(size=B4 * N * M4)
        dC.fill(9.0)
        BMM.batchMatMul([0], 1, dA.address, dB.address, dC.address, B4, N, M4, K, K4)
        gpu.Cuda.streamSynchronize(0)
        assert np.array_equal(dC.get((B4, N, M4)), R), BALANCED[tile]
        for x in (dA, dB, dC):
            x.free()


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_tiles_that_do_not_divide_among_the_workgroups_go_out_as_two_launches(gpu, variant):
    """Many 128 x 128 tiles, not a multiple of the compute units, K >= 3072: whole tiles first (every workgroup the
    same number), then the remaining tiles shared out in runs of stages -- two launches on the caller's stream.
    Every bit against the exact product (small integers), ragged rows and columns, and twice in a row (the
    second launch's arrival counters are back at zero)."""
    rng = np.random.default_rng(640 + variant)
    for (N, M, K) in ((3072, 3072, 3072), (2000, 5000, 3100), (3300, 2900, 3076)):
        assert gpu.choose_tile(variant, N, (M + 3) // 4 * 4, 1, (K + 3) // 4 * 4) == 21
        A, B = logical_operands(variant, rng, N, M, K, dist="int")
        R = oracle.matmul_f64(variant, A, B).astype(np.float32)
        for _ in range(2):
            C, Cp = gpu_matmul_2d(gpu, variant, A, B, fill=3.0)
            assert np.array_equal(C, R), "%s %s" % (VARIANT_NAMES[variant], (N, M, K))
            assert np.count_nonzero(Cp[N:, :]) == 0 and np.count_nonzero(Cp[:, M:]) == 0
