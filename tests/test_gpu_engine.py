"""The host-side engine (Engine / EngineCore / CudaFloat32EngineBase / Tensor mirror) on the
GPU, written the way the reference's own tests are (alpha-Dragon-v1.2/test/test/cuda/matMul/
Cuda_matMul_test.java:51-95, Cuda_batchMatMul_test.java:47-82): random inputs -> eg.tensor ->
eg.matMul -> eg.valueOf -> compare with the CPU loops by samePercent_relative."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=["direct", "pooled"])
def eg(gpu, request):
    """Every test runs on an engine that allocates each block on the device itself and on one with the
    reference's recycling pool (alpha.engine.memp1) behind its tensors and partial buffers."""
    from dragon_hip import engine
    e = engine.cuda_float32(0, 32, max_mem_size=(2 << 30) if request.param == "pooled" else 0)
    yield e
    e.close()


def check_correct(eg, N, M, K, rng):   # testCorrect(N, M, K) of the reference
    A = rng.random(N * K, dtype=np.float32)
    B = rng.random(K * M, dtype=np.float32)
    tA, tB = eg.tensor(A, N, K), eg.tensor(B, K, M)
    C1 = oracle.matmul(0, A.reshape(N, K), B.reshape(K, M)).reshape(-1)      # CPU
    tC1 = eg.matMul(tA, tB).c()                                               # GPU
    tC2 = eg.matMul(eg.empty(N, M).c(), tA, tB).c()
    C2, C3 = eg.valueOf(tC1), eg.valueOf(tC2)
    sp1, sp2 = oracle.samePercent_relative(C1, C2), oracle.samePercent_relative(C1, C3)
    assert sp1 >= 0.999 and sp2 >= 0.999, (N, M, K)
    assert np.array_equal(C2, C3)
    eg.delete(tA, tB, tC1, tC2)


def test_matMul_like_the_reference(eg):
    rng = np.random.default_rng(1)
    base = eg.get_param("live_blocks")
    for (N, M, K) in [(1, 1, 1), (20, 52, 2), (255, 255, 132), (64, 65, 517), (1024, 1148, 1024)]:
        check_correct(eg, N, M, K, rng)
    assert eg.get_param("live_blocks") == base        # nothing leaked


def test_tensor_layout(eg):
    t = eg.tensor(np.arange(33 * 257 * 129, dtype=np.float32), 33, 257, 129)
    assert (t.length, t.lengthv, t.length_4x) == (33 * 257 * 129, 33 * 257 * 132, 36 * 257 * 132)
    assert t.dim == [33, 257, 129] and t.address % 16 == 0
    assert np.array_equal(eg.valueOf(t), np.arange(33 * 257 * 129, dtype=np.float32))
    # the pad reads as zero on the device
    raw = np.empty(t.length_4x, np.float32)
    from dragon_hip import Cuda
    Cuda.get1D(0, t.address, raw, t.length_4x)
    raw = raw.reshape(36, 257, 132)
    assert not raw[:, :, 129:].any() and not raw[33:].any()
    v = eg.tensor(np.ones(10, np.float32), 10)
    assert (v.length, v.lengthv, v.length_4x) == (10, 12, 12)
    u = eg.tensor(np.ones(24, np.float32), -1, 6)       # one dimension inferred
    assert u.dim == [4, 6]
    eg.delete(t, v, u)


@pytest.mark.parametrize("sync", [True, False])
def test_three_products_and_async_mode(eg, sync):
    rng = np.random.default_rng(2)
    eg.sync(sync)
    try:
        N, M, K = 130, 70, 300
        A = rng.uniform(-1, 1, (N, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (K, M)).astype(np.float32)
        tA, tB = eg.tensor(A, N, K), eg.tensor(B, K, M)
        tAt, tBt = eg.tensor(A.T.copy(), K, N), eg.tensor(B.T.copy(), M, K)
        R = oracle.matmul(0, A, B)
        outs = [eg.matMul(tA, tB), eg.matMulT1(tAt, tB), eg.matMulT2(tA, tBt)]
        for t in outs:
            assert t.dim == [N, M]
            C = eg.valueOf(t).reshape(N, M)              # valueOf waits for the producer
            assert np.linalg.norm(C - R) / np.linalg.norm(R) <= 1e-5
        eg.delete(tA, tB, tAt, tBt, *outs)
    finally:
        eg.sync(True)


def test_split_k_through_the_engine_frees_its_buffer(eg):
    rng = np.random.default_rng(3)
    K, N, M = 16384, 256, 256
    A = rng.standard_normal((K, N)).astype(np.float32) * 0.05
    B = rng.standard_normal((K, M)).astype(np.float32) * 0.05
    tA, tB = eg.tensor(A, K, N), eg.tensor(B, K, M)
    base = eg.get_param("live_blocks")
    eg.sync(False)
    try:
        tC = eg.matMulT1(tA, tB)
        GZ = eg.get_param("last_gridZ")
        assert GZ == eg.gridZ(1, N, M, K) == oracle.gridZ(1, N, M, K, eg.get_param("multiProcessorCount"))
        assert GZ >= 2
        assert eg.get_param("live_blocks") == base + 2      # C and the partial-product buffer
        tC.c()                                               # SplitKSyncer.sync() frees Cbuf
        assert eg.get_param("live_blocks") == base + 1
    finally:
        eg.sync(True)
    C = eg.valueOf(tC).reshape(N, M)
    R = oracle.matmul_f64(1, A, B)
    assert np.linalg.norm(C - R) / np.linalg.norm(R) <= 1e-5
    eg.delete(tA, tB, tC)


def test_a_skinny_product_through_the_engine(eg, gpu):
    """Engine.matMul of 8 rows by a 2048 x 4096 matrix: the unchanged policy splits it (GridZ >= 2), the library
    declines the split and runs the skinny kernel; the engine's sequence (stage 1, fold, syncer, buffer release)
    is the same and the result is the exact product."""
    rng = np.random.default_rng(12)
    N, K, M = 8, 2048, 4096
    A = rng.integers(-3, 4, (N, K)).astype(np.float32)
    B = rng.integers(-3, 4, (K, M)).astype(np.float32)
    tA, tB = eg.tensor(A, N, K), eg.tensor(B, K, M)
    base = eg.get_param("live_blocks")
    before = gpu.declined_splits()
    tC = eg.matMul(tA, tB)
    assert eg.get_param("last_gridZ") >= 2
    assert gpu.declined_splits() == before + 1
    assert np.array_equal(eg.valueOf(tC).reshape(N, M), oracle.matmul_f64(0, A, B).astype(np.float32))
    assert eg.get_param("live_blocks") == base + 1          # the partial buffer went back
    eg.delete(tA, tB, tC)


def test_events_are_recycled(eg):
    """The syncers' events (CudaFloat32EngineBase.java:657-694, 1008-1054 create and destroy one per call) come
    from a pool and go back to it: after many calls, split and unsplit, in both modes, the pool holds a few idle
    events rather than one per call, and the results stay right."""
    rng = np.random.default_rng(5)
    K, N, M = 4096, 256, 256
    A = rng.integers(-3, 4, (K, N)).astype(np.float32)
    B = rng.integers(-3, 4, (K, M)).astype(np.float32)
    tA, tB = eg.tensor(A, K, N), eg.tensor(B, K, M)
    R = oracle.matmul(1, A, B)
    for sync in (True, False, True):
        eg.sync(sync)
        for _ in range(40):
            tC = eg.matMulT1(tA, tB)
            tS = eg.matMul(tC, tC)                           # an unsplit product behind the split one
            assert np.array_equal(eg.valueOf(tC).reshape(N, M), R)
            eg.delete(tC, tS)
    eg.sync(True)
    assert 1 <= eg.get_param("pooled_events") <= 8
    eg.delete(tA, tB)


def test_policy_follows_the_unit_count(eg):
    real = eg.get_param("multiProcessorCount")
    try:
        eg.set_param("multiProcessorCount", 38)
        assert eg.get_param("matMulT1_maxPart") == 40
        assert eg.gridZ(1, 256, 256, 131072) == 36
        eg.set_param("multiProcessorCount", 256)
        assert eg.get_param("matMul_splitK_maxPart") == 128
        assert eg.gridZ(1, 256, 256, 131072) == 128
        assert [eg.gridZ(k, 1000, 780, 1532) for k in range(3)] == [2, 2, 2]
        assert [eg.gridZ(k, 4096, 4096, 4096) for k in range(3)] == [1, 1, 1]
        eg.set_param("matMulT1_maxPart", 16)
        assert eg.gridZ(1, 256, 256, 131072) == 16
    finally:
        eg.set_param("multiProcessorCount", real)


def test_stream_counts_follow_nstream(eg):
    rng = np.random.default_rng(4)
    tA = eg.tensor(rng.random(1000 * 64, dtype=np.float32), 1000, 64)
    tB = eg.tensor(rng.random(64 * 777, dtype=np.float32), 64, 777)
    tC = eg.matMul(tA, tB)
    assert eg.get_param("last_stream_count") == oracle.nstream(1000, 780) == 10
    assert eg.get_param("stream_pool_size") == 32
    C = eg.valueOf(tC).reshape(1000, 777)
    R = oracle.matmul(0, eg.valueOf(tA).reshape(1000, 64), eg.valueOf(tB).reshape(64, 777))
    assert oracle.samePercent_relative(C, R) >= 0.999
    eg.delete(tA, tB, tC)


def test_batched_products_like_the_reference(eg):
    # Cuda_batchMatMul_test.java:47-82: 4-D tensors [Batch0, Batch1, N, K]
    rng = np.random.default_rng(5)
    B0, B1 = 5, 3
    for (N, M, K) in [(24, 21, 8), (82, 96, 9), (7, 5, 7), (130, 68, 36)]:
        A = rng.random((B0, B1, N, K), dtype=np.float32)
        B = rng.random((B0, B1, K, M), dtype=np.float32)
        tA, tB = eg.tensor(A, B0, B1, N, K), eg.tensor(B, B0, B1, K, M)
        tC = eg.batchMatMul(eg.empty(B0, B1, N, M), tA, tB).c()
        ref = np.stack([oracle.matmul(0, A.reshape(-1, N, K)[b], B.reshape(-1, K, M)[b])
                        for b in range(B0 * B1)])
        assert oracle.samePercent_relative(eg.valueOf(tC), ref) == 1.0
        # T1: A stored [.., K, N];  T2: B stored [.., M, K]
        tAt = eg.tensor(np.swapaxes(A, -1, -2).copy(), B0, B1, K, N)
        tBt = eg.tensor(np.swapaxes(B, -1, -2).copy(), B0, B1, M, K)
        tC1, tC2 = eg.batchMatMulT1(tAt, tB), eg.batchMatMulT2(tA, tBt)
        assert tC1.dim == [B0, B1, N, M] and tC2.dim == [B0, B1, N, M]
        assert oracle.samePercent_relative(eg.valueOf(tC1), ref) == 1.0
        assert oracle.samePercent_relative(eg.valueOf(tC2), ref) == 1.0
        eg.delete(tA, tB, tAt, tBt, tC, tC1, tC2)


def test_error_behaviour(eg):
    from dragon_hip import engine as E
    a = eg.tensor(np.ones(12, np.float32), 3, 4)
    b = eg.tensor(np.ones(15, np.float32), 5, 3)
    with pytest.raises(E.IllegalArgumentException):
        eg.matMul(a, b)                      # A.width != B.height
    with pytest.raises(E.NullPointerException):
        eg.matMul(a, None)
    with pytest.raises(E.IllegalArgumentException):
        eg.empty(3, 0)                       # dims must be positive
    with pytest.raises(E.IllegalArgumentException):
        eg.tensor(np.ones(7, np.float32), 2, 4)   # value.length != tensor.length
    with pytest.raises(E.IllegalArgumentException):
        eg.set_param("matMul_splitK_threshold", 500)   # must be a power of two
    with pytest.raises(E.IllegalArgumentException):
        eg.set_param("matMul_splitK_maxPart", 3)       # must be >= 4
    v3 = eg.tensor(np.ones(24, np.float32), 2, 3, 4)
    with pytest.raises(E.IllegalArgumentException):
        eg.batchMatMul(v3, eg.tensor(np.ones(40, np.float32), 2, 5, 4))   # K mismatch
    eg.delete(a, b, v3)
