"""The BASELINE workloads at their full sizes, on the documented seeded inputs, against
the CPU oracle (FP32 sequential = the reference's CPU matmul, and its FP64 twin), plus
size-independent properties.  Tolerances: relative Frobenius error <= 1e-5 and
per-element |err| <= 1e-4*sqrt(K)*max|A|*max|B|."""
import numpy as np
import pytest

from oracle import oracle
from helpers import NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, rel_fro

pytestmark = pytest.mark.gpu
p4 = lambda v: (v + 3) // 4 * 4


@pytest.fixture(scope="module")
def syn(gpu):
    from dragon_hip import synthetic
    return synthetic


def test_config_2_square_4096(gpu, syn):
    """A*B, A*B^T, A^T*B at 4096^3, Normal(0,1), C zero-initialised."""
    n = 4096
    g = syn.stream_for(2)
    A = g.normal((n, n), 0.0, 1.0)
    B = g.normal((n, n), 0.0, 1.0)
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(size=n * n)
    results = {}
    for variant, fn in ((NN, MM.matMul), (T2, MM.matMulT2), (T1, MM.matMulT1)):
        Cuda.memsetAsync(0, dC.address, 0, n * n * 4)
        fn([0], 1, dA.address, dB.address, dC.address, n, n, n)
        Cuda.streamSynchronize(0)
        C = dC.get((n, n))
        results[variant] = C
        R32 = oracle.matmul(variant, A, B)
        rf, me = assert_within_tolerance(C, R32, n, A, B, VARIANT_NAMES[variant] + " vs FP32 oracle")
        assert oracle.samePercent_relative(C[:256], R32[:256]) >= 0.999
    # FP64 twin for the plain product
    assert_within_tolerance(results[NN], oracle.matmul_f64(NN, A, B), n, A, B, "A*B vs FP64 oracle")
    # (A*B^T)^T computed as B*A^T: swap operands, same kernel family
    Cuda.memsetAsync(0, dC.address, 0, n * n * 4)
    MM.matMulT2([0], 1, dB.address, dA.address, dC.address, n, n, n)
    Cuda.streamSynchronize(0)
    assert rel_fro(dC.get((n, n)).T, results[T2]) < 2e-6
    # doubling B doubles C bit for bit at full size
    dB2 = gpu.DeviceArray((2 * B).astype(np.float32))
    MM.matMul([0], 1, dA.address, dB2.address, dC.address, n, n, n)
    Cuda.streamSynchronize(0)
    assert np.array_equal(dC.get((n, n)), 2 * results[NN])
    for x in (dA, dB, dB2, dC):
        x.free()


def test_config_3_tall_k_split(gpu, syn):
    """A^T*B with A, B of 131072 x 256, Normal(0, 0.05): split-K with the GridZ the
    unchanged host policy picks for this device, then the compensated reduction."""
    K, N, M = 131072, 256, 256
    g = syn.stream_for(3)
    A = g.normal((K, N), 0.0, 0.05)
    B = g.normal((K, M), 0.0, 0.05)
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    SM = Cuda.multiProcessorCount(0)
    GZ = oracle.gridZ(oracle.MATMUL_T1, N, M, K, SM)
    if SM == 256:
        assert GZ == 128 and oracle.SK_K_slice(K, GZ) == 1024
    assert GZ >= 2
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC, dCbuf = gpu.DeviceArray(size=N * M), gpu.DeviceArray(size=N * M * (GZ - 1))
    dC.fill(1.0)
    dCbuf.fill(1.0)
    MM.matMulT1SK([0], 1, GZ, dA.address, dB.address, dC.address, dCbuf.address, N, M, K)
    Cuda.streamSynchronize(0)
    C0, Cbuf = dC.get((N, M)), dCbuf.get((GZ - 1, N, M))
    MM.SKbuf_summary(0, dCbuf.address, dC.address, GZ - 1, N * M)
    Cuda.streamSynchronize(0)
    C = dC.get((N, M))
    # stage 2 on the device equals the reference-order Kahan fold of the device's partials
    assert np.array_equal(C, oracle.SKbuf_summary(Cbuf, C0, GZ - 1))
    R64 = oracle.matmul_f64(T1, A, B)
    R32 = oracle.matmul(T1, A, B)                       # the reference's sequential FP32 sum
    assert_within_tolerance(C, R64, K, A, B, "config 3 vs FP64 oracle")
    # The gate as stated: relative Frobenius error <= 1e-5 against the CPU matmul (the reference's
    # sequential FP32 sum).  That sum of 131072 terms carries a rounding error of its own of about the
    # size of the gate, so the device result is also required to be at least as close to the exact
    # product as the FP32 oracle is.
    e_dev, e_seq, e_gate = rel_fro(C, R64), rel_fro(R32, R64), rel_fro(C, R32)
    print("config 3: rel_fro(device, FP32 oracle) = %.3e (gate 1e-5), rel_fro(device, FP64) = %.3e, "
          "rel_fro(FP32 oracle, FP64) = %.3e" % (e_gate, e_dev, e_seq), flush=True)
    assert e_gate <= 1e-5
    assert e_dev <= e_seq
    assert float(np.abs(C.astype(np.float64) - R32).max()) <= \
        1e-4 * np.sqrt(K) * float(np.abs(A).max()) * float(np.abs(B).max())
    # each partial against the oracle's partial for the same slice
    O0, Obuf = oracle.matMulSK(T1, GZ, A, B)
    assert rel_fro(C0, O0) < 1e-5 and rel_fro(Cbuf, Obuf) < 1e-5
    # unsplit entry point on the same data
    MM.matMulT1([0], 1, dA.address, dB.address, dC.address, N, M, K)
    Cuda.streamSynchronize(0)
    assert_within_tolerance(dC.get((N, M)), R64, K, A, B, "config 3 unsplit vs FP64 oracle")
    for x in (dA, dB, dC, dCbuf):
        x.free()


def test_config_4_attention_like_batches(gpu, syn):
    """batch 64: Q.K^T (1024x64 each), scores.V (1024x1024 by 1024x64), A^T.B (64x1024 each);
    all inputs Normal(0, 0.02)."""
    BMM, Cuda = gpu.Cuda_batchMatMul, gpu.Cuda
    g = syn.stream_for(4)
    Bt, S, D = 64, 1024, 64
    Q = g.normal((Bt, S, D), 0.0, 0.02)
    Kt = g.normal((Bt, S, D), 0.0, 0.02)
    scores = g.normal((Bt, S, S), 0.0, 0.02)
    V = g.normal((Bt, S, D), 0.0, 0.02)
    A1 = g.normal((Bt, D, S), 0.0, 0.02)
    B1 = g.normal((Bt, D, S), 0.0, 0.02)
    cases = [
        ("Q.K^T", T2, BMM.batchMatMulT2_texture, Q, Kt, (S, S, S, D), (Bt, S, S), D),
        ("scores.V", NN, BMM.batchMatMul_texture, scores, V, (S, D, S, S), (Bt, S, D), S),
        ("A^T.B", T1, BMM.batchMatMulT1, A1, B1, (S, S, S, D), (Bt, S, S), D),
    ]
    for name, variant, fn, A, B, dims, cshape, K in cases:
        dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
        dC = gpu.DeviceArray(size=int(np.prod(cshape)))
        fn([0], 1, dA.address, dB.address, dC.address, Bt, *dims)
        Cuda.streamSynchronize(0)
        C = dC.get(cshape)
        R = oracle.bmm(variant, A, B, Bt, *dims)
        assert_within_tolerance(C, R, K, A, B, "config 4 " + name)
        # batched == the 2-D entry point on one batch, bit for bit (same kernel arithmetic)
        b = 17
        MM = gpu.Cuda_matMul
        d2 = gpu.DeviceArray(size=cshape[1] * cshape[2])
        f2 = {NN: MM.matMul, T1: MM.matMulT1, T2: MM.matMulT2}[variant]
        f2([0], 1, dA.address + b * A[0].size * 4, dB.address + b * B[0].size * 4, d2.address,
           cshape[1], cshape[2], K)
        Cuda.streamSynchronize(0)
        assert rel_fro(d2.get(cshape[1:]), C[b]) < 1e-6
        for x in (dA, dB, dC, d2):
            x.free()


def test_config_5_ragged(gpu, syn):
    """Shapes that are not multiples of 64: 2-D at rows 1000, cols 777, K 1531 (padded to
    1000/780/1532) and batchMatMul batch 33 (36) of 257x129 by 129x385; Uniform(-1,1)."""
    MM, BMM, Cuda = gpu.Cuda_matMul, gpu.Cuda_batchMatMul, gpu.Cuda
    g = syn.stream_for(5)
    N, M, K = 1000, 777, 1531
    A = g.uniform((N, K), -1, 1)
    B = g.uniform((K, M), -1, 1)
    ops = {NN: (A, B), T2: (A, np.ascontiguousarray(B.T)), T1: (np.ascontiguousarray(A.T), B)}
    for variant, (a, b) in ops.items():
        ap, bp = syn.to_device_layout(a, pad_first=True), syn.to_device_layout(b, pad_first=True)
        dA, dB, dC = gpu.DeviceArray(ap), gpu.DeviceArray(bp), gpu.DeviceArray(size=p4(N) * p4(M))
        dC.fill(3.0)
        fn = {NN: MM.matMul, T1: MM.matMulT1, T2: MM.matMulT2}[variant]
        fn([0], 1, dA.address, dB.address, dC.address, p4(N), p4(M), p4(K))
        Cuda.streamSynchronize(0)
        Cp = dC.get((p4(N), p4(M)))
        assert_within_tolerance(Cp[:N, :M], oracle.matmul(variant, a, b), K, a, b,
                                "config 5 " + VARIANT_NAMES[variant])
        assert np.count_nonzero(Cp[:, M:]) == 0        # columns 777..779 come out zero
        # the host policy splits this shape in two on a 256-CU device: same result
        GZ = oracle.gridZ(variant, p4(N), p4(M), p4(K), Cuda.multiProcessorCount(0))
        if GZ > 1:
            dCbuf = gpu.DeviceArray(size=p4(N) * p4(M) * (GZ - 1))
            sk = {NN: MM.matMulSK, T1: MM.matMulT1SK, T2: MM.matMulT2SK}[variant]
            sk([0], 1, GZ, dA.address, dB.address, dC.address, dCbuf.address, p4(N), p4(M), p4(K))
            MM.SKbuf_summary(0, dCbuf.address, dC.address, GZ - 1, p4(N) * p4(M))
            Cuda.streamSynchronize(0)
            assert_within_tolerance(dC.get((p4(N), p4(M)))[:N, :M], oracle.matmul(variant, a, b),
                                    K, a, b, "config 5 split " + VARIANT_NAMES[variant])
            dCbuf.free()
        for x in (dA, dB, dC):
            x.free()
    # batched: batch 33 -> 36, A[33,257,129] -> 36*257*132, B[33,129,385] -> 36*129*388
    Bt, n, k, m = 33, 257, 129, 385
    Ab = g.uniform((Bt, n, k), -1, 1)
    Bb = g.uniform((Bt, k, m), -1, 1)
    Ap, Bp = syn.to_device_layout(Ab, pad_first=True), syn.to_device_layout(Bb, pad_first=True)
    assert Ap.shape == (36, 257, 132) and Bp.shape == (36, 129, 388)
    dA, dB, dC = gpu.DeviceArray(Ap), gpu.DeviceArray(Bp), gpu.DeviceArray(size=36 * 257 * 388)
    dC.fill(3.0)
    BMM.batchMatMul_texture([0], 1, dA.address, dB.address, dC.address, 36, n, 388, k, 132)
    Cuda.streamSynchronize(0)
    C = dC.get((36, 257, 388))
    R = oracle.bmm(NN, Ap, Bp, 36, n, 388, k, 132)
    assert_within_tolerance(C, R, k, Ab, Bb, "config 5 batched")
    assert np.count_nonzero(C[33:]) == 0 and np.count_nonzero(C[:, :, 385:]) == 0
    for x in (dA, dB, dC):
        x.free()
