"""Shared helpers of the parity tests: error metrics with the stated tolerances and
host<->device plumbing at the C-ABI level."""
import numpy as np

from oracle import oracle

NN, T1, T2 = 0, 1, 2
VARIANT_NAMES = {NN: "A*B", T1: "A^T*B", T2: "A*B^T"}

# Tolerances of the path (FP32): relative Frobenius error <= 1e-5 and
# per-element |err| <= 1e-4 * sqrt(K) * max|A| * max|B|.
REL_FRO_TOL = 1e-5
ELEM_COEF = 1e-4


def rel_fro(C, R):
    C = np.asarray(C, dtype=np.float64)
    R = np.asarray(R, dtype=np.float64)
    den = np.linalg.norm(R)
    return float(np.linalg.norm(C - R) / den) if den > 0 else float(np.linalg.norm(C - R))


def elem_bound(K, A, B):
    return ELEM_COEF * np.sqrt(K) * float(np.abs(A).max()) * float(np.abs(B).max())


def assert_within_tolerance(C, R, K, A, B, what=""):
    C64 = np.asarray(C, dtype=np.float64)
    R64 = np.asarray(R, dtype=np.float64)
    assert np.isfinite(C64).all(), what + ": non-finite output"
    rf = rel_fro(C64, R64)
    me = float(np.abs(C64 - R64).max()) if C64.size else 0.0
    assert rf <= REL_FRO_TOL, "%s: relative Frobenius error %.3e > %.1e" % (what, rf, REL_FRO_TOL)
    eb = elem_bound(K, A, B)
    assert me <= eb, "%s: max element error %.3e > bound %.3e" % (what, me, eb)
    return rf, me


def logical_operands(variant, rng, N, M, K, dist="uniform"):
    """Random logical operands for C[N,M]: NN A[N,K],B[K,M]; T1 A[K,N],B[K,M]; T2 A[N,K],B[M,K]."""
    shA = (K, N) if variant == T1 else (N, K)
    shB = (M, K) if variant == T2 else (K, M)
    if dist == "uniform":
        return (rng.uniform(-1, 1, shA).astype(np.float32),
                rng.uniform(-1, 1, shB).astype(np.float32))
    if dist == "int":
        return (rng.integers(-3, 4, shA).astype(np.float32),
                rng.integers(-3, 4, shB).astype(np.float32))
    return (rng.standard_normal(shA).astype(np.float32),
            rng.standard_normal(shB).astype(np.float32))


def pad2(x):
    """[r, c] logical -> zero-padded [r4, c4] (the engine pads N, M and K to x4 for 2-D)."""
    r, c = x.shape
    out = np.zeros(((r + 3) // 4 * 4, (c + 3) // 4 * 4), np.float32)
    out[:r, :c] = x
    return out


def gpu_matmul_2d(dh, variant, A, B, gz=1, streams=(0,), fill=None):
    """Runs one 2-D product through the C ABI on padded copies of the logical operands and
    returns the logical C[N,M] plus the full padded C."""
    MM = dh.Cuda_matMul
    Ap, Bp = pad2(A), pad2(B)
    if variant == NN:
        (N4, K4), M4 = Ap.shape, Bp.shape[1]
    elif variant == T1:
        (K4, N4), M4 = Ap.shape, Bp.shape[1]
    else:
        (N4, K4), M4 = Ap.shape, Bp.shape[0]
    N, M = (A.shape[1] if variant == T1 else A.shape[0]), (B.shape[0] if variant == T2 else B.shape[1])
    dA, dB = dh.DeviceArray(Ap), dh.DeviceArray(Bp)
    dC = dh.DeviceArray(size=N4 * M4)
    if fill is not None:
        dC.fill(fill)
    s = list(streams)
    if gz == 1:
        [MM.matMul, MM.matMulT1, MM.matMulT2][variant](s, len(s), dA.address, dB.address,
                                                         dC.address, N4, M4, K4)
    else:
        dCbuf = dh.DeviceArray(size=N4 * M4 * (gz - 1))
        if fill is not None:
            dCbuf.fill(fill)
        [MM.matMulSK, MM.matMulT1SK, MM.matMulT2SK][variant](s, len(s), gz, dA.address, dB.address,
                                                               dC.address, dCbuf.address, N4, M4, K4)
        MM.SKbuf_summary(s[0], dCbuf.address, dC.address, gz - 1, N4 * M4)
        dh.Cuda.streamSynchronize(s[0])
        dCbuf.free()
    dh.Cuda.streamSynchronize(s[0])
    Cp = dC.get((N4, M4))
    for x in (dA, dB, dC):
        x.free()
    return Cp[:N, :M], Cp


def oracle_2d(variant, A, B):
    return oracle.matmul(variant, A, B)
