"""The split-K product that allocates nothing (dragon_Cuda_matMul_matMulSK_static): partials in the
library's static device workspace instead of a caller's Cbuf.  Same kernels, same partial layout and
the same Kahan fold as matMul*SK + SKbuf_summary, so every bit of C must agree -- on a first call and
on a second, smaller one that finds the first call's partials still in the workspace."""
import ctypes

import numpy as np
import pytest

from helpers import NN, T1, T2, VARIANT_NAMES, logical_operands, pad2

pytestmark = pytest.mark.gpu

OUT_OF_MEMORY = 2           # hipErrorOutOfMemory
STATIC_FLOATS = 8 << 20     # the limit the header states


def two_stage(gpu, variant, A, B, GZ, N, M, K, fill):
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC, dCbuf = gpu.DeviceArray(size=N * M), gpu.DeviceArray(size=N * M * max(GZ - 1, 1))
    dC.fill(fill)
    dCbuf.fill(fill)
    [MM.matMulSK, MM.matMulT1SK, MM.matMulT2SK][variant]([0], 1, GZ, dA.address, dB.address, dC.address,
                                                           dCbuf.address, N, M, K)
    MM.SKbuf_summary(0, dCbuf.address, dC.address, GZ - 1, N * M)
    Cuda.streamSynchronize(0)
    C = dC.get((N, M))
    for x in (dA, dB, dC, dCbuf):
        x.free()
    return C


def static_workspace(gpu, variant, A, B, GZ, N, M, K, fill):
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC = gpu.DeviceArray(size=N * M)
    dC.fill(fill)
    MM.matMulSK_static([0], 1, variant, GZ, dA.address, dB.address, dC.address, N, M, K)
    Cuda.streamSynchronize(0)
    C = dC.get((N, M))
    for x in (dA, dB, dC):
        x.free()
    return C


def padded_dims(variant, Ap, Bp):
    if variant == NN:
        (N, K), M = Ap.shape, Bp.shape[1]
    elif variant == T1:
        (K, N), M = Ap.shape, Bp.shape[1]
    else:
        (N, K), M = Ap.shape, Bp.shape[0]
    return N, M, K


@pytest.mark.parametrize("variant", [T1, NN, T2])
def test_two_calls_in_a_row_match_the_two_stage_entry_points_bitwise(gpu, variant):
    rng = np.random.default_rng(20 + variant)
    # the second call is smaller in every respect: fewer, shorter partials that overlay the first call's
    for (N, M, K), GZ in (((250, 132, 4100), 16), ((61, 40, 1000), 5)):
        A, B = logical_operands(variant, rng, N, M, K, dist="normal")
        Ap, Bp = pad2(A), pad2(B)
        N4, M4, K4 = padded_dims(variant, Ap, Bp)
        want = two_stage(gpu, variant, Ap, Bp, GZ, N4, M4, K4, fill=3.0)
        got = static_workspace(gpu, variant, Ap, Bp, GZ, N4, M4, K4, fill=-7.0)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), \
            "%s %dx%dx%d GridZ %d" % (VARIANT_NAMES[variant], N, M, K, GZ)


def test_the_largest_baseline_split_fits_and_one_slice_needs_no_workspace(gpu):
    # the tall-K weight gradient: 256 x 256, GridZ 128 -> 127 partials of 65536 floats, just inside
    # the limit; a K short enough to run here
    rng = np.random.default_rng(5)
    N = M = 256
    K, GZ = 8192, 128
    assert (GZ - 1) * N * M <= STATIC_FLOATS
    A = rng.standard_normal((K, N)).astype(np.float32)
    B = rng.standard_normal((K, M)).astype(np.float32)
    want = two_stage(gpu, T1, A, B, GZ, N, M, K, fill=1.0)
    got = static_workspace(gpu, T1, A, B, GZ, N, M, K, fill=2.0)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # GridZ = 1 is the plain product
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    dA, dB, dC, dD = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(size=N * M), gpu.DeviceArray(size=N * M)
    MM.matMulSK_static([0], 1, T1, 1, dA.address, dB.address, dC.address, N, M, K)
    MM.matMulT1([0], 1, dA.address, dB.address, dD.address, N, M, K)
    Cuda.streamSynchronize(0)
    assert np.array_equal(dC.get().view(np.uint32), dD.get().view(np.uint32))
    for x in (dA, dB, dC, dD):
        x.free()


def test_a_size_beyond_the_workspace_is_refused_and_nothing_runs(gpu, capfd):
    lib = gpu.lib
    s = (ctypes.c_int64 * 1)(0)
    N = M = 1024
    dA, dB, dC = gpu.DeviceArray(size=N * 64), gpu.DeviceArray(size=M * 64), gpu.DeviceArray(size=N * M)
    dC.fill(5.0)
    # 9 partials of 1 Mi floats > 8 Mi floats
    rc = lib.dragon_Cuda_matMul_matMulSK_static(s, 1, NN, 10, dA.address, dB.address, dC.address, N, M, 64)
    assert rc == OUT_OF_MEMORY
    assert "static workspace" in capfd.readouterr().err
    gpu.Cuda.streamSynchronize(0)
    assert np.all(dC.get() == 5.0)
    # 8 partials fit exactly
    assert lib.dragon_Cuda_matMul_matMulSK_static(s, 1, NN, 9, dA.address, dB.address, dC.address, N, M, 64) == 0
    gpu.Cuda.streamSynchronize(0)
    assert np.all(dC.get() == 0.0)
    for x in (dA, dB, dC):
        x.free()
