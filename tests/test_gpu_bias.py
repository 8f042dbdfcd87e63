"""The bias row of matMul_biased / fullconnect_biased on the GPU, through the C ABI.

Three layers, as in the reference: the native linear_dual2D_row against the oracle (bit-exact:
both evaluate alpha*x1 + beta*x2 + gamma with every operation rounded on its own), the fused
product+bias launch against the two separate launches it replaces (every bit equal, for every
tile shape), and the engine-level check the reference's own test makes
(alpha-Dragon-v1.2/test/test/cuda/matMul/Cuda_fullconect_test.java:23-50): fullconnect followed
by add_row must equal fullconnect_biased exactly.
"""
import numpy as np
import pytest

from oracle import oracle
from helpers import assert_within_tolerance, pad2

pytestmark = pytest.mark.gpu


def _row_case(rng, rows, width, garbage_pad=False):
    stride = (width + 3) // 4 * 4
    X1 = np.zeros((rows, stride), np.float32)
    X1[:, :width] = rng.standard_normal((rows, width)).astype(np.float32)
    if garbage_pad:
        X1[:, width:] = 3.5
    X2 = np.zeros(stride, np.float32)
    X2[:width] = rng.standard_normal(width).astype(np.float32)
    return X1, X2, stride


def _run_row(dh, X1, X2, alpha, beta, gamma, width, inplace):
    rows, stride = X1.shape
    d1, d2 = dh.DeviceArray(X1), dh.DeviceArray(X2)
    dy = d1 if inplace else dh.DeviceArray(size=X1.size)
    if not inplace:
        dy.fill(-7.0)
    dh.Cuda_function.linear_dual2D_row(0, d1.address, d2.address, stride, alpha, beta, gamma,
                                       dy.address, rows * stride, width, stride)
    dh.Cuda.streamSynchronize(0)
    Y = dy.get((rows, stride))
    d1.free(), d2.free()
    if not inplace:
        dy.free()
    return Y


# rows x width: tiny (under one workgroup), ragged widths, and more than 8192*512 floats, where the
# reference switches launch shapes
ROW_SHAPES = [(1, 1), (3, 7), (16, 4), (37, 50), (255, 129), (1000, 780), (2048, 2049)]


@pytest.mark.parametrize("rows,width", ROW_SHAPES)
@pytest.mark.parametrize("inplace", [False, True])
def test_bias_add_is_bit_exact(dh, gpu, rows, width, inplace):
    rng = np.random.default_rng(rows * 131 + width)
    X1, X2, _ = _row_case(rng, rows, width, garbage_pad=True)
    Y = _run_row(dh, X1, X2, 1.0, 1.0, 0.0, width, inplace)
    R = oracle.linear_dual2D_row(X1, X2, 1.0, 1.0, 0.0, width)
    assert np.array_equal(Y.view(np.uint32), R.view(np.uint32))
    assert not Y[:, width:].any()


def test_general_coefficients_match_the_oracle_bitwise(dh, gpu):
    rng = np.random.default_rng(77)
    X1, X2, _ = _row_case(rng, 300, 97)
    for (a, b, g) in [(0.37, -1.91, 0.123), (-2.0, 0.5, 0.0), (0.0, 1.0, -3.25)]:
        Y = _run_row(dh, X1, X2, a, b, g, 97, False)
        R = oracle.linear_dual2D_row(X1, X2, a, b, g, 97)
        assert np.array_equal(Y.view(np.uint32), R.view(np.uint32)), (a, b, g)


def test_row_vector_may_span_several_rows(dh, gpu):
    # row_lengthv a multiple of the stride: X2 holds a [3, stride] field repeated down X1
    rng = np.random.default_rng(5)
    stride, width, reps = 12, 10, 7
    X1 = np.zeros((3 * reps, stride), np.float32)
    X1[:, :width] = rng.standard_normal((3 * reps, width)).astype(np.float32)
    X2 = np.zeros((3, stride), np.float32)
    X2[:, :width] = rng.standard_normal((3, width)).astype(np.float32)
    d1, d2 = dh.DeviceArray(X1), dh.DeviceArray(X2)
    dy = dh.DeviceArray(size=X1.size)
    dh.Cuda_function.linear_dual2D_row(0, d1.address, d2.address, 3 * stride, 1.0, 1.0, 0.0,
                                       dy.address, X1.size, width, stride)
    dh.Cuda.streamSynchronize(0)
    Y = dy.get(X1.shape)
    assert np.array_equal(Y, X1 + np.tile(X2, (reps, 1)))
    for d in (d1, d2, dy):
        d.free()


def test_row_argument_errors(dh, gpu):
    d = dh.DeviceArray(size=64)
    ok = (0, d.address, d.address, 8, 1.0, 1.0, 0.0, d.address, 64, 8, 8)

    def call(**kw):
        names = ["stream", "X1", "X2", "row_lengthv", "alpha", "beta", "gamma", "Y", "lengthv", "width",
                 "stride"]
        args = dict(zip(names, ok))
        args.update(kw)
        dh.Cuda_function.linear_dual2D_row(*[args[n] for n in names])

    call()
    for bad in (dict(X1=0), dict(X2=0), dict(Y=0), dict(lengthv=0), dict(lengthv=62), dict(width=0),
                dict(width=9), dict(stride=6), dict(row_lengthv=12), dict(row_lengthv=24), dict(X1=d.address + 4)):
        with pytest.raises(dh.CudaException) as e:
            call(**bad)
        assert e.value.code == 1, bad
    dh.Cuda.streamSynchronize(0)
    d.free()


# ---- fused product + bias against the two launches it replaces ------------------------------------

def _biased_both_ways(dh, A, B, bias, tile):
    """Logical A[N,K], B[K,M], bias[M] -> (fused padded C, two-launch padded C)."""
    MM = dh.Cuda_matMul
    N, M = A.shape[0], B.shape[1]
    Ap, Bp = pad2(A), pad2(B)
    N4, K4, M4 = Ap.shape[0], Ap.shape[1], Bp.shape[1]
    bp = np.zeros(M4, np.float32)
    bp[:M] = bias
    dA, dB, db = dh.DeviceArray(Ap), dh.DeviceArray(Bp), dh.DeviceArray(bp)
    dC1, dC2 = dh.DeviceArray(size=N4 * M4), dh.DeviceArray(size=N4 * M4)
    dC1.fill(9.0), dC2.fill(9.0)
    lengthv = N * M4                     # C.lengthv: logical rows, padded row stride
    dh.force_tile(tile)
    try:
        MM.matMul_biased([0], 1, dA.address, dB.address, dC1.address, db.address, N4, M4, K4, lengthv, M)
        MM.matMul([0], 1, dA.address, dB.address, dC2.address, N4, M4, K4)
        dh.Cuda_function.linear_dual2D_row(0, dC2.address, db.address, M4, 1.0, 1.0, 0.0, dC2.address,
                                           lengthv, M, M4)
        dh.Cuda.streamSynchronize(0)
    finally:
        dh.force_tile(-1)
    C1, C2 = dC1.get((N4, M4)), dC2.get((N4, M4))
    for d in (dA, dB, db, dC1, dC2):
        d.free()
    return C1, C2


@pytest.mark.parametrize("tile", list(range(-1, 24)) + [25] + list(range(256, 266)))
def test_fused_bias_equals_two_launches_bitwise(dh, gpu, tile):
    rng = np.random.default_rng(1000 + tile)
    shapes = [(130, 203, 77), (1, 5, 300), (257, 64, 129)]
    if 18 <= tile < 24 or tile == 25:     # the balanced kernel: tiles whose sum is put together from several workgroups' pieces
        shapes += [(70, 130, 3001), (300, 260, 1030)]
    for (N, M, K) in shapes:
        A = rng.uniform(-1, 1, (N, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (K, M)).astype(np.float32)
        bias = rng.uniform(-2, 2, M).astype(np.float32)
        C1, C2 = _biased_both_ways(dh, A, B, bias, tile)
        assert np.array_equal(C1.view(np.uint32), C2.view(np.uint32)), (N, M, K, tile)
        # pad rows and columns of C are exact zeros: the bias is not added there
        assert not C1[N:].any() and not C1[:, M:].any()
        R = oracle.matmul(0, A, B)
        Rb = oracle.linear_dual2D_row(pad2(R)[:N], np.pad(bias, (0, C1.shape[1] - M)), 1.0, 1.0, 0.0, M)
        assert_within_tolerance(C1[:N, :M] - bias[None, :], R, K, A, B, "fused bias, tile %d" % tile)
        assert np.abs(C1[:N, :M] - Rb[:, :M]).max() <= 1e-4 * np.sqrt(K) + 1e-6


def test_fused_bias_on_skinny_products(dh, gpu):
    """A C of at most 8 rows or columns goes through the skinny kernel, whose epilogue adds the bias row like the
    tile kernels' does: the bits of the product followed by linear_dual2D_row, pads left at zero."""
    rng = np.random.default_rng(91)
    for (N, M, K) in ((8, 5000, 516), (5000, 8, 516), (3, 4097, 100), (4100, 5, 2052), (8, 4096, 4096)):
        assert dh.choose_tile(0, (N + 3) // 4 * 4, (M + 3) // 4 * 4, 1, (K + 3) // 4 * 4) == 27
        A = rng.integers(-3, 4, (N, K)).astype(np.float32)
        B = rng.integers(-3, 4, (K, M)).astype(np.float32)
        bias = rng.integers(-5, 6, M).astype(np.float32)
        C1, C2 = _biased_both_ways(dh, A, B, bias, -1)
        assert np.array_equal(C1.view(np.uint32), C2.view(np.uint32)), (N, M, K)
        assert np.array_equal(C1[:N, :M], oracle.matmul_f64(0, A, B).astype(np.float32) + bias[None, :])
        assert not C1[N:].any() and not C1[:, M:].any()
    # a sum of -0 and a bias of +0: the gamma term of the separate launch turns it into +0 in both
    A = np.zeros((8, 512), np.float32); A[:, 0] = -1.0
    B = np.zeros((512, 300), np.float32)
    C1, C2 = _biased_both_ways(dh, A, B, np.zeros(300, np.float32), -1)
    assert np.array_equal(C1.view(np.uint32), C2.view(np.uint32))


def test_fused_bias_through_two_launches_of_the_balanced_kernel(dh, gpu):
    """640 tiles of 128 x 128 for 256 compute units: whole tiles first, the remaining 128 in a second launch; the
    bias row is added once, by whoever stores a tile, in both."""
    rng = np.random.default_rng(77)
    N, M, K = 2000, 5000, 3100
    A = rng.integers(-3, 4, (N, K)).astype(np.float32)
    B = rng.integers(-3, 4, (K, M)).astype(np.float32)
    bias = rng.integers(-5, 6, M).astype(np.float32)
    C1, C2 = _biased_both_ways(dh, A, B, bias, -1)
    assert np.array_equal(C1.view(np.uint32), C2.view(np.uint32))
    assert np.array_equal(C1[:N, :M], oracle.matmul_f64(0, A, B).astype(np.float32) + bias[None, :])
    assert not C1[N:].any() and not C1[:, M:].any()


def test_fused_bias_large_and_negative_zero(dh, gpu):
    rng = np.random.default_rng(3)
    N, M, K = 1000, 780, 256
    A = rng.standard_normal((N, K)).astype(np.float32)
    B = rng.standard_normal((K, M)).astype(np.float32)
    bias = rng.standard_normal(M).astype(np.float32)
    A[5] = 0.0                      # a row of exact zeros in C ...
    bias[7] = -0.0                  # ... meets a negative-zero bias: both paths must give +0
    C1, C2 = _biased_both_ways(dh, A, B, bias, -1)
    assert np.array_equal(C1.view(np.uint32), C2.view(np.uint32))
    assert C1[5, 7] == 0 and not np.signbit(C1[5, 7])


def test_fused_bias_argument_errors(dh, gpu):
    d, dc = dh.DeviceArray(size=64), dh.DeviceArray(size=64)
    a, c = d.address, dc.address
    MM = dh.Cuda_matMul
    MM.matMul_biased([0], 1, a, a, c, a, 8, 8, 8, 64, 8)
    for bad in (dict(dBias=0), dict(lengthv=60), dict(lengthv=72), dict(width=0), dict(width=9),
                dict(lengthv=0), dict(dBias=a + 4)):
        args = dict(dBias=a, lengthv=64, width=8)
        args.update(bad)
        with pytest.raises(dh.CudaException) as e:
            MM.matMul_biased([0], 1, a, a, c, args["dBias"], 8, 8, 8, args["lengthv"], args["width"])
        assert e.value.code == 1, bad
    dh.Cuda.streamSynchronize(0)
    d.free(), dc.free()


# ---- engine level -----------------------------------------------------------------------------------

@pytest.fixture(scope="module", params=["direct", "pooled"])
def eg(gpu, request):
    """With and without the recycling device memory pool behind the tensors (recycled blocks are dirty)."""
    from dragon_hip import engine
    e = engine.cuda_float32(0, 32, max_mem_size=(2 << 30) if request.param == "pooled" else 0)
    yield e
    e.close()


def check_fullconnect(eg, rng, dimX, IW, OW):   # testCorrect(ih, iw, ...) of Cuda_fullconect_test
    n = int(np.prod(dimX))
    X = rng.random(n * IW, dtype=np.float32)
    W = rng.random(IW * OW, dtype=np.float32)
    Bv = rng.random(OW, dtype=np.float32)
    tX, tW, tB = eg.tensor(X, *dimX, IW), eg.tensor(W, IW, OW), eg.tensor(Bv, OW)
    tY1 = eg.fullconnect(tX, tW)
    tY1 = eg.add_row(True, tY1, tB)
    tY2 = eg.fullconnect_biased(tX, tW, tB)
    assert tY2.dim == list(dimX) + [OW]
    Y1, Y2 = eg.valueOf(tY1), eg.valueOf(tY2)
    assert np.array_equal(Y1, Y2), (dimX, IW, OW)          # samePercent_absolute == 1 in the reference
    R = oracle.matmul(0, X.reshape(n, IW), W.reshape(IW, OW)) + Bv[None, :]
    assert oracle.samePercent_relative(R.reshape(-1), Y2) >= 0.999
    # the pad of Y stays zero (rows beyond the logical count, columns beyond OW)
    raw = np.empty(tY2.length_4x, np.float32)
    from dragon_hip import Cuda
    Cuda.get1D(0, tY2.address, raw, tY2.length_4x)
    OW4 = (OW + 3) // 4 * 4
    raw = raw.reshape(-1, OW4)
    assert not raw[:, OW:].any() and not raw[n:].any()
    eg.delete(tX, tW, tB, tY1, tY2)


@pytest.mark.parametrize("fused", [1, 0])
def test_fullconnect_biased_like_the_reference(eg, fused):
    rng = np.random.default_rng(11)
    base = eg.get_param("live_blocks")
    eg.set_param("matMul_biased_fused", fused)
    try:
        for (dimX, IW, OW) in [((4,), 1, 1), ((4, 7), 33, 17), ((3, 5, 2), 64, 129), ((2, 128), 128, 100),
                               ((37,), 300, 5), ((2, 3), 1532, 780)]:
            check_fullconnect(eg, rng, dimX, IW, OW)
    finally:
        eg.set_param("matMul_biased_fused", 1)
    assert eg.get_param("live_blocks") == base


def test_matMul_biased_split_k_path(eg):
    # 1000 x 780 x 1532 splits in two on 256 units: product, Kahan fold, then the bias row
    rng = np.random.default_rng(12)
    N, M, K = 1000, 780, 1532
    A = rng.uniform(-1, 1, (N, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, M)).astype(np.float32)
    bias = rng.uniform(-1, 1, M).astype(np.float32)
    tA, tB, tb = eg.tensor(A, N, K), eg.tensor(B, K, M), eg.tensor(bias, M)
    assert eg.gridZ(3, 1000, 780, 1532) == oracle.gridZ(oracle.MATMUL_BIASED, 1000, 780, 1532,
                                                        eg.get_param("multiProcessorCount"))
    tC = eg.matMul_biased(tA, tB, tb)
    gz = eg.get_param("last_gridZ")
    assert gz == eg.gridZ(3, 1000, 780, 1532)
    tC2 = eg.matMul_biased(eg.empty(N, M).c(), tA, tB, tb)
    tD = eg.add_row(True, eg.matMul(tA, tB), tb)
    C, C2, D = (eg.valueOf(t).reshape(N, M) for t in (tC, tC2, tD))
    assert np.array_equal(C, C2)
    if gz == eg.gridZ(0, 1000, 780, 1532):      # same slices -> the same bits as product + add_row
        assert np.array_equal(C, D)
    R = oracle.matmul(0, A, B)
    assert_within_tolerance(C - bias[None, :], R, K, A, B, "matMul_biased split-K")
    eg.delete(tA, tB, tb, tC, tC2, tD)


def test_fullconnect_backward_products(eg):
    rng = np.random.default_rng(13)
    dimX, IW, OW = (3, 10), 70, 45
    n = 30
    X = rng.uniform(-1, 1, (n, IW)).astype(np.float32)
    W = rng.uniform(-1, 1, (IW, OW)).astype(np.float32)
    dY = rng.uniform(-1, 1, (n, OW)).astype(np.float32)
    tX, tW, tdY = eg.tensor(X, *dimX, IW), eg.tensor(W, IW, OW), eg.tensor(dY, *dimX, OW)
    tdX = eg.fullconnect_deltaX(tdY, tW)
    tdW = eg.fullconnect_deltaW(tX, tdY)
    assert tdX.dim == [3, 10, IW] and tdW.dim == [IW, OW]
    assert_within_tolerance(eg.valueOf(tdX).reshape(n, IW), oracle.matmul(2, dY, W), OW, dY, W, "deltaX")
    assert_within_tolerance(eg.valueOf(tdW).reshape(IW, OW), oracle.matmul(1, X, dY), n, X, dY, "deltaW")
    tY = eg.fullconnect(eg.empty(3, 10, OW).c(), tX, tW)
    assert_within_tolerance(eg.valueOf(tY).reshape(n, OW), oracle.matmul(0, X, W), IW, X, W, "fullconnect into")
    eg.delete(tX, tW, tdY, tdX, tdW, tY)


def test_bias_argument_checks(eg):
    from dragon_hip import engine
    tA = eg.tensor(np.ones(12, np.float32), 3, 4)
    tB = eg.tensor(np.ones(20, np.float32), 4, 5)
    tb_bad = eg.tensor(np.ones(4, np.float32), 4)
    tb = eg.tensor(np.ones(5, np.float32), 5)
    with pytest.raises(engine.IllegalArgumentException):
        eg.matMul_biased(tA, tB, tb_bad)
    with pytest.raises(engine.NullPointerException):
        eg.matMul_biased(tA, tB, None)
    with pytest.raises(engine.IllegalArgumentException):
        eg.add_row(False, tA, tb)                         # lastDim 4 != 5
    tC = eg.matMul_biased(tA, tB, tb)
    assert np.array_equal(eg.valueOf(tC), np.full(15, 5.0, np.float32))
    tD = eg.linear2_row(False, tC, tb, 2.0, -1.0, 0.5)
    assert np.array_equal(eg.valueOf(tD), np.full(15, 9.5, np.float32))
    eg.delete(tA, tB, tb_bad, tb, tC, tD)
