"""The steps between the two batched products of an attention block on the GPU: linear2D (sdiv),
the one-launch row softmax, and the whole chain through the engine mirror as the reference's
ChannelMHA runs it (nn/unit/complex/block/ChannelMHA.java:66-83).

Softmax tolerance, per element: against the FP64 softmax |y - r| <= 2^-24 * (|x - max| + 8) * r (the
subtraction x - max is rounded to float, the exponential lies within an ulp, the row sum and the
division add a few more); against the oracle |y - o| <= (2e-6 + 2^-24 * n) * o for rows of n terms:
the oracle sums the row left to right in float, whose guaranteed error grows with n, while the
device sums it pairwise (the FP64 bound is the tight one).  Rows must sum to 1 within 2e-6."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu
ABS = 1e-37


def rel_vs_oracle(n):
    return 2e-6 + 2.0 ** -24 * n


def check_softmax(Y, Xp, width, features=None, scale=1.0):
    """Y against the oracle and against the FP64 softmax of the same input."""
    rows, stride = Xp.shape
    features = width if features is None else features
    R = oracle.softmax2D(Xp, width, features=features, scale=scale)
    assert np.isfinite(Y).all()
    assert np.all(np.abs(Y - R) <= rel_vs_oracle(features) * R + ABS), np.abs(Y - R).max()
    assert not Y[:, width:].any()
    x = (Xp[:, :width].astype(np.float32) * np.float32(scale)).astype(np.float64).reshape(-1, features)
    d = x.max(1, keepdims=True) - x
    e = np.exp(-d)
    r = e / e.sum(1, keepdims=True)
    y = Y[:, :width].astype(np.float64).reshape(-1, features)
    assert np.all(np.abs(y - r) <= 2.0 ** -24 * (d + 8) * r + ABS), (np.abs(y - r) / (r + 1e-300)).max()
    assert np.abs(y.sum(1) - 1).max() <= 2e-6


def dev_layout(X):
    s = (X.shape[-1] + 3) // 4 * 4
    out = np.zeros(X.shape[:-1] + (s,), np.float32)
    out[..., :X.shape[-1]] = X
    return out


def run_softmax(dh, Xp, width, features=None, scale=1.0, inplace=False):
    rows, stride = Xp.shape
    features = width if features is None else features
    row_lengthv = features // width * stride
    dX = dh.DeviceArray(Xp)
    dY = dX if inplace else dh.DeviceArray(size=Xp.size)
    if not inplace:
        dY.fill(7.0)
    dh.Cuda_reduce.softmax2D(0, dX.address, dY.address, Xp.size // row_lengthv, row_lengthv, width, stride, scale)
    dh.Cuda.streamSynchronize(0)
    Y = dY.get(Xp.shape)
    dX.free()
    if not inplace:
        dY.free()
    return Y


# rows x width: every register-resident size class (256 .. 4096 floats per field), ragged widths,
# one column, and fields longer than a wavefront holds (two-pass kernel)
SOFTMAX_SHAPES = [(5, 1), (7, 3), (64, 64), (33, 129), (10, 256), (9, 300), (12, 777), (6, 1024), (5, 2047),
                  (3, 4096), (4, 4100), (2, 20000)]


@pytest.mark.parametrize("rows,width", SOFTMAX_SHAPES)
@pytest.mark.parametrize("inplace", [False, True])
def test_softmax_matches_oracle(dh, gpu, rows, width, inplace):
    rng = np.random.default_rng(rows * 31 + width)
    Xp = dev_layout((rng.standard_normal((rows, width)) * 4).astype(np.float32))
    Xp[:, width:] = 60.0                                     # garbage in the pad must not take part
    Y = run_softmax(dh, Xp, width, inplace=inplace)
    check_softmax(Y, Xp, width)


def test_softmax_exact_cases_scale_and_multi_row_fields(dh, gpu):
    U = np.full((3, 8), 2.5, np.float32)
    assert np.array_equal(run_softmax(dh, U, 8), np.full((3, 8), 0.125, np.float32))
    D = np.zeros((1, 4), np.float32); D[0, :3] = [0.0, 200.0, -5.0]
    assert np.array_equal(run_softmax(dh, D, 3)[0, :3], np.array([0.0, 1.0, 0.0], np.float32))
    big = np.zeros((2, 4), np.float32); big[:, :3] = [[3e38, 3e38, -3e38], [-3e38, -3e38, -3e38]]
    Yb = run_softmax(dh, big, 3)                            # extreme magnitudes stay finite
    assert np.array_equal(Yb[0, :3], np.array([0.5, 0.5, 0.0], np.float32))
    assert np.allclose(Yb[1, :3], 1 / 3, rtol=1e-6)
    rng = np.random.default_rng(1)
    Xp = dev_layout(rng.standard_normal((24, 50)).astype(np.float32))
    for scale in (0.125, 1 / np.sqrt(64.0), 3.0):
        check_softmax(run_softmax(dh, Xp, 50, scale=scale), Xp, 50, scale=scale)
    for features in (100, 150, 50 * 24):                    # fields of 2, 3 and all 24 memory rows
        check_softmax(run_softmax(dh, Xp, 50, features=features), Xp, 50, features=features)


def test_linear2D_is_bit_exact(dh, gpu):
    rng = np.random.default_rng(2)
    for (rows, width) in [(1, 1), (9, 7), (300, 97), (2048, 2049)]:
        Xp = dev_layout(rng.standard_normal((rows, width)).astype(np.float32))
        Xp[:, width:] = 5.0
        for (a, b) in [(1 / 8.0, 0.0), (0.37, -1.5), (-2.0, 0.25)]:
            dX = dh.DeviceArray(Xp); dY = dh.DeviceArray(size=Xp.size)
            dh.Cuda_function.linear2D(0, a, dX.address, b, dY.address, Xp.size, width, Xp.shape[1])
            dh.Cuda.streamSynchronize(0)
            Y = dY.get(Xp.shape)
            R = oracle.linear2D(a, Xp, b, width)
            assert np.array_equal(Y.view(np.uint32), R.view(np.uint32)), (rows, width, a, b)
            dX.free(), dY.free()


def test_argument_errors(dh, gpu):
    d = dh.DeviceArray(size=64)
    a = d.address
    R, F = dh.Cuda_reduce, dh.Cuda_function
    R.softmax2D(0, a, a, 8, 8, 7, 8, 1.0)
    F.linear2D(0, 1.0, a, 0.0, a, 64, 7, 8)
    for call in (lambda: R.softmax2D(0, 0, a, 8, 8, 7, 8), lambda: R.softmax2D(0, a, 0, 8, 8, 7, 8),
                 lambda: R.softmax2D(0, a, a, 0, 8, 7, 8), lambda: R.softmax2D(0, a, a, 8, 12, 7, 8),
                 lambda: R.softmax2D(0, a, a, 8, 8, 9, 8), lambda: R.softmax2D(0, a, a, 8, 8, 0, 8),
                 lambda: R.softmax2D(0, a, a, 8, 6, 5, 6), lambda: R.softmax2D(0, a + 4, a, 8, 8, 7, 8),
                 lambda: F.linear2D(0, 1.0, 0, 0.0, a, 64, 7, 8), lambda: F.linear2D(0, 1.0, a, 0.0, a, 62, 7, 8),
                 lambda: F.linear2D(0, 1.0, a, 0.0, a, 64, 9, 8), lambda: F.linear2D(0, 1.0, a, 0.0, a, 60, 7, 8)):
        with pytest.raises(dh.CudaException) as e:
            call()
        assert e.value.code == 1
    dh.Cuda.streamSynchronize(0)
    d.free()


@pytest.fixture(scope="module", params=["direct", "pooled"])
def eg(gpu, request):
    """With and without the recycling device memory pool behind the tensors (recycled blocks are dirty)."""
    from dragon_hip import engine
    e = engine.cuda_float32(0, 8, max_mem_size=(2 << 30) if request.param == "pooled" else 0)
    yield e
    e.close()


def test_engine_softmax_and_sdiv(eg):
    from dragon_hip import engine
    rng = np.random.default_rng(3)
    X = rng.standard_normal((4, 6, 33)).astype(np.float32)
    tX = eg.tensor(X, 4, 6, 33)
    e = np.exp(X.astype(np.float64)); R = e / e.sum(-1, keepdims=True)
    tY = eg.softmax(False, tX)
    assert np.allclose(eg.valueOf(tY).reshape(X.shape), R, rtol=5e-6, atol=0)
    tZ = eg.softmax(False, tX, features=6 * 33)              # over the last two dimensions together
    e2 = e.reshape(4, -1); R2 = (e2 / e2.sum(1, keepdims=True)).reshape(X.shape)
    assert np.allclose(eg.valueOf(tZ).reshape(X.shape), R2, rtol=5e-6, atol=0)
    tD = eg.sdiv(False, tX, 8.0)
    assert np.array_equal(eg.valueOf(tD).reshape(X.shape), X / np.float32(8.0))
    tS = eg.softmax(False, tX, scale=0.125)                  # softmax(sdiv(X, 8)) in one launch
    tS2 = eg.softmax(True, tD)
    assert tS2 is tD
    assert np.allclose(eg.valueOf(tS), eg.valueOf(tS2), rtol=1e-6, atol=0)
    with pytest.raises(engine.IllegalArgumentException):
        eg.softmax(False, tX, features=7)
    eg.delete(tX, tY, tZ, tD, tS)


def test_attention_chain_like_the_reference_block(eg):
    # ChannelMHA.java:66-83: view [N, L, head, d], transpose(1, 2), P = softmax(sdiv(sqrt(KC), Q.K^T)),
    # Y = P.V, transpose back
    rng = np.random.default_rng(4)
    N, QL, VL, head, d = 2, 37, 29, 4, 20
    KC = head * d
    Q = rng.uniform(-1, 1, (N, QL, head, d)).astype(np.float32)
    K = rng.uniform(-1, 1, (N, VL, head, d)).astype(np.float32)
    V = rng.uniform(-1, 1, (N, VL, head, d)).astype(np.float32)
    base = eg.get_param("live_blocks")
    tQ, tK, tV = (eg.tensor(x, *x.shape) for x in (Q, K, V))
    tQt, tKt, tVt = (eg.transpose(False, t, 1, 2) for t in (tQ, tK, tV))     # [N, head, L, d]
    tP = eg.batchMatMulT2(tQt, tKt)                                          # [N, head, QL, VL]
    assert tP.dim == [N, head, QL, VL]
    tP1 = eg.softmax(False, eg.sdiv(False, tP, float(np.sqrt(KC))))
    tP2 = eg.softmax(False, tP, scale=float(1 / np.sqrt(KC)))                # the same in one launch
    outs = []
    for P in (tP1, tP2):
        tY = eg.transpose(True, eg.batchMatMul(P, tVt), 1, 2)                # [N, QL, head, d]
        assert tY.dim == [N, QL, head, d]
        outs.append(eg.valueOf(tY).reshape(N, QL, head, d))
        eg.delete(tY)
    S = np.einsum("nqhd,nkhd->nhqk", Q.astype(np.float64), K.astype(np.float64)) / np.sqrt(KC)
    Pm = np.exp(S - S.max(-1, keepdims=True)); Pm /= Pm.sum(-1, keepdims=True)
    ref = np.einsum("nhqk,nkhd->nqhd", Pm, V.astype(np.float64))
    for got in outs:
        assert np.linalg.norm(got - ref) <= 1e-5 * np.linalg.norm(ref)
    assert np.abs(outs[0] - outs[1]).max() <= 1e-6
    eg.delete(tQ, tK, tV, tQt, tKt, tVt, tP, tP1, tP2)
    assert eg.get_param("live_blocks") <= base + 1            # the sdiv temporary was not kept by the test
