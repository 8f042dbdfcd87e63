"""Dimension swap (Cuda_expk2.transpose2D / 3D / 4D and Engine.transpose) on the GPU against the
oracle: pure data movement, so every comparison is bit for bit, pad included."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu


def dev_layout(X):
    s = (X.shape[-1] + 3) // 4 * 4
    out = np.zeros(X.shape[:-1] + (s,), np.float32)
    out[..., :X.shape[-1]] = X
    return out


def run_native(dh, X, i1, i2, poison=True):
    dims = list(X.shape)
    yd = list(dims)
    yd[i1], yd[i2] = yd[i2], yd[i1]
    Xp = dev_layout(X)
    sx, sy = Xp.shape[-1], (yd[-1] + 3) // 4 * 4
    ny = int(np.prod(yd[:-1])) * sy
    dX, dY = dh.DeviceArray(Xp), dh.DeviceArray(size=ny + 16)
    # the row-moving form copies X's zero pad; the tiled form writes Y's pad itself: poison both
    if poison:
        dY.fill(7.0)
    E = dh.Cuda_expk2
    n = X.size
    if len(dims) == 2:
        E.transpose2D(0, dX.address, dY.address, dims[1], yd[1], sx, sy, n)
    elif len(dims) == 3:
        E.transpose3D(0, dX.address, dY.address, dims[1], dims[2], yd[1], yd[2], i1, i2, sx, sy, n)
    else:
        E.transpose4D(0, dX.address, dY.address, dims[1], dims[2], dims[3], yd[1], yd[2], yd[3], i1, i2, sx,
                      sy, n)
    dh.Cuda.streamSynchronize(0)
    raw = dY.get()
    dX.free(), dY.free()
    assert np.all(raw[ny:] == (7.0 if poison else 0.0))        # nothing written past Y
    return raw[:ny].reshape(yd[:-1] + [sy])


CASES = [((1, 1), 0, 1), ((5, 7), 0, 1), ((7, 5), 1, 0), ((64, 64), 0, 1), ((257, 129), 0, 1), ((1000, 777), 0, 1),
         ((3, 1), 0, 1), ((1, 300), 0, 1),
         ((2, 3, 5), 0, 1), ((2, 3, 5), 1, 2), ((2, 3, 5), 0, 2), ((33, 257, 129), 1, 2), ((4, 100, 8), 2, 0),
         ((2, 3, 4, 6), 0, 1), ((2, 3, 4, 6), 1, 2), ((2, 3, 4, 6), 0, 2), ((2, 3, 4, 6), 2, 3), ((2, 3, 4, 6), 1, 3),
         ((2, 3, 4, 6), 0, 3), ((8, 128, 12, 64), 1, 2), ((8, 12, 128, 64), 2, 3), ((3, 70, 2, 65), 3, 1),
         # planes of many tiles, square and not: the diagonal tile order visits each tile once
         ((1024, 1024), 0, 1), ((2048, 1021), 0, 1), ((2, 1024, 2, 1024), 1, 3), ((1021, 3, 2048), 0, 2)]


@pytest.mark.parametrize("dims,i1,i2", CASES)
def test_native_transpose_matches_oracle_bitwise(dh, gpu, dims, i1, i2):
    X = np.random.default_rng(sum(dims) + i1 * 7 + i2).standard_normal(dims).astype(np.float32)
    Y = run_native(dh, X, i1, i2)
    R = oracle.transpose(dev_layout(X), dims, i1, i2)
    assert Y.shape == R.shape
    assert np.array_equal(Y.view(np.uint32), R.view(np.uint32))     # logical elements and zero pad


def test_transpose_argument_errors(dh, gpu):
    d = dh.DeviceArray(size=256)
    a = d.address
    E = dh.Cuda_expk2
    E.transpose2D(0, a, a + 512, 8, 4, 8, 4, 32)
    for call in (lambda: E.transpose2D(0, 0, a, 8, 4, 8, 4, 32), lambda: E.transpose2D(0, a, 0, 8, 4, 8, 4, 32),
                 lambda: E.transpose2D(0, a, a + 512, 8, 4, 8, 4, 30), lambda: E.transpose2D(0, a, a + 512, 8, 4, 6, 4, 32),
                 lambda: E.transpose2D(0, a, a + 512, 8, 4, 8, 3, 32), lambda: E.transpose2D(0, a + 4, a + 512, 8, 4, 8, 4, 32),
                 lambda: E.transpose3D(0, a, a + 512, 4, 4, 4, 4, 0, 3, 4, 4, 32),
                 lambda: E.transpose3D(0, a, a + 512, 4, 4, 4, 4, 0, 1, 4, 4, 32),      # Ydim1 must be 2 here
                 lambda: E.transpose4D(0, a, a + 512, 2, 2, 4, 2, 2, 4, 1, 1, 4, 4, 32)):
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


def test_engine_transpose(eg):
    from dragon_hip import engine
    rng = np.random.default_rng(8)
    base = eg.get_param("live_blocks")
    X = rng.standard_normal((6, 33, 5, 19)).astype(np.float32)
    tX = eg.tensor(X, 6, 33, 5, 19)
    for (i1, i2) in [(1, 2), (-1, -2), (0, 3), (2, 1), (1, -1)]:
        tY = eg.transpose(False, tX, i1, i2)
        R = np.swapaxes(X, i1, i2)
        assert tY.dim == list(R.shape)
        assert np.array_equal(eg.valueOf(tY).reshape(R.shape), R)
        eg.delete(tY)
    tC = eg.transpose(False, tX, 2, 2)                      # equal indices: a copy
    assert tC.address != tX.address and np.array_equal(eg.valueOf(tC), X.reshape(-1))
    assert eg.transpose(True, tX, 1, 1) is tX
    # in place: X takes the new shape and memory, the old block goes back
    old = tX.address
    assert eg.transpose(True, tX, 1, 3) is tX
    assert tX.dim == [6, 19, 5, 33] and tX.address != old
    assert np.array_equal(eg.valueOf(tX).reshape(6, 19, 5, 33), np.swapaxes(X, 1, 3))
    # attention-style use: Q.K^T through an explicit transpose equals the T2 product
    Q = rng.uniform(-1, 1, (4, 37, 20)).astype(np.float32)
    K = rng.uniform(-1, 1, (4, 29, 20)).astype(np.float32)
    tQ, tK = eg.tensor(Q, 4, 37, 20), eg.tensor(K, 4, 29, 20)
    tKt = eg.transpose(False, tK, 1, 2)
    S1, S2 = eg.batchMatMul(tQ, tKt), eg.batchMatMulT2(tQ, tK)
    ref = np.einsum("bik,bjk->bij", Q.astype(np.float64), K.astype(np.float64))
    for S in (S1, S2):
        got = eg.valueOf(S).reshape(4, 37, 29)
        assert np.linalg.norm(got - ref) <= 1e-5 * np.linalg.norm(ref)
    eg.delete(tX, tC, tQ, tK, tKt, S1, S2)
    assert eg.get_param("live_blocks") == base
    # checks
    t5 = eg.tensor(np.zeros(32, np.float32), 2, 2, 2, 2, 2)
    with pytest.raises(engine.IllegalArgumentException):
        eg.transpose(False, t5, 0, 1)
    t2 = eg.tensor(np.zeros(6, np.float32), 2, 3)
    with pytest.raises(engine.IllegalArgumentException):
        eg.transpose(False, t2, 0, 2)
    eg.delete(t5, t2)
