"""Tensor upload / download through a pinned staging buffer (the _v2 natives and the engine's
PinnedMempool): the device reads or writes the packed host data in place, chunk by chunk.
Data movement only, so every comparison is bit for bit; the pageable-buffer route (the
reference's own: CPU re-layout, one copy) is the cross-check."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# height x width: stride == width, one float, one row, ragged widths, a total that is not a
# multiple of 4, and sizes beyond one 2 Mi-float chunk (3 and 5 chunks)
SHAPES = [(7, 8), (1, 1), (1, 13), (13, 1), (2, 5), (3, 7), (50, 777), (257, 129), (3000, 1501), (9001, 1023)]


def _raw(Cuda, d, n):
    out = np.empty(n, np.float32)
    Cuda.get1D(0, d, out, n)
    return out


@pytest.mark.parametrize("h,w", SHAPES)
def test_2d_round_trip_through_pinned_buffer(gpu, h, w):
    Cuda = gpu.Cuda
    s = (w + 3) // 4 * 4
    X = np.random.default_rng(h * 7 + w).standard_normal((h, w)).astype(np.float32)
    d = Cuda.malloc(h * s * 4 + 64)
    buf = Cuda.mallocHost(h * s * 4)
    try:
        Cuda.set1D(0, d, 9.0, h * s + 16)              # poison, pad and a guard zone included
        Cuda.set2D_v2(0, d, X, buf, h, w, s)
        raw = _raw(Cuda, d, h * s + 16)
        assert np.all(raw[h * s:] == 9.0)              # nothing written past the tensor
        raw = raw[:h * s].reshape(h, s)
        assert np.array_equal(raw[:, :w].view(np.uint32), X.view(np.uint32))
        assert not raw[:, w:].any()                    # the device zeroed the pad
        back = np.full((h, w), -1.0, np.float32)
        Cuda.get2D_v2(0, d, back, buf, h, w, s)
        assert np.array_equal(back.view(np.uint32), X.view(np.uint32))
        # the same through a pageable staging buffer (CPU re-layout route) gives the same device bytes
        stage = np.empty(h * s, np.float32)
        Cuda.set1D(0, d, 9.0, h * s)
        Cuda.set2D_v2(0, d, X, stage.ctypes.data, h, w, s)
        assert np.array_equal(_raw(Cuda, d, h * s).reshape(h, s), raw)
        back2 = np.empty((h, w), np.float32)
        Cuda.get2D_v2(0, d, back2, stage.ctypes.data, h, w, s)
        assert np.array_equal(back2, X)
    finally:
        Cuda.free(d)
        Cuda.freeHost(buf)


@pytest.mark.parametrize("n", [1, 5, 4096, (2 << 20) + 3, 5 * (2 << 20)])
def test_1d_round_trip_through_pinned_buffer(gpu, n):
    Cuda = gpu.Cuda
    X = np.random.default_rng(n % 1000).standard_normal(n).astype(np.float32)
    d = Cuda.malloc(n * 4 + 64)
    buf = Cuda.mallocHost(n * 4)
    try:
        Cuda.set1D_v2(0, d, X, buf, n)
        assert np.array_equal(_raw(Cuda, d, n), X)
        back = np.empty(n, np.float32)
        Cuda.get1D_v2(0, d, back, buf, n)
        assert np.array_equal(back, X)
    finally:
        Cuda.free(d)
        Cuda.freeHost(buf)


def test_transfer_argument_errors(gpu):
    Cuda = gpu.Cuda
    d = Cuda.malloc(1024)
    buf = Cuda.mallocHost(1024)
    x = np.zeros(64, np.float32)
    for call in (lambda: Cuda.set2D_v2(0, d, x, 0, 4, 3, 4), lambda: Cuda.get2D_v2(0, d, x, 0, 4, 3, 4),
                 lambda: Cuda.set2D_v2(0, 0, x, buf, 4, 3, 4), lambda: Cuda.set2D_v2(0, d, x, buf, 4, 5, 4),
                 lambda: Cuda.set2D_v2(0, d, x, buf, 0, 3, 4), lambda: Cuda.set1D_v2(0, d, x, 0, 8),
                 lambda: Cuda.get1D_v2(0, d, x, buf, 0)):
        with pytest.raises(gpu.CudaException) as e:
            call()
        assert e.value.code == 1
    Cuda.set2D_v2(0, d, x, buf, 4, 3, 4)               # still works after the refusals
    Cuda.free(d)
    Cuda.freeHost(buf)


def test_engine_with_staging_pool(gpu):
    from dragon_hip import engine
    eg = engine.cuda_float32(0, 8, max_trans_buf_size=64 << 20)
    try:
        assert eg.get_param("buf_physical_blocks") == 0
        rng = np.random.default_rng(4)
        X = rng.standard_normal((300, 1001)).astype(np.float32)
        t = eg.tensor(X, 300, 1001)
        assert np.array_equal(eg.valueOf(t).reshape(300, 1001), X)
        # one pinned block serves upload and download of the same size, and is back in the pool
        assert eg.get_param("buf_physical_blocks") == 1
        assert eg.get_param("buf_buffered_blocks") == 1 and eg.get_param("buf_used_mem_size") == 0
        for _ in range(3):
            u = eg.tensor(X, 300, 1001)
            assert np.array_equal(eg.valueOf(u).reshape(300, 1001), X)
            eg.delete(u)
        assert eg.get_param("buf_physical_blocks") == 1
        # a request outside [size, 1.5*size] of every free block allocates a new one
        v = eg.tensor(np.ones(64, np.float32), 64)        # 1-D: the linear route
        assert np.array_equal(eg.valueOf(v), np.ones(64, np.float32))
        assert eg.get_param("buf_physical_blocks") == 2
        # products see the uploaded layout: a ragged product through the pooled transfers
        A = rng.uniform(-1, 1, (33, 45)).astype(np.float32)
        B = rng.uniform(-1, 1, (45, 29)).astype(np.float32)
        tA, tB = eg.tensor(A, 33, 45), eg.tensor(B, 45, 29)
        C = eg.valueOf(eg.matMul(tA, tB)).reshape(33, 29)
        assert np.linalg.norm(C - A.astype(np.float64) @ B) <= 1e-5 * np.linalg.norm(A.astype(np.float64) @ B)
        # beyond the budget the pool refuses (the Java pool would wait 10 s first)
        with pytest.raises(Exception):
            eg.tensor(np.zeros(20 << 20, np.float32), 4096, 5120)   # 80 MiB > 64 MiB
        eg.delete(t, v, tA, tB)
    finally:
        eg.close()
