"""The streaming kernels (linear2D, linear_dual2D_row, softmax2D, the dimension swaps) on tensors whose footprint
-- the tensor, twice that where the result goes elsewhere -- reaches 320 MiB: from there on they read and write
with non-temporal accesses (csrc/stream_policy.h), a different instantiation of each kernel than every other test
runs.  Same oracles, same bars: bit for bit for the linear maps and the swaps, the softmax tolerance of
test_gpu_softmax.py."""
import numpy as np
import pytest

from oracle import oracle
from test_gpu_softmax import check_softmax

pytestmark = pytest.mark.gpu

ROWS, WIDTH, STRIDE = 41000, 1021, 1024          # 41000 x 1024 floats = 160.2 MiB: 320.3 MiB with a separate result


def tensor(seed, rows=ROWS):
    rng = np.random.default_rng(seed)
    Xp = np.zeros((rows, STRIDE), np.float32)
    Xp[:, :WIDTH] = rng.standard_normal((rows, WIDTH), dtype=np.float32)
    return Xp


def test_linear2D_large_out_of_place_and_in_place(dh, gpu):
    Xp = tensor(1)
    Xp[:, WIDTH:] = 5.0
    dX, dY = dh.DeviceArray(Xp), dh.DeviceArray(size=Xp.size)
    dh.Cuda_function.linear2D(0, 0.37, dX.address, -1.5, dY.address, Xp.size, WIDTH, STRIDE)
    dh.Cuda.streamSynchronize(0)
    assert np.array_equal(dY.get(Xp.shape).view(np.uint32), oracle.linear2D(0.37, Xp, -1.5, WIDTH).view(np.uint32))
    dX.free(), dY.free()
    big = np.concatenate([Xp, Xp[::-1]])             # 320.3 MiB in place
    dX = dh.DeviceArray(big)
    dh.Cuda_function.linear2D(0, -2.0, dX.address, 0.25, dX.address, big.size, WIDTH, STRIDE)
    dh.Cuda.streamSynchronize(0)
    assert np.array_equal(dX.get(big.shape).view(np.uint32), oracle.linear2D(-2.0, big, 0.25, WIDTH).view(np.uint32))
    dX.free()


def test_linear_dual2D_row_large(dh, gpu):
    X1 = tensor(2)
    X2 = np.zeros(STRIDE, np.float32)
    X2[:WIDTH] = np.random.default_rng(3).standard_normal(WIDTH, dtype=np.float32)
    d1, d2, dY = dh.DeviceArray(X1), dh.DeviceArray(X2), dh.DeviceArray(size=X1.size)
    dh.Cuda_function.linear_dual2D_row(0, d1.address, d2.address, STRIDE, 0.5, 2.0, 0.125, dY.address, X1.size, WIDTH, STRIDE)
    dh.Cuda.streamSynchronize(0)
    R = oracle.linear_dual2D_row(X1, X2, 0.5, 2.0, 0.125, WIDTH)
    assert np.array_equal(dY.get(X1.shape).view(np.uint32), R.view(np.uint32))
    d1.free(), d2.free(), dY.free()


def test_softmax2D_large(dh, gpu):
    Xp = tensor(4) * np.float32(4.0)
    Xp[:, WIDTH:] = 60.0                              # garbage in the pad must not take part
    dX, dY = dh.DeviceArray(Xp), dh.DeviceArray(size=Xp.size)
    dh.Cuda_reduce.softmax2D(0, dX.address, dY.address, ROWS, STRIDE, WIDTH, STRIDE, 1.0)
    dh.Cuda.streamSynchronize(0)
    Y = dY.get(Xp.shape)
    dX.free(), dY.free()
    for lo in range(0, ROWS, 8200):                   # (in slabs: the FP64 reference of the whole tensor is 1.3 GB)
        check_softmax(Y[lo:lo + 8200], Xp[lo:lo + 8200], WIDTH)


@pytest.mark.parametrize("dims,i1,i2", [((16, 2050, 20, 64), 1, 2), ((6500, 6460), 0, 1), ((10, 66, 1000, 64), 1, 3)])
def test_transpose_large(dh, gpu, dims, i1, i2):
    from test_gpu_transpose import dev_layout, run_native
    X = np.random.default_rng(sum(dims)).standard_normal(dims, dtype=np.float32)
    assert X.size * 8 >= 320 << 20
    Y = run_native(dh, X, i1, i2)
    R = oracle.transpose(dev_layout(X), dims, i1, i2)
    assert Y.shape == R.shape
    assert np.array_equal(Y.view(np.uint32), R.view(np.uint32))
