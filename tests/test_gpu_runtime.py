"""Behaviour of the runtime bridge on the GPU: allocation, fills, strided transfer,
streams and events."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_device_reports_compute_units(gpu):
    assert gpu.Cuda.getDeviceCount() >= 1
    assert gpu.Cuda.getDeviceId() == 0
    assert gpu.Cuda.multiProcessorCount(0) >= 64


def test_malloc_memset_copy_free_round_trip(gpu):
    Cuda = gpu.Cuda
    n = 1 << 16
    a = Cuda.malloc(n * 4)
    b = Cuda.malloc(n * 4)
    assert a and b and a % 256 == 0
    host = np.arange(n, dtype=np.float32)
    Cuda.set1D(0, a, host, n)
    Cuda.memcpyAsyncDeviceToDevice(0, b, a, n * 4)
    Cuda.memsetAsync(0, a, 0, n * 4)
    out_a, out_b = np.empty(n, np.float32), np.empty(n, np.float32)
    Cuda.get1D(0, a, out_a, n)
    Cuda.get1D(0, b, out_b, n)
    assert not out_a.any() and np.array_equal(out_b, host)
    Cuda.set1D(0, a, 2.5, n)
    Cuda.get1D(0, a, out_a, n)
    assert np.all(out_a == 2.5)
    Cuda.free(a)
    Cuda.free(b)
    with pytest.raises(gpu.CudaException):
        Cuda.malloc(-1)


def test_strided_2d_transfer_round_trip(gpu):
    # width 777 in rows of stride 780: upload writes zeros into the pad, download drops it
    Cuda = gpu.Cuda
    h, w, s = 50, 777, 780
    X = np.random.default_rng(0).uniform(-1, 1, (h, w)).astype(np.float32)
    d = Cuda.malloc(h * s * 4)
    Cuda.set1D(0, d, 9.0, h * s)                      # poison, pad included
    Cuda.set2D(0, d, X, h, w, s)
    raw = np.empty(h * s, np.float32)
    Cuda.get1D(0, d, raw, h * s)
    raw = raw.reshape(h, s)
    assert np.array_equal(raw[:, :w], X) and not raw[:, w:].any()
    back = np.empty((h, w), np.float32)
    Cuda.get2D(0, d, back, h, w, s)
    assert np.array_equal(back, X)
    # constant fill of the logical width zeroes the pad as well
    Cuda.set1D(0, d, 9.0, h * s)
    Cuda.set2D(0, d, 1.5, h, w, s)
    Cuda.get1D(0, d, raw.reshape(-1), h * s)
    assert np.all(raw[:, :w] == 1.5) and not raw[:, w:].any()
    # pinned staging variants
    buf = Cuda.mallocHost(h * s * 4)
    assert gpu.lib.dragon_Cuda_set2D_v2(0, d, X.ctypes.data, buf, h, w, s) == 0
    back[:] = 0
    assert gpu.lib.dragon_Cuda_get2D_v2(0, d, back.ctypes.data, buf, h, w, s) == 0
    assert np.array_equal(back, X)
    Cuda.freeHost(buf)
    Cuda.free(d)


def test_events_order_work_across_streams(gpu):
    Cuda, MM = gpu.Cuda, gpu.Cuda_matMul
    s1, s2 = Cuda.newStream_Blocking(), Cuda.newStream_NonBlocking()
    n = 2048
    rng = np.random.default_rng(1)
    A = rng.integers(-2, 3, (n, n)).astype(np.float32)
    dA, dC, dD = gpu.DeviceArray(A), gpu.DeviceArray(size=n * n), gpu.DeviceArray(size=n * n)
    e0, e1 = Cuda.newEvent_Default(), Cuda.newEvent_Default()
    Cuda.eventRecord(e0, s1)
    MM.matMul([s1], 1, dA.address, dA.address, dC.address, n, n, n)      # on s1
    Cuda.eventRecord(e1, s1)
    Cuda.streamWaitEvent_default(s2, e1)
    Cuda.memcpyAsyncDeviceToDevice(s2, dD.address, dC.address, n * n * 4)  # on s2, after e1
    Cuda.streamSynchronize(s2)
    assert Cuda.streamQuery(s1) and Cuda.streamQuery(s2)
    exact = (A.astype(np.float64) @ A.astype(np.float64)).astype(np.float32)   # small integers: exact
    assert np.array_equal(dD.get((n, n)), exact)
    assert Cuda.eventElapsedTime(e0, e1) > 0
    # array form: the event completes after the work of every stream in the array
    done = Cuda.newEvent_DisableTiming()
    MM.matMul([s2], 1, dA.address, dA.address, dC.address, n, n, n)
    Cuda.eventRecord(done, [s1, s2])
    Cuda.eventSync_Del(done)
    assert Cuda.streamQuery(s2)
    for e in (e0, e1):
        Cuda.deleteEvent(e)
    Cuda.deleteStream(s1)
    Cuda.deleteStream(s2)


def test_error_reporting(gpu):
    Cuda = gpu.Cuda
    Cuda.getLastExceptionType()            # clear
    assert gpu.lib.dragon_Cuda_free(0x10) != 0     # not a device allocation
    code = Cuda.getLastExceptionType()
    assert code != 0
    assert gpu.lib.dragon_Cuda_getExceptionName(code)
    assert Cuda.getLastExceptionType() == 0        # reading clears it
