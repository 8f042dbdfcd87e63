"""Python access to the gfx950 FP32 matrix-multiplication engine.

Thin, one-to-one wrappers over the C ABI (no compute happens in Python):

  Cuda             -- runtime natives of the reference's z.dragon.engine.cuda.impl.Cuda
  Cuda_matMul      -- natives + heuristics of ...impl.math.Cuda_matMul
  Cuda_batchMatMul -- natives + heuristics of ...impl.math.Cuda_batchMatMul
  Cuda_conv3D      -- forward-convolution natives of ...impl.math.Cuda_conv3D
  Cuda_expk2       -- transpose2D / 3D / 4D of ...impl.Cuda_expk2 (dimension swap)
  Cuda_function    -- linear_dual2D_row of ...impl.math.Cuda_function (the bias row)
  CudaException    -- the error type the reference's natives throw

Method names and argument order follow the Java declarations
(source/alpha-Dragon-v1.2/src/z/dragon/engine/cuda/impl/Cuda.java,
 .../impl/math/Cuda_matMul.java, .../impl/math/Cuda_batchMatMul.java).
"""
import ctypes

import numpy as np

from . import _lib

lib = _lib.load()


class CudaException(RuntimeError):
    """Mirror of z.dragon.engine.cuda.impl.CudaException: carries the runtime error code."""

    def __init__(self, code):
        self.code = int(code)
        name = lib.dragon_Cuda_getExceptionName(self.code)
        info = lib.dragon_Cuda_getExceptionInfo(self.code)
        super().__init__("%s (%d): %s" % ((name or b"?").decode(), self.code,
                                           (info or b"").decode()))


def _check(code):
    if code != 0:
        raise CudaException(code)


def _stream_array(streams):
    arr = (ctypes.c_int64 * len(streams))(*[int(s) for s in streams])
    return arr, len(streams)


def _host_ptr(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


class Cuda:
    """Runtime natives (Cuda.java:66-194)."""

    @staticmethod
    def malloc(size):
        addr = lib.dragon_Cuda_malloc(int(size))
        if addr == 0:
            raise CudaException(lib.dragon_Cuda_getLastExceptionType() or 2)
        return addr

    @staticmethod
    def free(address):
        _check(lib.dragon_Cuda_free(address))

    @staticmethod
    def mallocHost(size):
        addr = lib.dragon_Cuda_mallocHost(int(size))
        if addr == 0:
            raise CudaException(lib.dragon_Cuda_getLastExceptionType() or 2)
        return addr

    @staticmethod
    def freeHost(address):
        _check(lib.dragon_Cuda_freeHost(address))

    @staticmethod
    def memsetAsync(stream, address, value, size):
        _check(lib.dragon_Cuda_memsetAsync(stream, address, value, size))

    @staticmethod
    def memcpyAsyncDeviceToDevice(stream, dst, src, size):
        _check(lib.dragon_Cuda_memcpyAsyncDeviceToDevice(stream, dst, src, size))

    @staticmethod
    def getDeviceId():
        return lib.dragon_Cuda_getDeviceId()

    @staticmethod
    def getDeviceCount():
        return lib.dragon_Cuda_getDeviceCount()

    @staticmethod
    def setDevice(dev_id):
        _check(lib.dragon_Cuda_setDevice(dev_id))

    @staticmethod
    def deviceSynchronize():
        _check(lib.dragon_Cuda_deviceSynchronize())

    @staticmethod
    def multiProcessorCount(dev_id=0):
        return lib.dragon_CudaDevice_multiProcessorCount(dev_id)

    @staticmethod
    def newStream_Blocking():
        s = lib.dragon_Cuda_newStream_Blocking()
        if s == 0:
            raise CudaException(lib.dragon_Cuda_getLastExceptionType() or 1)
        return s

    @staticmethod
    def newStream_NonBlocking():
        s = lib.dragon_Cuda_newStream_NonBlocking()
        if s == 0:
            raise CudaException(lib.dragon_Cuda_getLastExceptionType() or 1)
        return s

    @staticmethod
    def deleteStream(stream):
        _check(lib.dragon_Cuda_deleteStream(stream))

    @staticmethod
    def streamQuery(stream):
        r = lib.dragon_Cuda_streamQuery(stream)
        if r < 0:
            raise CudaException(lib.dragon_Cuda_getLastExceptionType() or 1)
        return bool(r)

    @staticmethod
    def streamSynchronize(stream):
        _check(lib.dragon_Cuda_streamSynchronize(stream))

    @staticmethod
    def newEvent_Default():
        return lib.dragon_Cuda_newEvent_Default()

    @staticmethod
    def newEvent_DisableTiming():
        return lib.dragon_Cuda_newEvent_DisableTiming()

    @staticmethod
    def deleteEvent(event):
        _check(lib.dragon_Cuda_deleteEvent(event))

    @staticmethod
    def eventRecord(event, stream_or_streams, length=None):
        if isinstance(stream_or_streams, (list, tuple)):
            arr, n = _stream_array(stream_or_streams)
            _check(lib.dragon_Cuda_eventRecord_streams(event, arr, n if length is None else length))
        else:
            _check(lib.dragon_Cuda_eventRecord(event, stream_or_streams))

    @staticmethod
    def eventSynchronize(event):
        _check(lib.dragon_Cuda_eventSynchronize(event))

    @staticmethod
    def eventSync_Del(event):
        _check(lib.dragon_Cuda_eventSync_Del(event))

    @staticmethod
    def eventElapsedTime(start_event, stop_event):
        ms = lib.dragon_Cuda_eventElapsedTime(start_event, stop_event)
        if ms < 0:
            raise CudaException(lib.dragon_Cuda_getLastExceptionType() or 1)
        return ms

    @staticmethod
    def streamWaitEvent_default(stream, event):
        _check(lib.dragon_Cuda_streamWaitEvent_default(stream, event))

    @staticmethod
    def getLastExceptionType():
        return lib.dragon_Cuda_getLastExceptionType()

    @staticmethod
    def set1D(stream, address, value, length):
        if isinstance(value, (int, float)):
            _check(lib.dragon_Cuda_set1D_value(stream, address, float(value), length))
        else:
            _check(lib.dragon_Cuda_set1D(stream, address, _host_ptr(value), length))

    @staticmethod
    def set2D(stream, address, value, height, width, stride):
        if isinstance(value, (int, float)):
            _check(lib.dragon_Cuda_set2D_value(stream, address, float(value), height, width, stride))
        else:
            _check(lib.dragon_Cuda_set2D(stream, address, _host_ptr(value), height, width, stride))

    @staticmethod
    def get1D(stream, address, value, length):
        _check(lib.dragon_Cuda_get1D(stream, address, _host_ptr(value), length))

    @staticmethod
    def get2D(stream, address, value, height, width, stride):
        _check(lib.dragon_Cuda_get2D(stream, address, _host_ptr(value), height, width, stride))

    # _v2: through a staging buffer of the caller's (an address from mallocHost, normally)
    @staticmethod
    def set1D_v2(stream, address, value, buf_address, length):
        _check(lib.dragon_Cuda_set1D_v2(stream, address, _host_ptr(value), buf_address, length))

    @staticmethod
    def set2D_v2(stream, address, value, buf_address, height, width, stride):
        _check(lib.dragon_Cuda_set2D_v2(stream, address, _host_ptr(value), buf_address, height, width,
                                        stride))

    @staticmethod
    def get1D_v2(stream, address, value, buf_address, length):
        _check(lib.dragon_Cuda_get1D_v2(stream, address, _host_ptr(value), buf_address, length))

    @staticmethod
    def get2D_v2(stream, address, value, buf_address, height, width, stride):
        _check(lib.dragon_Cuda_get2D_v2(stream, address, _host_ptr(value), buf_address, height, width,
                                        stride))


class Cuda_matMul:
    """Natives and helpers of Cuda_matMul.java."""

    blockNum = staticmethod(lambda N, M: lib.dragon_Cuda_matMul_blockNum(N, M))
    nstream = staticmethod(lambda N, M: lib.dragon_Cuda_matMul_nstream(N, M))

    @staticmethod
    def SKbuf_summary(stream, dCbuf, dC, part, sizeC):
        _check(lib.dragon_Cuda_matMul_SKbuf_summary(stream, dCbuf, dC, part, sizeC))

    @staticmethod
    def matMulSK_static(streams, length, variant, GridZ, dA, dB, dC, N, M, K):
        """Both split-K stages with the partials in the library's own static workspace (no allocation)."""
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulSK_static(arr, length, variant, GridZ, dA, dB, dC, N, M, K))

    @staticmethod
    def matMul(streams, length, dA, dB, dC, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMul(arr, length, dA, dB, dC, N, M, K))

    @staticmethod
    def matMulT1(streams, length, dA, dB, dC, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulT1(arr, length, dA, dB, dC, N, M, K))

    @staticmethod
    def matMulT2(streams, length, dA, dB, dC, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulT2(arr, length, dA, dB, dC, N, M, K))

    @staticmethod
    def matMulSK(streams, length, GZ, dA, dB, dC, dCbuf, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulSK(arr, length, GZ, dA, dB, dC, dCbuf, N, M, K))

    @staticmethod
    def matMulT1SK(streams, length, GZ, dA, dB, dC, dCbuf, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulT1SK(arr, length, GZ, dA, dB, dC, dCbuf, N, M, K))

    @staticmethod
    def matMulT2SK(streams, length, GZ, dA, dB, dC, dCbuf, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulT2SK(arr, length, GZ, dA, dB, dC, dCbuf, N, M, K))

    @staticmethod
    def matMul_biased(streams, length, dA, dB, dC, dBias, N, M, K, lengthv, width):
        """One launch for matMul followed by the bias row; no native of this name in the reference."""
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMul_biased(arr, length, dA, dB, dC, dBias, N, M, K,
                                                    lengthv, width))

    @staticmethod
    def matMul_mma(streams, length, dA, dB, dC, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMul_mma(arr, length, dA, dB, dC, N, M, K))

    @staticmethod
    def matMulT1_mma(streams, length, dA, dB, dC, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulT1_mma(arr, length, dA, dB, dC, N, M, K))

    @staticmethod
    def matMulT2_mma(streams, length, dA, dB, dC, N, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_matMul_matMulT2_mma(arr, length, dA, dB, dC, N, M, K))


class Cuda_function:
    """The natives of Cuda_function.java on the path: the bias row and the scalar linear map."""

    @staticmethod
    def linear2D(stream, alpha, dX, beta, dY, lengthv, width, stride):
        _check(lib.dragon_Cuda_function_linear2D(stream, alpha, dX, beta, dY, lengthv, width, stride))

    @staticmethod
    def linear_dual2D_row(stream, dX1, dX2, row_lengthv, alpha, beta, gamma, dY, lengthv, width,
                          stride):
        _check(lib.dragon_Cuda_function_linear_dual2D_row(stream, dX1, dX2, row_lengthv, alpha, beta,
                                                          gamma, dY, lengthv, width, stride))


class Cuda_conv3D:
    """Forward-convolution natives of Cuda_conv3D.java (every family runs the same implicit-GEMM kernel)."""

    @staticmethod
    def output_feature_dim(IH, IW, FH, FW, N, OC, sh, sw, ph, pw):
        return [N, (IH - FH + 2 * ph) // sh + 1, (IW - FW + 2 * pw) // sw + 1, OC]

    @staticmethod
    def conv3D(streams, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3D(arr, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh,
                                             sw, ph, pw))

    @staticmethod
    def conv3D_texture(streams, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3D_texture(arr, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC,
                                                     OC, sh, sw, ph, pw))

    @staticmethod
    def conv3D_np(streams, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3D_np(arr, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC,
                                                sh, sw))

    @staticmethod
    def conv3D_W1(streams, length, dX, IH, IW, dW, dY, N, IC, OC):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3D_W1(arr, length, dX, IH, IW, dW, dY, N, IC, OC))

    @staticmethod
    def conv3DV2(useTexture, streams, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3DV2(int(useTexture), arr, length, dX, IH, IW, dW, FH, FW, dY, OH,
                                               OW, N, IC, OC, sh, sw, ph, pw))

    @staticmethod
    def kernel_remode(stream, dW, dCW, FH, FW, OC, IC):
        _check(lib.dragon_Cuda_conv3D_kernel_remode(stream, dW, dCW, FH, FW, OC, IC))

    @staticmethod
    def conv3D_GemmR(streams, length, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3D_GemmR(arr, length, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW, N, IC,
                                                   OC, sh, sw, ph, pw))

    @staticmethod
    def conv3D_GemmR_W1(streams, length, dX, IH, IW, dW, dCW, dY, N, IC, OC):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3D_GemmR_W1(arr, length, dX, IH, IW, dW, dCW, dY, N, IC, OC))

    @staticmethod
    def conv3D_Im2col_Winograd_s8_R_texture(useTexture, streams, length, dX, IH, IW, dW, dCW, FH, FW, dY, OH,
                                            OW, N, IC, OC, ph, pw):
        arr, _ = _stream_array(streams)
        rc = lib.dragon_Cuda_conv3D_conv3D_Im2col_Winograd_s8_R_texture(
            int(useTexture), arr, length, dX, IH, IW, dW, dCW, FH, FW, dY, OH, OW, N, IC, OC, ph, pw)
        if rc < 0:
            raise CudaException(-rc)
        return rc == 1

    @staticmethod
    def conv3D_biased(streams, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC, sh, sw, ph, pw, dBias,
                      lengthv, width):
        """Convolution and bias row in one launch; no native of this name in the reference."""
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_conv3D_conv3D_biased(arr, length, dX, IH, IW, dW, FH, FW, dY, OH, OW, N, IC, OC,
                                                    sh, sw, ph, pw, dBias, lengthv, width))


class Cuda_reduce:
    """Row softmax in one launch (stands in for row_max + row_softmax + div2D_field)."""

    @staticmethod
    def softmax2D(stream, dX, dY, field_length, row_lengthv, width, stride, scale=1.0):
        _check(lib.dragon_Cuda_reduce_softmax2D(stream, dX, dY, field_length, row_lengthv, width, stride,
                                                scale))


class Cuda_attention:
    """softmax(scale * Q.K^T).V in one launch (stands in for the chain of ChannelMHA.java:66-83)."""

    @staticmethod
    def forward(streams, length, dQ, dK, dV, dY, N, head, QL, VL, dK4, dV4, head_inner, scale):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_attention_forward(arr, length, dQ, dK, dV, dY, N, head, QL, VL, dK4, dV4,
                                                 int(head_inner), scale))

    @staticmethod
    def forward_masked(streams, length, dQ, dK, dV, dMask, dY, N, head, QL, VL, dK4, dV4, head_inner, scale,
                       mask_pitch, mask_per_head):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_attention_forward_masked(arr, length, dQ, dK, dV, dMask, dY, N, head, QL, VL, dK4, dV4,
                                                        int(head_inner), scale, mask_pitch, int(mask_per_head)))


class Cuda_expk2:
    """The dimension-swap natives of Cuda_expk2.java."""

    @staticmethod
    def transpose2D(stream, dX, dY, Xdim1, Ydim1, strideX, strideY, length):
        _check(lib.dragon_Cuda_expk2_transpose2D(stream, dX, dY, Xdim1, Ydim1, strideX, strideY, length))

    @staticmethod
    def transpose3D(stream, dX, dY, Xdim1, Xdim2, Ydim1, Ydim2, dimIndex1, dimIndex2, strideX, strideY,
                    length):
        _check(lib.dragon_Cuda_expk2_transpose3D(stream, dX, dY, Xdim1, Xdim2, Ydim1, Ydim2, dimIndex1,
                                                 dimIndex2, strideX, strideY, length))

    @staticmethod
    def transpose4D(stream, dX, dY, Xdim1, Xdim2, Xdim3, Ydim1, Ydim2, Ydim3, dimIndex1, dimIndex2,
                    strideX, strideY, length):
        _check(lib.dragon_Cuda_expk2_transpose4D(stream, dX, dY, Xdim1, Xdim2, Xdim3, Ydim1, Ydim2, Ydim3,
                                                 dimIndex1, dimIndex2, strideX, strideY, length))


class Cuda_batchMatMul:
    """Natives and helpers of Cuda_batchMatMul.java."""

    streamSize = staticmethod(lambda N, M: lib.dragon_Cuda_batchMatMul_streamSize(N, M))

    @staticmethod
    def batchMatMul(streams, length, dA, dB, dC, Batch, N, M, BK, AK):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_batchMatMul_batchMatMul(arr, length, dA, dB, dC, Batch, N, M, BK, AK))

    @staticmethod
    def batchMatMul_texture(streams, length, dA, dB, dC, Batch, N, M, BK, AK):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_batchMatMul_batchMatMul_texture(arr, length, dA, dB, dC, Batch, N, M,
                                                               BK, AK))

    @staticmethod
    def batchMatMulT1(streams, length, dA, dB, dC, Batch, CN, AN, M, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_batchMatMul_batchMatMulT1(arr, length, dA, dB, dC, Batch, CN, AN, M, K))

    @staticmethod
    def batchMatMulT2(streams, length, dA, dB, dC, Batch, N, CM, BM, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_batchMatMul_batchMatMulT2(arr, length, dA, dB, dC, Batch, N, CM, BM, K))

    @staticmethod
    def batchMatMulT2_texture(streams, length, dA, dB, dC, Batch, N, CM, BM, K):
        arr, _ = _stream_array(streams)
        _check(lib.dragon_Cuda_batchMatMul_batchMatMulT2_texture(arr, length, dA, dB, dC, Batch, N,
                                                                 CM, BM, K))


def force_tile(tile):
    """Force one kernel tile shape (-1 = automatic).  Benchmark / test hook."""
    lib.dragon_gemm_force_tile(int(tile))


def skinny_form(form):
    """Force a form of the skinny kernel (0..4, -1 = automatic).  Benchmark / test hook."""
    lib.dragon_gemm_skinny_form(int(form))


def split_policy(mode):
    """How the split-K entries treat GridZ: -1 the estimate decides, 0 always as asked, 1 declined where possible."""
    lib.dragon_gemm_split_policy(int(mode))


def fold_skip(on):
    """Whether the no-op fold after a declined split is elided (default on).  Test hook."""
    lib.dragon_gemm_fold_skip(int(bool(on)))


def folds_skipped():
    return lib.dragon_gemm_folds_skipped()


def declined_splits():
    return lib.dragon_gemm_declined_splits()


def split_loses(variant, N, M, GZ, K, num_cu=256):
    return lib.dragon_gemm_split_loses(variant, N, M, GZ, K, num_cu)


def estimate_us(variant, rows, cols, nz, k, num_cu=256):
    return lib.dragon_gemm_estimate_us(variant, rows, cols, nz, k, num_cu)


def workspace_count():
    return lib.dragon_gemm_workspace_count()


def workspaces_refused():
    return lib.dragon_gemm_workspaces_refused()


def release_workspaces():
    """Frees every per-stream workspace of the balanced kernel; returns how many there were."""
    return lib.dragon_gemm_release_workspaces()


def mem_get_info():
    """(free, total) bytes of device memory on the current device."""
    import ctypes
    f, t = ctypes.c_int64(0), ctypes.c_int64(0)
    _check(lib.dragon_test_mem_get_info(ctypes.byref(f), ctypes.byref(t)))
    return f.value, t.value


def choose_tile(variant, rows, cols, nz, k, num_cu=256):
    """The tile shape the automatic choice takes (host arithmetic only)."""
    return lib.dragon_gemm_choose_tile(variant, rows, cols, nz, k, num_cu)


class DeviceArray:
    """A float32 device allocation filled from / read back into a numpy array.

    Test and benchmark plumbing: owns one Cuda.malloc block of `a.size` floats."""

    def __init__(self, host=None, size=None, zero=True):
        n = int(host.size if host is not None else size)
        self.size = n
        self.address = Cuda.malloc(max(n, 4) * 4)
        if host is not None:
            h = np.ascontiguousarray(host, dtype=np.float32).reshape(-1)
            Cuda.set1D(0, self.address, h, n)
        elif zero:
            Cuda.memsetAsync(0, self.address, 0, n * 4)
            Cuda.streamSynchronize(0)

    def get(self, shape=None):
        out = np.empty(self.size, dtype=np.float32)
        Cuda.get1D(0, self.address, out, self.size)
        return out.reshape(shape) if shape is not None else out

    def fill(self, value):
        Cuda.set1D(0, self.address, float(value), self.size)
        Cuda.streamSynchronize(0)

    def free(self):
        if self.address:
            Cuda.free(self.address)
            self.address = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
