"""Python face of the host-side engine mirror: Engine / Tensor with the reference's method
names (alpha.engine.cuda_float32, eg.tensor, eg.matMul, eg.batchMatMulT2, eg.valueOf ...).
All logic lives in the C++ classes behind include/dragon_hip_engine.h."""
import ctypes

import numpy as np

from . import lib, CudaException


class NullPointerException(RuntimeError):
    pass


class IllegalArgumentException(ValueError):
    pass


def _raise(code):
    msg = (lib.dragon_engine_last_error() or b"").decode()
    if code == 1:
        raise NullPointerException(msg)
    if code == 2:
        raise IllegalArgumentException(msg)
    if code == 3:
        raise CudaException(lib.dragon_engine_last_cuda_code())
    raise RuntimeError(msg)


def _last_code():
    # pointer-returning entry points report through the thread's last error only
    msg = (lib.dragon_engine_last_error() or b"").decode()
    return msg


def _dims(dim):
    arr = (ctypes.c_int32 * len(dim))(*[int(d) for d in dim])
    return arr, len(dim)


class Tensor:
    def __init__(self, eg, handle):
        self._eg, self._h = eg, handle

    def c(self):
        rc = lib.dragon_tensor_c(self._h)
        if rc:
            _raise(rc)
        return self

    @property
    def dim(self):
        return [lib.dragon_tensor_dim(self._h, i) for i in range(lib.dragon_tensor_ndim(self._h))]

    def ndim(self):
        return lib.dragon_tensor_ndim(self._h)

    length = property(lambda self: lib.dragon_tensor_length(self._h))
    lengthv = property(lambda self: lib.dragon_tensor_lengthv(self._h))
    length_4x = property(lambda self: lib.dragon_tensor_length_4x(self._h))
    address = property(lambda self: lib.dragon_tensor_address(self._h))

    def value(self):
        return self._eg.valueOf(self)


MATMUL, MATMUL_T1, MATMUL_T2, BMM, BMM_T1, BMM_T2 = range(6)


class Engine:
    """alpha.engine.cuda_float32(deviceId, ...)"""

    def __init__(self, device_id=0, stream_pool_size=32, max_trans_buf_size=0, max_mem_size=0):
        """max_trans_buf_size > 0: pinned staging pool for uploads / downloads; max_mem_size > 0: device
        memory pool (alpha.engine.memp1) behind tensors and split-K partial buffers."""
        if max_mem_size > 0:
            self._h = lib.dragon_engine_cuda_float32_pooled(device_id, stream_pool_size, max_mem_size,
                                                            max_trans_buf_size)
        elif max_trans_buf_size > 0:
            self._h = lib.dragon_engine_cuda_float32_buffered(device_id, stream_pool_size,
                                                              max_trans_buf_size)
        else:
            self._h = lib.dragon_engine_cuda_float32(device_id, stream_pool_size)
        if not self._h:
            _raise(lib.dragon_engine_last_status() or 4)

    def close(self):
        if self._h:
            lib.dragon_engine_delete(self._h)
            self._h = None

    def check(self, flag):
        lib.dragon_engine_check(self._h, int(flag))
        return self

    def sync(self, flag):
        lib.dragon_engine_sync(self._h, int(flag))
        return self

    def set_param(self, name, value):
        rc = lib.dragon_engine_set_param(self._h, name.encode(), int(value))
        if rc:
            _raise(rc)
        return self

    def get_param(self, name):
        return lib.dragon_engine_get_param(self._h, name.encode())

    def gridZ(self, kind, N, M, K):
        return lib.dragon_engine_gridZ(self._h, kind, N, M, K)

    # ---- tensors ----
    def _wrap(self, h):
        if not h:
            _raise(lib.dragon_engine_last_status() or 4)
        return Tensor(self, h)

    def empty(self, *dim):
        arr, n = _dims(dim)
        return self._wrap(lib.dragon_engine_empty(self._h, arr, n))

    def zeros(self, *dim):
        arr, n = _dims(dim)
        return self._wrap(lib.dragon_engine_zeros(self._h, arr, n))

    def tensor(self, value, *dim):
        v = np.ascontiguousarray(value, dtype=np.float32).reshape(-1)
        arr, n = _dims(dim)
        return self._wrap(lib.dragon_engine_tensor(self._h, v.ctypes.data, v.size, arr, n))

    def valueOf(self, ts):
        out = np.empty(ts.length, dtype=np.float32)
        rc = lib.dragon_engine_valueOf(self._h, ts._h, out.ctypes.data, out.size)
        if rc:
            _raise(rc)
        return out

    def delete(self, *tensors):
        for t in tensors:
            if t is not None and t._h:
                lib.dragon_engine_delete_tensor(self._h, t._h)
                t._h = None

    # ---- products ----
    def _product(self, op, args, likeA=True):
        hs = [a._h if a is not None else None for a in args]
        if len(args) == 2:
            return self._wrap(lib.dragon_engine_product(self._h, op, int(likeA), hs[0], hs[1]))
        rc = lib.dragon_engine_product_into(self._h, op, hs[0], hs[1], hs[2])
        if rc:
            _raise(rc)
        return args[0]

    def matMul(self, *t):
        return self._product(MATMUL, t)

    def matMulT1(self, *t):
        return self._product(MATMUL_T1, t)

    def matMulT2(self, *t):
        return self._product(MATMUL_T2, t)

    def batchMatMul(self, *t, likeA=True):
        return self._product(BMM, t, likeA)

    def batchMatMulT1(self, *t, likeA=True):
        return self._product(BMM_T1, t, likeA)

    def batchMatMulT2(self, *t, likeA=True):
        return self._product(BMM_T2, t, likeA)

    # ---- fully connected layer and bias row ----
    def _fullconnect(self, op, t, n_in):
        """t = inputs, or (output, inputs...) when one more tensor than n_in is given."""
        hs = [a._h if a is not None else None for a in t]
        if len(t) == n_in:
            hs += [None] * (3 - n_in)
            return self._wrap(lib.dragon_engine_fullconnect(self._h, op, hs[0], hs[1], hs[2]))
        hs += [None] * (4 - len(hs))
        rc = lib.dragon_engine_fullconnect_into(self._h, op, hs[0], hs[1], hs[2], hs[3])
        if rc:
            _raise(rc)
        return t[0]

    def fullconnect(self, *t):
        return self._fullconnect(0, t, 2)

    def fullconnect_biased(self, *t):
        return self._fullconnect(1, t, 3)

    def fullconnect_deltaX(self, deltaY, W):
        return self._fullconnect(2, (deltaY, W), 2)

    def fullconnect_deltaW(self, X, deltaY):
        return self._fullconnect(3, (X, deltaY), 2)

    def matMul_biased(self, *t):
        return self._fullconnect(4, t, 3)

    # ---- forward convolution over NHWC tensors (Engine.java:2076-2204) ----
    def conv3D(self, *a, Bias=None):
        """conv3D(Y, X, W, sh, sw[, ph, pw]) writes into Y (padding derived from the shapes when omitted);
        conv3D(X, W, sh, sw, ph, pw) or conv3D(X, W, OH, OW, sh, sw, ph, pw) creates Y."""
        n_t = sum(1 for x in a if isinstance(x, Tensor) or x is None)
        ts, num = a[:n_t], [int(v) for v in a[n_t:]]
        hs = [x._h if x is not None else None for x in ts]
        hb = Bias._h if Bias is not None else None
        if n_t == 3:
            sh, sw, ph, pw = num if len(num) == 4 else (num[0], num[1], -1, -1)
            rc = lib.dragon_engine_conv3D_into(self._h, hs[0], hs[1], hs[2], sh, sw, ph, pw, hb)
            if rc:
                _raise(rc)
            return ts[0]
        OH, OW, sh, sw, ph, pw = num if len(num) == 6 else [-1, -1] + num
        return self._wrap(lib.dragon_engine_conv3D(self._h, hs[0], hs[1], OH, OW, sh, sw, ph, pw, hb))

    @staticmethod
    def conv3D_GEMM_nstream(GM, OC):
        return lib.dragon_policy_conv3D_GEMM_nstream(GM, OC)

    def conv3D_biased(self, *a):
        """The argument lists of conv3D with the Bias tensor last."""
        if a[-1] is None:
            raise NullPointerException("Bias is null")
        return self.conv3D(*a[:-1], Bias=a[-1])

    def linear2_row(self, inplace, X1, X2, alpha, beta, gamma):
        h = lib.dragon_engine_linear2_row(self._h, int(inplace), X1._h if X1 else None,
                                          X2._h if X2 else None, alpha, beta, gamma)
        if inplace and h:
            return X1
        return self._wrap(h)

    def linear(self, inplace, alpha, X, beta):
        h = lib.dragon_engine_linear(self._h, int(inplace), alpha, X._h if X else None, beta)
        return X if (inplace and h) else self._wrap(h)

    def sdiv(self, inplace, X, C):
        return self.linear(inplace, 1.0 / C, X, 0.0)

    def softmax(self, inplace, X, features=-1, scale=1.0):
        h = lib.dragon_engine_softmax(self._h, int(inplace), X._h if X else None, features, scale)
        return X if (inplace and h) else self._wrap(h)

    def attention(self, Q, K, V, head, scale=0.0, mask=None):
        """softmax(scale * Q.K^T).V per head in one launch; scale = 0: 1/sqrt(Q.lastDim).  mask: a tensor
        [QL, VL] or [N, head, QL, VL] that multiplies the probabilities after the softmax."""
        hs = [x._h if x is not None else None for x in (Q, K, V)]
        if mask is not None:
            return self._wrap(lib.dragon_engine_attention_masked(self._h, hs[0], hs[1], hs[2], mask._h, head, scale))
        return self._wrap(lib.dragon_engine_attention(self._h, hs[0], hs[1], hs[2], head, scale))

    def transpose(self, inplace, X, dimIdx1, dimIdx2):
        h = lib.dragon_engine_transpose(self._h, int(inplace), X._h if X else None, dimIdx1, dimIdx2)
        if h and X is not None and h == X._h:
            return X
        return self._wrap(h)

    def add_row(self, inplace, X1, X2):
        return self.linear2_row(inplace, X1, X2, 1.0, 1.0, 0.0)


def cuda_float32(device_id=0, stream_pool_size=32, max_trans_buf_size=0, max_mem_size=0):
    return Engine(device_id, stream_pool_size, max_trans_buf_size, max_mem_size)
