"""ctypes access to the CPU oracle (oracle/dragon_oracle.c) -- TEST INFRASTRUCTURE.

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg import this
module.  The shipped library never does.  If liboracle.so is not built yet it is built
with the Makefile next to this file (gcc only, no GPU needed).
"""
import ctypes
import os
import subprocess
from ctypes import c_int, c_float, c_void_p, POINTER, byref

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libref_micro.so")

NN, T1, T2 = 0, 1, 2


def build():
    subprocess.run(["make", "-C", _HERE, "-s"], check=True, stdout=subprocess.DEVNULL,
                   stderr=subprocess.DEVNULL)


if not os.path.exists(_SO):
    build()
_o = ctypes.CDLL(_SO)

_P = c_void_p
for _name, _res, _args in [
    ("oracle_multiply", None, [_P, _P, _P, c_int, c_int, c_int]),
    ("oracle_multiplyT1", None, [_P, _P, _P, c_int, c_int, c_int]),
    ("oracle_multiplyT2", None, [_P, _P, _P, c_int, c_int, c_int]),
    ("oracle_matMul_fast", c_int, [c_int, _P, _P, _P, c_int, c_int, c_int]),
    ("oracle_matMul_f64", c_int, [c_int, _P, _P, _P, c_int, c_int, c_int]),
    ("oracle_bmm", None, [_P, _P, _P] + [c_int] * 5),
    ("oracle_bmmT1", None, [_P, _P, _P] + [c_int] * 5),
    ("oracle_bmmT2", None, [_P, _P, _P] + [c_int] * 5),
    ("oracle_bmm_fast", c_int, [c_int, _P, _P, _P] + [c_int] * 5),
    ("oracle_SK_K_slice", c_int, [c_int, c_int]),
    ("oracle_SK_bounds", None, [c_int, c_int, c_int, POINTER(c_int), POINTER(c_int)]),
    ("oracle_matMulSK", c_int, [c_int, c_int, _P, _P, _P, _P, c_int, c_int, c_int]),
    ("oracle_SKbuf_summary", None, [_P, _P, c_int, c_int]),
    ("oracle_blockNum", c_int, [c_int, c_int]),
    ("oracle_nstream", c_int, [c_int, c_int]),
    ("oracle_streamSize", c_int, [c_int, c_int]),
    ("oracle_smooth_maxPart", c_int, [c_int]),
    ("oracle_gridZ", c_int, [c_int] * 6 + [c_float, c_float, c_int]),
    ("oracle_linear_dual2D_row", None, [_P, _P, c_int, c_float, c_float, c_float, _P, c_int, c_int, c_int]),
    ("oracle_linear2D", None, [c_float, _P, c_float, _P, c_int, c_int, c_int]),
    ("oracle_softmax2D", None, [_P, _P, c_int, c_int, c_int, c_int, c_float]),
    ("oracle_conv3D", None, [_P, c_int, c_int, _P, c_int, c_int, _P] + [c_int] * 10),
    ("oracle_transpose4D", None, [_P, _P, POINTER(c_int), c_int, c_int, c_int, c_int]),
    ("oracle_samePercent_relative", c_float, [_P, _P, c_int, c_float]),
    ("oracle_num_threads", c_int, []),
]:
    _f = getattr(_o, _name)
    _f.restype = _res
    _f.argtypes = _args


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_P)


def num_threads():
    return _o.oracle_num_threads()


# ---- 2-D products -----------------------------------------------------------------
def _shapes(variant, A, B):
    if variant == NN:
        (N, K), (K2, M) = A.shape, B.shape
    elif variant == T1:
        (K, N), (K2, M) = A.shape, B.shape
    else:
        (N, K), (M, K2) = A.shape, B.shape
    assert K == K2, "contraction lengths differ"
    return N, M, K


def multiply_literal(variant, A, B):
    """The reference's k,i,j triple loop, single thread (MM/test.cuh:60-82)."""
    A, pa = _f32(A)
    B, pb = _f32(B)
    N, M, K = _shapes(variant, A, B)
    C = np.zeros((N, M), np.float32)
    fn = [_o.oracle_multiply, _o.oracle_multiplyT1, _o.oracle_multiplyT2][variant]
    fn(pa, pb, C.ctypes.data_as(_P), N, M, K)
    return C


def matmul(variant, A, B):
    """Bit-identical to multiply_literal, cache-blocked and multi-threaded."""
    A, pa = _f32(A)
    B, pb = _f32(B)
    N, M, K = _shapes(variant, A, B)
    C = np.zeros((N, M), np.float32)
    rc = _o.oracle_matMul_fast(variant, pa, pb, C.ctypes.data_as(_P), N, M, K)
    assert rc == 0
    return C


def matmul_f64(variant, A, B):
    """FP64-accumulate twin (exact products, double sum); returns float64."""
    A, pa = _f32(A)
    B, pb = _f32(B)
    N, M, K = _shapes(variant, A, B)
    C = np.zeros((N, M), np.float64)
    rc = _o.oracle_matMul_f64(variant, pa, pb, C.ctypes.data_as(_P), N, M, K)
    assert rc == 0
    return C


# ---- batched products, arrays in the reference's padded memory layout ---------------
def bmm_literal(variant, A, B, Batch, d0, d1, d2, d3):
    """variant NN: (N, CM, BK, AK); T1: (CN, AN, CM, K); T2: (N, CM, BM, K).
    A and B are flat float32 buffers laid out as the reference lays them out."""
    A, pa = _f32(A)
    B, pb = _f32(B)
    rows, cols = (d0, d1) if variant != T1 else (d0, d2)
    C = np.zeros((Batch, rows, cols), np.float32)
    fn = [_o.oracle_bmm, _o.oracle_bmmT1, _o.oracle_bmmT2][variant]
    fn(pa, pb, C.ctypes.data_as(_P), Batch, d0, d1, d2, d3)
    return C


def bmm(variant, A, B, Batch, d0, d1, d2, d3):
    A, pa = _f32(A)
    B, pb = _f32(B)
    rows, cols = (d0, d1) if variant != T1 else (d0, d2)
    C = np.zeros((Batch, rows, cols), np.float32)
    rc = _o.oracle_bmm_fast(variant, pa, pb, C.ctypes.data_as(_P), Batch, d0, d1, d2, d3)
    assert rc == 0
    return C


# ---- split-K -------------------------------------------------------------------------
def SK_K_slice(K, GZ):
    return _o.oracle_SK_K_slice(K, GZ)


def SK_bounds(K, GZ, z):
    a, b = c_int(), c_int()
    _o.oracle_SK_bounds(K, GZ, z, byref(a), byref(b))
    return a.value, b.value


def matMulSK(variant, GZ, A, B):
    """Stage 1: returns (C, Cbuf) with slice 0 in C and slices 1.. in Cbuf[GZ-1, N, M]."""
    A, pa = _f32(A)
    B, pb = _f32(B)
    N, M, K = _shapes(variant, A, B)
    C = np.zeros((N, M), np.float32)
    Cbuf = np.zeros((max(GZ - 1, 1), N, M), np.float32)
    rc = _o.oracle_matMulSK(variant, GZ, pa, pb, C.ctypes.data_as(_P), Cbuf.ctypes.data_as(_P),
                            N, M, K)
    assert rc == 0
    return C, Cbuf[:GZ - 1]


def SKbuf_summary(Cbuf, C, part):
    """Stage 2 (Kahan, p ascending); returns the folded C (input left untouched)."""
    Cbuf, pb = _f32(Cbuf)
    out = np.array(C, dtype=np.float32, copy=True, order="C")
    _o.oracle_SKbuf_summary(pb, out.ctypes.data_as(_P), part, out.size)
    return out


# ---- heuristics ------------------------------------------------------------------------
blockNum = _o.oracle_blockNum
nstream = _o.oracle_nstream
streamSize = _o.oracle_streamSize
smooth_maxPart = _o.oracle_smooth_maxPart

MATMUL, MATMUL_T1, MATMUL_T2, MATMUL_BIASED = 0, 1, 2, 3


def gridZ(kind, N, M, K, SM, threshold=512, minBlock=None, maxBlock=4.0, maxPart=None):
    """Split-K decision of CudaFloat32EngineBase (1 = no split) with its defaults."""
    if minBlock is None:
        minBlock = 1.14 if kind == MATMUL_T1 else 1.2
    if maxPart is None:
        maxPart = smooth_maxPart(SM)
    return _o.oracle_gridZ(kind, N, M, K, SM, threshold, minBlock, maxBlock, maxPart)


def linear_dual2D_row(X1, X2, alpha, beta, gamma, width):
    """X1: device-layout matrix [rows, stride] (stride a multiple of 4), X2: row vector of
    `stride` floats.  Returns alpha*X1 + beta*X2 + gamma with columns >= width times zero."""
    X1, p1 = _f32(X1)
    X2, p2 = _f32(np.ravel(X2))
    rows, stride = X1.shape
    assert stride % 4 == 0 and X2.size == stride and 0 < width <= stride
    Y = np.empty_like(X1)
    _o.oracle_linear_dual2D_row(p1, p2, stride, alpha, beta, gamma, Y.ctypes.data_as(_P),
                                rows * stride, width, stride)
    return Y


def linear2D(alpha, Xp, beta, width):
    """Xp: device-layout [rows, stride].  alpha*X + beta with the pad columns times zero."""
    Xp, px = _f32(Xp)
    stride = Xp.shape[-1]
    Y = np.empty_like(Xp)
    _o.oracle_linear2D(alpha, px, beta, Y.ctypes.data_as(_P), Xp.size, width, stride)
    return Y


def softmax2D(Xp, width, features=None, scale=1.0):
    """Xp: device-layout [rows, stride]; softmax of scale*X over groups of `features` logical
    elements (a multiple of width; default one memory row).  Pad of the result is zero."""
    Xp, px = _f32(Xp)
    rows, stride = Xp.shape
    features = width if features is None else features
    assert features % width == 0 and rows % (features // width) == 0
    row_lengthv = features // width * stride
    Y = np.empty_like(Xp)
    _o.oracle_softmax2D(px, Y.ctypes.data_as(_P), Xp.size // row_lengthv, row_lengthv, width, stride, scale)
    return Y


def attention(Q, K, V, alpha, mask=None):
    """Y = softmax(alpha * Q.K^T).V per batch entry, as the reference chains its operators
    (nn/unit/complex/block/ChannelMHA.java:74-78: batchMatMulT2, sdiv, softmax, [mask], batchMatMul).
    Logical float32 arrays Q[B, QL, dk], K[B, VL, dk], V[B, VL, dv] -> Y[B, QL, dv].  mask: a float32
    array [QL, VL] or [B, QL, VL] that multiplies the probabilities element by element after the softmax
    (one float32 product each, what an element-wise mask unit computes)."""
    def pad_last(x):
        s = (x.shape[-1] + 3) // 4 * 4
        out = np.zeros(x.shape[:-1] + (s,), np.float32)
        out[..., :x.shape[-1]] = x
        return out
    B, QL, dk = Q.shape
    VL, dv = V.shape[1], V.shape[2]
    Qp, Kp, Vp = pad_last(Q), pad_last(K), pad_last(V)
    VL4, dk4, dv4 = (VL + 3) // 4 * 4, Qp.shape[-1], Vp.shape[-1]
    P = bmm(T2, Qp, Kp, B, QL, VL4, VL, dk4)                       # [B, QL, VL4], columns >= VL zero
    P = linear2D(alpha, P.reshape(B * QL, VL4), 0.0, VL)           # sdiv(C, P) = linear(1/C, P, 0)
    P = softmax2D(P, VL)
    if mask is not None:
        Mp = np.zeros((B, QL, VL4), np.float32)
        Mp[:, :, :VL] = np.broadcast_to(np.asarray(mask, np.float32), (B, QL, VL))
        P = (P.reshape(B, QL, VL4) * Mp).astype(np.float32)
    Y = bmm(NN, P.reshape(B, QL, VL4), Vp, B, QL, dv4, VL, VL4)    # [B, QL, dv4]
    return Y[:, :, :dv]


def conv3D(X, W, sh, sw, ph, pw, OH=None, OW=None, acc32=False):
    """X[N, IH, IW, IC], W[OC, FH, FW, IC] logical arrays -> Y[N, OH, OW, OC]."""
    X, px = _f32(X)
    W, pw_ = _f32(W)
    N, IH, IW, IC = X.shape
    OC, FH, FW, IC2 = W.shape
    assert IC == IC2
    OH = (IH - FH + 2 * ph) // sh + 1 if OH is None else OH
    OW = (IW - FW + 2 * pw) // sw + 1 if OW is None else OW
    Y = np.zeros((N, OH, OW, OC), np.float32)
    _o.oracle_conv3D(px, IH, IW, pw_, FH, FW, Y.ctypes.data_as(_P), OH, OW, N, IC, OC, sh, sw, ph, pw,
                     1 if acc32 else 0)
    return Y


def transpose(Xp, dims, i1, i2):
    """Xp: device-layout array [..., stride] of a tensor with logical dims `dims` (2 to 4 of them,
    stride = last dim rounded up to 4).  Returns the device-layout array of the tensor with
    dimensions i1 and i2 exchanged, pad zero."""
    dims = list(dims)
    nd = len(dims)
    assert 2 <= nd <= 4
    Xp, px = _f32(Xp)
    d4 = [1] * (4 - nd) + dims
    a, b = i1 + 4 - nd, i2 + 4 - nd
    yd = list(dims)
    yd[i1], yd[i2] = yd[i2], yd[i1]
    sx, sy = (dims[-1] + 3) // 4 * 4, (yd[-1] + 3) // 4 * 4
    assert Xp.size == int(np.prod(dims[:-1])) * sx
    Y = np.zeros(yd[:-1] + [sy], np.float32)
    arr = (c_int * 4)(*d4)
    _o.oracle_transpose4D(px, Y.ctypes.data_as(_P), arr, a, b, sx, sy)
    return Y


def samePercent_relative(a, b, threshold=1e-3):
    a, pa = _f32(np.ravel(a))
    b, pb = _f32(np.ravel(b))
    return float(_o.oracle_samePercent_relative(pa, pb, min(a.size, b.size), threshold))


# ---- oracle/_ref: the reference's own micro.cuh helpers, when built ------------------------
def load_ref():
    """Returns the ctypes handle of oracle/_ref/libref_micro.so or None if it is not built."""
    if not os.path.exists(_REF_SO):
        return None
    try:
        return ctypes.CDLL(_REF_SO)
    except OSError:
        return None
