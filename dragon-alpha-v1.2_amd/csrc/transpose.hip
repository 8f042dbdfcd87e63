// Swap of two dimensions of a 2-D .. 4-D tensor: Y[.., x_j, .., x_i, ..] = X[.., x_i, .., x_j, ..].
// Replaces the transpose natives of the reference's Cuda_expk2 library
// (source/engine-cuda-base/Cuda_expk2/Cuda_expk2/Cuda_transpose.cuh:13-75; dispatchers
// Cuda_transpose2D.cuh:69-84, Cuda_transpose3D.cuh:125-155, Cuda_transpose4D.cuh:125-153), the
// layout step either side of the batched products in attention blocks.
//
// Tensors are row-major with the LAST dimension stored at a stride rounded up to 4 floats, pad zero.
// Every case is handled as 4-D (missing leading dimensions are 1) by one of two kernels:
//   * the swap leaves the last dimension alone: whole padded rows move, 16 bytes per lane, reads
//     and writes both contiguous (transpose_rows_kernel);
//   * the swap involves the last dimension: 64x64 tiles of the (swapped dimension, last dimension)
//     plane go through LDS, so that the reads run along X's last dimension and the writes along
//     Y's (transpose_last_kernel).  The reference's general kernel gathers element by element with
//     strided stores (its own comments quote a third of the row-copy rate for it).
// Both are bound by HBM: one read and one write of the tensor (non-temporal for large tensors, stream_policy.h).
#include <hip/hip_runtime.h>
#include "runtime_internal.h"
#include "stream_policy.h"
#include <stdint.h>
#include "../../include/dragon_hip_gemm.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

struct Dims4 { int d[4]; };

// rows of `stride` floats; X rows indexed (x0, x1, x2), two of them swapped in Y
template <bool NT>
__global__ __launch_bounds__(256) void transpose_rows_kernel(const float* __restrict__ X, float* __restrict__ Y,
                                                             Dims4 xd, Dims4 yd, int i1, int i2, int stride,
                                                             long long rows) {
    const int c4n = stride >> 2;
    const long long n = rows * c4n;
    const long long step = (long long)gridDim.x * blockDim.x;
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < n; q += step) {
        const long long row = q / c4n;
        const int c4 = (int)(q - row * c4n);
        int x[3];
        long long t = row;
        x[2] = (int)(t % xd.d[2]); t /= xd.d[2];
        x[1] = (int)(t % xd.d[1]); t /= xd.d[1];
        x[0] = (int)t;
        const int s = x[i1]; x[i1] = x[i2]; x[i2] = s;
        const long long yrow = ((long long)x[0] * yd.d[1] + x[1]) * yd.d[2] + x[2];
        dragon::stream_store4<NT>(Y + yrow * stride + 4 * c4, dragon::stream_load4<NT>(X + row * stride + 4 * c4));
    }
}

// dimension a (0..2) swapped with the last one.  A workgroup moves one 64x64 tile of the
// (x_a, x_3) plane for one value of the two other indices.
constexpr int TP = 64;
template <bool NT>
__global__ __launch_bounds__(256) void transpose_last_kernel(const float* __restrict__ X, float* __restrict__ Y,
                                                             Dims4 xd, Dims4 yd, int a, int strideX, int strideY,
                                                             int tiles_p, int tiles_q) {
    __shared__ float tile[TP][TP + 1];
    long long b = blockIdx.x;
    // tiles are walked along diagonals of the (p, q) plane: from one workgroup to the next both the tile row
    // and the tile column move on, so neighbours differ in their X rows, X columns, Y rows and Y columns, which
    // spreads power-of-two strides over the HBM channels on both sides
    const int tq = (int)(b % tiles_q); b /= tiles_q;
    const int tp = (int)((b % tiles_p + tq) % tiles_p); b /= tiles_p;
    // the two dimensions that stay in place, o1 < o2
    const int o1 = (a == 0) ? 1 : 0, o2 = (a == 2) ? 1 : 2;
    int x[4];
    x[o2] = (int)(b % xd.d[o2]);
    x[o1] = (int)(b / xd.d[o2]);
    const int p0 = tp * TP, q0 = tq * TP;
    const int P = xd.d[a], Q = xd.d[3];

    // read: 16 lanes x 16 bytes along X's last dimension, 16 tile rows per pass.  Reading up to
    // the stride is safe and gives zeros beyond the width (the pad is zero).
    // lane -> (16-byte column lx, row ly): each half-wave covers 8 columns x 4 rows, which with the
    // row stride of 65 floats puts its 32 four-byte LDS accesses on 32 different banks, for the
    // row-wise stores here and for the column-wise loads below alike
    const int lx = (threadIdx.x & 7) | ((threadIdx.x >> 2) & 8);
    const int ly = ((threadIdx.x >> 3) & 3) | ((threadIdx.x >> 4) & 12);
    x[3] = q0 + 4 * lx;
#pragma unroll
    for (int i = 0; i < TP; i += 16) {
        x[a] = p0 + ly + i;
        v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (x[a] < P && x[3] < strideX)
            v = dragon::stream_load4<NT>(X + (((long long)x[0] * xd.d[1] + x[1]) * xd.d[2] + x[2]) * strideX + x[3]);
        tile[ly + i][4 * lx + 0] = v.x; tile[ly + i][4 * lx + 1] = v.y;
        tile[ly + i][4 * lx + 2] = v.z; tile[ly + i][4 * lx + 3] = v.w;
    }
    __syncthreads();
    // write: 16 lanes x 16 bytes along Y's last dimension (= X's dimension a); columns of the tile
    // beyond X's extent hold zeros, which is what the pad of Y's rows gets
    int y[4];
    y[o1] = x[o1]; y[o2] = x[o2];
    y[3] = p0 + 4 * lx;
#pragma unroll
    for (int i = 0; i < TP; i += 16) {
        y[a] = q0 + ly + i;
        if (y[a] < Q && y[3] < strideY) {
            const v4f v = {tile[4 * lx + 0][ly + i], tile[4 * lx + 1][ly + i], tile[4 * lx + 2][ly + i],
                           tile[4 * lx + 3][ly + i]};
            dragon::stream_store4<NT>(Y + (((long long)y[0] * yd.d[1] + y[1]) * yd.d[2] + y[2]) * strideY + y[3], v);
        }
    }
}

inline bool aligned16(int64_t a) { return (a & 15) == 0; }

// dims of X as 4-D, i1 < i2 indices into them
int transpose_launch(int64_t stream, int64_t dX, int64_t dY, Dims4 xd, int i1, int i2, int strideX, int strideY,
                     long long length) {
    if (dX == 0 || dY == 0 || !aligned16(dX) || !aligned16(dY)) return hipErrorInvalidValue;
    if (i1 > i2) { const int t = i1; i1 = i2; i2 = t; }
    if (i1 < 0 || i2 > 3 || i1 == i2) return hipErrorInvalidValue;
    for (int k = 0; k < 4; k++)
        if (xd.d[k] <= 0) return hipErrorInvalidValue;
    if ((long long)xd.d[0] * xd.d[1] * xd.d[2] * xd.d[3] != length) return hipErrorInvalidValue;
    if (strideX < xd.d[3] || (strideX & 3) || (strideY & 3)) return hipErrorInvalidValue;
    Dims4 yd = xd;
    yd.d[i1] = xd.d[i2]; yd.d[i2] = xd.d[i1];
    if (strideY < yd.d[3]) return hipErrorInvalidValue;
    hipStream_t s = (hipStream_t)(intptr_t)stream;
    const float* X = (const float*)(intptr_t)dX;
    float* Y = (float*)(intptr_t)dY;
    dragon::split_ledger_touch(Y, (size_t)yd.d[0] * yd.d[1] * yd.d[2] * (size_t)strideY * 4);
    const bool nt = dragon::stream_nt(X, Y, (long long)yd.d[0] * yd.d[1] * yd.d[2] * (long long)strideY * 4);
    if (i2 < 3) {
        if (strideX != strideY) return hipErrorInvalidValue;
        const long long rows = (long long)xd.d[0] * xd.d[1] * xd.d[2];
        const long long blocks = (rows * (strideX >> 2) + 255) / 256;   // one 16-byte element per thread, in address order
        if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
        if (nt) hipLaunchKernelGGL(transpose_rows_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, X, Y, xd, yd, i1, i2,
                                   strideX, rows);
        else hipLaunchKernelGGL(transpose_rows_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, X, Y, xd, yd, i1, i2,
                                strideX, rows);
    } else {
        const int tiles_p = (strideY + TP - 1) / TP;      // along Y's rows, pad included
        const int tiles_q = (xd.d[3] + TP - 1) / TP;
        const int o1 = (i1 == 0) ? 1 : 0, o2 = (i1 == 2) ? 1 : 2;
        const long long blocks = (long long)tiles_p * tiles_q * xd.d[o1] * xd.d[o2];
        if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
        if (nt) hipLaunchKernelGGL(transpose_last_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, X, Y, xd, yd, i1,
                                   strideX, strideY, tiles_p, tiles_q);
        else hipLaunchKernelGGL(transpose_last_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, X, Y, xd, yd, i1,
                                strideX, strideY, tiles_p, tiles_q);
    }
    return hipGetLastError();
}

}  // namespace

extern "C" {

int dragon_Cuda_expk2_transpose2D(int64_t stream, int64_t dX, int64_t dY, int32_t Xdim1, int32_t Ydim1,
                                  int32_t strideX, int32_t strideY, int32_t length) {
    if (Xdim1 <= 0 || Ydim1 <= 0 || length <= 0 || (long long)Xdim1 * Ydim1 != length)
        return hipErrorInvalidValue;
    Dims4 xd = {{1, 1, Ydim1, Xdim1}};       // X[Ydim1][Xdim1] -> Y[Xdim1][Ydim1]
    return transpose_launch(stream, dX, dY, xd, 2, 3, strideX, strideY, length);
}

int dragon_Cuda_expk2_transpose3D(int64_t stream, int64_t dX, int64_t dY, int32_t Xdim1, int32_t Xdim2,
                                  int32_t Ydim1, int32_t Ydim2, int32_t dimIndex1, int32_t dimIndex2,
                                  int32_t strideX, int32_t strideY, int32_t length) {
    if (Xdim1 <= 0 || Xdim2 <= 0 || length <= 0 || length % (Xdim1 * (long long)Xdim2) != 0)
        return hipErrorInvalidValue;
    if (dimIndex1 < 0 || dimIndex1 > 2 || dimIndex2 < 0 || dimIndex2 > 2) return hipErrorInvalidValue;
    Dims4 xd = {{1, (int)(length / (Xdim1 * (long long)Xdim2)), Xdim1, Xdim2}};
    Dims4 yd = xd;
    yd.d[dimIndex1 + 1] = xd.d[dimIndex2 + 1]; yd.d[dimIndex2 + 1] = xd.d[dimIndex1 + 1];
    if (yd.d[2] != Ydim1 || yd.d[3] != Ydim2) return hipErrorInvalidValue;
    return transpose_launch(stream, dX, dY, xd, dimIndex1 + 1, dimIndex2 + 1, strideX, strideY, length);
}

int dragon_Cuda_expk2_transpose4D(int64_t stream, int64_t dX, int64_t dY, int32_t Xdim1, int32_t Xdim2,
                                  int32_t Xdim3, int32_t Ydim1, int32_t Ydim2, int32_t Ydim3,
                                  int32_t dimIndex1, int32_t dimIndex2, int32_t strideX, int32_t strideY,
                                  int32_t length) {
    if (Xdim1 <= 0 || Xdim2 <= 0 || Xdim3 <= 0 || length <= 0) return hipErrorInvalidValue;
    const long long inner = (long long)Xdim1 * Xdim2 * Xdim3;
    if (length % inner != 0) return hipErrorInvalidValue;
    if (dimIndex1 < 0 || dimIndex1 > 3 || dimIndex2 < 0 || dimIndex2 > 3) return hipErrorInvalidValue;
    Dims4 xd = {{(int)(length / inner), Xdim1, Xdim2, Xdim3}};
    Dims4 yd = xd;
    yd.d[dimIndex1] = xd.d[dimIndex2]; yd.d[dimIndex2] = xd.d[dimIndex1];
    if (yd.d[1] != Ydim1 || yd.d[2] != Ydim2 || yd.d[3] != Ydim3) return hipErrorInvalidValue;
    return transpose_launch(stream, dX, dY, xd, dimIndex1, dimIndex2, strideX, strideY, length);
}

}  // extern "C"
