// The element-wise and row-wise steps between the two batched products of an attention block
// (reference: nn/unit/complex/block/ChannelMHA.java:74-78: P = softmax(Q.K^T / sqrt(d)), Y = P.V):
//   * linear2D: Y = alpha*X + beta, pad columns multiplied by zero
//     (Cuda_function.linear2D, engine-cuda-base/Cuda_function/Cuda_function/A.cu:170-183;
//     Engine.sdiv / Engine.linear call it);
//   * softmax2D: Y = softmax(scale * X) over each field of row_lengthv floats, in ONE launch that
//     reads X once and writes Y once.  The reference runs three launches with two temporary
//     buffers (row_max, row_softmax, div2D_field: CudaFloat32EngineBase.java:5738-5774) and moves
//     the tensor five times; the optional scale folds the preceding sdiv launch in as well.
// Both are bound by HBM; tensors far larger than the Infinity Cache pass through non-temporally (stream_policy.h).
#include <hip/hip_runtime.h>
#include "runtime_internal.h"
#include "stream_policy.h"
#include <stdint.h>
#include "../../include/dragon_hip_gemm.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

#pragma clang fp contract(off)
template <bool NT>
__global__ __launch_bounds__(256) void linear2D_kernel(float alpha, const float* __restrict__ X, float beta,
                                                       float* __restrict__ Y, int length4, int width, int stride) {
    const int step = gridDim.x * blockDim.x;
    for (int i4 = blockIdx.x * blockDim.x + threadIdx.x; i4 < length4; i4 += step) {
        const int index = i4 << 2;
        v4f y = alpha * dragon::stream_load4<NT>(X + index) + beta;
        const int c0 = index % stride;
        y.x *= (c0 + 0 < width) ? 1.0f : 0.0f;   // the reference multiplies by the 0/1 flag
        y.y *= (c0 + 1 < width) ? 1.0f : 0.0f;   // (Cuda_function/micro.cuh:61-65)
        y.z *= (c0 + 2 < width) ? 1.0f : 0.0f;
        y.w *= (c0 + 3 < width) ? 1.0f : 0.0f;
        dragon::stream_store4<NT>(Y + index, y);
    }
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// what pad elements and idle lanes hold: below every input, and exp(NEG_BIG - max) is an exact 0
#define NEG_BIG (-__builtin_inff())

// One wavefront per field; the field (at most 256*NV floats) stays in registers between the
// three steps max -> exp and sum -> divide.  Four fields per workgroup.
template <int NV, bool NT>
__global__ __launch_bounds__(256) void softmax_wave_kernel(const float* __restrict__ X, float* __restrict__ Y,
                                                           int field_length, int row_lengthv, int width,
                                                           int stride, float scale) {
    const int lane = threadIdx.x & 63;
    const int field = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (field >= field_length) return;
    const float* x = X + (size_t)field * row_lengthv;
    float* y = Y + (size_t)field * row_lengthv;
    v4f v[NV];
    float m = NEG_BIG;
#pragma unroll
    for (int s = 0; s < NV; s++) {
        const int i = (s * 64 + lane) * 4;
        v[s] = (v4f)(NEG_BIG);
        if (i < row_lengthv) {
            const v4f t = dragon::stream_load4<NT>(x + i) * scale;
            const int c0 = i % stride;
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (c0 + j < width) v[s][j] = t[j];
        }
        m = fmaxf(m, fmaxf(fmaxf(v[s].x, v[s].y), fmaxf(v[s].z, v[s].w)));
    }
    m = wave_max(m);
    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < NV; s++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // pad elements hold -inf: exp gives an exact 0, which is also what the pad of Y gets
            v[s][j] = expf(v[s][j] - m);
            sum += v[s][j];
        }
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int s = 0; s < NV; s++) {
        const int i = (s * 64 + lane) * 4;
        if (i < row_lengthv) dragon::stream_store4<NT>(y + i, v[s] / sum);
    }
}

// Long fields: one workgroup per field, two passes over X (the second mostly from cache): running
// maximum and rescaled sum first, then exp / sum.
__global__ __launch_bounds__(256) void softmax_block_kernel(const float* __restrict__ X, float* __restrict__ Y,
                                                            int row_lengthv, int width, int stride, float scale) {
    __shared__ float red_m[4], red_s[4];
    const float* x = X + (size_t)blockIdx.x * row_lengthv;
    float* y = Y + (size_t)blockIdx.x * row_lengthv;
    float m = NEG_BIG, sum = 0.0f;
    for (int i = threadIdx.x * 4; i < row_lengthv; i += 1024) {
        const v4f t = *(const v4f*)(x + i) * scale;
        const int c0 = i % stride;
        float lm = NEG_BIG;
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (c0 + j < width) lm = fmaxf(lm, t[j]);
        if (lm > m) { sum *= expf(m - lm); m = lm; }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (c0 + j < width) sum += expf(t[j] - m);
    }
    const float wm = wave_max(m);
    sum = wave_sum(sum * expf(m - wm));
    if ((threadIdx.x & 63) == 0) { red_m[threadIdx.x >> 6] = wm; red_s[threadIdx.x >> 6] = sum; }
    __syncthreads();
    const float M = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
    const float S = red_s[0] * expf(red_m[0] - M) + red_s[1] * expf(red_m[1] - M) +
                    red_s[2] * expf(red_m[2] - M) + red_s[3] * expf(red_m[3] - M);
    for (int i = threadIdx.x * 4; i < row_lengthv; i += 1024) {
        const v4f t = *(const v4f*)(x + i) * scale;
        const int c0 = i % stride;
        v4f o;
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = (c0 + j < width) ? expf(t[j] - M) / S : 0.0f;
        *(v4f*)(y + i) = o;
    }
}

inline bool aligned16(int64_t a) { return (a & 15) == 0; }

}  // namespace

extern "C" {

int dragon_Cuda_function_linear2D(int64_t stream, float alpha, int64_t dX, float beta, int64_t dY,
                                  int32_t lengthv, int32_t width, int32_t stride) {
    if (dX == 0 || dY == 0 || !aligned16(dX) || !aligned16(dY)) return hipErrorInvalidValue;
    if (lengthv <= 0 || (lengthv & 3) || stride <= 0 || (stride & 3) || width <= 0 || width > stride ||
        lengthv % stride != 0)
        return hipErrorInvalidValue;
    dragon::split_ledger_touch((const void*)(intptr_t)dY, (size_t)lengthv * 4);
    const int length4 = lengthv >> 2;
    // one 16-byte element per thread, workgroups in address order: measured on a 1 GiB tensor in place 6.0 TB/s,
    // against 4.7 for 8192 workgroups that stride over the tensor (neighbours in time then touch addresses far apart)
    const int blocks = (length4 + 255) / 256;
    const float* X = (const float*)(intptr_t)dX;
    float* Y = (float*)(intptr_t)dY;
    if (dragon::stream_nt(X, Y, (long long)lengthv * 4))
        hipLaunchKernelGGL(linear2D_kernel<true>, dim3(blocks), dim3(256), 0, (hipStream_t)(intptr_t)stream, alpha, X, beta, Y,
                           length4, width, stride);
    else
        hipLaunchKernelGGL(linear2D_kernel<false>, dim3(blocks), dim3(256), 0, (hipStream_t)(intptr_t)stream, alpha, X, beta, Y,
                           length4, width, stride);
    return hipGetLastError();
}

int dragon_Cuda_reduce_softmax2D(int64_t stream, int64_t dX, int64_t dY, int32_t field_length,
                                 int32_t row_lengthv, int32_t width, int32_t stride, float scale) {
    if (dX == 0 || dY == 0 || !aligned16(dX) || !aligned16(dY)) return hipErrorInvalidValue;
    if (field_length <= 0 || row_lengthv <= 0 || stride <= 0 || (stride & 3) || width <= 0 || width > stride ||
        row_lengthv % stride != 0 || (long long)field_length * row_lengthv > 0x7fffffffLL)
        return hipErrorInvalidValue;
    hipStream_t s = (hipStream_t)(intptr_t)stream;
    const float* X = (const float*)(intptr_t)dX;
    float* Y = (float*)(intptr_t)dY;
    dragon::split_ledger_touch(Y, (size_t)field_length * row_lengthv * 4);
    const dim3 grid4((field_length + 3) / 4), block(256);
    const bool nt = dragon::stream_nt(X, Y, (long long)field_length * row_lengthv * 4);
#define WAVE_CASE(NV)                                                                                              \
    do {                                                                                                           \
        if (nt) hipLaunchKernelGGL((softmax_wave_kernel<NV, true>), grid4, block, 0, s, X, Y, field_length, row_lengthv, \
                                   width, stride, scale);                                                          \
        else hipLaunchKernelGGL((softmax_wave_kernel<NV, false>), grid4, block, 0, s, X, Y, field_length, row_lengthv,   \
                                width, stride, scale);                                                             \
    } while (0)
    if (row_lengthv <= 256) WAVE_CASE(1);
    else if (row_lengthv <= 512) WAVE_CASE(2);
    else if (row_lengthv <= 1024) WAVE_CASE(4);
    else if (row_lengthv <= 2048) WAVE_CASE(8);
    else if (row_lengthv <= 4096) WAVE_CASE(16);
    else
        hipLaunchKernelGGL(softmax_block_kernel, dim3(field_length), block, 0, s, X, Y, row_lengthv, width,
                           stride, scale);
#undef WAVE_CASE
    return hipGetLastError();
}

}  // extern "C"
