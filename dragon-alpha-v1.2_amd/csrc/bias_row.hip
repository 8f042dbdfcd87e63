// Y[i] = alpha*X1[i] + beta*X2[i % row_lengthv] + gamma, row vector X2 broadcast over the rows of X1,
// elements in the pad of a row (column >= width) multiplied by zero.  The reference's
// linear_dual2D_row (source/engine-cuda-base/Cuda_function/Cuda_function/type1_linear_dual2D_row.cuh:43-84),
// the second launch of matMul_biased: with alpha = beta = 1, gamma = 0 it adds the bias row to C
// (CudaFloat32EngineBase.java:1626-1634).  The expression is evaluated as written, each product
// and sum rounded on its own; for the (1, 1, 0) bias case every grouping gives the same bits.
//
// HBM-bound: reads lengthv floats, writes lengthv floats (the row vector stays in cache).
#include <hip/hip_runtime.h>
#include "gemm_mfma.h"
#include "stream_policy.h"

namespace dragon {

typedef float v4f __attribute__((ext_vector_type(4)));

#pragma clang fp contract(off)
template <bool NT>
__global__ __launch_bounds__(256) void linear_dual2D_row_kernel(const float* __restrict__ X1,
                                                                const float* __restrict__ X2,
                                                                int row_lengthv, float alpha,
                                                                float beta, float gamma,
                                                                float* __restrict__ Y, int length4,
                                                                int width, int stride) {
    const int step = gridDim.x * blockDim.x;
    for (int i4 = blockIdx.x * blockDim.x + threadIdx.x; i4 < length4; i4 += step) {
        const int index = i4 << 2;
        const v4f x1 = stream_load4<NT>(X1 + index);
        const v4f x2 = *(const v4f*)(X2 + index % row_lengthv);
        v4f y = (alpha * x1 + beta * x2) + gamma;
        const int c0 = index % stride;      // stride is a multiple of 4: the four share a row
        y.x *= (c0 + 0 < width) ? 1.0f : 0.0f;   // the reference multiplies by the 0/1 flag
        y.y *= (c0 + 1 < width) ? 1.0f : 0.0f;   // (Cuda_function/micro.cuh:61-65)
        y.z *= (c0 + 2 < width) ? 1.0f : 0.0f;
        y.w *= (c0 + 3 < width) ? 1.0f : 0.0f;
        stream_store4<NT>(Y + index, y);
    }
}

hipError_t linear_dual2D_row_launch(hipStream_t stream, const float* X1, const float* X2,
                                    int row_lengthv, float alpha, float beta, float gamma, float* Y,
                                    int lengthv, int width, int stride) {
    const int length4 = lengthv >> 2;
    if (length4 <= 0) return hipSuccess;
    // one 16-byte element per thread, workgroups in address order: measured on a 1 GiB tensor in place 6.0 TB/s,
    // against 4.7 for 8192 workgroups that stride over the tensor (neighbours in time then touch addresses far apart)
    const int blocks = (length4 + 255) / 256;
    if (stream_nt(X1, Y, (long long)lengthv * 4))
        hipLaunchKernelGGL(linear_dual2D_row_kernel<true>, dim3(blocks), dim3(256), 0, stream, X1, X2, row_lengthv,
                           alpha, beta, gamma, Y, length4, width, stride);
    else
        hipLaunchKernelGGL(linear_dual2D_row_kernel<false>, dim3(blocks), dim3(256), 0, stream, X1, X2, row_lengthv,
                           alpha, beta, gamma, Y, length4, width, stride);
    return hipGetLastError();
}

}  // namespace dragon
