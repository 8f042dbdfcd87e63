// Stage 2 of the two-stage split-K product: fold the partial products into C.
//   C[i] += sum_{p < part} Cbuf[p*sizeC + i]
// with Kahan compensation, p ascending, starting from the value already in C --
// the operation order of the reference's buf_summary_kernel4
// (source/engine-cuda-base/Cuda_matMul/Cuda_matMul/SKbufsum.cuh:29-68), so the
// result is bit-identical to it.  The additions carry no multiply, so there is
// nothing for the compiler to contract; reassociation is off by default.
//
// HBM-bound: reads part*sizeC floats once.  One float4 per thread per partial;
// the loads of 8 partials are issued before the dependent Kahan chain consumes
// them so that enough bytes are in flight.
#include <hip/hip_runtime.h>
#include "gemm_mfma.h"

namespace dragon {

typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void kahan_step(v4f& v, v4f& c, v4f vbuf) {
    vbuf = vbuf - c;          // subtract the error of the previous addition
    const v4f t = v + vbuf;
    c = (t - v) - vbuf;       // recover what the addition lost
    v = t;
}

__global__ __launch_bounds__(256) void skbuf_summary_kernel(const float* __restrict__ Cbuf,
                                                            float* __restrict__ C,
                                                            int part, int size4, size_t sizeC) {
    const int stride = gridDim.x * blockDim.x;
    for (int i4 = blockIdx.x * blockDim.x + threadIdx.x; i4 < size4; i4 += stride) {
        const size_t at = (size_t)i4 * 4;
        v4f v = *(const v4f*)(C + at);
        v4f c = {0.f, 0.f, 0.f, 0.f};
        const float* src = Cbuf + at;
        int p = 0;
        for (; p + 8 <= part; p += 8) {
            v4f b[8];
#pragma unroll
            for (int u = 0; u < 8; u++)
                b[u] = __builtin_nontemporal_load((const v4f*)(src + (size_t)(p + u) * sizeC));
#pragma unroll
            for (int u = 0; u < 8; u++) kahan_step(v, c, b[u]);
        }
        for (; p < part; p++)
            kahan_step(v, c, __builtin_nontemporal_load((const v4f*)(src + (size_t)p * sizeC)));
        *(v4f*)(C + at) = v;
    }
}

hipError_t skbuf_summary_launch(hipStream_t stream, const float* Cbuf, float* C, int part,
                                int sizeC) {
    const int size4 = sizeC >> 2;
    if (size4 <= 0) return hipSuccess;
    // 64 threads per workgroup spreads a small C over many compute units.
    const int threads = 64;
    int blocks = (size4 + threads - 1) / threads;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(skbuf_summary_kernel, dim3(blocks), dim3(threads), 0, stream, Cbuf, C, part,
                       size4, (size_t)sizeC);
    return hipGetLastError();
}

}  // namespace dragon
