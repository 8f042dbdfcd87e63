// Stage 2 of the two-stage split-K product: fold the partial products into C.
//   C[i] += sum_{p < part} Cbuf[p*sizeC + i]
// with Kahan compensation, p ascending, starting from the value already in C --
// the operation order of the reference's buf_summary_kernel4
// (source/engine-cuda-base/Cuda_matMul/Cuda_matMul/SKbufsum.cuh:29-68), so the
// result is bit-identical to it.  The additions carry no multiply, so there is
// nothing for the compiler to contract; reassociation is off by default.
//
// HBM-bound: reads part*sizeC floats once.  The sum over the partials is a serial
// chain per element, so the bytes in flight come from the elements: a C of at least
// 1M floats uses one float4 per thread, a smaller one a single float per thread (four
// times the threads), and the loads of 16 partials (64 for a small C with 48 partials or more) are issued ahead
// of the chain.
#include <hip/hip_runtime.h>
#include "gemm_mfma.h"

namespace dragon {

typedef float v4f __attribute__((ext_vector_type(4)));

template <typename V>
__device__ __forceinline__ void kahan_step(V& v, V& c, V vbuf) {
    vbuf = vbuf - c;          // subtract the error of the previous addition
    const V t = v + vbuf;
    c = (t - v) - vbuf;       // recover what the addition lost
    v = t;
}

template <typename V, int AHEAD>
__global__ __launch_bounds__(256) void skbuf_summary_kernel(const float* __restrict__ Cbuf,
                                                            float* __restrict__ C,
                                                            int part, int nvec, size_t sizeC) {
    constexpr int W = sizeof(V) / sizeof(float);
    const int stride = gridDim.x * blockDim.x;
    for (int iv = blockIdx.x * blockDim.x + threadIdx.x; iv < nvec; iv += stride) {
        const size_t at = (size_t)iv * W;
        V v = *(const V*)(C + at);
        V c = (V)(0.0f);
        const float* src = Cbuf + at;
        int p = 0;
        for (; p + AHEAD <= part; p += AHEAD) {
            V b[AHEAD];
#pragma unroll
            for (int u = 0; u < AHEAD; u++)
                b[u] = __builtin_nontemporal_load((const V*)(src + (size_t)(p + u) * sizeC));
#pragma unroll
            for (int u = 0; u < AHEAD; u++) kahan_step(v, c, b[u]);
        }
        if (p < part) {      // the remainder: its loads go out together as well
            V b[AHEAD - 1];
#pragma unroll
            for (int u = 0; u < AHEAD - 1; u++)
                if (p + u < part) b[u] = __builtin_nontemporal_load((const V*)(src + (size_t)(p + u) * sizeC));
#pragma unroll
            for (int u = 0; u < AHEAD - 1; u++)
                if (p + u < part) kahan_step(v, c, b[u]);
        }
        *(V*)(C + at) = v;
    }
}

hipError_t skbuf_summary_launch(hipStream_t stream, const float* Cbuf, float* C, int part,
                                int sizeC) {
    if (sizeC <= 0) return hipSuccess;
    const int threads = 64;   // small workgroups spread a small C over many compute units
    if (sizeC >= (1 << 20)) {
        const int nvec = sizeC >> 2;
        int blocks = (nvec + threads - 1) / threads;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL((skbuf_summary_kernel<v4f, 16>), dim3(blocks), dim3(threads), 0, stream, Cbuf,
                           C, part, nvec, (size_t)sizeC);
    } else {
        const int blocks = (sizeC + threads - 1) / threads;
        // many partials of a small C (the tall-K weight gradient: 127 x 65536): few elements, so each thread keeps
        // 64 loads on their way (8.8 -> 6.4 us); the remainder's loads are predicated one by one, which a short
        // fold does not earn back (part = 1: 4.9 -> 12.8 us), so it keeps 16
        if (part >= 48)
            hipLaunchKernelGGL((skbuf_summary_kernel<float, 64>), dim3(blocks), dim3(threads), 0, stream, Cbuf,
                               C, part, sizeC, (size_t)sizeC);
        else
            hipLaunchKernelGGL((skbuf_summary_kernel<float, 16>), dim3(blocks), dim3(threads), 0, stream, Cbuf,
                               C, part, sizeC, (size_t)sizeC);
    }
    return hipGetLastError();
}

}  // namespace dragon
