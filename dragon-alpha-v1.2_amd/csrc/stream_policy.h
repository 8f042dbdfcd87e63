// Cache policy of the kernels that stream a tensor through once (element-wise, row-wise, dimension swaps).
// A tensor far larger than the 256 MB Infinity Cache gains nothing from being kept on its way through, and the
// lines it displaces are lost to everyone else: from 320 MiB of footprint on (the tensor, twice that when the
// result goes elsewhere) such kernels read and write non-temporally -- measured on 1 GiB in place 6.0 -> 6.55 TB/s
// (linear2D), 5.7 -> 6.3 (softmax2D).  Below that the caches are left to work: a 256 MiB tensor that the previous
// kernel has just written is largely served by them (7.3 TB/s in place, 6.5 with non-temporal accesses).
#pragma once
#include <hip/hip_runtime.h>

namespace dragon {

typedef float sp_v4f __attribute__((ext_vector_type(4)));

constexpr long long STREAM_NT_BYTES = 320LL << 20;

inline bool stream_nt(const void* x, const void* y, long long bytes_each) {
    return (x == y ? bytes_each : 2 * bytes_each) >= STREAM_NT_BYTES;
}

template <bool NT> __device__ __forceinline__ sp_v4f stream_load4(const float* p) {
    if constexpr (NT) return __builtin_nontemporal_load((const sp_v4f*)p);
    else return *(const sp_v4f*)p;
}
template <bool NT> __device__ __forceinline__ void stream_store4(float* p, sp_v4f v) {
    if constexpr (NT) __builtin_nontemporal_store(v, (sp_v4f*)p);
    else *(sp_v4f*)p = v;
}

}  // namespace dragon
