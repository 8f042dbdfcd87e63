// Runtime bridge (declared in include/dragon_hip_runtime.h): device memory,
// streams, events and float tensor transfer over the HIP runtime, one thin wrapper
// per native of the reference's Cuda class (reference implementation:
// source/engine-cuda-base/Cuda/Cuda/Cuda_memory.cuh, Cuda_Stream.cuh, Cuda_Event.cuh,
// Cuda_Device.cuh, Cuda_Exception.cuh, Cuda_float.cuh).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <atomic>
#include <vector>
#include "../../include/dragon_hip_runtime.h"
#include "../../include/dragon_hip_testing.h"
#include "runtime_internal.h"

namespace dragon {
void gemm_streamk_release_workspace(hipStream_t stream);   // gemm_mfma_streamk.hip
}
namespace {
// per host thread, like the runtime's own last error (cudaGetLastError in the reference,
// Cuda/Cuda/Cuda_Exception.cuh:21-27): one thread never takes another thread's error code
thread_local int t_last_error = 0;
}
namespace dragon_rt {
int note(hipError_t e) {
    if (e != hipSuccess) t_last_error = (int)e;
    return (int)e;
}
}  // namespace dragon_rt

namespace {

inline int note(hipError_t e) { return dragon_rt::note(e); }
inline hipStream_t as_stream(int64_t s) { return (hipStream_t)(intptr_t)s; }
inline hipEvent_t as_event(int64_t e) { return (hipEvent_t)(intptr_t)e; }
inline void* as_ptr(int64_t a) { return (void*)(intptr_t)a; }

typedef float v4f __attribute__((ext_vector_type(4)));

// X[i] = value, i < length
__global__ void fill1d_kernel(float* __restrict__ X, float value, int length) {
    const int stride = gridDim.x * blockDim.x;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < length; i += stride) X[i] = value;
}

// X[y*stride + x] = value for x < width and 0 for the pad width <= x < stride
// (reference: Cuda_float_set2D.cuh masks the value to zero outside the width).
__global__ void fill2d_kernel(float* __restrict__ X, float value, int height, int width,
                              int stride) {
    const int total = height * stride;
    const int step = gridDim.x * blockDim.x;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
        const int x = i % stride;
        X[i] = (x < width) ? value : 0.0f;
    }
}

// dst[i] = src[i] as float4: the plain copy that HBM byte counters are calibrated against
__global__ void copy4_kernel(v4f* __restrict__ dst, const v4f* __restrict__ src, long long n4) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride)
        dst[i] = src[i];
}

int launch_blocks(long long n, int threads) {
    long long b = (n + threads - 1) / threads;
    if (b < 1) b = 1;
    if (b > 4096) b = 4096;
    return (int)b;
}

}  // namespace

extern "C" {

// ---- memory --------------------------------------------------------------------
int64_t dragon_Cuda_malloc(int64_t size) {
    void* p = nullptr;
    if (size <= 0) { note(hipErrorInvalidValue); return 0; }
    if (note(hipMalloc(&p, (size_t)size)) != 0) return 0;
    return (int64_t)(intptr_t)p;
}
int dragon_Cuda_free(int64_t address) {
    dragon::split_ledger_touch(as_ptr(address), 0);
    return note(hipFree(as_ptr(address)));
}
int64_t dragon_Cuda_mallocHost(int64_t size) {
    void* p = nullptr;
    if (size <= 0) { note(hipErrorInvalidValue); return 0; }
    if (note(hipHostMalloc(&p, (size_t)size, hipHostMallocDefault)) != 0) return 0;
    return (int64_t)(intptr_t)p;
}
int dragon_Cuda_freeHost(int64_t address) { return note(hipHostFree(as_ptr(address))); }
int dragon_Cuda_memsetAsync(int64_t stream, int64_t address, int32_t value, int64_t size) {
    dragon::split_ledger_touch(as_ptr(address), (size_t)size);
    return note(hipMemsetAsync(as_ptr(address), value, (size_t)size, as_stream(stream)));
}
static int copy_async(int64_t stream, int64_t dst, int64_t src, int64_t size, hipMemcpyKind kind) {
    dragon::split_ledger_touch(as_ptr(dst), (size_t)size);   // a host destination never matches a device range
    return note(hipMemcpyAsync(as_ptr(dst), as_ptr(src), (size_t)size, kind, as_stream(stream)));
}
int dragon_Cuda_memcpyAsyncHostToDevice(int64_t s, int64_t dst, int64_t src, int64_t size) {
    return copy_async(s, dst, src, size, hipMemcpyHostToDevice);
}
int dragon_Cuda_memcpyAsyncHostToHost(int64_t s, int64_t dst, int64_t src, int64_t size) {
    return copy_async(s, dst, src, size, hipMemcpyHostToHost);
}
int dragon_Cuda_memcpyAsyncDeviceToHost(int64_t s, int64_t dst, int64_t src, int64_t size) {
    return copy_async(s, dst, src, size, hipMemcpyDeviceToHost);
}
int dragon_Cuda_memcpyAsyncDeviceToDevice(int64_t s, int64_t dst, int64_t src, int64_t size) {
    return copy_async(s, dst, src, size, hipMemcpyDeviceToDevice);
}
int dragon_Cuda_memcpyAsyncDefault(int64_t s, int64_t dst, int64_t src, int64_t size) {
    return copy_async(s, dst, src, size, hipMemcpyDefault);
}

// ---- device --------------------------------------------------------------------
int32_t dragon_Cuda_getDeviceId(void) {
    int d = -1;
    if (note(hipGetDevice(&d)) != 0) return -1;
    return d;
}
int32_t dragon_Cuda_getDeviceCount(void) {
    int n = 0;
    if (note(hipGetDeviceCount(&n)) != 0) return 0;
    return n;
}
int dragon_Cuda_setDevice(int32_t dev_id) { return note(hipSetDevice(dev_id)); }
int dragon_Cuda_deviceSynchronize(void) { return note(hipDeviceSynchronize()); }
int32_t dragon_CudaDevice_multiProcessorCount(int32_t dev_id) {
    int n = 0;
    if (note(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev_id)) != 0)
        return 0;
    return n;
}

// ---- streams (default priority only) ---------------------------------------------
int64_t dragon_Cuda_newStream_Blocking(void) {
    hipStream_t s = nullptr;
    if (note(hipStreamCreateWithFlags(&s, hipStreamDefault)) != 0) return 0;
    return (int64_t)(intptr_t)s;
}
int64_t dragon_Cuda_newStream_NonBlocking(void) {
    hipStream_t s = nullptr;
    if (note(hipStreamCreateWithFlags(&s, hipStreamNonBlocking)) != 0) return 0;
    return (int64_t)(intptr_t)s;
}
// A stream that has launched the balanced product kernel owns a workspace in device memory (the library's only
// allocation); it goes with the stream.
int dragon_Cuda_deleteStream(int64_t stream) {
    if (stream == 0) return 0;  // the default stream is never destroyed
    dragon::gemm_streamk_release_workspace(as_stream(stream));
    return note(hipStreamDestroy(as_stream(stream)));
}
int dragon_Cuda_deleteStreams(const int64_t* streams, int32_t length) {
    int rc = 0;
    for (int i = 0; i < length; i++) {
        if (streams[i] == 0) continue;
        dragon::gemm_streamk_release_workspace(as_stream(streams[i]));
        int e = note(hipStreamDestroy(as_stream(streams[i])));
        if (e && !rc) rc = e;
    }
    return rc;
}
int32_t dragon_Cuda_streamQuery(int64_t stream) {
    hipError_t e = hipStreamQuery(as_stream(stream));
    if (e == hipSuccess) return 1;
    if (e == hipErrorNotReady) return 0;
    note(e);
    return -1;
}
int dragon_Cuda_streamSynchronize(int64_t stream) {
    return note(hipStreamSynchronize(as_stream(stream)));
}
int dragon_Cuda_streamsSynchronize(const int64_t* streams, int32_t length) {
    int rc = 0;
    for (int i = 0; i < length; i++) {
        int e = note(hipStreamSynchronize(as_stream(streams[i])));
        if (e && !rc) rc = e;
    }
    return rc;
}

// ---- events ----------------------------------------------------------------------
static int64_t new_event(unsigned flags) {
    hipEvent_t ev = nullptr;
    if (note(hipEventCreateWithFlags(&ev, flags)) != 0) return 0;
    return (int64_t)(intptr_t)ev;
}
int64_t dragon_Cuda_newEvent_Default(void) { return new_event(hipEventDefault); }
int64_t dragon_Cuda_newEvent_BlockingSync(void) { return new_event(hipEventBlockingSync); }
int64_t dragon_Cuda_newEvent_DisableTiming(void) { return new_event(hipEventDisableTiming); }
int dragon_Cuda_deleteEvent(int64_t event) { return note(hipEventDestroy(as_event(event))); }
int dragon_Cuda_eventRecord(int64_t event, int64_t stream) {
    return note(hipEventRecord(as_event(event), as_stream(stream)));
}
int dragon_Cuda_eventRecord_streams(int64_t event, const int64_t* streams, int32_t length) {
    if (streams == nullptr || length < 1) return note(hipErrorInvalidValue);
    // join streams[1..] into streams[0], then record there
    for (int i = 1; i < length; i++) {
        if (streams[i] == streams[0]) continue;
        hipEvent_t j = nullptr;
        int e = note(hipEventCreateWithFlags(&j, hipEventDisableTiming));
        if (e) return e;
        e = note(hipEventRecord(j, as_stream(streams[i])));
        if (!e) e = note(hipStreamWaitEvent(as_stream(streams[0]), j, 0));
        hipError_t d = hipEventDestroy(j);  // destruction is deferred until the event completes
        if (e) return e;
        if (d != hipSuccess) return note(d);
    }
    return note(hipEventRecord(as_event(event), as_stream(streams[0])));
}
int dragon_Cuda_eventSynchronize(int64_t event) {
    return note(hipEventSynchronize(as_event(event)));
}
int dragon_Cuda_eventSync_Del(int64_t event) {
    int e = note(hipEventSynchronize(as_event(event)));
    int d = note(hipEventDestroy(as_event(event)));
    return e ? e : d;
}
float dragon_Cuda_eventElapsedTime(int64_t start_event, int64_t stop_event) {
    float ms = -1.0f;
    if (note(hipEventElapsedTime(&ms, as_event(start_event), as_event(stop_event))) != 0)
        return -1.0f;
    return ms;
}
int dragon_Cuda_streamWaitEvent_default(int64_t stream, int64_t event) {
    return note(hipStreamWaitEvent(as_stream(stream), as_event(event), 0));
}
int dragon_Cuda_streamsWaitEvent_default(const int64_t* streams, int32_t length, int64_t event) {
    int rc = 0;
    for (int i = 0; i < length; i++) {
        int e = note(hipStreamWaitEvent(as_stream(streams[i]), as_event(event), 0));
        if (e && !rc) rc = e;
    }
    return rc;
}

// ---- errors ----------------------------------------------------------------------
const char* dragon_Cuda_getExceptionName(int32_t type) { return hipGetErrorName((hipError_t)type); }
const char* dragon_Cuda_getExceptionInfo(int32_t type) { return hipGetErrorString((hipError_t)type); }
int32_t dragon_Cuda_getLastExceptionType(void) {
    const int e = t_last_error;
    t_last_error = 0;
    hipError_t h = hipGetLastError();
    return e ? e : (int)h;
}

// ---- float fill / transfer ---------------------------------------------------------
int dragon_Cuda_set1D_value(int64_t stream, int64_t address, float value, int32_t length) {
    if (address == 0 || length <= 0) return note(hipErrorInvalidValue);
    dragon::split_ledger_touch(as_ptr(address), (size_t)length * 4);
    hipLaunchKernelGGL(fill1d_kernel, dim3(launch_blocks(length, 256)), dim3(256), 0,
                       as_stream(stream), (float*)as_ptr(address), value, length);
    return note(hipGetLastError());
}
int dragon_Cuda_set2D_value(int64_t stream, int64_t address, float value, int32_t height,
                            int32_t width, int32_t stride) {
    if (address == 0 || height <= 0 || width <= 0 || stride < width) return note(hipErrorInvalidValue);
    dragon::split_ledger_touch(as_ptr(address), (size_t)height * stride * 4);
    hipLaunchKernelGGL(fill2d_kernel, dim3(launch_blocks((long long)height * stride, 256)),
                       dim3(256), 0, as_stream(stream), (float*)as_ptr(address), value, height,
                       width, stride);
    return note(hipGetLastError());
}

int dragon_test_mem_get_info(int64_t* free_bytes, int64_t* total_bytes) {
    size_t f = 0, t = 0;
    const int e = note(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = (int64_t)f;
    if (total_bytes) *total_bytes = (int64_t)t;
    return e;
}
int dragon_test_copy1D_kernel(int64_t stream, int64_t dst, int64_t src, int64_t length) {
    if (dst == 0 || src == 0 || length <= 0 || (length & 3) || ((dst | src) & 15))
        return note(hipErrorInvalidValue);
    const long long n4 = length >> 2;
    dragon::split_ledger_touch(as_ptr(dst), (size_t)length * 4);
    hipLaunchKernelGGL(copy4_kernel, dim3(launch_blocks(n4, 256)), dim3(256), 0, as_stream(stream),
                       (v4f*)as_ptr(dst), (const v4f*)as_ptr(src), n4);
    return note(hipGetLastError());
}

}  // extern "C"
