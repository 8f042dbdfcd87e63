// Host <-> device transfer of float tensors: the get/set natives of the reference's Cuda class
// (source/engine-cuda-base/Cuda/Cuda/Cuda_float.cuh:45-165 download, :214-368 upload; declared in
// include/dragon_hip_runtime.h).
//
// The reference stages through a host buffer: upload = CPU loop that spreads packed rows of
// `width` floats to rows of `stride` floats, then ONE copy of height*stride floats, then a wait;
// download the reverse.  With a pinned staging buffer (the _v2 natives, fed by the engine's
// PinnedMempool) this file does it differently:
//   * the staging buffer holds the PACKED data and a kernel reads it (or writes it) in place over
//     the host link: the pad never crosses the link, and the re-layout costs no CPU time;
//   * the transfer is cut into chunks, so the CPU copy of chunk i+1 between the caller's array and
//     the staging buffer overlaps the device's transfer of chunk i; long transfers share the CPU
//     copies between the calling thread and one helper.  Every chunk has its own region
//     of the staging buffer (it is as large as the whole tensor), so no region is reused and the
//     only synchronisation is "chunk i has arrived" on the download side.
// Device rows are written whole: the pad columns of an upload are zeroed by the device.
// A staging buffer that is not pinned host memory (or none: the plain natives) takes the
// reference's route, since a kernel must not touch pageable memory.
// All entry points return after the data has arrived (stream-synchronous, like the reference's).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <atomic>
#include <thread>
#include <vector>
#include "../../include/dragon_hip_runtime.h"
#include "runtime_internal.h"

namespace {

using dragon_rt::note;
typedef float v4f __attribute__((ext_vector_type(4)));

inline hipStream_t as_stream(int64_t s) { return (hipStream_t)(intptr_t)s; }
inline void* as_ptr(int64_t a) { return (void*)(intptr_t)a; }

constexpr long long CHUNK_FLOATS = 2LL << 20;   // 8 MiB per chunk
constexpr int MAX_CHUNKS = 64;

// packed[i0 .. i0+count) -> dst[(i / width) * stride + i % width]; i0 and count multiples of 4
// except at the very end.  One aligned 16-byte load per thread from the packed source (the host
// buffer, read over the link: a wave reads 1 KiB of consecutive bytes), four 4-byte stores.
__global__ __launch_bounds__(256) void spread_rows_kernel(const float* __restrict__ packed,
                                                          float* __restrict__ dst, long long i0,
                                                          long long count, long long total, int width,
                                                          int stride) {
    const long long n4 = (count + 3) >> 2;
    const long long step = (long long)gridDim.x * blockDim.x;
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < n4; q += step) {
        const long long i = i0 + 4 * q;
        const v4f v = *(const v4f*)(packed + i);     // the buffer holds at least ceil4(total) floats
        long long row = i / width;
        int col = (int)(i - row * width);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (i + j < total) dst[row * stride + col] = v[j];
            if (++col == width) { col = 0; row++; }
        }
    }
}

// zeros in the pad columns width..stride-1 of every row
__global__ __launch_bounds__(256) void zero_pad_kernel(float* __restrict__ dst, int height, int width,
                                                       int stride) {
    const int pad = stride - width;
    const long long n = (long long)height * pad;
    const long long step = (long long)gridDim.x * blockDim.x;
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < n; q += step) {
        const long long row = q / pad;
        dst[row * stride + width + (int)(q - row * pad)] = 0.0f;
    }
}

// src[(i / width) * stride + i % width] -> packed[i0 .. i0+count): four 4-byte loads from device
// memory, one aligned 16-byte store per thread into the host buffer.
__global__ __launch_bounds__(256) void gather_rows_kernel(const float* __restrict__ src,
                                                          float* __restrict__ packed, long long i0,
                                                          long long count, long long total, int width,
                                                          int stride) {
    const long long n4 = (count + 3) >> 2;
    const long long step = (long long)gridDim.x * blockDim.x;
    for (long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x; q < n4; q += step) {
        const long long i = i0 + 4 * q;
        long long row = i / width;
        int col = (int)(i - row * width);
        v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (i + j < total) v[j] = src[row * stride + col];
            if (++col == width) { col = 0; row++; }
        }
        *(v4f*)(packed + i) = v;
    }
}

int blocks_for(long long n, int threads) {
    long long b = (n + threads - 1) / threads;
    return (int)(b < 1 ? 1 : (b > 2048 ? 2048 : b));
}

// true if a kernel on the current device may dereference p (pinned / registered host memory)
bool device_can_touch(const void* p) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();   // a pageable pointer is not an error of the caller's
        return false;
    }
    return attr.type == hipMemoryTypeHost && attr.devicePointer != nullptr;
}

// chunk i of n floats: [lo, hi), boundaries multiples of 4
struct Chunks {
    long long n, size;
    int count;
    explicit Chunks(long long total) : n(total) {
        size = CHUNK_FLOATS;
        if ((n + size - 1) / size > MAX_CHUNKS) size = (((n + MAX_CHUNKS - 1) / MAX_CHUNKS) + 3) & ~3LL;
        count = (int)((n + size - 1) / size);
        if (count < 1) count = 1;
    }
    long long lo(int i) const { return i * size; }
    long long hi(int i) const { long long h = (i + 1) * size; return h < n ? h : n; }
};

int sync(hipStream_t s) { return note(hipStreamSynchronize(s)); }

// Runs body(i) for every chunk i, on the calling thread alone for short transfers and shared with
// one helper thread for long ones (one core's memcpy is slower than the host link).  The chunks are
// independent: each has its own region of the staging buffer and of the tensor.  Returns the first
// failure; the helper works on the caller's device.
template <typename F>
int for_each_chunk(int count, F body) {
    if (count < 4) {
        for (int i = 0; i < count; i++)
            if (int e = body(i)) return e;
        return 0;
    }
    int dev = 0;
    (void)hipGetDevice(&dev);
    std::atomic<int> next{0}, err{0};
    auto work = [&] {
        for (;;) {
            const int i = next.fetch_add(1);
            if (i >= count || err.load()) return;
            if (int e = body(i)) { err.store(e); return; }
        }
    };
    std::thread helper([&] { if (hipSetDevice(dev) == hipSuccess) work(); });
    work();
    helper.join();
    return err.load();
}

// ---- the reference's route: CPU re-layout in the staging buffer, one copy ----------------------
void expand_rows(float* dst, const float* src, int height, int width, int stride) {
    for (int y = 0; y < height; y++) {
        memcpy(dst + (size_t)y * stride, src + (size_t)y * width, sizeof(float) * (size_t)width);
        for (int x = width; x < stride; x++) dst[(size_t)y * stride + x] = 0.0f;
    }
}
void compact_rows(float* dst, const float* src, int height, int width, int stride) {
    for (int y = 0; y < height; y++)
        memcpy(dst + (size_t)y * width, src + (size_t)y * stride, sizeof(float) * (size_t)width);
}
int upload_staged(hipStream_t s, float* dX, const float* value, float* buf, int height, int width,
                  int stride) {
    expand_rows(buf, value, height, width, stride);
    int e = note(hipMemcpyAsync(dX, buf, sizeof(float) * (size_t)height * stride, hipMemcpyHostToDevice, s));
    return e ? e : sync(s);
}
int download_staged(hipStream_t s, const float* dX, float* value, float* buf, int height, int width,
                    int stride) {
    int e = note(hipMemcpyAsync(buf, dX, sizeof(float) * (size_t)height * stride, hipMemcpyDeviceToHost, s));
    if (e || (e = sync(s))) return e;
    compact_rows(value, buf, height, width, stride);
    return 0;
}

// ---- contiguous data through a pinned buffer, chunk by chunk --------------------------------------
int upload_linear(hipStream_t s, float* dX, const float* value, float* buf, long long n) {
    const Chunks c(n);
    const int e = for_each_chunk(c.count, [&](int i) {
        const long long lo = c.lo(i), cnt = c.hi(i) - lo;
        memcpy(buf + lo, value + lo, sizeof(float) * (size_t)cnt);
        return note(hipMemcpyAsync(dX + lo, buf + lo, sizeof(float) * (size_t)cnt, hipMemcpyHostToDevice, s));
    });
    const int w = sync(s);     // also on failure: nothing may still read the buffer when we return
    return e ? e : w;
}

struct EventList {
    std::vector<hipEvent_t> ev;
    ~EventList() { for (hipEvent_t e : ev) (void)hipEventDestroy(e); }
    int add(hipStream_t s) {
        hipEvent_t e;
        int rc = note(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        if (rc) return rc;
        ev.push_back(e);
        return note(hipEventRecord(e, s));
    }
};

// chunk i has arrived in the staging buffer when its event has completed: copy it out
int drain(hipStream_t s, const Chunks& c, EventList& done, float* value, const float* buf) {
    const int e = for_each_chunk(c.count, [&](int i) {
        if (int w = note(hipEventSynchronize(done.ev[i]))) return w;
        const long long lo = c.lo(i);
        memcpy(value + lo, buf + lo, sizeof(float) * (size_t)(c.hi(i) - lo));
        return 0;
    });
    if (e) (void)hipStreamSynchronize(s);
    return e;
}

int download_linear(hipStream_t s, const float* dX, float* value, float* buf, long long n) {
    const Chunks c(n);
    EventList done;
    for (int i = 0; i < c.count; i++) {
        const long long lo = c.lo(i), cnt = c.hi(i) - lo;
        int e = note(hipMemcpyAsync(buf + lo, dX + lo, sizeof(float) * (size_t)cnt, hipMemcpyDeviceToHost, s));
        if (!e) e = done.add(s);
        if (e) { (void)hipStreamSynchronize(s); return e; }
    }
    return drain(s, c, done, value, buf);
}

// ---- strided rows through a pinned buffer that the device reads / writes in place ----------------
int upload_rows(hipStream_t s, float* dX, const float* value, float* buf, int height, int width, int stride) {
    const long long n = (long long)height * width;
    const Chunks c(n);
    hipLaunchKernelGGL(zero_pad_kernel, dim3(blocks_for((long long)height * (stride - width), 256)), dim3(256),
                       0, s, dX, height, width, stride);
    int e = note(hipGetLastError());
    if (!e) e = for_each_chunk(c.count, [&](int i) {
        const long long lo = c.lo(i), cnt = c.hi(i) - lo;
        memcpy(buf + lo, value + lo, sizeof(float) * (size_t)cnt);
        hipLaunchKernelGGL(spread_rows_kernel, dim3(blocks_for((cnt + 3) >> 2, 256)), dim3(256), 0, s,
                           (const float*)buf, dX, lo, cnt, n, width, stride);
        return note(hipGetLastError());
    });
    const int w = sync(s);     // also on failure: nothing may still read the buffer when we return
    return e ? e : w;
}
int download_rows(hipStream_t s, const float* dX, float* value, float* buf, int height, int width, int stride) {
    const long long n = (long long)height * width;
    const Chunks c(n);
    EventList done;
    int e = 0;
    for (int i = 0; i < c.count && !e; i++) {
        const long long lo = c.lo(i), cnt = c.hi(i) - lo;
        hipLaunchKernelGGL(gather_rows_kernel, dim3(blocks_for((cnt + 3) >> 2, 256)), dim3(256), 0, s, dX,
                           buf, lo, cnt, n, width, stride);
        e = note(hipGetLastError());
        if (!e) e = done.add(s);
    }
    if (e) { (void)hipStreamSynchronize(s); return e; }
    return drain(s, c, done, value, buf);
}

bool bad2d(int64_t address, const void* value, int height, int width, int stride) {
    return address == 0 || value == nullptr || height <= 0 || width <= 0 || stride < width ||
           (long long)height * stride > 0x7fffffffLL;
}

}  // namespace

extern "C" {

int dragon_Cuda_get1D(int64_t stream, int64_t address, float* value, int32_t length) {
    if (address == 0 || value == nullptr || length <= 0) return note(hipErrorInvalidValue);
    hipStream_t s = as_stream(stream);
    int e = note(hipMemcpyAsync(value, as_ptr(address), sizeof(float) * (size_t)length, hipMemcpyDeviceToHost, s));
    return e ? e : sync(s);
}
int dragon_Cuda_set1D(int64_t stream, int64_t address, const float* value, int32_t length) {
    if (address == 0 || value == nullptr || length <= 0) return note(hipErrorInvalidValue);
    dragon::split_ledger_touch(as_ptr(address), (size_t)length * 4);
    hipStream_t s = as_stream(stream);
    int e = note(hipMemcpyAsync(as_ptr(address), value, sizeof(float) * (size_t)length, hipMemcpyHostToDevice, s));
    return e ? e : sync(s);
}
int dragon_Cuda_get1D_v2(int64_t stream, int64_t address, float* value, int64_t buf, int32_t length) {
    if (address == 0 || value == nullptr || buf == 0 || length <= 0) return note(hipErrorInvalidValue);
    return download_linear(as_stream(stream), (const float*)as_ptr(address), value, (float*)as_ptr(buf), length);
}
int dragon_Cuda_set1D_v2(int64_t stream, int64_t address, const float* value, int64_t buf, int32_t length) {
    if (address == 0 || value == nullptr || buf == 0 || length <= 0) return note(hipErrorInvalidValue);
    dragon::split_ledger_touch(as_ptr(address), (size_t)length * 4);
    return upload_linear(as_stream(stream), (float*)as_ptr(address), value, (float*)as_ptr(buf), length);
}

int dragon_Cuda_get2D_v2(int64_t stream, int64_t address, float* value, int64_t buf, int32_t height,
                         int32_t width, int32_t stride) {
    if (bad2d(address, value, height, width, stride) || buf == 0) return note(hipErrorInvalidValue);
    hipStream_t s = as_stream(stream);
    const float* dX = (const float*)as_ptr(address);
    float* b = (float*)as_ptr(buf);
    if (width == stride) return download_linear(s, dX, value, b, (long long)height * width);
    if (device_can_touch(b) && (buf & 15) == 0) return download_rows(s, dX, value, b, height, width, stride);
    return download_staged(s, dX, value, b, height, width, stride);
}
int dragon_Cuda_set2D_v2(int64_t stream, int64_t address, const float* value, int64_t buf, int32_t height,
                         int32_t width, int32_t stride) {
    if (bad2d(address, value, height, width, stride) || buf == 0) return note(hipErrorInvalidValue);
    dragon::split_ledger_touch(as_ptr(address), (size_t)height * stride * 4);
    hipStream_t s = as_stream(stream);
    float* dX = (float*)as_ptr(address);
    float* b = (float*)as_ptr(buf);
    if (width == stride) return upload_linear(s, dX, value, b, (long long)height * width);
    if (device_can_touch(b) && (buf & 15) == 0) return upload_rows(s, dX, value, b, height, width, stride);
    return upload_staged(s, dX, value, b, height, width, stride);
}

// no staging buffer from the caller: the reference allocates a pageable one per call, so does this
int dragon_Cuda_get2D(int64_t stream, int64_t address, float* value, int32_t height, int32_t width,
                      int32_t stride) {
    if (bad2d(address, value, height, width, stride)) return note(hipErrorInvalidValue);
    if (width == stride) return dragon_Cuda_get1D(stream, address, value, height * width);
    std::vector<float> staging((size_t)height * stride);
    return download_staged(as_stream(stream), (const float*)as_ptr(address), value, staging.data(), height,
                           width, stride);
}
int dragon_Cuda_set2D(int64_t stream, int64_t address, const float* value, int32_t height, int32_t width,
                      int32_t stride) {
    if (bad2d(address, value, height, width, stride)) return note(hipErrorInvalidValue);
    if (width == stride) return dragon_Cuda_set1D(stream, address, value, height * width);
    dragon::split_ledger_touch(as_ptr(address), (size_t)height * stride * 4);
    std::vector<float> staging((size_t)height * stride);
    return upload_staged(as_stream(stream), (float*)as_ptr(address), value, staging.data(), height, width,
                         stride);
}

}  // extern "C"
