// C-ABI entry points of the matrix-multiplication engine (declared in
// include/dragon_hip_gemm.h).  Each one validates its arguments, translates the
// reference's (N, M, K, ...) argument list into the operand bounds of the one
// guarded kernel, and launches on streams[0].
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <atomic>
#include <mutex>
#include <vector>
#include "gemm_mfma.h"
#include "runtime_internal.h"
#include "../../include/dragon_hip_gemm.h"
#include "../../include/dragon_hip_testing.h"

using namespace dragon;

namespace {

constexpr int MAX_STREAMS = 10;  // the reference copies the handles into jlong streams[10]

inline bool aligned16(int64_t a) { return (a & 15) == 0; }

// How the split-K entry points treat the caller's GridZ: -1 the estimate decides (gemm_split_loses), 0 always
// as asked, 1 declined wherever the unsplit product can take the balanced kernel.  A test hook, per thread.
thread_local int t_split_policy = -1;
std::atomic<long long> g_declined{0};   // split-K calls that ran unsplit (read by tests)

// ---- the ledger of declined splits ------------------------------------------------------------------------
// A declined split leaves the whole product in C and zeros in the partial buffers; the fold the host then asks
// for (SKbuf_summary with the same stream, Cbuf, C, part and sizeC) would add zeros to C: a launch, three
// passes over C, and no change.  The entry point remembers the call here, and SKbuf_summary, finding its exact
// arguments, returns without launching.  An entry dies with its first use, with any write the library sees to
// its C or its partial buffers (every entry point that writes device memory reports the range), with a free of
// that memory, and when 64 younger ones exist; the buffers hold their zeros in any case, so a fold that does run
// (another stream, other arguments, an entry that died) is right as well.
struct DeclinedSplit { int dev; hipStream_t stream; uintptr_t cbuf, cbuf_end, c, c_end; int part, sizeC; };
std::mutex g_led_mutex;
std::vector<DeclinedSplit> g_led;
std::atomic<int> g_led_n{0};
std::atomic<int> g_fold_skip{1};          // test hook: 0 = every fold is launched
std::atomic<long long> g_folds_skipped{0};

void ledger_note(hipStream_t stream, int64_t dCbuf, int64_t dC, int part, int sizeC) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return;
    const uintptr_t cb = (uintptr_t)dCbuf, c = (uintptr_t)dC;
    std::lock_guard<std::mutex> lock(g_led_mutex);
    if (g_led.size() >= 64) g_led.erase(g_led.begin());
    g_led.push_back({dev, stream, cb, cb + (uintptr_t)part * (uintptr_t)sizeC * 4, c, c + (uintptr_t)sizeC * 4, part, sizeC});
    g_led_n.store((int)g_led.size(), std::memory_order_release);
}

// true: this fold is the no-op that follows a declined split
bool ledger_fold_is_noop(hipStream_t stream, int64_t dCbuf, int64_t dC, int part, int sizeC) {
    if (g_led_n.load(std::memory_order_acquire) == 0) return false;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    std::lock_guard<std::mutex> lock(g_led_mutex);
    for (size_t i = 0; i < g_led.size(); i++) {
        const DeclinedSplit& e = g_led[i];
        if (e.cbuf != (uintptr_t)dCbuf) continue;
        const bool same = e.dev == dev && e.stream == stream && e.c == (uintptr_t)dC && e.part == part && e.sizeC == sizeC;
        g_led.erase(g_led.begin() + i);
        g_led_n.store((int)g_led.size(), std::memory_order_release);
        return same && g_fold_skip.load(std::memory_order_relaxed) != 0;
    }
    return false;
}

inline void touch(int64_t address, long long floats) { split_ledger_touch((const void*)(intptr_t)address, (size_t)floats * 4); }

bool split_declined(int variant, int N, int M, int gz, int K, int k_slice, int num_cu) {
    if (gemm_forced_tile() != TILE_AUTO || t_split_policy == 0) return false;
    if (t_split_policy == 1) return k_slice >= 32 && gemm_choose_streamk(N, M, 1, K, num_cu, variant) >= 0;
    return gemm_split_loses(variant, N, M, gz, K, k_slice, num_cu);
}
inline bool x4(int v) { return (v & 3) == 0; }

int check_common(const int64_t* streams, int length, int64_t dA, int64_t dB, int64_t dC) {
    if (streams == nullptr || length < 1 || length > MAX_STREAMS) return hipErrorInvalidValue;
    if (dA == 0 || dB == 0 || dC == 0) return hipErrorInvalidValue;
    if (!aligned16(dA) || !aligned16(dB) || !aligned16(dC)) return hipErrorInvalidValue;
    return hipSuccess;
}

// 2-D products, optionally cut into gz K slices.  sk_ws: a workspace of GEMM_SK_WS_FLOATS_256CU floats for the
// balanced kernel, from a caller that may not allocate (the kernel otherwise makes one per stream at its first
// launch there).
int matmul_2d(int variant, const int64_t* streams, int length, int gz, int64_t dA, int64_t dB,
              int64_t dC, int64_t dCbuf, int N, int M, int K, int64_t dBias = 0, int bias_rows = 0,
              int bias_width = 0, float* sk_ws = nullptr) {
    int e = check_common(streams, length, dA, dB, dC);
    if (e) return e;
    if (N <= 0 || M <= 0 || K <= 0 || gz < 1) return hipErrorInvalidValue;
    if (!x4(N) || !x4(M) || !x4(K)) return hipErrorInvalidValue;
    if (gz > 1 && (dCbuf == 0 || !aligned16(dCbuf))) return hipErrorInvalidValue;
    if ((long long)N * M > 0x7fffffffLL) return hipErrorInvalidValue;

    touch(dC, (long long)N * M);
    if (gz > 1) touch(dCbuf, (long long)(gz - 1) * N * M);
    GemmParams p = {};
    p.A = (const float*)(intptr_t)dA;
    p.B = (const float*)(intptr_t)dB;
    p.C = (float*)(intptr_t)dC;
    p.Cbuf = (float*)(intptr_t)dCbuf;
    p.rows = N;
    p.cols = M;
    p.k_total = K;
    p.ldc = M;
    switch (variant) {
        case GEMM_NN:  // A[N,K], B[K,M]
            p.lda = K; p.a_outer = N; p.a_inner = K;
            p.ldb = M; p.b_outer = K; p.b_inner = M;
            break;
        case GEMM_T1:  // A[K,N], B[K,M]
            p.lda = N; p.a_outer = K; p.a_inner = N;
            p.ldb = M; p.b_outer = K; p.b_inner = M;
            break;
        default:       // GEMM_T2: A[N,K], B[M,K]
            p.lda = K; p.a_outer = N; p.a_inner = K;
            p.ldb = K; p.b_outer = M; p.b_inner = K;
            break;
    }
    p.bias = (const float*)(intptr_t)dBias;
    p.bias_rows = dBias ? bias_rows : 0;
    p.bias_width = dBias ? bias_width : 0;
    p.nz = gz;
    if (gz > 1) {
        // K_slice = (K / GZ) >> 3 << 3   (reference: MM/micro.cuh:92)
        p.k_slice = ((K / gz) >> 3) << 3;
        p.sizeC = (long long)N * M;
        p.split = 1;  // a zero K_slice leaves every slice but the last empty: they write zeros
    }
    if (!gemm_pitches_addressable(p)) return hipErrorInvalidValue;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    p.sk_ws_given = sk_ws;
    p.sk_ws_given_floats = sk_ws != nullptr ? GEMM_SK_WS_FLOATS_256CU : 0;
    hipStream_t stream = (hipStream_t)(intptr_t)streams[0];
    // A split that loses is declined: the balanced kernel deals equal runs of stages to the compute units by
    // itself, and where the unsplit product through it is estimated to beat the slices plus their fold, the
    // whole product goes to C and the partial buffers get zeros -- SKbuf_summary then adds zeros and leaves C
    // as it is (the caller sees the sum it asked for; which slice holds what is the kernel's business).  A
    // forced tile shape (tests, tuning) always honours the split.
    // A skinny product (a C of 4 ... 32 columns or rows, ...) that the host policy asks to split -- it does, by 4 to 16,
    // for the shapes with few lines: 8 x 4096 x 4096 gets GridZ 16 -- goes to the skinny kernel whole, which cuts K
    // among its workgroups itself; the partial buffers get zeros from the same launch and the fold is elided.
    if (gz > 1 && dBias == 0 && sk_ws == nullptr && gemm_forced_tile() == TILE_AUTO && t_split_policy != 0 &&
        gemm_choose_skinny(N, M, 1, K, variant, num_cu) >= 0) {
        GemmParams q = p;
        q.nz = 1; q.split = 0; q.k_slice = 0; q.sizeC = 0; q.Cbuf = nullptr;
        q.zero_buf = p.Cbuf;
        q.zero_floats = (long long)(gz - 1) * N * M;
        const hipError_t e1 = gemm_launch_skinny(variant, q, stream);
        if (e1 != hipErrorOutOfMemory) {
            if (e1 == hipSuccess) {
                g_declined.fetch_add(1, std::memory_order_relaxed);
                ledger_note(stream, dCbuf, dC, gz - 1, N * M);
            }
            return e1;
        }
        (void)hipGetLastError();
    }
    if (gz > 1 && dBias == 0 && split_declined(variant, N, M, gz, K, p.k_slice, num_cu)) {
        GemmParams q = p;
        q.nz = 1; q.split = 0; q.k_slice = 0; q.sizeC = 0; q.Cbuf = nullptr;
        q.zero_buf = p.Cbuf;
        q.zero_floats = (long long)(gz - 1) * N * M;
        const int tile1 = gemm_choose_streamk(N, M, 1, K, num_cu, variant);
        const hipError_t e1 = gemm_launch_streamk(variant, q, tile1, stream);
        if (e1 != hipErrorOutOfMemory) {
            if (e1 == hipSuccess) {
                g_declined.fetch_add(1, std::memory_order_relaxed);
                if (sk_ws == nullptr) ledger_note(stream, dCbuf, dC, gz - 1, N * M);   // (the static entry folds nothing)
            }
            return e1;
        }
        (void)hipGetLastError();   // no workspace may be made now (a capturing stream): the slices as asked
    }
    // K slices are tiles like batches are: (slice, tile of C) pairs, each slice k_slice long
    const int k_tile = p.split && p.k_slice > 0 ? p.k_slice : p.k_total;
    const int tile = gemm_choose_tile(p.rows, p.cols, p.nz, k_tile, num_cu, variant);
    return gemm_launch(variant, p, tile, stream);
}

}  // namespace

namespace dragon {
void split_ledger_touch(const void* ptr, size_t bytes) {
    if (g_led_n.load(std::memory_order_acquire) == 0) return;
    const uintptr_t lo = (uintptr_t)ptr, hi = bytes == 0 ? ~(uintptr_t)0 : lo + bytes;
    std::lock_guard<std::mutex> lock(g_led_mutex);
    for (size_t i = 0; i < g_led.size();) {
        const DeclinedSplit& e = g_led[i];
        if ((lo < e.cbuf_end && e.cbuf < hi) || (lo < e.c_end && e.c < hi)) g_led.erase(g_led.begin() + i);
        else i++;
    }
    g_led_n.store((int)g_led.size(), std::memory_order_release);
}
}  // namespace dragon

extern "C" {

int dragon_Cuda_matMul_matMul(const int64_t* streams, int32_t length, int64_t dA, int64_t dB,
                              int64_t dC, int32_t N, int32_t M, int32_t K) {
    return matmul_2d(GEMM_NN, streams, length, 1, dA, dB, dC, 0, N, M, K);
}
int dragon_Cuda_matMul_matMulT1(const int64_t* streams, int32_t length, int64_t dA, int64_t dB,
                                int64_t dC, int32_t N, int32_t M, int32_t K) {
    return matmul_2d(GEMM_T1, streams, length, 1, dA, dB, dC, 0, N, M, K);
}
int dragon_Cuda_matMul_matMulT2(const int64_t* streams, int32_t length, int64_t dA, int64_t dB,
                                int64_t dC, int32_t N, int32_t M, int32_t K) {
    return matmul_2d(GEMM_T2, streams, length, 1, dA, dB, dC, 0, N, M, K);
}

int dragon_Cuda_matMul_matMulSK(const int64_t* streams, int32_t length, int32_t GridZ, int64_t dA,
                                int64_t dB, int64_t dC, int64_t dCbuf, int32_t N, int32_t M,
                                int32_t K) {
    return matmul_2d(GEMM_NN, streams, length, GridZ, dA, dB, dC, dCbuf, N, M, K);
}
int dragon_Cuda_matMul_matMulT1SK(const int64_t* streams, int32_t length, int32_t GridZ,
                                  int64_t dA, int64_t dB, int64_t dC, int64_t dCbuf, int32_t N,
                                  int32_t M, int32_t K) {
    return matmul_2d(GEMM_T1, streams, length, GridZ, dA, dB, dC, dCbuf, N, M, K);
}
int dragon_Cuda_matMul_matMulT2SK(const int64_t* streams, int32_t length, int32_t GridZ,
                                  int64_t dA, int64_t dB, int64_t dC, int64_t dCbuf, int32_t N,
                                  int32_t M, int32_t K) {
    return matmul_2d(GEMM_T2, streams, length, GridZ, dA, dB, dC, dCbuf, N, M, K);
}

int dragon_Cuda_matMul_SKbuf_summary(int64_t stream, int64_t dCbuf, int64_t dC, int32_t part,
                                     int32_t sizeC) {
    if (dC == 0 || sizeC <= 0 || part < 0 || !x4(sizeC) || !aligned16(dC))
        return hipErrorInvalidValue;
    if (part > 0 && (dCbuf == 0 || !aligned16(dCbuf))) return hipErrorInvalidValue;
    if (part == 0) return hipSuccess;
    // the fold that follows a declined split adds zeros: nothing to launch
    if (ledger_fold_is_noop((hipStream_t)(intptr_t)stream, dCbuf, dC, part, sizeC)) {
        g_folds_skipped.fetch_add(1, std::memory_order_relaxed);
        return hipSuccess;
    }
    touch(dC, sizeC);
    return skbuf_summary_launch((hipStream_t)(intptr_t)stream, (const float*)(intptr_t)dCbuf,
                                (float*)(intptr_t)dC, part, sizeC);
}

// ---- the whole split-K product with the partials in memory the library already holds ------------

}  // extern "C"

namespace {

// Scratch memory of dragon_Cuda_matMul_matMulSK_static, one copy per GPU, held until the process ends:
//   [0, SK_STATIC_FLOATS)          the partial products, slice z >= 1 at (z-1)*N*M, exactly the layout of the
//                                  caller's Cbuf in the two-stage entry points;
//   [SK_STATIC_FLOATS, + GEMM_SK_WS_FLOATS_256CU)
//                                  the balanced kernel's workspace (arrival counters, pieces of shared tiles),
//                                  which the other entry points keep per stream in allocated memory.  The
//                                  counters start at zero with the array (a device variable without an
//                                  initialiser is zero) and every launch leaves them there.
// In host code the array's name is only a handle for hipGetSymbolAddress: the kernels get the device address
// that call returns.
constexpr long long SK_STATIC_FLOATS = 8ll << 20;   // 32 MiB
static __device__ __align__(256) __attribute__((used)) float scratch[SK_STATIC_FLOATS + GEMM_SK_WS_FLOATS_256CU];

constexpr int MAX_DEVICES = 64;
std::atomic<float*> g_scratch_ptr[MAX_DEVICES];

// The device address of `scratch` on the current device, looked up once per device.
int static_scratch(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    float* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (ptr == nullptr) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // concurrent first calls store the same value
    }
    *out = ptr;
    return hipSuccess;
}

}  // namespace

extern "C" {

int dragon_Cuda_matMul_matMulSK_static(const int64_t* streams, int32_t length, int32_t variant, int32_t GridZ,
                                       int64_t dA, int64_t dB, int64_t dC, int32_t N, int32_t M, int32_t K) {
    if (variant < GEMM_NN || variant > GEMM_T2) return hipErrorInvalidValue;
    int e = check_common(streams, length, dA, dB, dC);
    if (e) return e;
    if (N <= 0 || M <= 0 || K <= 0 || GridZ < 1 || !x4(N) || !x4(M) || !x4(K)) return hipErrorInvalidValue;
    if ((long long)N * M > 0x7fffffffLL) return hipErrorInvalidValue;
    const long long need = (long long)(GridZ - 1) * N * M;
    if (need > SK_STATIC_FLOATS) {
        fprintf(stderr,
                "dragon_Cuda_matMul_matMulSK_static: (GridZ-1)*N*M = %lld floats of partial products do not fit "
                "the static workspace of %lld floats\n", need, SK_STATIC_FLOATS);
        return hipErrorOutOfMemory;
    }
    float* ptr = nullptr;
    e = static_scratch(&ptr);
    if (e) return e;
    float* sk_ws = ptr + SK_STATIC_FLOATS;
    // While the stream is capturing, the balanced kernel stays out of it: replays of a graph may overlap with
    // each other or with eager calls, and two launches at a time on the one static workspace would mix their
    // pieces and could leave its arrival counters off zero for every later call.  The tile-per-workgroup
    // kernels need no workspace; the partials still go to the static array.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)(intptr_t)streams[0], &cap) != hipSuccess) {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusActive;
    }
    if (cap != hipStreamCaptureStatusNone) sk_ws = nullptr;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    // a split that loses is declined as in the two-stage entry points; here nobody folds afterwards, so the
    // unsplit product is the whole call
    if (GridZ > 1 && sk_ws != nullptr && split_declined(variant, N, M, GridZ, K, ((K / GridZ) >> 3) << 3, num_cu)) GridZ = 1;
    if (GridZ == 1) return matmul_2d(variant, streams, length, 1, dA, dB, dC, 0, N, M, K, 0, 0, 0, sk_ws);
    // stage 1 writes every float of the GridZ-1 partials it later reads, so nothing has to be cleared
    e = matmul_2d(variant, streams, length, GridZ, dA, dB, dC, (int64_t)(intptr_t)ptr, N, M, K, 0, 0, 0, sk_ws);
    if (e) return e;
    return skbuf_summary_launch((hipStream_t)(intptr_t)streams[0], ptr, (float*)(intptr_t)dC, GridZ - 1, N * M);
}

int dragon_Cuda_matMul_matMul_biased(const int64_t* streams, int32_t length, int64_t dA, int64_t dB,
                                     int64_t dC, int64_t dBias, int32_t N, int32_t M, int32_t K,
                                     int32_t lengthv, int32_t width) {
    if (dBias == 0 || !aligned16(dBias) || width <= 0 || width > M || lengthv <= 0 || M <= 0 ||
        lengthv % M != 0 || lengthv / M > N)
        return hipErrorInvalidValue;
    return matmul_2d(GEMM_NN, streams, length, 1, dA, dB, dC, 0, N, M, K, dBias, lengthv / M, width);
}

int dragon_Cuda_function_linear_dual2D_row(int64_t stream, int64_t dX1, int64_t dX2,
                                           int32_t row_lengthv, float alpha, float beta, float gamma,
                                           int64_t dY, int32_t lengthv, int32_t width, int32_t stride) {
    if (dX1 == 0 || dX2 == 0 || dY == 0 || !aligned16(dX1) || !aligned16(dX2) || !aligned16(dY))
        return hipErrorInvalidValue;
    if (lengthv <= 0 || row_lengthv <= 0 || stride <= 0 || width <= 0 || width > stride ||
        !x4(lengthv) || !x4(row_lengthv) || !x4(stride) || lengthv % stride != 0 ||
        lengthv % row_lengthv != 0 || row_lengthv % stride != 0)
        return hipErrorInvalidValue;
    touch(dY, lengthv);
    return linear_dual2D_row_launch((hipStream_t)(intptr_t)stream, (const float*)(intptr_t)dX1,
                                    (const float*)(intptr_t)dX2, row_lengthv, alpha, beta, gamma,
                                    (float*)(intptr_t)dY, lengthv, width, stride);
}

// ---- batched ---------------------------------------------------------------------

int dragon_Cuda_batchMatMul_batchMatMul(const int64_t* streams, int32_t length, int64_t dA,
                                        int64_t dB, int64_t dC, int32_t Batch, int32_t N,
                                        int32_t M, int32_t BK, int32_t AK) {
    int e = check_common(streams, length, dA, dB, dC);
    if (e) return e;
    if (Batch <= 0 || N <= 0 || M <= 0 || BK <= 0 || AK < BK) return hipErrorInvalidValue;
    if (!x4(M) || !x4(AK)) return hipErrorInvalidValue;
    GemmParams p = {};
    p.A = (const float*)(intptr_t)dA;   // A[Batch, N, AK]
    p.B = (const float*)(intptr_t)dB;   // B[Batch, BK, M]
    p.C = (float*)(intptr_t)dC;         // C[Batch, N, M]
    // A is read up to the last 16-byte chunk that holds a k below BK: its columns beyond are never touched
    // (the reference's loop stops at BK, BMM/batchMatMul.cuh:15)
    const int k_read = (BK + 3) / 4 * 4 < AK ? (BK + 3) / 4 * 4 : AK;
    p.rows = N; p.cols = M; p.k_total = k_read;
    p.lda = AK; p.a_outer = N;  p.a_inner = k_read;
    p.ldb = M;  p.b_outer = BK; p.b_inner = M;
    p.ldc = M;
    p.sA = (long long)N * AK; p.sB = (long long)BK * M; p.sC = (long long)N * M;
    p.nz = Batch;
    touch(dC, p.sC * Batch);
    if (!gemm_pitches_addressable(p)) return hipErrorInvalidValue;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const int tile = gemm_choose_tile(p.rows, p.cols, p.nz, p.k_total, num_cu, GEMM_NN);
    return gemm_launch(GEMM_NN, p, tile, (hipStream_t)(intptr_t)streams[0]);
}

int dragon_Cuda_batchMatMul_batchMatMul_texture(const int64_t* streams, int32_t length,
                                                int64_t dA, int64_t dB, int64_t dC, int32_t Batch,
                                                int32_t N, int32_t M, int32_t BK, int32_t AK) {
    return dragon_Cuda_batchMatMul_batchMatMul(streams, length, dA, dB, dC, Batch, N, M, BK, AK);
}

int dragon_Cuda_batchMatMul_batchMatMulT1(const int64_t* streams, int32_t length, int64_t dA,
                                          int64_t dB, int64_t dC, int32_t Batch, int32_t CN,
                                          int32_t AN, int32_t M, int32_t K) {
    int e = check_common(streams, length, dA, dB, dC);
    if (e) return e;
    if (Batch <= 0 || CN <= 0 || AN < CN || M <= 0 || K <= 0) return hipErrorInvalidValue;
    if (!x4(AN) || !x4(M)) return hipErrorInvalidValue;
    GemmParams p = {};
    p.A = (const float*)(intptr_t)dA;   // A[Batch, K, AN]
    p.B = (const float*)(intptr_t)dB;   // B[Batch, K, M]
    p.C = (float*)(intptr_t)dC;         // C[Batch, CN, M]
    p.rows = CN; p.cols = M; p.k_total = K;
    p.lda = AN; p.a_outer = K; p.a_inner = AN;
    p.ldb = M;  p.b_outer = K; p.b_inner = M;
    p.ldc = M;
    p.sA = (long long)K * AN; p.sB = (long long)K * M; p.sC = (long long)CN * M;
    p.nz = Batch;
    touch(dC, p.sC * Batch);
    if (!gemm_pitches_addressable(p)) return hipErrorInvalidValue;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const int tile = gemm_choose_tile(p.rows, p.cols, p.nz, p.k_total, num_cu, GEMM_T1);
    return gemm_launch(GEMM_T1, p, tile, (hipStream_t)(intptr_t)streams[0]);
}

int dragon_Cuda_batchMatMul_batchMatMulT2(const int64_t* streams, int32_t length, int64_t dA,
                                          int64_t dB, int64_t dC, int32_t Batch, int32_t N,
                                          int32_t CM, int32_t BM, int32_t K) {
    int e = check_common(streams, length, dA, dB, dC);
    if (e) return e;
    if (Batch <= 0 || N <= 0 || CM <= 0 || BM <= 0 || BM > CM || K <= 0) return hipErrorInvalidValue;
    if (!x4(CM) || !x4(K)) return hipErrorInvalidValue;
    GemmParams p = {};
    p.A = (const float*)(intptr_t)dA;   // A[Batch, N, K]
    p.B = (const float*)(intptr_t)dB;   // B[Batch, BM, K]
    p.C = (float*)(intptr_t)dC;         // C[Batch, N, CM]
    p.rows = N; p.cols = CM; p.k_total = K;
    p.lda = K; p.a_outer = N;  p.a_inner = K;
    p.ldb = K; p.b_outer = BM; p.b_inner = K;
    p.ldc = CM;
    p.sA = (long long)N * K; p.sB = (long long)BM * K; p.sC = (long long)N * CM;
    p.nz = Batch;
    touch(dC, p.sC * Batch);
    if (!gemm_pitches_addressable(p)) return hipErrorInvalidValue;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const int tile = gemm_choose_tile(p.rows, p.cols, p.nz, p.k_total, num_cu, GEMM_T2);
    return gemm_launch(GEMM_T2, p, tile, (hipStream_t)(intptr_t)streams[0]);
}

int dragon_Cuda_batchMatMul_batchMatMulT2_texture(const int64_t* streams, int32_t length,
                                                  int64_t dA, int64_t dB, int64_t dC,
                                                  int32_t Batch, int32_t N, int32_t CM,
                                                  int32_t BM, int32_t K) {
    return dragon_Cuda_batchMatMul_batchMatMulT2(streams, length, dA, dB, dC, Batch, N, CM, BM, K);
}

// ---- *_mma: forward to the FP32 path ---------------------------------------------

int dragon_Cuda_matMul_matMul_mma(const int64_t* streams, int32_t length, int64_t dA, int64_t dB,
                                  int64_t dC, int32_t N, int32_t M, int32_t K) {
    return dragon_Cuda_matMul_matMul(streams, length, dA, dB, dC, N, M, K);
}
int dragon_Cuda_matMul_matMulT1_mma(const int64_t* streams, int32_t length, int64_t dA,
                                    int64_t dB, int64_t dC, int32_t N, int32_t M, int32_t K) {
    return dragon_Cuda_matMul_matMulT1(streams, length, dA, dB, dC, N, M, K);
}
int dragon_Cuda_matMul_matMulT2_mma(const int64_t* streams, int32_t length, int64_t dA,
                                    int64_t dB, int64_t dC, int32_t N, int32_t M, int32_t K) {
    return dragon_Cuda_matMul_matMulT2(streams, length, dA, dB, dC, N, M, K);
}
int dragon_Cuda_batchMatMul_batchMatMul_mma(int32_t, const int64_t* streams, int32_t length,
                                            int64_t dA, int64_t dB, int64_t dC, int32_t Batch,
                                            int32_t N, int32_t M, int32_t BK, int32_t AK) {
    return dragon_Cuda_batchMatMul_batchMatMul(streams, length, dA, dB, dC, Batch, N, M, BK, AK);
}
int dragon_Cuda_batchMatMul_batchMatMulT1_mma(const int64_t* streams, int32_t length, int64_t dA,
                                              int64_t dB, int64_t dC, int32_t Batch, int32_t CN,
                                              int32_t AN, int32_t M, int32_t K) {
    return dragon_Cuda_batchMatMul_batchMatMulT1(streams, length, dA, dB, dC, Batch, CN, AN, M, K);
}
int dragon_Cuda_batchMatMul_batchMatMulT2_mma(int32_t, const int64_t* streams, int32_t length,
                                              int64_t dA, int64_t dB, int64_t dC, int32_t Batch,
                                              int32_t N, int32_t CM, int32_t BM, int32_t K) {
    return dragon_Cuda_batchMatMul_batchMatMulT2(streams, length, dA, dB, dC, Batch, N, CM, BM, K);
}

// ---- host heuristics ---------------------------------------------------------------

static int tile_classes(int n, bool count_full) {
    // Number of tile classes (128, 64, 32, 16, 8, 4) a dimension decomposes into; the
    // 128 class counts once per full tile when count_full is set.
    int c = 0;
    if (n > 127) c += count_full ? (n >> 7) : 1;
    n &= 127;
    for (int bit = 64; bit >= 4; bit >>= 1)
        if (n & bit) c++;
    return c;
}

int32_t dragon_Cuda_matMul_blockNum(int32_t N, int32_t M) {
    return tile_classes(N, true) * tile_classes(M, true);
}

static int stream_classes(int n) { return ((n & (n - 1)) == 0) ? 1 : tile_classes(n, false); }

int32_t dragon_Cuda_matMul_nstream(int32_t N, int32_t M) {
    const int size = stream_classes(N) * stream_classes(M);
    return size < MAX_STREAMS ? size : MAX_STREAMS;
}

int32_t dragon_Cuda_batchMatMul_streamSize(int32_t N, int32_t M) {
    int size = stream_classes(N) * stream_classes(M);
    if (size < 1) size = 1;
    return size < MAX_STREAMS ? size : MAX_STREAMS;
}

void dragon_gemm_force_tile(int32_t tile) { gemm_force_tile(tile); }
void dragon_gemm_skinny_form(int32_t form) { gemm_skinny_form(form); }
int32_t dragon_gemm_release_workspaces(void) { return gemm_streamk_release_workspaces(); }
int32_t dragon_gemm_workspace_count(void) { return gemm_streamk_workspace_count(); }
int64_t dragon_gemm_workspaces_refused(void) { return gemm_streamk_workspaces_refused(); }
void dragon_gemm_fold_skip(int32_t on) { g_fold_skip.store(on ? 1 : 0, std::memory_order_relaxed); }
int64_t dragon_gemm_folds_skipped(void) { return g_folds_skipped.load(std::memory_order_relaxed); }
void dragon_gemm_split_policy(int32_t mode) { t_split_policy = mode < -1 || mode > 1 ? -1 : mode; }
int64_t dragon_gemm_declined_splits(void) { return g_declined.load(std::memory_order_relaxed); }
int32_t dragon_gemm_split_loses(int32_t variant, int32_t N, int32_t M, int32_t GridZ, int32_t K, int32_t num_cu) {
    if (variant < GEMM_NN || variant > GEMM_T2 || GridZ < 1 || N <= 0 || M <= 0 || K <= 0 || num_cu <= 0) return -1;
    return gemm_split_loses(variant, N, M, GridZ, K, ((K / GridZ) >> 3) << 3, num_cu) ? 1 : 0;
}
double dragon_gemm_estimate_us(int32_t variant, int32_t rows, int32_t cols, int32_t nz, int32_t k, int32_t num_cu) {
    return gemm_estimate_us(rows, cols, nz, k, num_cu, variant);
}
void dragon_gemm_tile_divisor(uint32_t d, uint32_t* mul, uint32_t* shift) {
    unsigned m = 0, s = 0;
    gemm_magic_divisor(d, m, s);
    if (mul) *mul = m;
    if (shift) *shift = s;
}
int32_t dragon_gemm_paired_form_fits(int32_t variant, int32_t GridZ, int32_t N, int32_t M, int32_t K) {
    if (variant < GEMM_NN || variant > GEMM_T2 || GridZ < 1 || N <= 0 || M <= 0 || K <= 0) return -1;
    GemmParams p = {};
    p.k_total = K;
    p.lda = variant == GEMM_T1 ? N : K;
    p.ldb = variant == GEMM_T2 ? K : M;
    p.nz = GridZ;
    p.split = GridZ > 1;
    p.k_slice = ((K / GridZ) >> 3) << 3;
    return gemm_paired_form_fits(variant != GEMM_T1, variant == GEMM_T2, p) ? 1 : 0;
}
int32_t dragon_gemm_choose_tile(int32_t variant, int32_t rows, int32_t cols, int32_t nz, int32_t k, int32_t num_cu) {
    if (rows <= 0 || cols <= 0 || nz <= 0 || k <= 0 || num_cu <= 0) return -1;
    return gemm_choose_tile(rows, cols, nz, k, num_cu, variant);
}

}  // extern "C"
