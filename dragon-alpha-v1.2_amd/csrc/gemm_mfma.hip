// FP32 GEMM for gfx950 (MI355X / CDNA4) on the FP32 matrix cores.
//
// One kernel template covers the three products of Dragon-Alpha's matMul path
//   NN: C = A  * B     A[rows,K]  B[K,cols]     (reference: MM/matMul.cuh:47-119)
//   T1: C = A^T * B    A[K,rows]  B[K,cols]     (reference: MM/matMulT1.cuh:42-89)
//   T2: C = A  * B^T   A[rows,K]  B[cols,K]     (reference: MM/matMulT2.cuh:44-107)
// their batched forms (grid depth = batch; BMM/batchMatMul*.cuh) and their split-K
// forms (grid depth = K slices; MM/matMulSK_kernel.cuh:124-131).  MM and BMM are
// source/engine-cuda-base/Cuda_matMul/Cuda_matMul and .../Cuda_batchMatMul/Cuda_batchMatMul
// of the reference tree.
//
// Where the reference carves C into power-of-two tile classes on the host and
// launches one unguarded kernel per class, this kernel guards its own edges:
// every operand load is predicated on exact bounds (out-of-range lanes read zero
// through the buffer descriptor's range check) and every store is predicated, so
// one launch covers any shape.
//
// Arithmetic: v_mfma_f32_32x32x2_f32 -- IEEE FP32 multiply, FP32 accumulate.
//
// Operand layouts.  An operand is either "K-inner" (k is the contiguous index:
// A of NN/T2, B of T2) or "K-outer" (k is the row index: B of NN/T1, A of T1).
// Neither is transposed on its way through LDS:
//   K-inner tile  -> LDS [row][k] (+4 floats of row padding); a lane reads 4
//                    consecutive k with one ds_read_b128 and feeds 4 MFMA steps.
//   K-outer tile  -> LDS [k][row]; a lane reads T consecutive rows with one
//                    ds_read, and those T values belong to T different MFMA
//                    blocks (block b of a wave holds rows {T*p + b}).  The
//                    interleave makes the lane's accumulators cover T adjacent
//                    columns of C, which become one vector store.
// The MFMA step q of a group of 8 k consumes k = 4*h + q from lane half h, for
// both operands, which is what lets a K-inner and a K-outer operand be paired.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "gemm_mfma.h"

namespace dragon {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

static constexpr int NTHREADS = 256;          // 4 wavefronts of 64
static constexpr int OOB_OFFSET = 0x7ffffff0; // >= num_records: the load returns 0
static constexpr int RSRC_RECORDS = 0x7ffffff0;
static constexpr int RSRC_FLAGS = 0x00020000; // raw buffer, 32-bit data format

__device__ __forceinline__ v4f buffer_load_f4(const float* base, int byte_offset) {
    __amdgpu_buffer_rsrc_t r =
        __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, RSRC_RECORDS, RSRC_FLAGS);
    v4u x = __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, 0, 0);
    return __builtin_bit_cast(v4f, x);
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with a private L2.
// Re-number them so that one XCD owns a contiguous range of logical ids.
__device__ __forceinline__ int xcd_contiguous_id(int pid, int nwg) {
    const int xcd = pid & 7, local = pid >> 3;
    const int per = nwg >> 3, rem = nwg & 7;
    return xcd * per + (xcd < rem ? xcd : rem) + local;
}

// ---------------------------------------------------------------------------
// Tile staging: global -> registers -> LDS
// ---------------------------------------------------------------------------

// K-inner operand: R rows of KT consecutive k.  LDS row stride KT+4 floats.
template <int R, int KT>
struct KInner {
    static constexpr int CPR = KT / 4;            // float4 chunks per row
    static constexpr int RPP = NTHREADS / CPR;    // rows per pass
    static constexpr int PASSES = R / RPP;
    static constexpr int LDS_STRIDE = KT + 4;
    static constexpr int LDS_FLOATS = R * LDS_STRIDE;
    static_assert(R % RPP == 0 && PASSES >= 1, "tile does not divide over the workgroup");

    int off[PASSES];   // byte offset of this thread's chunk, or OOB_OFFSET if its row is outside
    int kcol;          // k offset of this thread's chunk inside the tile
    int lds_at;        // float index of the first chunk in the LDS tile

    __device__ __forceinline__ void init(int t, int row0, int outer_bound, int ld) {
        const int c = t % CPR, r0 = t / CPR;
        kcol = c * 4;
        lds_at = r0 * LDS_STRIDE + c * 4;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int r = r0 + s * RPP;
            off[s] = (row0 + r < outer_bound) ? (r * ld + c * 4) * 4 : OOB_OFFSET;
        }
    }
    // base points at (row0, k) of the operand; k_left = k_limit - k
    __device__ __forceinline__ void load(v4f (&reg)[PASSES], const float* base, int k_left) const {
        const bool kok = kcol < k_left;
#pragma unroll
        for (int s = 0; s < PASSES; s++) reg[s] = buffer_load_f4(base, kok ? off[s] : OOB_OFFSET);
    }
    __device__ __forceinline__ void store(const v4f (&reg)[PASSES], float* lds) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++) *(v4f*)(lds + lds_at + s * RPP * LDS_STRIDE) = reg[s];
    }
    __device__ __forceinline__ static const float* tile_base(const float* X, int row0, int k, int ld) {
        return X + (size_t)row0 * ld + k;
    }
    __device__ __forceinline__ static size_t k_advance(int ld) { return KT; }
};

// K-outer operand: KT rows (k) of R consecutive outputs.  LDS row stride R floats.
template <int R, int KT>
struct KOuter {
    static constexpr int CPR = R / 4;
    static constexpr int RPP = NTHREADS / CPR;    // k rows per pass
    static constexpr int PASSES = KT / RPP;
    static constexpr int LDS_STRIDE = R;
    static constexpr int LDS_FLOATS = KT * LDS_STRIDE;
    static_assert(KT % RPP == 0 && PASSES >= 1, "tile does not divide over the workgroup");

    int off[PASSES];
    int krow;          // k row of the first pass
    int lds_at;

    __device__ __forceinline__ void init(int t, int col0, int inner_bound, int ld) {
        const int c = t % CPR, k0 = t / CPR;
        krow = k0;
        lds_at = k0 * LDS_STRIDE + c * 4;
        const bool ok = col0 + c * 4 < inner_bound;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int kr = k0 + s * RPP;
            off[s] = ok ? (kr * ld + c * 4) * 4 : OOB_OFFSET;
        }
    }
    __device__ __forceinline__ void load(v4f (&reg)[PASSES], const float* base, int k_left) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++)
            reg[s] = buffer_load_f4(base, (krow + s * RPP < k_left) ? off[s] : OOB_OFFSET);
    }
    __device__ __forceinline__ void store(const v4f (&reg)[PASSES], float* lds) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++) *(v4f*)(lds + lds_at + s * RPP * LDS_STRIDE) = reg[s];
    }
    __device__ __forceinline__ static const float* tile_base(const float* X, int col0, int k, int ld) {
        return X + (size_t)k * ld + col0;
    }
    __device__ __forceinline__ static size_t k_advance(int ld) { return (size_t)KT * ld; }
};

// ---------------------------------------------------------------------------
// Fragment reads: LDS -> MFMA operands for one group of 8 k
//   frag[b][q]: operand of block b for MFMA step q (k = 8*g + 4*h + q)
// ---------------------------------------------------------------------------
template <int T, int KT>
__device__ __forceinline__ void read_frag_kinner(float (&frag)[T][4], const float* lds,
                                                 int wave_row0, int g, int r, int h) {
    constexpr int S = KT + 4;
#pragma unroll
    for (int b = 0; b < T; b++) {
        const v4f v = *(const v4f*)(lds + (wave_row0 + b * 32 + r) * S + g * 8 + h * 4);
        frag[b][0] = v.x; frag[b][1] = v.y; frag[b][2] = v.z; frag[b][3] = v.w;
    }
}

template <int T, int R>
__device__ __forceinline__ void read_frag_kouter(float (&frag)[T][4], const float* lds,
                                                 int wave_row0, int g, int r, int h) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const float* p = lds + (g * 8 + h * 4 + q) * R + wave_row0 + T * r;
        if constexpr (T == 1) {
            frag[0][q] = p[0];
        } else if constexpr (T == 2) {
            const v2f v = *(const v2f*)p;
            frag[0][q] = v.x; frag[1][q] = v.y;
        } else {
            static_assert(T == 4, "blocks per wave along a K-outer operand: 1, 2 or 4");
            const v4f v = *(const v4f*)p;
            frag[0][q] = v.x; frag[1][q] = v.y; frag[2][q] = v.z; frag[3][q] = v.w;
        }
    }
}

// ---------------------------------------------------------------------------
// The kernel
//   A_KIN / B_KIN : operand is K-inner
//   WM x WN       : wavefront grid in the workgroup (WM*WN == 4)
//   TM x TN       : 32x32 MFMA blocks per wavefront
//   KT            : k per LDS stage
// ---------------------------------------------------------------------------
template <bool A_KIN, bool B_KIN, int WM, int WN, int TM, int TN, int KT>
__global__ __launch_bounds__(NTHREADS) void gemm_f32_mfma(const GemmParams p) {
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    using LoadA = typename std::conditional<A_KIN, KInner<BM, KT>, KOuter<BM, KT>>::type;
    using LoadB = typename std::conditional<B_KIN, KInner<BN, KT>, KOuter<BN, KT>>::type;

    __shared__ __attribute__((aligned(16))) float As[2][LoadA::LDS_FLOATS];
    __shared__ __attribute__((aligned(16))) float Bs[2][LoadB::LDS_FLOATS];

    // ---- which tile, which batch / K slice -------------------------------------
    const int tiles = p.tiles_m * p.tiles_n;
    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int z = lid / tiles;
    int tt = lid - z * tiles;
    // bands of 8 tile rows, walked row-fastest, keep one XCD's concurrent tiles compact
    constexpr int BAND = 8;
    const int band_sz = BAND * p.tiles_n;
    const int band = tt / band_sz;
    const int first_m = band * BAND;
    const int band_rows = (p.tiles_m - first_m < BAND) ? (p.tiles_m - first_m) : BAND;
    tt -= band * band_sz;
    const int tile_m = first_m + tt % band_rows;
    const int tile_n = tt / band_rows;
    const int row0 = tile_m * BM, col0 = tile_n * BN;

    const float* A = p.A;
    const float* B = p.B;
    float* C = p.C;
    int k0 = 0, k1 = p.k_total;
    if (p.split) {                   // split-K: z is the slice
        k0 = z * p.k_slice;
        if (z != p.nz - 1) k1 = k0 + p.k_slice;
        if (z != 0) C = p.Cbuf + (size_t)(z - 1) * p.sizeC;
    } else {                          // batched: z is the batch
        A += (size_t)z * p.sA;
        B += (size_t)z * p.sB;
        C += (size_t)z * p.sC;
    }
    // k range each operand may touch
    const int ka_lim = min(k1, A_KIN ? p.a_inner : p.a_outer);
    const int kb_lim = min(k1, B_KIN ? p.b_inner : p.b_outer);

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    LoadA la;
    LoadB lb;
    la.init(t, row0, A_KIN ? p.a_outer : p.a_inner, p.lda);
    lb.init(t, col0, B_KIN ? p.b_outer : p.b_inner, p.ldb);
    const float* a_ptr = LoadA::tile_base(A, row0, k0, p.lda);
    const float* b_ptr = LoadB::tile_base(B, col0, k0, p.ldb);
    const size_t a_step = LoadA::k_advance(p.lda), b_step = LoadB::k_advance(p.ldb);

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    v4f ra[LoadA::PASSES], rb[LoadB::PASSES];
    const int ntile = (k1 - k0 + KT - 1) / KT;

    // prologue: stage 0
    la.load(ra, a_ptr, ka_lim - k0);
    lb.load(rb, b_ptr, kb_lim - k0);
    la.store(ra, As[0]);
    lb.store(rb, Bs[0]);
    __syncthreads();

    for (int it = 0; it < ntile; it++) {
        const int cur = it & 1;
        const int knext = k0 + (it + 1) * KT;
        if (it + 1 < ntile) {        // prefetch the next stage into registers
            a_ptr += a_step;
            b_ptr += b_step;
            la.load(ra, a_ptr, ka_lim - knext);
            lb.load(rb, b_ptr, kb_lim - knext);
        }
        const float* as = As[cur];
        const float* bs = Bs[cur];
#pragma unroll
        for (int g = 0; g < KT / 8; g++) {
            float fa[TM][4], fb[TN][4];
            if constexpr (A_KIN) read_frag_kinner<TM, KT>(fa, as, wm * TM * 32, g, r, h);
            else                 read_frag_kouter<TM, BM>(fa, as, wm * TM * 32, g, r, h);
            if constexpr (B_KIN) read_frag_kinner<TN, KT>(fb, bs, wn * TN * 32, g, r, h);
            else                 read_frag_kouter<TN, BN>(fb, bs, wn * TN * 32, g, r, h);
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q],
                                                                         acc[i][j], 0, 0, 0);
        }
        if (it + 1 < ntile) {
            la.store(ra, As[cur ^ 1]);
            lb.store(rb, Bs[cur ^ 1]);
        }
        __syncthreads();
    }

    // ---- epilogue: predicated stores ------------------------------------------
    // MFMA block element e of lane (r,h): block row = 8*(e/4) + 4*h + e%4, block col = r.
    // K-inner operand: block b covers 32 consecutive outputs; K-outer: outputs {T*x + b}.
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int mrow = 8 * (e / 4) + 4 * h + (e % 4);
            const int row = row0 + wm * TM * 32 + (A_KIN ? (i * 32 + mrow) : (TM * mrow + i));
            if (row >= p.rows) continue;
            float* crow = C + (size_t)row * p.ldc;
            if constexpr (B_KIN) {
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const int col = col0 + wn * TN * 32 + j * 32 + r;
                    if (col < p.cols) crow[col] = acc[i][j][e];
                }
            } else {
                const int col = col0 + wn * TN * 32 + TN * r;
                if (col < p.cols) {
                    if constexpr (TN == 1) {
                        crow[col] = acc[i][0][e];
                    } else if constexpr (TN == 2) {
                        v2f v = {acc[i][0][e], acc[i][1][e]};
                        *(v2f*)(crow + col) = v;
                    } else {
                        v4f v = {acc[i][0][e], acc[i][1][e], acc[i][2][e], acc[i][3][e]};
                        *(v4f*)(crow + col) = v;
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Host side: tile choice and launch
// ---------------------------------------------------------------------------
template <bool A_KIN, bool B_KIN, int WM, int WN, int TM, int TN, int KT>
static hipError_t launch_cfg(GemmParams p, hipStream_t stream) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    p.tiles_m = (p.rows + BM - 1) / BM;
    p.tiles_n = (p.cols + BN - 1) / BN;
    const long long nwg = (long long)p.tiles_m * p.tiles_n * p.nz;
    if (nwg <= 0 || nwg > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((gemm_f32_mfma<A_KIN, B_KIN, WM, WN, TM, TN, KT>), dim3((unsigned)nwg),
                       dim3(NTHREADS), 0, stream, p);
    return hipGetLastError();
}

template <bool A_KIN, bool B_KIN>
static hipError_t launch_variant(const GemmParams& p, int tile, hipStream_t stream) {
    switch (tile) {
        case TILE_128x128: return launch_cfg<A_KIN, B_KIN, 2, 2, 2, 2, 16>(p, stream);
        case TILE_64x64:   return launch_cfg<A_KIN, B_KIN, 2, 2, 1, 1, 16>(p, stream);
        case TILE_256x64:  return launch_cfg<A_KIN, B_KIN, 4, 1, 2, 2, 16>(p, stream);
        case TILE_64x256:  return launch_cfg<A_KIN, B_KIN, 1, 4, 2, 2, 16>(p, stream);
        case TILE_128x64:  return launch_cfg<A_KIN, B_KIN, 2, 2, 2, 1, 16>(p, stream);
        case TILE_64x128:  return launch_cfg<A_KIN, B_KIN, 2, 2, 1, 2, 16>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

static int g_forced_tile = TILE_AUTO;
void gemm_force_tile(int tile) { g_forced_tile = tile; }

static const int kTileM[TILE_COUNT] = {128, 64, 256, 64, 128, 64};
static const int kTileN[TILE_COUNT] = {128, 64, 64, 256, 64, 128};

// Pick the tile shape with the lowest estimated cost: work actually issued to the
// matrix cores (padded tiles), stretched by how unevenly the workgroups fill the
// compute units.
int gemm_choose_tile(int rows, int cols, int nz, int num_cu) {
    if (g_forced_tile != TILE_AUTO) return g_forced_tile;
    int best = TILE_128x128;
    double best_cost = 1e300;
    for (int tile = 0; tile < TILE_COUNT; tile++) {
        const int bm = kTileM[tile], bn = kTileN[tile];
        const long long tm = (rows + bm - 1) / bm, tn = (cols + bn - 1) / bn;
        const long long nwg = tm * tn * nz;
        // workgroups resident per CU: the small tiles leave room for more
        const int resident = (bm * bn >= 128 * 128) ? 2 : 4;
        const long long slots = (long long)num_cu * resident;
        const long long rounds = (nwg + slots - 1) / slots;
        // time ~ rounds * (tile work / resident sharing) ; small tiles pay a fixed overhead
        const double per_tile = (double)bm * bn * (1.0 + 1024.0 / (bm * bn) * 4.0);
        const double cost = (double)rounds * per_tile * resident;
        if (cost < best_cost * 0.999) { best_cost = cost; best = tile; }
    }
    return best;
}

hipError_t gemm_launch(int variant, const GemmParams& p, int tile, hipStream_t stream) {
    switch (variant) {
        case GEMM_NN: return launch_variant<true, false>(p, tile, stream);
        case GEMM_T1: return launch_variant<false, false>(p, tile, stream);
        case GEMM_T2: return launch_variant<true, true>(p, tile, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace dragon
