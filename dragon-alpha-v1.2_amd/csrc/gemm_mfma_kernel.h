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
//   K-inner tile  -> LDS [row][k] in 16-byte chunks, chunk c of row r stored at chunk
//                    position c ^ swizzle(r) so that both the staging stores (lanes
//                    walk along a row) and the fragment reads (lanes walk down the
//                    rows) touch every bank once; a lane reads 4 consecutive k with
//                    one ds_read_b128 and feeds 4 MFMA steps.  As the B operand its
//                    rows are staged interleaved (LDS row 32*b + r = tile row T*r + b),
//                    which gives the lane the same T adjacent columns as below.
//   K-outer tile  -> LDS [k][row]; a lane reads T consecutive rows with one
//                    ds_read, and those T values belong to T different MFMA
//                    blocks (block b of a wave holds rows {T*p + b}).  The
//                    interleave makes the lane's accumulators cover T adjacent
//                    columns of C, which become one vector store.
// The MFMA step q of a group of 8 k consumes k = 4*h + q from lane half h, for
// both operands, which is what lets a K-inner and a K-outer operand be paired.
//
// This header holds the kernel template and its launcher; gemm_mfma.hip instantiates the plain
// products, gemm_mfma_biased.hip the NN product with the bias row in its epilogue (two
// translation units so that they compile side by side).
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <type_traits>
#include <utility>
#include <stdint.h>
#include "gemm_mfma.h"

namespace dragon {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

static constexpr int NTHREADS = 256;          // 4 wavefronts of 64
static constexpr int OOB_OFFSET = 0x7ffffff0; // >= num_records: the load returns 0
static constexpr int RSRC_RECORDS = 0x7ffffff0;
static constexpr int RSRC_FLAGS = 0x00020000; // raw buffer, 32-bit data format

// byte_offset is the lane's part, scalar_offset a wave-uniform part on top of it; the hardware checks
// their sum against the descriptor's size (measured on gfx950)
__device__ __forceinline__ v4f buffer_load_f4(const float* base, int byte_offset, int scalar_offset = 0) {
    __amdgpu_buffer_rsrc_t r =
        __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, RSRC_RECORDS, RSRC_FLAGS);
    v4u x = __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, scalar_offset, 0);
    return __builtin_bit_cast(v4f, x);
}

// 16 bytes per lane from global memory straight into LDS: lane l of the wave writes
// lds_wave_base + 16*l (the base must be the same for the whole wave; it travels in M0).  A lane
// whose offset is out of range writes zeros.  Completion is counted by vmcnt like any other
// vector-memory load.
// Written as inline assembly on purpose: the compiler then knows nothing of a transfer in flight
// and inserts no waits of its own before LDS reads (its alias analysis gives up on merged
// ds_read2 instructions and would wait for EVERY transfer, serialising the pipeline); the kernel
// waits explicitly.  Transfers the compiler does not know of can only make the waits it inserts
// for its own loads and stores longer, never too short, because vmcnt retires in issue order.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // M0 is "reserved": it is exactly what this changes
__device__ __forceinline__ void dma_f4(const float* base, float* lds_wave_base, int byte_offset) {
    const unsigned long long b = (unsigned long long)base;
    const v4u rsrc = {(unsigned)b, (unsigned)(b >> 32) & 0xffffu, (unsigned)RSRC_RECORDS, (unsigned)RSRC_FLAGS};
    const unsigned lds_addr = __builtin_amdgcn_readfirstlane(
        (unsigned)(unsigned long long)(__attribute__((address_space(3))) void*)lds_wave_base);
    // one wait state is required between writing M0 and the transfer that reads it
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_addr), "v"(byte_offset), "s"(rsrc)
                 : "memory", "m0");
}
// The same transfer for callers that keep the descriptor in registers and the LDS address as an
// integer (a wave-uniform base plus a compile-time distance): three instructions per transfer.
template <int LDS_IMM>
__device__ __forceinline__ void dma_f4_lean(v4u rsrc, unsigned lds_wave_base, int byte_offset) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_wave_base), "v"(byte_offset), "s"(rsrc), "n"(LDS_IMM)
                 : "memory", "m0", "scc");
}
__device__ __forceinline__ v4u dma_descriptor(const float* base) {
    const unsigned long long b = (unsigned long long)base;
    const v4u rsrc = {(unsigned)b, (unsigned)(b >> 32) & 0xffffu, (unsigned)RSRC_RECORDS, (unsigned)RSRC_FLAGS};
    return rsrc;
}
// advance a descriptor's base by `bytes` (addresses stay below 2^48, so the carry never reaches the
// stride field above the base)
__device__ __forceinline__ void dma_descriptor_advance(v4u& rsrc, unsigned long long bytes) {
    unsigned long long b = ((unsigned long long)rsrc.y << 32) | rsrc.x;
    b += bytes;
    rsrc.x = (unsigned)b;
    rsrc.y = (unsigned)(b >> 32);
}
#pragma clang diagnostic pop

// compile-time loop: f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N-1>)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// s_waitcnt for the vector-memory counter alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14,
// expcnt 6:4 and lgkmcnt 11:8 left at "no wait")
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// The value as if it had just been read: the compiler works out what depends on it HERE instead of once
// at the top of the kernel and keeping the results in registers all the way (the lanes' row offsets of a
// tile's loads, needed once per tile: kept live, they were what the 128 x 128 kernels spilled).
__device__ __forceinline__ int fresh(int v) {
    asm volatile("" : "+s"(v));
    return v;
}

// Workgroup ids are dealt round-robin to the 8 XCDs, each with a private L2.
// Re-number them so that one XCD owns a contiguous range of logical ids.
__device__ __forceinline__ int xcd_contiguous_id(int pid, int nwg) {
    const int xcd = pid & 7, local = pid >> 3;
    const int per = nwg >> 3, rem = nwg & 7;
    return xcd * per + (xcd < rem ? xcd : rem) + local;
}

// The tile a persistent workgroup takes after `lid`, or -1.  full_end = (total / G) * G.  The rounds in
// which every workgroup has a tile are walked in the XCD-contiguous numbering; the tiles of the last,
// partial round are dealt by the hardware's own workgroup id instead, which spreads them evenly over
// the XCDs and their compute units (in the contiguous numbering they would all land on the first XCDs).
__device__ __forceinline__ int next_tile(int lid, int G, int full_end, int total, int block) {
    if (lid + G < full_end) return lid + G;
    if (lid >= full_end) return -1;                       // that was the extra tile
    const int extra = full_end + block;
    return extra < total ? extra : -1;
}

// ---------------------------------------------------------------------------
// Tile staging: global -> registers -> LDS
// ---------------------------------------------------------------------------

// Chunk swizzle of a K-inner tile.  Rows hold CPR = KT/4 chunks of 16 bytes, no padding.
// Measured on gfx950: a ds_read_b128 serves 16 lanes per cycle from 16 chunk slots (256
// bytes wide), a ds_write_b128 8 lanes per cycle from 8 slots.  The fragment reads walk
// DOWN the rows (16 consecutive rows, same logical chunk), the staging stores walk ALONG
// a row; XOR-ing the chunk index with the index of the row's 256-byte group puts the 16
// rows of a read on 16 different slots and leaves the stores a permutation of a
// contiguous run.
template <int KT>
__device__ __forceinline__ int kin_swizzle(int row) {
    static_assert(KT == 16 || KT == 32 || KT == 64 || KT == 128 || KT == 256, "k per row: 16, 32, 64, 128 or 256");
    return (KT == 16) ? ((row >> 2) & 3) : (KT == 32) ? ((row >> 1) & 7) : (row & 15);
}

// Which tile row an LDS row of a K-inner operand holds.  IL == 1: the same row.  IL > 1 (the B
// operand, IL = the wavefront's MFMA blocks along the columns): inside each run of IL*32 rows, LDS row
// 32*j + r holds tile row IL*r + j, so that lane r's IL blocks are IL CONSECUTIVE columns of C and leave
// in one vector store, as they do for a K-outer operand.  Only the global side of the staging sees
// this; the LDS layout, its swizzle and the fragment reads are the same for every IL.
template <int IL>
__device__ __forceinline__ int kin_tile_row(int lds_row) {
    if constexpr (IL == 1) return lds_row;
    const int local = lds_row % (IL * 32);
    return lds_row - local + IL * (local % 32) + local / 32;
}

// K-inner operand: R rows of KT consecutive k.  LDS row stride KT floats, chunks swizzled.
template <int R, int KT, int IL = 1>
struct KInner {
    static constexpr int CPR = KT / 4;            // float4 chunks per row
    static constexpr int RPP = NTHREADS / CPR;    // rows per pass
    static constexpr int PASSES = R / RPP;
    static constexpr int LDS_STRIDE = KT;
    static constexpr int LDS_FLOATS = R * LDS_STRIDE;
    static_assert(R % RPP == 0 && PASSES >= 1, "tile does not divide over the workgroup");

    int off[PASSES];   // byte offset of this thread's chunk, or OOB_OFFSET if its row is outside
    int kcol;          // k offset of this thread's chunk inside the tile
    int row_first;     // tile row of the first pass
    int chunk;         // logical chunk index in the row

    __device__ __forceinline__ void init(int t, int row0, int outer_bound, int ld) {
        const int c = t % CPR, r0 = t / CPR;
        kcol = c * 4;
        row_first = r0;
        chunk = c;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int r = kin_tile_row<IL>(r0 + s * RPP);
            off[s] = (row0 + r < outer_bound) ? (r * ld + c * 4) * 4 : OOB_OFFSET;
        }
    }
    // base points at (row0, k) of the operand; k_left = k_limit - k
    // GUARD false: the caller knows that the whole stage lies inside K (k_left >= KT), and the per-lane
    // test, which costs vector instructions between the MFMAs, is left out
    // soff: a wave-uniform byte offset on top of base (the stage's distance from the tile's first one)
    template <bool GUARD = true>
    __device__ __forceinline__ void load(v4f (&reg)[PASSES], const float* base, int k_left, int soff = 0) const {
        const bool kok = !GUARD || kcol < k_left;
#pragma unroll
        for (int s = 0; s < PASSES; s++) reg[s] = buffer_load_f4(base, kok ? off[s] : OOB_OFFSET, soff);
    }
    __device__ __forceinline__ void store(const v4f (&reg)[PASSES], float* lds) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int r = row_first + s * RPP;
            *(v4f*)(lds + r * LDS_STRIDE + 4 * (chunk ^ kin_swizzle<KT>(r))) = reg[s];
        }
    }
    // ---- direct global -> LDS staging (no registers).  The hardware places lane l's 16 bytes at
    // (wave's LDS base) + 16*l, so thread t fills LDS chunk position s*NTHREADS + t and the swizzle
    // moves to the global side: the thread at slot c of row r fetches logical chunk c ^ swizzle(r).
    int dma_kcol[PASSES];
    __device__ __forceinline__ void init_dma(int t, int row0, int outer_bound, int ld) {
        const int slot = t % CPR, r0 = t / CPR;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int c = slot ^ kin_swizzle<KT>(r0 + s * RPP);
            const int r = kin_tile_row<IL>(r0 + s * RPP);
            dma_kcol[s] = c * 4;
            off[s] = (row0 + r < outer_bound) ? (r * ld + c * 4) * 4 : OOB_OFFSET;
        }
    }
    __device__ __forceinline__ void issue(float* lds, const float* base, int k_left, int wave) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++)
            dma_f4(base, lds + (s * NTHREADS + wave * 64) * 4, dma_kcol[s] < k_left ? off[s] : OOB_OFFSET);
    }
    // one of the PASSES transfers of a stage, for callers that place them between other instructions
    __device__ __forceinline__ void issue_pass(int s, float* lds, const float* base, int k_left, int wave) const {
        dma_f4(base, lds + (s * NTHREADS + wave * 64) * 4, dma_kcol[s] < k_left ? off[s] : OOB_OFFSET);
    }
    // the lane's byte offset for transfer s of a stage with k_left k still inside the operand
    __device__ __forceinline__ int dma_offset(int s, int k_left) const { return dma_kcol[s] < k_left ? off[s] : OOB_OFFSET; }
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
    template <bool GUARD = true>
    __device__ __forceinline__ void load(v4f (&reg)[PASSES], const float* base, int k_left, int soff = 0) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++)
            reg[s] = buffer_load_f4(base, (!GUARD || krow + s * RPP < k_left) ? off[s] : OOB_OFFSET, soff);
    }
    __device__ __forceinline__ void store(const v4f (&reg)[PASSES], float* lds) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++) *(v4f*)(lds + lds_at + s * RPP * LDS_STRIDE) = reg[s];
    }
    // direct global -> LDS staging: thread t's chunk of pass s already sits at LDS chunk s*NTHREADS + t
    __device__ __forceinline__ void init_dma(int t, int col0, int inner_bound, int ld) { init(t, col0, inner_bound, ld); }
    __device__ __forceinline__ void issue(float* lds, const float* base, int k_left, int wave) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++)
            dma_f4(base, lds + (s * NTHREADS + wave * 64) * 4, (krow + s * RPP < k_left) ? off[s] : OOB_OFFSET);
    }
    __device__ __forceinline__ void issue_pass(int s, float* lds, const float* base, int k_left, int wave) const {
        dma_f4(base, lds + (s * NTHREADS + wave * 64) * 4, (krow + s * RPP < k_left) ? off[s] : OOB_OFFSET);
    }
    __device__ __forceinline__ int dma_offset(int s, int k_left) const { return (krow + s * RPP < k_left) ? off[s] : OOB_OFFSET; }
    __device__ __forceinline__ static const float* tile_base(const float* X, int col0, int k, int ld) {
        return X + (size_t)k * ld + col0;
    }
    __device__ __forceinline__ static size_t k_advance(int ld) { return (size_t)KT * ld; }
};

// Implicit-GEMM convolution: the A operand of Y[GM, OC] = A[GM, GK] * W[OC, GK]^T is never
// materialised.  Row m = (n, oh, ow) and column k = (fh, fw, ic) of A is X[n, oh*sh - ph + fh,
// ow*sw - pw + fw, ic], or zero when that pixel lies in the padding.  IC is a multiple of 4, so a
// 16-byte chunk of 4 consecutive k stays inside one pixel; the chunk's address is
// row part (fixed per tile) + k part (changes per stage), and "in the padding" / "row outside" /
// "k beyond GK" all become the out-of-range offset that makes the load return zeros.
// Same LDS layout and swizzle as KInner, so the fragment reads do not know the difference.
template <int R, int KT>
struct ConvInner {
    static constexpr int CPR = KT / 4;
    static constexpr int RPP = NTHREADS / CPR;
    static constexpr int PASSES = R / RPP;
    static constexpr int LDS_STRIDE = KT;
    static constexpr int LDS_FLOATS = R * LDS_STRIDE;
    static_assert(R % RPP == 0 && PASSES >= 1, "tile does not divide over the workgroup");

    int base[PASSES];   // element offset of pixel (n, oh*sh - ph, ow*sw - pw), channel kcol
    int ih0[PASSES];    // oh*sh - ph, or far below zero for a row outside the matrix
    int iw0[PASSES];
    int kcol, row_first, chunk;

    __device__ __forceinline__ void init_conv(int t, int row0, int gm, const GemmParams& p) {
        const int c = t % CPR, r0 = t / CPR;
        kcol = c * 4;
        row_first = r0;
        chunk = c;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int m = row0 + r0 + s * RPP;
            const int q = m / p.cv_OW, ow = m - q * p.cv_OW;
            const int n = q / p.cv_OH, oh = q - n * p.cv_OH;
            const int ih = oh * p.cv_sh - p.cv_ph, iw = ow * p.cv_sw - p.cv_pw;
            ih0[s] = (m < gm) ? ih : -(1 << 30);
            iw0[s] = iw;
            base[s] = ((n * p.cv_IH + ih) * p.cv_IW + iw) * p.cv_IC + kcol;
        }
    }
    // k = first k of the stage; k_left = GK - k
    __device__ __forceinline__ void load_conv(v4f (&reg)[PASSES], const float* X, int k_left, int k,
                                              const GemmParams& p) const {
        const int kk = k + kcol;                     // < 2^24, checked by the host
        // kk = (fh * FW + fw) * IC + ic by float reciprocals with an exact integer correction
        int pix = (int)((float)kk * p.cv_rcp_IC);
        int ic = kk - pix * p.cv_IC;
        if (ic < 0) { pix--; ic += p.cv_IC; }
        if (ic >= p.cv_IC) { pix++; ic -= p.cv_IC; }
        int fh = (int)((float)pix * p.cv_rcp_FW);
        int fw = pix - fh * p.cv_FW;
        if (fw < 0) { fh--; fw += p.cv_FW; }
        if (fw >= p.cv_FW) { fh++; fw -= p.cv_FW; }
        const int koff = (fh * p.cv_IW + fw) * p.cv_IC + ic - kcol;
        const bool kok = kcol < k_left;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const bool ok = kok && (unsigned)(ih0[s] + fh) < (unsigned)p.cv_IH &&
                            (unsigned)(iw0[s] + fw) < (unsigned)p.cv_IW;
            reg[s] = buffer_load_f4(X, ok ? (base[s] + koff) * 4 : OOB_OFFSET);
        }
    }
    // The same for a stage that lies inside one filter tap (IC a multiple of KT): the tap (fh, fw)
    // and the stage's first channel ic0 are the same for every lane, so the caller keeps them in
    // scalar registers and the lanes are left with two compares and one add per row.
    __device__ __forceinline__ void load_conv_tap(v4f (&reg)[PASSES], const float* X, int fh, int fw, int ic0,
                                                  const GemmParams& p) const {
        const int koff4 = ((fh * p.cv_IW + fw) * p.cv_IC + ic0) * 4;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const bool ok = (unsigned)(ih0[s] + fh) < (unsigned)p.cv_IH &&
                            (unsigned)(iw0[s] + fw) < (unsigned)p.cv_IW;
            reg[s] = buffer_load_f4(X, ok ? base[s] * 4 + koff4 : OOB_OFFSET);
        }
    }
    __device__ __forceinline__ void store(const v4f (&reg)[PASSES], float* lds) const {
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int r = row_first + s * RPP;
            *(v4f*)(lds + r * LDS_STRIDE + 4 * (chunk ^ kin_swizzle<KT>(r))) = reg[s];
        }
    }
    // the descriptor's base is X itself: every offset is absolute (X holds fewer than 2^29 floats)
    __device__ __forceinline__ static const float* tile_base(const float* X, int, int, int) { return X; }
    __device__ __forceinline__ static size_t k_advance(int) { return 0; }
};

// ---------------------------------------------------------------------------
// Fragment reads: LDS -> MFMA operands for one group of 8 k
//   frag[b][q]: operand of block b for MFMA step q (k = 8*g + 4*h + q)
// ---------------------------------------------------------------------------
template <int T, int KT>
__device__ __forceinline__ void read_frag_kinner(float (&frag)[T][4], const float* lds,
                                                 int wave_row0, int g, int r, int h) {
    // wave_row0 and b*32 are multiples of 32, so the swizzle depends on r alone
    const int chunk = (g * 2 + h) ^ kin_swizzle<KT>(r);
#pragma unroll
    for (int b = 0; b < T; b++) {
        const v4f v = *(const v4f*)(lds + (wave_row0 + b * 32 + r) * KT + chunk * 4);
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
// Epilogue shared by the kernels: predicated streaming stores of one tile's accumulators.
// ---------------------------------------------------------------------------
// MFMA block element e of lane (r,h): block row = 8*(e/4) + 4*h + e%4, block col = r.
// A operand, K-inner: block b covers 32 consecutive rows; K-outer: rows {TM*x + b}.  B operand, either
// layout: block b of lane r is column TN*r + b (the K-inner staging interleaves its rows for this), so a
// lane's TN values of one row are consecutive columns and leave in one vector store.
// BIAS: the bias row is added before the store (the lane's columns are the same for all of its
// rows); "+ 0.0f" is the gamma term of the separate bias launch this replaces: it turns a -0 sum
// into +0, so fused and unfused results share every bit.  A template parameter rather than a
// run-time test, so the plain products carry none of it.
// The stores go through a buffer descriptor whose base is the tile's origin: a lane outside C gets
// an out-of-range offset and the hardware drops its store, so the whole epilogue is straight-line
// code -- no branch per store and 32-bit offset arithmetic only.
template <bool A_KIN, bool B_KIN, int TM, int TN, bool BIAS>
__device__ __forceinline__ void store_tile(const v16f (&acc)[TM][TN], const GemmParams& p, int row0,
                                           int col0, float* c_ptr, int wm, int wn, int r, int h) {
    constexpr int NT_STORE = 2;   // cache policy bit "nt": C is written once and not read back here
    float bias_v[TN];
    if constexpr (BIAS) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = col0 + wn * TN * 32 + TN * r + j;
            bias_v[j] = col < p.bias_width ? p.bias[col] : 0.0f;
        }
    }
    // A store's address = tile origin (descriptor) + lane part (vector offset: the lane's first row
    // and its column) + row part (scalar offset: a compile-time row count times the row pitch).  The
    // hardware checks vector + scalar offset against the descriptor's size, which ends behind C's last
    // row: the rows of the tile beyond C are dropped there, with no instruction spent on them; a lane
    // whose columns lie beyond C carries an offset that is out of range from the start.
    const int ldc4 = p.ldc * 4;
    const int rows_left = p.rows - row0, cols_left = p.cols - col0;
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(c_ptr + (size_t)row0 * p.ldc + col0), 0, rows_left > 0 ? (rows_left > 256 ? 256 : rows_left) * ldc4 : 0, RSRC_FLAGS);   // a tile has at most 256 rows
    const int lane_row = wm * TM * 32 + (A_KIN ? 4 * h : TM * 4 * h);
    const int lcol = wn * TN * 32 + TN * r;
    const int lane_off = (lcol < cols_left) ? lane_row * ldc4 + lcol * 4 : OOB_OFFSET;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int crow = A_KIN ? (i * 32 + 8 * (e / 4) + (e % 4)) : (TM * (8 * (e / 4) + (e % 4)) + i);
            const int row_soff = crow * ldc4;
            float out[TN];
#pragma unroll
            for (int j = 0; j < TN; j++) {
                out[j] = acc[i][j][e];
                if constexpr (BIAS)
                    if (row0 + lane_row + crow < p.bias_rows) out[j] = (out[j] + bias_v[j]) + 0.0f;
            }
            if constexpr (TN == 1) {
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, out[0]), rsrc, lane_off, row_soff,
                                                      NT_STORE);
            } else if constexpr (TN == 2) {
                typedef unsigned int v2u __attribute__((ext_vector_type(2)));
                const v2f v = {out[0], out[1]};
                __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u, v), rsrc, lane_off, row_soff, NT_STORE);
            } else {
                const v4f v = {out[0], out[1], out[2], out[3]};
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), rsrc, lane_off, row_soff, NT_STORE);
            }
        }
    }
}

// One group of 8 k: fragments from LDS, then 4 MFMA steps over the wave's TM x TN blocks.
template <bool A_KIN, bool B_KIN, int TM, int TN, int BM, int BN, int KT>
__device__ __forceinline__ void mma_group(v16f (&acc)[TM][TN], const float* as, const float* bs, int wm,
                                          int wn, int g, int r, int h) {
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
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q], acc[i][j], 0, 0, 0);
}

// The same for a tile's last stage, of which only `k_here` k exist from this group on (>= 1): the steps
// whose k lie beyond for both lane halves are left out (their operands would be zeros).
template <bool A_KIN, bool B_KIN, int TM, int TN, int BM, int BN, int KT>
__device__ __forceinline__ void mma_group_upto(v16f (&acc)[TM][TN], const float* as, const float* bs, int wm,
                                               int wn, int g, int r, int h, int k_here) {
    float fa[TM][4], fb[TN][4];
    if constexpr (A_KIN) read_frag_kinner<TM, KT>(fa, as, wm * TM * 32, g, r, h);
    else                 read_frag_kouter<TM, BM>(fa, as, wm * TM * 32, g, r, h);
    if constexpr (B_KIN) read_frag_kinner<TN, KT>(fb, bs, wn * TN * 32, g, r, h);
    else                 read_frag_kouter<TN, BN>(fb, bs, wn * TN * 32, g, r, h);
#pragma unroll
    for (int q = 0; q < 4; q++)
        if (q < k_here) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q], acc[i][j], 0, 0, 0);
        }
}

// ---------------------------------------------------------------------------
// The rim: the last 1..4 rows and / or columns of a C whose extent is that much past a multiple of
// the tile.  A whole row or column of tiles for them would be all but empty (257 x 385 in 64 x 64
// tiles: 35 tiles where 24 hold all but one row and one column); the reference carves such edges
// down to tiles of 4 (MM/matMul.cuh:24-43) and has kernels for a C of 4 columns
// (MM/matMul_sernel.cuh:17-30).  Here the tiles cover the part of C that fills them, and the first
// rim_wgs workgroups of the same launch compute the rim with plain FMAs, straight from memory: the
// rim's matrix work is tiny (a few rows), what it needs is every byte of one operand once more, and
// that comes out of the L2 while the tiles run.
// One job = 64 outputs along the rim x up to 4 across it: the workgroup's four wavefronts each take a
// quarter of K (contiguous, so a lane that walks along a row of its own stays on a cache line), the
// quarters meet in LDS and are added in k order.  Row jobs: rows R0 .. R0+rr-1, 64 columns; column
// jobs: 64 rows below R0, columns C0 .. C0+rc-1.
// Four consecutive k of one operand line: a K-inner line (k contiguous, padded to a multiple of 4 in memory)
// in one 16-byte load, a K-outer one (k is the row) in four loads that stop where the operand ends.
template <bool KIN>
__device__ __forceinline__ v4f rim_load4(const float* line, size_t sk, int k, int k_end) {
    if constexpr (KIN) {
        return *(const v4f*)(line + k);
    } else {
        // every load is made (of the operand's last k where its own lies beyond) and the value dropped
        // afterwards: no branch around a load, so that they all are on their way together
        const int last = k_end - 1;
        v4f v;
        v.x = line[(size_t)min(k + 0, last) * sk];
        v.y = line[(size_t)min(k + 1, last) * sk];
        v.z = line[(size_t)min(k + 2, last) * sk];
        v.w = line[(size_t)min(k + 3, last) * sk];
        v.y = k + 1 < k_end ? v.y : 0.0f;
        v.z = k + 2 < k_end ? v.z : 0.0f;
        v.w = k + 3 < k_end ? v.w : 0.0f;
        return v;
    }
}

// acc[x] += sum over k in [k0, k1) of walk(k) * fixed[x](k) for x < NX: `walk` is the lane's own operand line
// (64 lanes, 64 lines), the `fixed` ones are the same for every lane.  16 k per turn, the loads ahead of the
// FMAs.  NX = 1 for a rim of a single row or column (the commonest: an extent one past a multiple of 64): a
// quarter of the loads and FMAs of NX = 4, and these vector instructions keep the SIMD's MFMAs waiting.
template <bool WALK_KIN, bool FIXED_KIN, int NX>
__device__ __forceinline__ void rim_dot(float (&acc)[4], const float* walk, size_t w_sk, const float* const (&fixed)[4],
                                        size_t f_sk, int k0, int k1, int k_end) {
#pragma unroll 4
    for (int k = k0; k < k1; k += 4) {
        const v4f w = rim_load4<WALK_KIN>(walk, w_sk, k, k_end);
#pragma unroll
        for (int x = 0; x < NX; x++) {
            const v4f f = rim_load4<FIXED_KIN>(fixed[x], f_sk, k, k_end);
            acc[x] = fmaf(w.x, f.x, acc[x]);
            acc[x] = fmaf(w.y, f.y, acc[x]);
            acc[x] = fmaf(w.z, f.z, acc[x]);
            acc[x] = fmaf(w.w, f.w, acc[x]);
        }
    }
}

template <bool A_KIN, bool B_KIN, bool BIAS>
__device__ __forceinline__ void rim_job(const GemmParams& p, float* lds, int job) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int R0 = p.rows, C0 = p.cols;                    // the tiles' part of C
    const int rr = p.rim_rows, rc = p.rim_cols;
    const int row_jobs = rr > 0 ? (C0 + rc + 63) / 64 : 0, col_jobs = rc > 0 ? (R0 + 63) / 64 : 0;
    const int per_z = row_jobs + col_jobs;
    const int z = job / per_z;
    if (z >= p.nz) return;                                 // the job count is rounded up to whole groups of 8
    int seg = job - z * per_z;
    const bool row_job = seg < row_jobs;
    if (!row_job) seg -= row_jobs;
    const float* A = p.A + (size_t)z * p.sA;
    const float* B = p.B + (size_t)z * p.sB;
    float* C = p.C + (size_t)z * p.sC;
    const size_t a_si = A_KIN ? p.lda : 1, a_sk = A_KIN ? 1 : p.lda;     // A(i, k) = A[i * a_si + k * a_sk]
    const size_t b_sk = B_KIN ? 1 : p.ldb, b_sj = B_KIN ? p.ldb : 1;     // B(k, j) = B[k * b_sk + j * b_sj]
    const int a_rows = A_KIN ? p.a_outer : p.a_inner, b_cols = B_KIN ? p.b_outer : p.b_inner;   // that exist in memory
    // the k both operands have; a K-inner operand's lines are padded with zeros to a multiple of 4
    const int K = min(p.k_total, min(A_KIN ? p.a_inner : p.a_outer, B_KIN ? p.b_inner : p.b_outer));
    const int kq = (K + 15) / 16 * 4;                      // a quarter of K, in whole groups of 4
    const int k0 = wave * kq, k1 = min(K, k0 + kq);
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    bool ok;
    if (row_job) {      // rows R0 .. R0+rr-1 of A against the lane's column of B
        const int j = seg * 64 + lane;
        ok = j < b_cols;
        const float* const fixed[4] = {A + (size_t)min(R0, a_rows - 1) * a_si, A + (size_t)min(R0 + (1 < rr ? 1 : 0), a_rows - 1) * a_si,
                                       A + (size_t)min(R0 + (2 < rr ? 2 : 0), a_rows - 1) * a_si,
                                       A + (size_t)min(R0 + (3 < rr ? 3 : 0), a_rows - 1) * a_si};
        if (rr == 1) rim_dot<B_KIN, A_KIN, 1>(acc, B + (ok ? (size_t)j * b_sj : 0), b_sk, fixed, a_sk, k0, k1, K);
        else         rim_dot<B_KIN, A_KIN, 4>(acc, B + (ok ? (size_t)j * b_sj : 0), b_sk, fixed, a_sk, k0, k1, K);
    } else {            // the lane's row of A against columns C0 .. C0+rc-1 of B
        const int i = seg * 64 + lane;
        ok = i < R0 && i < a_rows;
        const float* const fixed[4] = {B + (size_t)min(C0, b_cols - 1) * b_sj, B + (size_t)min(C0 + (1 < rc ? 1 : 0), b_cols - 1) * b_sj,
                                       B + (size_t)min(C0 + (2 < rc ? 2 : 0), b_cols - 1) * b_sj,
                                       B + (size_t)min(C0 + (3 < rc ? 3 : 0), b_cols - 1) * b_sj};
        if (rc == 1) rim_dot<A_KIN, B_KIN, 1>(acc, A + (ok ? (size_t)i * a_si : 0), a_sk, fixed, b_sk, k0, k1, K);
        else         rim_dot<A_KIN, B_KIN, 4>(acc, A + (ok ? (size_t)i * a_si : 0), a_sk, fixed, b_sk, k0, k1, K);
    }
#pragma unroll
    for (int x = 0; x < 4; x++) lds[(wave * 4 + x) * 64 + lane] = acc[x];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int x = 0; x < 4; x++) {
        const float sum = ((lds[(0 * 4 + x) * 64 + lane] + lds[(1 * 4 + x) * 64 + lane]) + lds[(2 * 4 + x) * 64 + lane]) +
                          lds[(3 * 4 + x) * 64 + lane];
        // a row of A or a column of B that does not exist in memory (the operand's own padding) gives zeros
        const int i = row_job ? R0 + x : seg * 64 + lane, j = row_job ? seg * 64 + lane : C0 + x;
        const bool inside = row_job ? (x < rr && j < C0 + rc) : (x < rc && i < R0);
        float value = (ok && (row_job ? i < a_rows : j < b_cols)) ? sum : 0.0f;
        if constexpr (BIAS) {   // as the tiles' epilogue adds it (see store_tile)
            if (inside && i < p.bias_rows) value = (value + (j < p.bias_width ? p.bias[j] : 0.0f)) + 0.0f;
        }
        if (inside) C[(size_t)i * p.ldc + j] = value;
    }
}

// ---------------------------------------------------------------------------
// The kernel
//   A_KIN / B_KIN : operand is K-inner
//   WM x WN       : wavefront grid in the workgroup (WM*WN == 4)
//   TM x TN       : 32x32 MFMA blocks per wavefront
//   KT            : k per LDS stage
//
// Workgroups are persistent: workgroup w works on the logical tiles w, w+G, w+2G, ...
// (G = grid size, chosen by the launcher as what the device keeps resident).  The
// first LDS stage of the next tile is fetched during the last k-step of the current
// one, and the stores of a finished tile drain while the next tile computes, so a
// stream of short tiles (small K, large C) keeps the matrix cores busy.
// ---------------------------------------------------------------------------
struct TileCtx {
    const float* a_ptr;   // A at (row0, k0) of this tile's batch / slice
    const float* b_ptr;
    float* c_ptr;         // C (or split-K partial) of this tile's batch / slice
    int row0, col0;
    int k0;               // first k of the slice
    int ka_lim, kb_lim;   // first k each operand may no longer touch
    int nstage;           // LDS stages to run (>= 1; an empty slice runs one all-zero stage)
};

// n / d for 0 <= n < 2^31 with the pair gemm_fill_tile_divisors made for d
__device__ __forceinline__ int div_by(int n, unsigned mul, unsigned shift) {
    return (int)(__umulhi((unsigned)n << 1, mul) >> shift);
}

template <bool A_KIN, bool B_KIN, int BM, int BN, int KT, typename LoadA, typename LoadB>
__device__ __forceinline__ TileCtx decode_tile(const GemmParams& p, int lid) {
    TileCtx c;
    // the three divisions are multiply-and-shift with host-made constants: a division by a run-time
    // value costs some 25 instructions, and this runs between the matrix work of two tiles
    const int tiles = p.tiles_m * p.tiles_n;
    const int z = div_by(lid, p.div_tiles_mul, p.div_tiles_shift);
    int tt = lid - z * tiles;
    // bands of 8 tile rows, walked row-fastest, keep one XCD's concurrent tiles compact
    constexpr int BAND = 8;
    const int band_sz = BAND * p.tiles_n;
    const int band = div_by(tt, p.div_band_mul, p.div_band_shift);
    const int first_m = band * BAND;
    const bool short_band = p.tiles_m - first_m < BAND;
    const int band_rows = short_band ? (p.tiles_m - first_m) : BAND;
    tt -= band * band_sz;
    const int tile_n = short_band ? div_by(tt, p.div_last_mul, p.div_last_shift) : (tt >> 3);
    const int tile_m = first_m + (tt - tile_n * band_rows);
    c.row0 = tile_m * BM;
    c.col0 = tile_n * BN;
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
    c.k0 = k0;
    c.ka_lim = min(k1, A_KIN ? p.a_inner : p.a_outer);
    c.kb_lim = min(k1, B_KIN ? p.b_inner : p.b_outer);
    const int n = (k1 - k0 + KT - 1) / KT;
    c.nstage = n > 0 ? n : 1;
    c.a_ptr = LoadA::tile_base(A, c.row0, k0, p.lda);
    c.b_ptr = LoadB::tile_base(B, c.col0, k0, p.ldb);
    c.c_ptr = C;
    return c;
}

// Wavefronts per SIMD the register allocator should leave room for: as many workgroups
// as the LDS footprint lets a compute unit hold (160 KiB), at most 4.
template <bool A_KIN, bool B_KIN, int BM, int BN, int KT>
constexpr int target_occupancy() {
    const int lds = 2 * 4 * (BM * KT + BN * KT);
    const int fit = (160 * 1024) / lds;
    return fit > 4 ? 4 : (fit < 1 ? 1 : fit);
}

template <bool A_KIN, bool B_KIN, int WM, int WN, int TM, int TN, int KT, bool BIAS, bool CONV = false,
          bool PAIRED = false, bool RIM = false>
__global__ __launch_bounds__(NTHREADS, (target_occupancy<A_KIN, B_KIN, WM * TM * 32, WN * TN * 32, KT>()))
void gemm_f32_mfma(const GemmParams p) {
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    static_assert(!CONV || (A_KIN && B_KIN), "the convolution is the A * B^T form with a gathered A");
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    using LoadA = typename std::conditional<
        CONV, ConvInner<BM, KT>,
        typename std::conditional<A_KIN, KInner<BM, KT>, KOuter<BM, KT>>::type>::type;
    using LoadB = typename std::conditional<B_KIN, KInner<BN, KT, TN>, KOuter<BN, KT>>::type;

    __shared__ __attribute__((aligned(16))) float As[2][LoadA::LDS_FLOATS];
    __shared__ __attribute__((aligned(16))) float Bs[2][LoadB::LDS_FLOATS];
    // The single-block wavefronts (64 x 64 tiles) reach the two arrays through a pointer, the others by
    // name.  No difference in meaning; the compiler's code for the paired 64 x 64 kernel is 9 % faster
    // this way (A*B 1000x777x1531: 35.8 -> 32.7 us) and for 128 x 64 2.6 % slower, so each keeps the
    // form that measured better.
    constexpr bool LDS_BY_POINTER = TM * TN == 1;
    float (*As_ptr)[LoadA::LDS_FLOATS] = As;
    float (*Bs_ptr)[LoadB::LDS_FLOATS] = Bs;

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    const size_t a_step = LoadA::k_advance(p.lda), b_step = LoadB::k_advance(p.ldb);
    // the same in bytes, for the paired form (whose launcher checks that K times this fits 32 bits)
    const int a_step4 = (int)(a_step * 4), b_step4 = (int)(b_step * 4);

    const int total = p.tiles_m * p.tiles_n * p.nz;
    int block = blockIdx.x, G = gridDim.x;
    if constexpr (RIM) {
        // the launch's first workgroups compute the rim of C (see rim_job); the others are the tiles'
        static_assert(LoadA::LDS_FLOATS >= 1024, "the rim's partial sums take 1024 floats of LDS");
        if (block < p.rim_wgs) {
            rim_job<A_KIN, B_KIN, BIAS>(p, &As[0][0], block);
            return;
        }
        block -= p.rim_wgs;
        G -= p.rim_wgs;
    }
    int lid = xcd_contiguous_id(block, G);   // G <= total, so lid is a valid tile
    const int full_end = (total / G) * G;

    TileCtx cur = decode_tile<A_KIN, B_KIN, BM, BN, KT, LoadA, LoadB>(p, lid);
    LoadA la;
    LoadB lb;
    if constexpr (CONV) la.init_conv(t, cur.row0, p.a_outer, p);
    else la.init(t, cur.row0, A_KIN ? p.a_outer : p.a_inner, p.lda);
    lb.init(t, cur.col0, B_KIN ? p.b_outer : p.b_inner, p.ldb);

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = (v16f)(0.0f);

    v4f ra[LoadA::PASSES], rb[LoadB::PASSES];

    // Convolution: the order in which the K chunks of a tile are visited.  In storage order
    // (filter row, filter column, channel) two uses of the same input element are IC/KT stages
    // apart, and by then the other workgroups of the XCD have pushed it out of the L2.  With the
    // filter column running fastest, consecutive stages read the same pixels shifted by one, so
    // all but 1/OW of a stage's input is what the previous stage fetched.  Any order gives the
    // same sum up to rounding; whole chunks only, so IC must be a multiple of KT -- and then a
    // stage lies inside one filter tap, which the scalar unit tracks (cv_fh, cv_fw, cv_ic).
    const int cv_nic = CONV ? p.cv_IC / KT : 0;
    const bool cv_walk = CONV && p.cv_walk && (p.cv_IC % KT == 0);
    int cv_fh = 0, cv_fw = 0, cv_ic = 0, cv_k = 0;

    // stage 0 of the first tile
    if constexpr (CONV) {
        if (cv_walk) la.load_conv_tap(ra, cur.a_ptr, 0, 0, 0, p);
        else la.load_conv(ra, cur.a_ptr, cur.ka_lim - cur.k0, cur.k0, p);
    } else la.load(ra, cur.a_ptr, cur.ka_lim - cur.k0);
    lb.load(rb, cur.b_ptr, cur.kb_lim - cur.k0);
    la.store(ra, LDS_BY_POINTER ? As_ptr[0] : As[0]);
    lb.store(rb, LDS_BY_POINTER ? Bs_ptr[0] : Bs[0]);
    __syncthreads();
    int buf = 0;

    for (;;) {
        const int next_lid = next_tile(lid, G, full_end, total, block);
        const bool has_next = next_lid >= 0;
        TileCtx nxt = cur;
        const float* a_ptr = cur.a_ptr;
        const float* b_ptr = cur.b_ptr;
        if constexpr (CONV) { cv_fh = 0; cv_fw = 0; cv_ic = 0; cv_k = 0; }

        // One stage: the following stage goes global -> registers, the matrix work runs on LDS buffer
        // `b`, the registers go into the other buffer, barrier.
        //   b      the buffer multiplied from: an int, or an integral_constant where the caller knows it
        //          (the LDS addresses are then immediates instead of vector arithmetic per stage)
        //   inner  true_type where the caller knows that the stage fetched belongs to this tile and
        //          lies wholly inside K: no "last stage?" branch and no per-lane K test
        auto stage = [&](int it, auto b_sel, auto inner_tag) __attribute__((always_inline)) {
            constexpr bool INNER = decltype(inner_tag)::value;
            const int b = b_sel;
            const bool last = !INNER && (it + 1 == cur.nstage);
            bool fetched = false;
            constexpr bool BY_OFFSET = INNER && !CONV;
            if constexpr (!CONV) {
                if constexpr (INNER) {
                    // next stage of this tile -> registers; the stage's distance from the tile's first
                    // stage travels as the loads' scalar offset (one scalar add per operand and stage,
                    // where an advancing pointer has the descriptor rebuilt from it each time)
                    la.template load<false>(ra, cur.a_ptr, KT, (it + 1) * a_step4);
                    lb.template load<false>(rb, cur.b_ptr, KT, (it + 1) * b_step4);
                    fetched = true;
                }
            }
            if (BY_OFFSET) {
            } else if (!last) {          // next stage of this tile -> registers
                a_ptr += a_step;
                int knext;
                if constexpr (CONV) {
                    if (cv_walk) {       // next filter column; then next channel chunk; then next filter row
                        cv_k += p.cv_IC;
                        if (++cv_fw == p.cv_FW) {
                            cv_fw = 0;
                            cv_k += KT - p.cv_FW * p.cv_IC;
                            if (++cv_ic == cv_nic) { cv_ic = 0; cv_fh++; cv_k += (p.cv_FW - 1) * p.cv_IC; }
                        }
                    } else cv_k += KT;
                    knext = cv_k;
                    b_ptr = cur.b_ptr + cv_k;
                } else {
                    b_ptr += b_step;
                    knext = cur.k0 + (it + 1) * KT;
                }
                if constexpr (CONV) {
                    if (cv_walk) la.load_conv_tap(ra, a_ptr, cv_fh, cv_fw, cv_ic * KT, p);
                    else la.load_conv(ra, a_ptr, cur.ka_lim - knext, knext, p);
                } else la.template load<!INNER>(ra, a_ptr, cur.ka_lim - knext);
                lb.template load<!INNER>(rb, b_ptr, cur.kb_lim - knext);
                fetched = true;
            } else if (has_next) {       // first stage of the next tile -> registers
                nxt = decode_tile<A_KIN, B_KIN, BM, BN, KT, LoadA, LoadB>(p, next_lid);
                if constexpr (CONV) la.init_conv(t, nxt.row0, p.a_outer, p);
                else la.init(t, nxt.row0, A_KIN ? p.a_outer : p.a_inner, fresh(p.lda));
                lb.init(t, nxt.col0, B_KIN ? p.b_outer : p.b_inner, fresh(p.ldb));
                if constexpr (CONV) {
                    if (cv_walk) la.load_conv_tap(ra, nxt.a_ptr, 0, 0, 0, p);
                    else la.load_conv(ra, nxt.a_ptr, nxt.ka_lim - nxt.k0, nxt.k0, p);
                } else la.load(ra, nxt.a_ptr, nxt.ka_lim - nxt.k0);
                lb.load(rb, nxt.b_ptr, nxt.kb_lim - nxt.k0);
                fetched = true;
            }
            // the prefetch must be in flight before the matrix work starts: keep the scheduler
            // from sinking the loads down to their first use
            __builtin_amdgcn_sched_barrier(0);
            const float* as = LDS_BY_POINTER ? As_ptr[b] : As[b];
            const float* bs = LDS_BY_POINTER ? Bs_ptr[b] : Bs[b];
            // A tile's last stage: only the k that exist (K = 129 ends one k into its ninth stage of 16).  For the
            // single-block wavefronts only: in the larger tiles the second form of the matrix work costs registers
            // (the 128 x 128 paired kernels spilled some 200 with it), and a short K is not their business.
            if (TM * TN == 1 && !CONV && last) {
                const int k_stage = min(cur.ka_lim, cur.kb_lim) - (cur.k0 + it * KT);
#pragma unroll
                for (int g = 0; g < KT / 8; g++)
                    if (g * 8 < k_stage)
                        mma_group_upto<A_KIN, B_KIN, TM, TN, BM, BN, KT>(acc, as, bs, wm, wn, g, r, h, k_stage - g * 8);
            } else {
#pragma unroll
                for (int g = 0; g < KT / 8; g++)
                    mma_group<A_KIN, B_KIN, TM, TN, BM, BN, KT>(acc, as, bs, wm, wn, g, r, h);
            }
            if (fetched) {
                // one wait for all of the stage's loads (issued a whole stage of matrix work ago) instead
                // of one per staging register: vmcnt(0), the other counters left alone
                if constexpr (INNER) __builtin_amdgcn_s_waitcnt(0x0F70);
                la.store(ra, LDS_BY_POINTER ? As_ptr[b ^ 1] : As[b ^ 1]);
                lb.store(rb, LDS_BY_POINTER ? Bs_ptr[b ^ 1] : Bs[b ^ 1]);
            }
            __syncthreads();
        };

        int it = 0;
        if constexpr (PAIRED) {
            // Stages whose successor is an inner stage run in pairs with the buffer index known at
            // compile time; one single stage first if the tile starts on the odd buffer.  The rest
            // (the stages before a partial or the last stage, and the last one, which fetches for the
            // next tile) take the general form.  Measured at 4096^3: 33 instead of 49 instructions
            // beside the 32 MFMAs of a stage, 93 % instead of 90 % of the matrix peak; the extra
            // copies of the stage cost registers, which a short K does not earn back (the tile choice
            // takes this form from K = 512 on).
            int inner = (min(cur.ka_lim, cur.kb_lim) - cur.k0) / KT;   // whole stages inside K
            if (inner > cur.nstage) inner = cur.nstage;
            if (buf == 1 && it + 1 < inner) {
                stage(it, std::integral_constant<int, 1>(), std::true_type());
                it++;
                buf = 0;
            }
            if (buf == 0)
                for (; it + 2 < inner; it += 2) {
                    stage(it, std::integral_constant<int, 0>(), std::true_type());
                    stage(it + 1, std::integral_constant<int, 1>(), std::true_type());
                }
            if constexpr (!CONV) {   // the inner stages left the pointers alone
                a_ptr = cur.a_ptr + (size_t)it * a_step;
                b_ptr = cur.b_ptr + (size_t)it * b_step;
            }
        }
        for (; it < cur.nstage; it++) {
            stage(it, buf, std::false_type());
            buf ^= 1;
        }

        // ---- epilogue: predicated streaming stores (C is written once and never read back
        // here; they drain while the next tile computes) ----
        store_tile<A_KIN, B_KIN, TM, TN, BIAS>(acc, p, cur.row0, cur.col0, cur.c_ptr, wm, wn, r, h);
        if (!has_next) break;
        for (int i = 0; i < TM; i++)
            for (int j = 0; j < TN; j++) acc[i][j] = (v16f)(0.0f);
        cur = nxt;
        lid = next_lid;
    }
}

// ---------------------------------------------------------------------------
// The same product with the operands staged global -> LDS directly (buffer_load ... lds) through
// NS stage buffers, NS-1 stages in flight ahead of the one being multiplied.  No staging
// registers, no LDS stores by the waves, one barrier per stage.  The stream of stages runs across
// tile boundaries: while the last stages of a tile are multiplied the first stages of the
// workgroup's next tile are already on their way.
//
// Each stage buffer is its own __shared__ array and the buffer index is a compile-time constant
// at every use (the stage loop is unrolled NS times): that is what lets the compiler tell which
// in-flight transfer a fragment read depends on, instead of waiting for all of them.
//
// Synchronisation per stage: every wave waits until ITS OWN transfers of the stage have landed
// (vmcnt; transfers complete in order, so "at most the (NS-2) younger stages outstanding" is
// enough -- later stores only make the wait longer, never shorter), then the workgroup barrier
// makes all four waves' parts visible and at the same time guarantees that everybody has
// finished reading the buffer that the next transfer overwrites.  A stage slot with nothing
// left to fetch still issues its transfers with every lane out of range (zeros, no memory
// traffic) so that the count of younger transfers is the same constant everywhere.
// ---------------------------------------------------------------------------
template <bool A_KIN, bool B_KIN, int BM, int BN, int KT, int NS>
constexpr int target_occupancy_dma() {
    const int lds = NS * 4 * (BM * KT + BN * KT);
    const int fit = (160 * 1024) / lds;
    return fit > 4 ? 4 : (fit < 1 ? 1 : fit);
}

template <bool A_KIN, bool B_KIN, int WM, int WN, int TM, int TN, int KT, int NS, bool BIAS>
__global__ __launch_bounds__(NTHREADS, (target_occupancy_dma<A_KIN, B_KIN, WM * TM * 32, WN * TN * 32, KT, NS>()))
void gemm_f32_mfma_dma(const GemmParams p) {
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    static_assert(NS >= 3 && NS <= 4, "stage buffers: 3 or 4");
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    using LoadA = typename std::conditional<A_KIN, KInner<BM, KT>, KOuter<BM, KT>>::type;
    using LoadB = typename std::conditional<B_KIN, KInner<BN, KT, TN>, KOuter<BN, KT>>::type;
    constexpr int STAGE_FLOATS = LoadA::LDS_FLOATS + LoadB::LDS_FLOATS;
    constexpr int XFERS = LoadA::PASSES + LoadB::PASSES;      // transfers per wave per stage
    static_assert((NS - 2) * XFERS <= 63, "vmcnt holds 6 bits");

    __shared__ __attribute__((aligned(16))) float S0[STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float S1[STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float S2[STAGE_FLOATS];
    __shared__ __attribute__((aligned(16))) float S3[NS > 3 ? STAGE_FLOATS : 4];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    const size_t a_step = LoadA::k_advance(p.lda), b_step = LoadB::k_advance(p.ldb);

    const int total = p.tiles_m * p.tiles_n * p.nz;
    const int G = gridDim.x;
    int lid = xcd_contiguous_id(blockIdx.x, G);   // G <= total, so lid is a valid tile

    // ---- producer: the stage to fetch next ----
    int f_lid = lid;
    TileCtx ft = decode_tile<A_KIN, B_KIN, BM, BN, KT, LoadA, LoadB>(p, f_lid);
    LoadA la;
    LoadB lb;
    la.init_dma(t, ft.row0, A_KIN ? p.a_outer : p.a_inner, p.lda);
    lb.init_dma(t, ft.col0, B_KIN ? p.b_outer : p.b_inner, p.ldb);
    const float* fa_ptr = ft.a_ptr;
    const float* fb_ptr = ft.b_ptr;
    int f_it = 0;
    bool f_live = true;

    auto fetch = [&](float* stage) {
        const int k = ft.k0 + f_it * KT;
        la.issue(stage, fa_ptr, f_live ? ft.ka_lim - k : 0, wave);
        lb.issue(stage + LoadA::LDS_FLOATS, fb_ptr, f_live ? ft.kb_lim - k : 0, wave);
        if (f_live) {
            f_it++;
            fa_ptr += a_step;
            fb_ptr += b_step;
            if (f_it == ft.nstage) {
                f_lid += G;
                if (f_lid < total) {
                    ft = decode_tile<A_KIN, B_KIN, BM, BN, KT, LoadA, LoadB>(p, f_lid);
                    la.init_dma(t, ft.row0, A_KIN ? p.a_outer : p.a_inner, p.lda);
                    lb.init_dma(t, ft.col0, B_KIN ? p.b_outer : p.b_inner, p.ldb);
                    fa_ptr = ft.a_ptr;
                    fb_ptr = ft.b_ptr;
                    f_it = 0;
                } else {
                    f_live = false;
                }
            }
        }
    };
    auto stage_buf = [&](int s) -> float* { return s == 0 ? S0 : s == 1 ? S1 : s == 2 ? S2 : S3; };

    // ---- consumer: the tile being multiplied ----
    TileCtx cur = ft;
    int it = 0;
    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = (v16f)(0.0f);

#pragma unroll
    for (int s = 0; s < NS - 1; s++) fetch(stage_buf(s));

    bool running = true;
    while (running) {
#pragma unroll
        for (int s = 0; s < NS; s++) {
            if (!running) break;
            __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * XFERS));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            fetch(stage_buf((s + NS - 1) % NS));
            __builtin_amdgcn_sched_barrier(0);
            const float* as = stage_buf(s);
            const float* bs = as + LoadA::LDS_FLOATS;
#pragma unroll
            for (int g = 0; g < KT / 8; g++)
                mma_group<A_KIN, B_KIN, TM, TN, BM, BN, KT>(acc, as, bs, wm, wn, g, r, h);
            if (++it == cur.nstage) {
                store_tile<A_KIN, B_KIN, TM, TN, BIAS>(acc, p, cur.row0, cur.col0, cur.c_ptr, wm, wn, r, h);
                lid += G;
                if (lid < total) {
                    cur = decode_tile<A_KIN, B_KIN, BM, BN, KT, LoadA, LoadB>(p, lid);
                    it = 0;
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++) acc[i][j] = (v16f)(0.0f);
                } else {
                    running = false;
                }
            }
        }
    }
    // nothing of this wave may still be on its way into LDS when the wave ends
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
}

// ---------------------------------------------------------------------------
// Host side: tile choice and launch
// ---------------------------------------------------------------------------
// Workgroups of `kernel` a compute unit keeps resident, asked of the runtime once per instantiation
// (concurrent first calls store the same value).
template <typename Kernel>
static int resident_workgroups(std::atomic<int>& cache, Kernel kernel) {
    int n = cache.load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, NTHREADS, 0) != hipSuccess || n < 1) n = 1;
        cache.store(n, std::memory_order_relaxed);
    }
    return n;
}

template <bool A_KIN, bool B_KIN, bool BIAS, int WM, int WN, int TM, int TN, int KT, bool CONV = false,
          bool PAIRED = false, bool RIM = false>
static hipError_t launch_cfg(GemmParams p, hipStream_t stream) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    auto kernel = gemm_f32_mfma<A_KIN, B_KIN, WM, WN, TM, TN, KT, BIAS, CONV, PAIRED, RIM>;
    if constexpr (RIM) {
        // the tiles take the part of C that fills them; the rim's jobs (64 outputs along it each) go first
        // in the grid, in whole groups of 8 so that the tiles' workgroups keep their places on the XCDs
        static_assert(BM == 64 && BN == 64, "the rim's jobs are 64 outputs long");
        const int row_jobs = p.rim_rows > 0 ? (p.cols + 63) / 64 : 0, col_jobs = p.rim_cols > 0 ? (p.rows - p.rim_rows + 63) / 64 : 0;
        p.rows -= p.rim_rows;
        p.cols -= p.rim_cols;
        p.rim_wgs = (int)((((long long)(row_jobs + col_jobs) * p.nz) + 7) / 8 * 8);
    }
    p.tiles_m = (p.rows + BM - 1) / BM;
    p.tiles_n = (p.cols + BN - 1) / BN;
    const long long total = (long long)p.tiles_m * p.tiles_n * p.nz;
    if (total <= 0 || total > 0x7fffffffLL) return hipErrorInvalidValue;
    gemm_fill_tile_divisors(p);
    // workgroups the device keeps resident: one persistent workgroup per slot
    static std::atomic<int> resident_cache{0};   // per instantiation
    const int resident_per_cu = resident_workgroups(resident_cache, kernel);
    // One persistent workgroup per resident slot: every compute unit holds the same number of
    // workgroups, and the tiles of the last, partial round go one each to workgroups spread over the
    // units (next_tile), so that no unit has more than one tile above the average.
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const long long slots = (long long)num_cu * resident_per_cu;
    const long long grid = (total < slots ? total : slots) + (RIM ? p.rim_wgs : 0);
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
    return hipGetLastError();
}

template <bool A_KIN, bool B_KIN, bool BIAS, bool CONV = false>
static hipError_t launch_variant(const GemmParams& p, int tile, hipStream_t stream) {
    const bool paired = (tile & TILE_PAIRED) != 0 && gemm_paired_form_fits(A_KIN, B_KIN, p);
    switch (tile & ~TILE_PAIRED) {
        case TILE_128x128: return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 2, 16, CONV, true>(p, stream)
                                         : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 2, 16, CONV>(p, stream);
        case TILE_64x64:
            if constexpr (!CONV) {
                GemmParams q = p;
                if (!paired && gemm_rim_applies(q)) return launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 16, CONV, false, true>(q, stream);
            }
            return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 16, CONV, true>(p, stream)
                          : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 16, CONV>(p, stream);
        case TILE_256x64:  return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 4, 1, 2, 2, 16, CONV, true>(p, stream)
                                         : launch_cfg<A_KIN, B_KIN, BIAS, 4, 1, 2, 2, 16, CONV>(p, stream);
        case TILE_64x256:  return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 1, 4, 2, 2, 16, CONV, true>(p, stream)
                                         : launch_cfg<A_KIN, B_KIN, BIAS, 1, 4, 2, 2, 16, CONV>(p, stream);
        case TILE_128x64:  return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 1, 16, CONV, true>(p, stream)
                                         : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 1, 16, CONV>(p, stream);
        case TILE_64x128:  return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 2, 16, CONV, true>(p, stream)
                                         : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 2, 16, CONV>(p, stream);
        case TILE_128x128_K32: return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 2, 32, CONV, true>(p, stream)
                                             : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 2, 32, CONV>(p, stream);
        case TILE_64x64_K32:
            if constexpr (!CONV) {
                GemmParams q = p;
                if (!paired && gemm_rim_applies(q)) return launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 32, CONV, false, true>(q, stream);
            }
            return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 32, CONV, true>(p, stream)
                          : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 32, CONV>(p, stream);
        case TILE_128x64_K32:  return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 1, 32, CONV, true>(p, stream)
                                             : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 1, 32, CONV>(p, stream);
        case TILE_64x128_K32:  return paired ? launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 2, 32, CONV, true>(p, stream)
                                             : launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 2, 32, CONV>(p, stream);
        case TILE_64x64_K64:   return launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 64, CONV>(p, stream);
        case TILE_64x64_K128:  return launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 128, CONV>(p, stream);
        case TILE_128x128_K64: return launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 2, 64, CONV>(p, stream);
        case TILE_128x64_K64:  return launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 2, 1, 64, CONV>(p, stream);
        case TILE_64x128_K64:  return launch_cfg<A_KIN, B_KIN, BIAS, 2, 2, 1, 2, 64, CONV>(p, stream);
        default: return hipErrorInvalidValue;
    }
}


template <bool A_KIN, bool B_KIN, bool BIAS, int WM, int WN, int TM, int TN, int KT, int NS>
static hipError_t launch_cfg_dma(GemmParams p, hipStream_t stream) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    auto kernel = gemm_f32_mfma_dma<A_KIN, B_KIN, WM, WN, TM, TN, KT, NS, BIAS>;
    p.tiles_m = (p.rows + BM - 1) / BM;
    p.tiles_n = (p.cols + BN - 1) / BN;
    const long long total = (long long)p.tiles_m * p.tiles_n * p.nz;
    if (total <= 0 || total > 0x7fffffffLL) return hipErrorInvalidValue;
    gemm_fill_tile_divisors(p);
    static std::atomic<int> resident_cache{0};   // per instantiation
    const int resident_per_cu = resident_workgroups(resident_cache, kernel);
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const long long slots = (long long)num_cu * resident_per_cu;
    long long grid = total;
    if (total > slots) {
        const long long rounds = (total + slots - 1) / slots;
        grid = (total + rounds - 1) / rounds;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
    return hipGetLastError();
}

template <bool A_KIN, bool B_KIN, bool BIAS>
static hipError_t launch_variant_dma(const GemmParams& p, int tile, hipStream_t stream) {
    switch (tile) {
        case TILE_DMA_128x128_S4:   return launch_cfg_dma<A_KIN, B_KIN, BIAS, 2, 2, 2, 2, 16, 4>(p, stream);
        case TILE_DMA_64x64_S4:     return launch_cfg_dma<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 16, 4>(p, stream);
        case TILE_DMA_64x64_K32_S4: return launch_cfg_dma<A_KIN, B_KIN, BIAS, 2, 2, 1, 1, 32, 4>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace
}  // namespace dragon
