// Skinny products: a C of at most 32 columns (N x 4 ... N x 32) or at most 32 rows (4 x M ... 32 x M) under a long
// other side -- matrix times a few vectors.  The reference sends a C of 4 columns to kernels of their own
// (MM/matMul_sernel.cuh:17-30, dispatched at MM/matMul.cuh:100-102) and thin row strips to k18 / k14 / k12
// (MM/matMul.cuh:104-106).
//
// Such a product reads its long operand X (L lines of K) once and does next to nothing with it: it is bound by
// HBM, and a 64 x 64 MFMA tile would multiply sixteen times the columns that exist.  Here every wavefront streams
// lines of X from memory straight into registers -- no LDS, no barrier in the stream, two register buffers so that
// the loads of one run under the arithmetic of the other -- and multiplies them with v_mfma_f32_4x4x1_16B_f32:
// sixteen independent 4 x 4 x 1 products per instruction, i.e. 64 lanes' values of X against 4 lines of the short
// operand S with no padded work.
//   X K-outer (k is the row: A of A^T*B, B of A*B and A^T*B): a lane owns W lines (W = 1 or 4 consecutive outputs);
//       the wavefront reads 64 W consecutive floats of a k row per instruction and adds k after k into the same
//       4 x 4 blocks.  The sum of an output runs k-ascending.
//   X K-inner (k contiguous: A of A*B and A*B^T, B of A*B^T): per instruction the wavefront reads 8 lines x 128
//       bytes: lane l holds the 4 k at 4 * (l >> 3) of line (l & 7), two such instructions (lines 0-7, 8-15) make
//       the 16 lines of a wavefront.  The 8 classes of k of a line meet at the end through three lane exchanges.
// With 8 or more short lines (and a long operand of at most 512 MiB, or a K-inner one) the same stream feeds
// v_mfma_f32_16x16x4_f32 instead: 16 lines of X against 16 short lines over 4 k per instruction, the k classes
// added inside the instruction (gemm_f32_skinny16 below; 20 ... 32 short lines as two groups of 16).
// S's values come from memory as well (they stay in the L1: a few floats per k, the same for every wavefront).
// Where the lines are too few to give every compute unit enough wavefronts, the 4 or 16 wavefronts of a workgroup
// share their lines and split K; their sums meet in LDS and are added share after share, a fixed order.  With
// fewer runs of lines than compute units K is cut across up to 8 workgroups per run as well: each leaves its sum
// in the stream's workspace (the balanced kernel's, with its arrival counters) and the one counted last adds them
// in k order -- one launch, the same bits every time.
#include "gemm_mfma_kernel.h"

namespace dragon {
namespace {

struct SkinnyParams {
    const float* X;     // the long operand: L lines of K
    const float* S;     // the short operand: T lines of K
    float* C;
    int L, K;           // lines of X (exact), contraction length (a multiple of 4)
    int ldx, lds, ldc;  // leading strides in floats
    int x_lines;        // lines X has in memory (rows of a K-inner X / row length of a K-outer one)
    int s_lines;        // the same for S (<= T)
    int k_share;        // 0: a wavefront takes its lines' whole K; else the k of each wavefront of a workgroup (a multiple of 32)
    int out_rows;       // the short side is C's row index (C is T x L), else its column index (C is L x T)
    // K cut across workgroups (few lines under a long K): k_cuts workgroups per run of lines take k_cut k each (a
    // multiple of 128, shared among a workgroup's wavefronts as k_share says); their sums meet in ws, counted in count
    int k_cuts, k_cut, units;
    float* ws;
    int* count;
    // a split-K call whose split was declined: zero_floats floats (a multiple of 4) of the caller's partial buffers get zeros
    float* zero_buf;
    long long zero_floats;
    // optional row vector added to C[i][j] for i < bias_rows, j < bias_width (the forward product's bias)
    const float* bias;
    int bias_rows, bias_width;
    int short_stored;   // lines C stores on its short side (4, 8, 12 or 16; >= s_lines)
};

typedef float sk_v4f __attribute__((ext_vector_type(4)));
typedef float sk_v2f __attribute__((ext_vector_type(2)));
constexpr int SKINNY_MAX_CUTS = 8;    // workgroups that cut one run's K
constexpr int SKINNY16_MAX_CUTS = 16; // the same for the 32-line runs of the 16 x 16 x 4 kernel
constexpr int SKINNY_STAGED_FLOATS = 12288;   // of a K-inner short operand in LDS (48 KiB)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t skinny_rsrc(const float* base, long long bytes) {
    const long long capped = bytes > 0xfffffff0LL ? 0xfffffff0LL : (bytes < 0 ? 0 : bytes);
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)(unsigned)capped, RSRC_FLAGS);
}
// AUX: the load's cache policy bits (2 = non-temporal)
template <int AUX = 0>
__device__ __forceinline__ float ld1(__amdgpu_buffer_rsrc_t r, int off, int soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, soff, AUX));
}
template <int AUX = 0>
__device__ __forceinline__ sk_v4f ld4(__amdgpu_buffer_rsrc_t r, int off, int soff) {
    return __builtin_bit_cast(sk_v4f, __builtin_amdgcn_raw_buffer_load_b128(r, off, soff, AUX));
}
template <int AUX = 0>
__device__ __forceinline__ sk_v2f ld2(__amdgpu_buffer_rsrc_t r, int off, int soff) {
    return __builtin_bit_cast(sk_v2f, __builtin_amdgcn_raw_buffer_load_b64(r, off, soff, AUX));
}
template <int W> struct XVal;
template <> struct XVal<1> { float v; __device__ __forceinline__ float at(int) const { return v; } };
template <> struct XVal<2> { sk_v2f v; __device__ __forceinline__ float at(int c) const { const float value = v[c]; return value; } };
template <> struct XVal<4> { sk_v4f v; __device__ __forceinline__ float at(int c) const { const float value = v[c]; return value; } };

__device__ __forceinline__ void skinny_put(const SkinnyParams& p, int line, int col, float value) {
    if (line < p.L) {
        const int ci = p.out_rows ? col : line, cj = p.out_rows ? line : col;      // row and column of C
        // the bias row as the tile kernels' epilogue adds it: "+ 0.0f" is the gamma term of the separate launch
        if (p.bias != nullptr && ci < p.bias_rows) value = (value + (cj < p.bias_width ? p.bias[cj] : 0.0f)) + 0.0f;
        p.C[(size_t)ci * p.ldc + cj] = value;
    }
}

// W: floats of a K-outer X a lane reads per k row (1 or 4), or sets of 8 lines of a K-inner X per wavefront (2 or 4).
// CL: classes of k among the lanes of a K-outer X with W = 1 (2: lanes 0-31 take the even k rows of 32 lines, lanes
// 32-63 the odd ones).  NW: wavefronts of a workgroup.
// SL: the workgroup's part of a K-inner S (T lines x its k range, at most 48 KiB) is staged in LDS once and read from
// there: the short operand's lines are K floats apart -- with K a power of two, lines of the L1 that fall into one set.
// NT: X is read with non-temporal loads -- an operand far larger than the 256 MB Infinity Cache passes through the
// caches once and is not kept (262144 x 4 x 1024: 180 -> 154 us); a smaller one is better left to them (8192 x 8 x
// 4096, served by that cache from launch to launch in a loop: 22.8 -> 32.4 us).
template <bool X_KIN, bool S_KIN, int T, int W, int NW, int CL = 1, bool SL = false, bool NT = false>
__global__ __launch_bounds__(NW * 64)
void gemm_f32_skinny(const SkinnyParams p) {
    static_assert(!SL || (!X_KIN && S_KIN && W == 1 && NW == 4 && CL == 1), "the staged form");
    static_assert(!NT || (W == 4 && NW == 4 && CL == 1 && !SL), "non-temporal reads: the long forms");
    constexpr int XA = NT ? 2 : 0;
    static_assert(T == 4 || T == 8 || T == 12 || T == 16, "4, 8, 12 or 16 short lines");
    static_assert(X_KIN ? (W == 2 || W == 4) && CL == 1 : (W == 1 || W == 4) && (CL == 1 || ((CL == 2 || CL == 4) && W == 1)), "forms");
    constexpr int LS = 8, PK = 32;                         // K-inner X: lines per read, k per panel
    constexpr int H = T / 4;                               // groups of 4 short lines
    constexpr int LINES = X_KIN ? LS * W : 64 * W / CL;    // lines of X per wavefront
    constexpr int ACCS = W * H;                            // 4 x 4 accumulator blocks per lane
    constexpr int MEET_LANES = X_KIN ? LS : 64 / CL;       // lanes that hold outputs once the classes of k have met
    __shared__ float meet_lds[NW][ACCS * 4][MEET_LANES];
    constexpr int SL_KMAX = SL ? SKINNY_STAGED_FLOATS / T : 4;     // k per short line in LDS; 4 zeros behind each line
    constexpr int SL_KS = SL_KMAX + 4;
    __shared__ __attribute__((aligned(16))) float s_lds[SL ? T * SL_KS + 64 : 4];

    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const bool shared = p.k_share > 0;
    // which run of LINES lines; neighbouring runs of a shared K read the halves of the same 128-byte lines: one XCD
    const int wg = shared ? xcd_contiguous_id(blockIdx.x, gridDim.x) : 0;
    const int cut = p.k_cuts > 1 ? wg / p.units : 0;           // neighbouring workgroups: neighbouring lines, the same k
    const int unit = shared ? wg - cut * p.units : blockIdx.x * NW + wave;
    const int line0 = unit * LINES;
    const int k_begin = shared ? cut * p.k_cut + wave * p.k_share : 0;
    const int k_end = shared ? min(min(p.K, (cut + 1) * p.k_cut), k_begin + p.k_share) : p.K;
    const int j = lane & 3;

    // S(k, j): rows beyond K (K-outer) or lines beyond those S has (K-inner) lie beyond the descriptor's end
    const __amdgpu_buffer_rsrc_t rs = skinny_rsrc(p.S, S_KIN ? (long long)p.s_lines * p.lds * 4 : ((long long)(p.K - 1) * p.lds + p.s_lines) * 4);
    sk_v4f d[ACCS];
#pragma unroll
    for (int a = 0; a < ACCS; a++) d[a] = (sk_v4f){0.0f, 0.0f, 0.0f, 0.0f};

    if (p.zero_floats > 0) {
        sk_v4f* const z = (sk_v4f*)p.zero_buf;
        const long long n4 = p.zero_floats >> 2, step = (long long)gridDim.x * (NW * 64);
        for (long long i = (long long)blockIdx.x * (NW * 64) + t; i < n4; i += step) z[i] = (sk_v4f){0.0f, 0.0f, 0.0f, 0.0f};
    }
    // the workgroup's k range of S, line after line (the launcher made sure that it fits)
    const int k_wg0 = (shared && p.k_cuts > 1) ? cut * p.k_cut : 0;
    if constexpr (SL) {
        const int k_len = min(p.K, (shared && p.k_cuts > 1) ? k_wg0 + p.k_cut : p.K) - k_wg0;
        const int chunks = k_len >> 2;
        for (int idx = t; idx < T * chunks; idx += NW * 64) {
            const int jj = idx / chunks, c = idx - jj * chunks;
            const sk_v4f v = ld4(rs, jj < p.s_lines ? (jj * p.lds + k_wg0 + 4 * c) * 4 : OOB_OFFSET, 0);
            *(sk_v4f*)&s_lds[jj * SL_KS + 4 * c] = v;
        }
        if (t < T) *(sk_v4f*)&s_lds[t * SL_KS + SL_KMAX] = (sk_v4f){0.0f, 0.0f, 0.0f, 0.0f};
        __syncthreads();
    }

    if (line0 < p.L && k_begin < k_end) {
        if constexpr (!X_KIN) {
            // ---- a lane owns W lines: X[k][line0 + W * lane + c] (CL = 2: X[k + class][line0 + (lane & 31)]);
            //      U loads (U * CL k rows) per register buffer ----
            constexpr int U = (W == 4 || (NW == 16 && H > 2)) ? 8 : 16;     // (the workgroups of 16 wavefronts have 128 registers a lane)
            const int cls = CL == 4 ? lane >> 4 : CL == 2 ? lane >> 5 : 0;
            const __amdgpu_buffer_rsrc_t rx = skinny_rsrc(p.X, ((long long)(p.K - 1) * p.ldx + p.x_lines) * 4);
            const int x_step = p.ldx * 4;
            const int x_off = CL > 1 ? (line0 + (lane & (64 / CL - 1))) * 4 + cls * x_step : (line0 + W * lane) * 4;
            // the lane's short line j (and j + 4) at k: K-outer S[k][j], K-inner S[j][k]
            const int s_step = S_KIN ? 4 : p.lds * 4;
            int s_off[H];
#pragma unroll
            for (int h = 0; h < H; h++)
                s_off[h] = (4 * h + j < p.s_lines) ? (S_KIN ? (4 * h + j) * p.lds * 4 : (4 * h + j) * 4) + cls * s_step : OOB_OFFSET;
            int sl_base[H];      // staged S: the lane's line, as an index that k - k_wg0 is added to
#pragma unroll
            for (int h = 0; h < H; h++) sl_base[h] = (4 * h + j) * SL_KS;
            struct Buf { XVal<W> x[U]; float s[H][U]; };
            // k rows at or beyond k_end are not this wavefront's (another share's, or beyond K): zeros instead.  K and
            // the shares are even, so the two classes of a load stand or fall together.
            auto load = [&](Buf& b, int k) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int off = (k + CL * u < k_end) ? x_off : OOB_OFFSET;
                    if constexpr (W == 4) b.x[u].v = ld4<XA>(rx, off, (k + CL * u) * x_step);
                    else b.x[u].v = ld1<XA>(rx, off, (k + CL * u) * x_step);
                }
#pragma unroll
                for (int h = 0; h < H; h++) {
                    if constexpr (SL) {
#pragma unroll
                        for (int u = 0; u < U; u += 4) {     // beyond k_end: the zeros behind the line
                            const sk_v4f v = *(const sk_v4f*)&s_lds[sl_base[h] + ((k + u < k_end) ? k + u - k_wg0 : SL_KMAX)];
                            b.s[h][u] = v.x; b.s[h][u + 1] = v.y; b.s[h][u + 2] = v.z; b.s[h][u + 3] = v.w;
                        }
                    } else if constexpr (S_KIN && CL == 1) {
#pragma unroll
                        for (int u = 0; u < U; u += 4) {
                            const sk_v4f v = ld4(rs, (k + u < k_end) ? s_off[h] : OOB_OFFSET, (k + u) * 4);
                            b.s[h][u] = v.x; b.s[h][u + 1] = v.y; b.s[h][u + 2] = v.z; b.s[h][u + 3] = v.w;
                        }
                    } else {   // (single floats also for the two classes of a K-inner S: measured faster than four k per read)
#pragma unroll
                        for (int u = 0; u < U; u++) b.s[h][u] = ld1(rs, (k + CL * u < k_end) ? s_off[h] : OOB_OFFSET, (k + CL * u) * s_step);
                    }
                }
            };
            auto compute = [&](const Buf& b) {
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int c = 0; c < W; c++)
#pragma unroll
                        for (int h = 0; h < H; h++)
                            d[c * H + h] = __builtin_amdgcn_mfma_f32_4x4x1f32(b.x[u].at(c), b.s[h][u], d[c * H + h], 0, 0, 0);
            };
            Buf b0, b1;
            load(b0, k_begin);
            // (the scheduling barriers keep the phases apart: left alone, the compiler moves the arithmetic on a
            // buffer up to right behind that buffer's loads and waits for them there)
            for (int k = k_begin; k < k_end; k += 2 * U * CL) {
                load(b1, k + U * CL);
                __builtin_amdgcn_sched_barrier(0);
                compute(b0);
                __builtin_amdgcn_sched_barrier(0);
                load(b0, k + 2 * U * CL);
                __builtin_amdgcn_sched_barrier(0);
                compute(b1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (CL > 1) {   // the classes of k meet: lanes l, l ^ 32 (and l ^ 16) hold the same outputs
#pragma unroll
                for (int a = 0; a < ACCS; a++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        float v = d[a][r];
                        if constexpr (CL == 4) v += __shfl_xor(v, 16);
                        v += __shfl_xor(v, 32);
                        d[a][r] = v;
                    }
            }
        } else {
            // ---- per instruction 8 lines x 8 classes of k: X[line0 + 8 * set + (lane & 7)][k0 + 4 * (lane >> 3) + 0 .. 3];
            //      U 32-k panels per register buffer ----
            constexpr int U = (NW == 16 && H > 2) ? 1 : (NW == 16 || W == 4) ? 2 : 4;
            const __amdgpu_buffer_rsrc_t rx = skinny_rsrc(p.X, (long long)p.x_lines * p.ldx * 4);
            const int kk4 = 4 * (lane / LS);
            int x_off[W];
#pragma unroll
            for (int set = 0; set < W; set++) x_off[set] = ((line0 + LS * set + (lane & (LS - 1))) * p.ldx + kk4) * 4;
            int s_off[H];
#pragma unroll
            for (int h = 0; h < H; h++)
                s_off[h] = (4 * h + j < p.s_lines) ? (S_KIN ? ((4 * h + j) * p.lds + kk4) * 4 : (kk4 * p.lds + 4 * h + j) * 4) : OOB_OFFSET;
            const int s_step = S_KIN ? 4 : p.lds * 4;
            struct Buf { sk_v4f x[U][W]; sk_v4f s[H][U]; };
            // a lane's 4 k at or beyond k_end are not read (what lies there is the next line, or another share)
            auto load = [&](Buf& b, int k) {
#pragma unroll
                for (int q = 0; q < U; q++) {
                    const bool on = k + PK * q + kk4 < k_end;
#pragma unroll
                    for (int set = 0; set < W; set++) b.x[q][set] = ld4<XA>(rx, on ? x_off[set] : OOB_OFFSET, (k + PK * q) * 4);
#pragma unroll
                    for (int h = 0; h < H; h++) {
                        if constexpr (S_KIN) {
                            b.s[h][q] = ld4(rs, on ? s_off[h] : OOB_OFFSET, (k + PK * q) * 4);
                        } else {
                            const int so = on ? s_off[h] : OOB_OFFSET, ss = (k + PK * q) * s_step;
                            sk_v4f v;
                            v.x = ld1(rs, so, ss);
                            v.y = ld1(rs, so, ss + s_step);
                            v.z = ld1(rs, so, ss + 2 * s_step);
                            v.w = ld1(rs, so, ss + 3 * s_step);
                            b.s[h][q] = v;
                        }
                    }
                }
            };
            auto compute = [&](const Buf& b) {
#pragma unroll
                for (int q = 0; q < U; q++)
#pragma unroll
                    for (int u = 0; u < 4; u++)
#pragma unroll
                        for (int set = 0; set < W; set++)
#pragma unroll
                            for (int h = 0; h < H; h++) {
                                const float xv = b.x[q][set][u], sv = b.s[h][q][u];
                                d[set * H + h] = __builtin_amdgcn_mfma_f32_4x4x1f32(xv, sv, d[set * H + h], 0, 0, 0);
                            }
            };
            Buf b0, b1;
            load(b0, k_begin);
            for (int k = k_begin; k < k_end; k += 2 * PK * U) {
                load(b1, k + PK * U);
                __builtin_amdgcn_sched_barrier(0);
                compute(b0);
                __builtin_amdgcn_sched_barrier(0);
                load(b0, k + 2 * PK * U);
                __builtin_amdgcn_sched_barrier(0);
                compute(b1);
                __builtin_amdgcn_sched_barrier(0);
            }
            // the eight classes of k meet: lanes l, l ^ 8, l ^ 16, ... hold the same outputs
#pragma unroll
            for (int a = 0; a < ACCS; a++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float v = d[a][r];
                    v += __shfl_xor(v, 8);
                    v += __shfl_xor(v, 16);
                    v += __shfl_xor(v, 32);
                    d[a][r] = v;
                }
        }
    }

    if (shared) {
        // the wavefronts' shares of K meet in LDS and are added in k order by the first
        if (lane < MEET_LANES) {
#pragma unroll
            for (int a = 0; a < ACCS; a++)
#pragma unroll
                for (int r = 0; r < 4; r++) { const float value = d[a][r]; meet_lds[wave][a * 4 + r][lane] = value; }
        }
        __syncthreads();
        if (wave != 0) return;
        if (lane < MEET_LANES) {
#pragma unroll
            for (int a = 0; a < ACCS; a++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float v = meet_lds[0][a * 4 + r][lane];
                    for (int w = 1; w < NW; w++) v += meet_lds[w][a * 4 + r][lane];
                    d[a][r] = v;
                }
        }
        if constexpr (W == (X_KIN ? 2 : 1) && CL == 1 && NW == 4) if (p.k_cuts > 1) {    // the narrow forms only
            // The workgroups that cut this run's K meet in memory: every one leaves its sum in its slot and is
            // counted; whoever is counted last adds the slots -- its own included -- in k order and stores.  The
            // hand-over is the balanced kernel's (gemm_mfma_streamk.hip, store_partial): device-scope stores that
            // have all been acknowledged (vmcnt 0) before this wavefront's count, device-scope loads after it.
            float* const slots = p.ws + (size_t)unit * p.k_cuts * (ACCS * 4 * MEET_LANES);
            if (lane < MEET_LANES) {
                float* const mine = slots + (size_t)cut * (ACCS * 4 * MEET_LANES) + lane;
#pragma unroll
                for (int a = 0; a < ACCS; a++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float value = d[a][r];
                        __hip_atomic_store(mine + (a * 4 + r) * MEET_LANES, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            asm volatile("" ::: "memory");
            int arrived = 0;
            if (lane == 0) {
                arrived = atomicAdd(p.count + unit, 1);
                if (arrived == p.k_cuts - 1) atomicExch(p.count + unit, 0);     // zero again for the next launch
            }
            arrived = __builtin_amdgcn_readfirstlane(arrived);
            if (arrived != p.k_cuts - 1) return;
            asm volatile("" ::: "memory");
            if (lane < MEET_LANES) {
                // eight outputs of a lane at a time: every cut's floats of them are read before any is added
                constexpr int CH = ACCS * 4 < 8 ? ACCS * 4 : 8;
#pragma unroll
                for (int base = 0; base < ACCS * 4; base += CH) {
                    float v[SKINNY_MAX_CUTS][CH];
#pragma unroll
                    for (int c = 0; c < SKINNY_MAX_CUTS; c++)
                        if (c < p.k_cuts) {
#pragma unroll
                            for (int i = 0; i < CH; i++)
                                v[c][i] = __hip_atomic_load(slots + (size_t)c * (ACCS * 4 * MEET_LANES) + (base + i) * MEET_LANES + lane,
                                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
#pragma unroll
                    for (int i = 0; i < CH; i++) {
                        float sum = v[0][i];
#pragma unroll
                        for (int c = 1; c < SKINNY_MAX_CUTS; c++)
                            if (c < p.k_cuts) sum += v[c][i];
                        d[(base + i) / 4][(base + i) % 4] = sum;
                    }
                }
            }
        }
    }
    // the lane's outputs.  K-outer X: accumulator c * H + h, element r is line line0 + W * (4 * (lane >> 2) + r) + c;
    // K-inner X (lanes 0 .. 7): accumulator set * H + h, element r is line line0 + 8 * set + 4 * (lane >> 2) + r;
    // both at the short line 4 * h + j
    if (lane < MEET_LANES) {
#pragma unroll
        for (int a = 0; a < ACCS; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int h = a % H, hi = a / H;
                const int line = X_KIN ? line0 + LS * hi + 4 * (lane >> 2) + r : line0 + W * (4 * (lane >> 2) + r) + hi;
                const float value = d[a][r];
                skinny_put(p, line, 4 * h + j, value);
            }
    }
}

// Sixteen short lines at once: v_mfma_f32_16x16x4_f32 multiplies 16 lines of X by the 16 lines of S over 4 k per
// instruction (lane l supplies line l & 15 at k class l >> 4 of either operand; element v of the result in lane l
// is X line 4 * (l >> 4) + v against S line l & 15).  A quarter of the 4 x 4 x 1 blocks' instructions per byte of X
// for 16 short lines, the k classes add up inside the instruction (no lane exchange), and the lanes of a line's
// outputs are 16 consecutive floats of C.  Fewer short lines than 16 are multiplied as zeros and not stored.
//   X K-inner: per set of 16 lines and 32 k two reads of 8 whole 128-byte lines each (a lane's 16 bytes are 4 k and
//       feed four instructions); what the instruction wants 8 lanes away comes by a row rotation.  (Reading 16 lines x
//       64 bytes per instruction, everything in place, is level with ordinary loads and loses with non-temporal
//       ones, which keep nothing for the second half of a line: 223 us against 178 on 262144 x 16 x 1024.)
//   X K-outer: a lane reads W consecutive lines at row k0 + 4 * (l >> 4) + m, m = 0 .. 3 (4 rows x 64 W bytes per
//       instruction); its W floats feed W accumulators (lines W * i + e, i the MFMA's row).
// ROWS: the short side is C's row index (C is 16 x L).  Then S is the instruction's first operand and X its second:
// element v of the result in lane l is S line 4 * (l >> 4) + v against X line l & 15 -- the lanes of a store run
// along a row of C.
// G: groups of 16 short lines (1, or 2 for 20 ... 32 short lines: every value of X feeds G instructions).
// NT: X is read with non-temporal loads (see gemm_f32_skinny).
template <bool X_KIN, bool S_KIN, int W, int NW, bool ROWS, int G = 1, bool NT = false, int U = (W == 4 ? 2 : 4)>
__global__ __launch_bounds__(NW * 64)
void gemm_f32_skinny16(const SkinnyParams p) {
    static_assert(W == 2 || W == 4, "sets of 16 lines (K-inner X) or floats a lane reads of a row (K-outer X)");

    constexpr int XA = NT ? 2 : 0;
    static_assert(G == 1 || G == 2, "up to 32 short lines");
    constexpr int LINES = 16 * W, PK = 16;                 // U: 16-k panels per register buffer
    __shared__ float meet_lds[NW][W * G * 4][64];

    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const bool shared = p.k_share > 0;
    const int wg = shared ? xcd_contiguous_id(blockIdx.x, gridDim.x) : 0;
    const int cut = p.k_cuts > 1 ? wg / p.units : 0;           // neighbouring workgroups: neighbouring lines, the same k
    const int unit = shared ? wg - cut * p.units : blockIdx.x * NW + wave;
    const int line0 = unit * LINES;
    const int k_begin = shared ? cut * p.k_cut + wave * p.k_share : 0;
    const int k_end = shared ? min(min(p.K, (cut + 1) * p.k_cut), k_begin + p.k_share) : p.K;
    const int r = lane & 15, c4 = 4 * (lane >> 4);

    const __amdgpu_buffer_rsrc_t rs = skinny_rsrc(p.S, S_KIN ? (long long)p.s_lines * p.lds * 4 : ((long long)(p.K - 1) * p.lds + p.s_lines) * 4);
    sk_v4f d[W][G];
#pragma unroll
    for (int a = 0; a < W; a++)
#pragma unroll
        for (int g = 0; g < G; g++) d[a][g] = (sk_v4f){0.0f, 0.0f, 0.0f, 0.0f};

    if (p.zero_floats > 0) {
        sk_v4f* const z = (sk_v4f*)p.zero_buf;
        const long long n4 = p.zero_floats >> 2, step = (long long)gridDim.x * (NW * 64);
        for (long long i = (long long)blockIdx.x * (NW * 64) + t; i < n4; i += step) z[i] = (sk_v4f){0.0f, 0.0f, 0.0f, 0.0f};
    }

    if (line0 < p.L && k_begin < k_end) {
        // the lane's short line 16 g + r at its class of k: K-inner S[line][k + c4 + m], K-outer S[k + c4 + m][line]
        int s_off[G];
#pragma unroll
        for (int g = 0; g < G; g++)
            s_off[g] = 16 * g + r < p.s_lines ? (S_KIN ? ((16 * g + r) * p.lds + c4) * 4 : (c4 * p.lds + 16 * g + r) * 4) : OOB_OFFSET;
        const int s_step = S_KIN ? 4 : p.lds * 4;
        auto load_s = [&](int g, int k, bool on) {
            sk_v4f v;
            if constexpr (S_KIN) {
                v = ld4(rs, on ? s_off[g] : OOB_OFFSET, k * 4);
            } else {
                const int so = on ? s_off[g] : OOB_OFFSET, ss = k * s_step;
                v.x = ld1(rs, so, ss);
                v.y = ld1(rs, so, ss + s_step);
                v.z = ld1(rs, so, ss + 2 * s_step);
                v.w = ld1(rs, so, ss + 3 * s_step);
            }
            return v;
        };
        auto mfma = [&](sk_v4f& acc, float xv, float sv) {
            acc = ROWS ? __builtin_amdgcn_mfma_f32_16x16x4f32(sv, xv, acc, 0, 0, 0)
                       : __builtin_amdgcn_mfma_f32_16x16x4f32(xv, sv, acc, 0, 0, 0);
        };
        if constexpr (X_KIN) {
            // Two reads per set of 16 lines and 32 k, each of 8 whole 128-byte lines: in read i the lane takes line
            // 8 i + (r & 7) at the 4 k at 16 (r >> 3) + c4.  The instruction wants line r at c4 (first 16 k) and at
            // 16 + c4 (second 16 k) in lane r: half of that is in place, the other half sits 8 lanes away in the
            // other read's register -- one row rotation (DPP) per operand.
            static_assert(U % 2 == 0, "panels of 32 k");
            constexpr int UP = U / 2;
            const __amdgpu_buffer_rsrc_t rx = skinny_rsrc(p.X, (long long)p.x_lines * p.ldx * 4);
            const int kh = 16 * (r >> 3) + c4;
            int x_off[W][2];
#pragma unroll
            for (int set = 0; set < W; set++)
#pragma unroll
                for (int i = 0; i < 2; i++) x_off[set][i] = ((line0 + 16 * set + 8 * i + (r & 7)) * p.ldx + kh) * 4;
            struct Buf { sk_v4f x[UP][W][2]; sk_v4f s[UP][2][G]; };
            // a lane's 4 k at or beyond k_end are not read (what lies there is the next line, or another share)
            auto load = [&](Buf& b, int k) {
#pragma unroll
                for (int q = 0; q < UP; q++)
#pragma unroll
                    for (int set = 0; set < W; set++)
#pragma unroll
                        for (int i = 0; i < 2; i++)
                            b.x[q][set][i] = ld4<XA>(rx, (k + 32 * q + kh < k_end) ? x_off[set][i] : OOB_OFFSET, (k + 32 * q) * 4);
#pragma unroll
                for (int q = 0; q < UP; q++)
#pragma unroll
                    for (int h = 0; h < 2; h++)
#pragma unroll
                        for (int g = 0; g < G; g++) b.s[q][h][g] = load_s(g, k + 32 * q + 16 * h, k + 32 * q + 16 * h + c4 < k_end);
            };
            auto rotated = [](float keep, float take, bool upper) {      // lanes 8 .. 15 (upper) or 0 .. 7 of a row take `take` from 8 lanes away
                const int k = __builtin_bit_cast(int, keep), t = __builtin_bit_cast(int, take);
                return __builtin_bit_cast(float, upper ? __builtin_amdgcn_update_dpp(k, t, 0x128, 0xf, 0xc, false)
                                                       : __builtin_amdgcn_update_dpp(k, t, 0x128, 0xf, 0x3, false));
            };
            auto compute = [&](const Buf& b) {
#pragma unroll
                for (int q = 0; q < UP; q++)
#pragma unroll
                    for (int h = 0; h < 2; h++)
#pragma unroll
                        for (int m = 0; m < 4; m++)
#pragma unroll
                            for (int set = 0; set < W; set++) {
                                const float x0 = b.x[q][set][0][m], x1 = b.x[q][set][1][m];
                                const float xv = h == 0 ? rotated(x0, x1, true) : rotated(x1, x0, false);
#pragma unroll
                                for (int g = 0; g < G; g++) {
                                    const float sv = b.s[q][h][g][m];
                                    mfma(d[set][g], xv, sv);
                                }
                            }
            };
            Buf b0, b1;
            load(b0, k_begin);
            for (int k = k_begin; k < k_end; k += 2 * PK * U) {
                load(b1, k + PK * U);
                __builtin_amdgcn_sched_barrier(0);
                compute(b0);
                __builtin_amdgcn_sched_barrier(0);
                load(b0, k + 2 * PK * U);
                __builtin_amdgcn_sched_barrier(0);
                compute(b1);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            const __amdgpu_buffer_rsrc_t rx = skinny_rsrc(p.X, ((long long)(p.K - 1) * p.ldx + p.x_lines) * 4);
            const int x_step = p.ldx * 4;
            const int x_off = (c4 * p.ldx + line0 + W * r) * 4;
            struct Buf { XVal<W> x[U][4]; sk_v4f s[U][G]; };
            // (K and the shares are multiples of 4: the lane's rows k + c4 + 0 .. 3 stand or fall together)
            auto load = [&](Buf& b, int k) {
#pragma unroll
                for (int q = 0; q < U; q++) {
                    const bool on = k + PK * q + c4 < k_end;
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        if constexpr (W == 4) b.x[q][m].v = ld4<XA>(rx, on ? x_off : OOB_OFFSET, (k + PK * q + m) * x_step);
                        else b.x[q][m].v = ld2<XA>(rx, on ? x_off : OOB_OFFSET, (k + PK * q + m) * x_step);
                    }
#pragma unroll
                    for (int g = 0; g < G; g++) b.s[q][g] = load_s(g, k + PK * q, on);
                }
            };
            auto compute = [&](const Buf& b) {
#pragma unroll
                for (int q = 0; q < U; q++)
#pragma unroll
                    for (int m = 0; m < 4; m++)
#pragma unroll
                        for (int e = 0; e < W; e++)
#pragma unroll
                            for (int g = 0; g < G; g++) {
                                const float xv = b.x[q][m].at(e), sv = b.s[q][g][m];
                                mfma(d[e][g], xv, sv);
                            }
            };
            Buf b0, b1;
            load(b0, k_begin);
            for (int k = k_begin; k < k_end; k += 2 * PK * U) {
                load(b1, k + PK * U);
                __builtin_amdgcn_sched_barrier(0);
                compute(b0);
                __builtin_amdgcn_sched_barrier(0);
                load(b0, k + 2 * PK * U);
                __builtin_amdgcn_sched_barrier(0);
                compute(b1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    if (shared) {
        // the wavefronts' shares of K meet in LDS and are added in k order by the first
#pragma unroll
        for (int a = 0; a < W; a++)
#pragma unroll
            for (int g = 0; g < G; g++)
#pragma unroll
                for (int v = 0; v < 4; v++) { const float value = d[a][g][v]; meet_lds[wave][(a * G + g) * 4 + v][lane] = value; }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int a = 0; a < W; a++)
#pragma unroll
            for (int g = 0; g < G; g++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    float sum = meet_lds[0][(a * G + g) * 4 + v][lane];
                    for (int w = 1; w < NW; w++) sum += meet_lds[w][(a * G + g) * 4 + v][lane];
                    d[a][g][v] = sum;
                }
        if constexpr (W == 2 && NW == 4) if (p.k_cuts > 1) {    // the 32-line runs only
            // The workgroups that cut this run's K meet in memory exactly as in gemm_f32_skinny: every one leaves
            // its sum in its slot and is counted; whoever is counted last adds the slots in k order and stores.
            constexpr int ACC = W * G * 4;
            float* const slots = p.ws + (size_t)unit * p.k_cuts * (ACC * 64);
            float* const mine = slots + (size_t)cut * (ACC * 64) + lane;
#pragma unroll
            for (int a = 0; a < W; a++)
#pragma unroll
                for (int g = 0; g < G; g++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const float value = d[a][g][v];
                        __hip_atomic_store(mine + ((a * G + g) * 4 + v) * 64, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            asm volatile("" ::: "memory");
            int arrived = 0;
            if (lane == 0) {
                arrived = atomicAdd(p.count + unit, 1);
                if (arrived == p.k_cuts - 1) atomicExch(p.count + unit, 0);     // zero again for the next launch
            }
            arrived = __builtin_amdgcn_readfirstlane(arrived);
            if (arrived != p.k_cuts - 1) return;
            asm volatile("" ::: "memory");
            // four outputs of a lane at a time: every cut's floats of them are read before any is added
#pragma unroll
            for (int base = 0; base < ACC; base += 4) {
                float part[SKINNY16_MAX_CUTS][4];
#pragma unroll
                for (int c = 0; c < SKINNY16_MAX_CUTS; c++)
                    if (c < p.k_cuts) {
#pragma unroll
                        for (int i = 0; i < 4; i++)
                            part[c][i] = __hip_atomic_load(slots + (size_t)c * (ACC * 64) + (base + i) * 64 + lane,
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float sum = part[0][i];
#pragma unroll
                    for (int c = 1; c < SKINNY16_MAX_CUTS; c++)
                        if (c < p.k_cuts) sum += part[c][i];
                    d[(base + i) / (G * 4)][((base + i) / 4) % G][(base + i) % 4] = sum;
                }
            }
        }
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
        if constexpr (!ROWS) {
            // element v of accumulator a: K-inner X line line0 + 16 * a + c4 + v, K-outer X line line0 + W * (c4 + v) + a;
            // the short line is 16 g + r
            if (16 * g + r < p.short_stored) {
#pragma unroll
                for (int a = 0; a < W; a++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const int line = X_KIN ? line0 + 16 * a + c4 + v : line0 + W * (c4 + v) + a;
                        const float value = d[a][g][v];
                        skinny_put(p, line, 16 * g + r, value);
                    }
            }
        } else {
            // element v of accumulator a: short line 16 g + c4 + v at K-inner X line line0 + 16 * a + r, K-outer X line
            // line0 + W * r + a -- there a lane's W accumulators are W consecutive floats of a row of C
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = 16 * g + c4 + v;
                if (row >= p.short_stored) continue;
                if constexpr (!X_KIN && W == 4) {
                    const int line = line0 + W * r;
                    if (p.bias == nullptr && line + 3 < p.L) {
                        const sk_v4f out = {d[0][g][v], d[1][g][v], d[2][g][v], d[3][g][v]};
                        *(sk_v4f*)&p.C[(size_t)row * p.ldc + line] = out;
                        continue;
                    }
                }
#pragma unroll
                for (int a = 0; a < W; a++) {
                    const int line = X_KIN ? line0 + 16 * a + r : line0 + W * r + a;
                    const float value = d[a][g][v];
                    skinny_put(p, line, row, value);
                }
            }
        }
    }
}

// cuts > 1 (the shared 32-line runs only): that many workgroups per run take a part of K each and meet through the
// stream's workspace, as in launch_one below
template <bool X_KIN, bool S_KIN, int W, int NW, int G, int U = (W == 4 ? 2 : 4)>
hipError_t launch_16(SkinnyParams p, bool shared, hipStream_t stream, bool nt = false, int cuts = 1) {
    if ((p.ldc & 3) != 0 || ((size_t)p.C & 15) != 0) return hipErrorInvalidValue;
    constexpr int LINES = 16 * W;
    constexpr int SLOT = W * G * 4 * 64;       // floats a workgroup leaves in the workspace
    const long long units = ((long long)p.L + LINES - 1) / LINES;
    p.k_share = shared ? ((p.K + NW - 1) / NW + 31) / 32 * 32 : 0;
    p.units = (int)units;
    p.k_cuts = 1;
    p.k_cut = p.K;
    long long grid = shared ? units : (units + NW - 1) / NW;
    if (shared && cuts > 1 && W == 2 && NW == 4 && units <= 65536) {
        if (cuts > SKINNY16_MAX_CUTS) cuts = SKINNY16_MAX_CUTS;
        const int k_cut = ((p.K + cuts - 1) / cuts + 32 * NW - 1) / (32 * NW) * (32 * NW);
        const int real = (p.K + k_cut - 1) / k_cut;
        size_t floats = 0;
        float* ws = real > 1 ? gemm_streamk_workspace(stream, &floats) : nullptr;
        if (ws != nullptr && 65536 + (size_t)units * real * SLOT <= floats) {
            p.k_cuts = real;
            p.k_cut = k_cut;
            p.k_share = k_cut / NW;
            p.count = (int*)ws;          // the workspace's arrival counters, zero between launches
            p.ws = ws + 65536;
            grid = units * real;
        }
    }
    if (grid <= 0 || grid > 0x7fffffffLL) return hipErrorInvalidValue;
    {
        if (nt) {
            if (p.out_rows) hipLaunchKernelGGL((gemm_f32_skinny16<X_KIN, S_KIN, W, NW, true, G, true, U>), dim3((unsigned)grid), dim3(NW * 64), 0, stream, p);
            else hipLaunchKernelGGL((gemm_f32_skinny16<X_KIN, S_KIN, W, NW, false, G, true, U>), dim3((unsigned)grid), dim3(NW * 64), 0, stream, p);
            return hipGetLastError();
        }
    }
    if (p.out_rows) hipLaunchKernelGGL((gemm_f32_skinny16<X_KIN, S_KIN, W, NW, true, G, false, U>), dim3((unsigned)grid), dim3(NW * 64), 0, stream, p);
    else hipLaunchKernelGGL((gemm_f32_skinny16<X_KIN, S_KIN, W, NW, false, G, false, U>), dim3((unsigned)grid), dim3(NW * 64), 0, stream, p);
    return hipGetLastError();
}

// cuts > 1: that many workgroups per run of lines take a part of K each (narrow forms only, at most
// SKINNY_MAX_CUTS); they meet through the stream's workspace of the balanced kernel -- without one (the stream
// is being captured before it has one, the table is full) the run's K stays with one workgroup.
template <bool X_KIN, bool S_KIN, int T, int W, int NW, int CL = 1>
hipError_t launch_one(SkinnyParams p, bool shared, hipStream_t stream, int cuts = 1, bool nt = false) {
    constexpr int LINES = X_KIN ? 8 * W : 64 * W / CL;
    constexpr int SLOT = W * (T / 4) * 4 * (X_KIN ? 8 : 64 / CL);      // floats a workgroup leaves in the workspace
    const long long units = ((long long)p.L + LINES - 1) / LINES;
    p.k_share = shared ? ((p.K + NW - 1) / NW + 31) / 32 * 32 : 0;
    p.units = (int)units;
    p.k_cuts = 1;
    p.k_cut = p.K;
    long long grid = shared ? units : (units + NW - 1) / NW;
    if (shared && cuts > 1 && NW == 4 && W == (X_KIN ? 2 : 1) && CL == 1 && units <= 65536) {
        if (cuts > SKINNY_MAX_CUTS) cuts = SKINNY_MAX_CUTS;
        const int k_cut = ((p.K + cuts - 1) / cuts + 32 * NW - 1) / (32 * NW) * (32 * NW);
        const int real = (p.K + k_cut - 1) / k_cut;
        size_t floats = 0;
        float* ws = real > 1 ? gemm_streamk_workspace(stream, &floats) : nullptr;
        if (ws != nullptr && 65536 + (size_t)units * real * SLOT <= floats) {
            p.k_cuts = real;
            p.k_cut = k_cut;
            p.k_share = k_cut / NW;
            p.count = (int*)ws;          // the workspace's arrival counters, zero between launches
            p.ws = ws + 65536;
            grid = units * real;
        }
    }
    if (grid <= 0 || grid > 0x7fffffffLL) return hipErrorInvalidValue;
    if constexpr (!X_KIN && S_KIN && W == 1 && NW == 4 && CL == 1) {
        // the wavefronts share their lines and the workgroup's part of S is small enough: S from LDS
        if (shared && (p.k_cuts > 1 ? p.k_cut : p.K) <= SKINNY_STAGED_FLOATS / T) {
            hipLaunchKernelGGL((gemm_f32_skinny<X_KIN, S_KIN, T, W, NW, CL, true>), dim3((unsigned)grid), dim3(NW * 64), 0, stream, p);
            return hipGetLastError();
        }
    }
    if constexpr (W == 4 && NW == 4 && CL == 1) {
        if (nt) {
            hipLaunchKernelGGL((gemm_f32_skinny<X_KIN, S_KIN, T, W, NW, CL, false, true>), dim3((unsigned)grid), dim3(NW * 64), 0, stream, p);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((gemm_f32_skinny<X_KIN, S_KIN, T, W, NW, CL>), dim3((unsigned)grid), dim3(NW * 64), 0, stream, p);
    return hipGetLastError();
}

thread_local int t_skinny_form = -1, t_skinny_cuts = 0, t_skinny_nt = -1;
constexpr long long SKINNY_NT_BYTES = 320LL << 20;     // long operands from this size on are read non-temporally

static bool skinny_nt(const SkinnyParams& p) {
    return t_skinny_nt >= 0 ? t_skinny_nt != 0 : (long long)p.L * p.K * 4 >= SKINNY_NT_BYTES;
}

// Which form (gemm_skinny_form's numbering): enough wavefronts on every compute unit with the widest reads that
// allow it.  With too few runs of lines the wavefronts of a workgroup share a run and split K, sixteen of them
// where even that leaves compute units without a run.
template <bool X_KIN, bool S_KIN, int T>
hipError_t launch_skinny(const SkinnyParams& p, hipStream_t stream) {
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    int form = t_skinny_form;
    constexpr int W0 = X_KIN ? 2 : 1;     // the narrow form: 16 lines of a K-inner X, 64 of a K-outer one
    if (form < 0) {
        // measured on 134 MB ... 1 GiB operands: the long runs wherever they give every compute unit a workgroup;
        // a K-inner X also then prefers the four wavefronts of a workgroup on the same lines (a K-outer one only
        // below four runs per compute unit); short of that the narrow runs, and 32-line runs of a K-outer X
        const long long narrow = ((long long)p.L + (X_KIN ? 15 : 63)) / (X_KIN ? 16 : 64);
        const long long wide = ((long long)p.L + (X_KIN ? 31 : 255)) / (X_KIN ? 32 : 256);
        if (p.K < 128) form = wide >= 4LL * num_cu ? 3 : 0;
        else if (wide >= 4LL * num_cu) form = X_KIN ? 4 : 3;
        else if (wide >= num_cu) form = 4;
        // (8 or more lines of a K-inner S beside a K-outer X: K cut so that a workgroup's part of S fits the LDS,
        // 8 x 16384 x 2048 35.8 -> 28.9 us; with 4 lines the cut costs more than the staging gives, 43.6 -> 47.2)
        else if (!X_KIN && S_KIN && T >= 8 && p.K >= 512 && narrow < 4LL * num_cu && p.K > SKINNY_STAGED_FLOATS / T &&
                 (p.K + SKINNY_STAGED_FLOATS / T - 1) / (SKINNY_STAGED_FLOATS / T) <= SKINNY_MAX_CUTS) form = 7;
        else if (narrow >= num_cu || p.K < 512) form = 1;
        // fewer narrow runs than compute units: K is cut across workgroups as well -- except for 128 ... 255 runs of
        // a K-outer X beside a K-outer S, where sixteen wavefronts on 32-line runs measured 10 % ahead
        else if (!X_KIN && !S_KIN && 2 * narrow >= num_cu) form = 5;
        else form = 7;
    }
    switch (form) {
        case 0: return launch_one<X_KIN, S_KIN, T, W0, 4>(p, false, stream);
        case 1: return launch_one<X_KIN, S_KIN, T, W0, 4>(p, true, stream);
        case 2: return launch_one<X_KIN, S_KIN, T, W0, 16>(p, true, stream);
        case 3: return launch_one<X_KIN, S_KIN, T, 4, 4>(p, false, stream, 1, skinny_nt(p));
        case 4: return launch_one<X_KIN, S_KIN, T, 4, 4>(p, true, stream, 1, skinny_nt(p));
        case 6:
            if constexpr (X_KIN) return launch_one<X_KIN, S_KIN, T, W0, 16>(p, true, stream);
            else return launch_one<X_KIN, S_KIN, T, 1, 16, 4>(p, true, stream);
        case 7: {   // two workgroups per compute unit
            const long long narrow = ((long long)p.L + (X_KIN ? 15 : 63)) / (X_KIN ? 16 : 64);
            long long cuts = t_skinny_cuts > 0 ? t_skinny_cuts : narrow < 2LL * num_cu ? (2LL * num_cu + narrow - 1) / narrow : 1;
            // a K-inner S beside a K-outer X is staged in LDS where a cut's part of it fits: enough cuts for that
            if (!X_KIN && S_KIN && t_skinny_cuts == 0) {
                const long long fit = ((long long)p.K + SKINNY_STAGED_FLOATS / T - 1) / (SKINNY_STAGED_FLOATS / T);
                if (fit > cuts && fit <= SKINNY_MAX_CUTS) cuts = fit;
            }
            return launch_one<X_KIN, S_KIN, T, W0, 4>(p, true, stream, (int)cuts);
        }
        default:
            if constexpr (X_KIN) return launch_one<X_KIN, S_KIN, T, W0, 16>(p, true, stream);
            else return launch_one<X_KIN, S_KIN, T, 1, 16, 2>(p, true, stream);
    }
}

template <bool X_KIN, bool S_KIN>
hipError_t launch_skinny_t(const SkinnyParams& p, int T, hipStream_t stream) {
    int form = t_skinny_form;
    if (form < 0) {
        // The 16-line blocks, measured against the 4 x 4 blocks on 32 MB ... 1 GiB operands: always for 12 or 16
        // short lines (16 x 65536 x 4096 192 - 268 -> 176 - 187 us), except 12 beside a long K-outer operand
        // (level); for 8 beside a K-inner long operand (65536 x 8 x 1024 50 -> 41 us) and beside a K-outer one up to
        // 512 MiB (8192 x 8 x 4096 29.8 -> 23.9; 1 GiB, non-temporal reads: 154 us with the 4 x 4 blocks against
        // 161); not for 4 (level), nor under 32 lines per compute unit.
        const int num_cu = gemm_device_num_cu();
        if (num_cu <= 0) return hipErrorNoDevice;
        const long long runs = ((long long)p.L + 63) / 64;
        bool blocks16 = false;
        if (T >= 12) blocks16 = X_KIN || T >= 16 || p.L < 256LL * num_cu;
        // (8 short lines over fewer than 32 lines per unit under a long K: the 32-line runs with K cut across
        // workgroups, 8 x 4096 x 32768 108 - 140 -> 97 - 112 us, 8 x 2048 x 16384 33 - 37 -> 25, 8 x 1024 x 65536
        // 64 - 130 -> 44 - 46)
        else if (T == 8) blocks16 = (p.L >= 32LL * num_cu && (X_KIN || (long long)p.L * p.K <= (1LL << 27))) ||
                                    (p.L < 32LL * num_cu && p.K >= 2048);
        // (4 short lines: only the very few lines under a very long K, 4 x 1024 x 65536 48 - 77 -> 42 - 45 us)
        else if (T == 4) blocks16 = p.L <= 8LL * num_cu && p.K >= 8192;
        if (blocks16) {
            if (p.K < 128) form = runs >= 4LL * num_cu ? 8 : 10;
            else form = runs >= 4LL * num_cu ? (X_KIN ? 9 : 8) : runs >= num_cu ? 9 : 11;
        }
    }
    if (T > 16 && (form < 8 || form > 11)) form = 9;        // (the 4 x 4 blocks stop at 16 short lines)
    switch (form) {     // the 16-line blocks: runs of 64 lines with the whole K, or shared; runs of 32
        case 8: return T > 16 ? launch_16<X_KIN, S_KIN, 4, 4, 2>(p, false, stream, skinny_nt(p)) : launch_16<X_KIN, S_KIN, 4, 4, 1>(p, false, stream, skinny_nt(p));
        case 9: return T > 16 ? launch_16<X_KIN, S_KIN, 4, 4, 2>(p, true, stream, skinny_nt(p)) : launch_16<X_KIN, S_KIN, 4, 4, 1>(p, true, stream, skinny_nt(p));
        case 10: return T > 16 ? launch_16<X_KIN, S_KIN, 2, 4, 2>(p, false, stream, skinny_nt(p)) : launch_16<X_KIN, S_KIN, 2, 4, 1>(p, false, stream, skinny_nt(p));
        case 11: {
            // at most three runs per four compute units under a long K: K is cut across workgroups as well, a workgroup
            // per unit (16 x 4096 x 32768: 173 - 180 -> 105 - 115 us, 16 x 4096 x 8192: 46 -> 26 - 27; two workgroups per
            // unit measured 0 - 15 % behind that, and 250 runs are better left whole)
            const int num_cu = gemm_device_num_cu();
            const long long runs32 = ((long long)p.L + 31) / 32;
            int cuts = t_skinny_cuts > 0 ? t_skinny_cuts : 1;
            if (t_skinny_cuts == 0 && t_skinny_form < 0 && num_cu > 0 && 4 * runs32 <= 3LL * num_cu && p.K >= 2048)
                cuts = (int)((num_cu + runs32 - 1) / runs32);
            return T > 16 ? launch_16<X_KIN, S_KIN, 2, 4, 2>(p, true, stream, skinny_nt(p), cuts)
                          : launch_16<X_KIN, S_KIN, 2, 4, 1>(p, true, stream, skinny_nt(p), cuts);
        }
        default: break;
    }
    switch (T) {
        case 4: return launch_skinny<X_KIN, S_KIN, 4>(p, stream);
        case 8: return launch_skinny<X_KIN, S_KIN, 8>(p, stream);
        case 12: return launch_skinny<X_KIN, S_KIN, 12>(p, stream);
        case 16: return launch_skinny<X_KIN, S_KIN, 16>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

// Force a form of the skinny kernel for the calling thread's launches: 0 = a wavefront per run of lines (64 of a
// K-outer long operand, 16 of a K-inner one) with the whole K, 1 = the four wavefronts of a workgroup share a run
// and split K, 2 = sixteen wavefronts do, 3 and 4 = as 0 and 1 with runs four (K-inner: two) times as long,
// 5 and 6 = as 2 with runs of 32 and 16 lines of a K-outer operand (two and four classes of k among the lanes;
// K-inner: as 2), 7 = as 1 with K cut across workgroups too (two workgroups per compute unit; 100 + c: c cuts);
// 8 ... 11 = the 16-line blocks: 8 = a wavefront per run of 64 lines with the whole K, 9 = the four wavefronts of a
// workgroup share a run, 10 and 11 = as 8 and 9 with runs of 32 lines (200 + c: as 11 with c cuts of K across
// workgroups); -1 = the automatic choice.
void gemm_skinny_form(int form) {
    t_skinny_nt = form >= 2000 ? 0 : form >= 1000 ? 1 : -1;      // 1000 + form: non-temporal reads of X, 2000 + form: none
    if (form >= 1000) form %= 1000;
    if (form == 999) form = -1;                                   // (1999 / 2999: the automatic form with that policy)
    t_skinny_cuts = form >= 100 ? form % 100 : 0;
    if (form >= 200) form = 11;                                   // 200 + c: the 16-line blocks' 32-line runs with c cuts of K
    else if (form >= 100) form = 7;
    t_skinny_form = (form >= 0 && form <= 11) ? form : -1;
}

// 4, 8, ... 32 stored lines on the short side
static bool skinny_short(int n) { return n >= 4 && n <= 32 && n % 4 == 0; }

// 4 or 8 short lines: every layout from 256 lines on.  12 or 16: from 16 lines of the long operand per compute unit
// on (4096 x 16 x 4096 20 - 24 us against the tile kernels' 24; 2048 x 16 x 8192 33 - 45 against 24 - 26).  20 ... 32:
// from 32 lines per compute unit on and a K of at least 256 (8192 x 32 x 4096 31 - 35 us against 39 - 41), from 16
// lines per unit on under a K of 2048 or more; 12 ... 32 under such a K from 8 lines per unit on.
int gemm_choose_skinny(int rows, int cols, int nz, int k, int variant, int num_cu) {
    (void)variant;
    if (nz != 1) return -1;
    const bool thin_cols = skinny_short(cols) && rows >= 256;
    const bool thin_rows = !thin_cols && skinny_short(rows) && cols >= 256;
    if (!thin_cols && !thin_rows) return -1;
    const int t = thin_cols ? cols : rows;
    if (t <= 8) return TILE_SKINNY;
    if (t > 16 && k < 256) return -1;      // (16384 x 32 x 128: 8.1 us against the balanced kernel's 5.2)
    // (with a K of 2048 or more, which is cut across workgroups, from 8 lines per unit on: 2048 x 16 x 8192 16 - 17 us
    // against 25 - 26, 4096 x 32 x 8192 36 - 38 against 39 - 44)
    // (and 12 or 16 short lines over any 256 lines or more under a K of 8192 or more, cut up to 16 times: 16 x 1024 x
    // 65536 72 - 79 -> 46 - 49 us, 1024 x 16 x 8192 20 -> 10 - 12)
    if (t <= 16 && k >= 8192) return TILE_SKINNY;
    return (long long)(thin_cols ? rows : cols) >= (k >= 2048 ? 8LL : t <= 16 ? 16LL : 32LL) * num_cu ? TILE_SKINNY : -1;
}

// True where the product is one for the skinny kernel: one unsplit 2-D product (a bias row on A*B only) whose C has
// 4 ... 32 stored columns under at least 256 rows, or 4 ... 32 stored rows over at least 256 columns, and whose
// operands' byte offsets (with the reads a register buffer runs ahead, and the lines of a last, partly filled
// run) fit 32 bits.
static bool gemm_skinny_applies(int variant, const GemmParams& p) {
    // (a forced choice takes every shape the kernel can run: up to 16 short lines in every layout)
    const bool thin_cols = skinny_short(p.cols) && p.rows >= 256;
    if (p.split || p.nz != 1 || (p.bias != nullptr && variant != GEMM_NN) || !(thin_cols || (skinny_short(p.rows) && p.cols >= 256))) return false;
    const bool a_kin = variant != GEMM_T1, b_kin = variant == GEMM_T2;
    // a K-inner operand is addressed line * ld + k, a K-outer one k * ld + line
    const long long a_span = a_kin ? (long long)(thin_cols ? p.rows : 32) * p.lda : (long long)p.k_total * p.lda;
    const long long b_span = b_kin ? (long long)(thin_cols ? 32 : p.cols) * p.ldb : (long long)p.k_total * p.ldb;
    const long long ld = p.lda > p.ldb ? p.lda : p.ldb;
    return ld <= (1 << 20) && (a_span + 64 * ld) * 4 < 0x7fff0000LL && (b_span + 64 * ld) * 4 < 0x7fff0000LL;
}

hipError_t gemm_launch_skinny(int variant, const GemmParams& g, hipStream_t stream) {
    if (!gemm_skinny_applies(variant, g)) return hipErrorOutOfMemory;   // the caller takes a tile kernel
    const bool a_kin = variant != GEMM_T1, b_kin = variant == GEMM_T2;
    const bool thin_cols = skinny_short(g.cols) && g.rows >= 256;
    SkinnyParams p = {};
    p.C = g.C; p.ldc = g.ldc;
    p.zero_buf = g.zero_buf; p.zero_floats = g.zero_floats;
    p.bias = g.bias; p.bias_rows = g.bias_rows; p.bias_width = g.bias_width;
    p.K = min(g.k_total, min(a_kin ? g.a_inner : g.a_outer, b_kin ? g.b_inner : g.b_outer));
    if (p.K <= 0) return hipErrorInvalidValue;
    if (thin_cols) {          // X = A (lines = rows of C), S = B (lines = columns of C)
        p.X = g.A; p.ldx = g.lda; p.x_lines = a_kin ? g.a_outer : g.a_inner;
        p.S = g.B; p.lds = g.ldb; p.s_lines = min(b_kin ? g.b_outer : g.b_inner, g.cols);
        p.L = g.rows; p.out_rows = 0; p.short_stored = g.cols;
        switch ((a_kin ? 2 : 0) | (b_kin ? 1 : 0)) {
            case 0: return launch_skinny_t<false, false>(p, g.cols, stream);
            case 1: return launch_skinny_t<false, true>(p, g.cols, stream);
            case 2: return launch_skinny_t<true, false>(p, g.cols, stream);
            default: return launch_skinny_t<true, true>(p, g.cols, stream);
        }
    }
    // X = B (lines = columns of C), S = A (lines = rows of C)
    p.X = g.B; p.ldx = g.ldb; p.x_lines = b_kin ? g.b_outer : g.b_inner;
    p.S = g.A; p.lds = g.lda; p.s_lines = min(a_kin ? g.a_outer : g.a_inner, g.rows);
    p.L = g.cols; p.out_rows = 1; p.short_stored = g.rows;
    switch ((b_kin ? 2 : 0) | (a_kin ? 1 : 0)) {
        case 0: return launch_skinny_t<false, false>(p, g.rows, stream);
        case 1: return launch_skinny_t<false, true>(p, g.rows, stream);
        case 2: return launch_skinny_t<true, false>(p, g.rows, stream);
        default: return launch_skinny_t<true, true>(p, g.rows, stream);
    }
}

}  // namespace dragon
