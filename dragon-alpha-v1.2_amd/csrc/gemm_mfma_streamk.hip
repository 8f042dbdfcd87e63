// The balanced kernel: one workgroup per compute unit (two in two of its shapes), and the work dealt out in
// equal runs of LDS stages instead of in whole tiles.  Written for shapes with FEWER TILES THAN THE CHIP HAS
// COMPUTE UNITS (or barely more), where whole tiles leave units idle; its stage loop, which carries no
// vector-ALU instruction, turned out to be the fastest for large products as well (gemm_choose_streamk), and
// it also runs the K slices of a split-K launch ((slice, tile) pairs as its tiles) and the forward
// convolution (ConvDirect: the gathered operand staged a filter tap at a time).
//
// Unit of work = one LDS stage (KT k) of one tile; the tiles' stages are numbered tile by tile
// (tile order of decode_tile) and workgroup w takes the contiguous run [u0(w), u0(w+1)), every run
// within one unit of the others.  A run may start and end in the middle of a tile's K range: a
// tile whose stages all fall to one workgroup is stored to C as usual, a tile shared by several
// workgroups has each of them write its partial sum to a workspace slot (two slots per workgroup:
// one for a piece of the tile its run starts in, one for a piece of a later tile) and count itself
// on the tile's arrival counter; the workgroup that arrives last adds the tile's pieces in run
// order and stores it.  No workgroup ever waits for another.  The split is a pure function of the
// shape and the unit count and the pieces are added in run order whoever does it, so every bit of
// the result is the same from run to run.  The reference's answer to the same problem is the host-side split-K policy
// (CudaFloat32EngineBase.java:1523-1562), which on 256 units still leaves most of them idle or
// unevenly loaded on such shapes.
//
// A workgroup that has a compute unit to itself has nobody to hide its waits behind, so the stage
// loop is built for that case:
//   * operands go global -> LDS directly (buffer_load ... lds) through NS stage buffers, NS-2
//     stages in flight beyond the one that has just landed; no staging registers;
//   * ONE barrier per stage, placed before the matrix work of the stage's LAST k group: by then
//     the fragments of that group are in registers, so after the barrier the wavefront first
//     issues the transfers of a later stage and the fragment reads of the NEXT stage's first
//     group, and only then multiplies -- the LDS latency that otherwise sits between a barrier and
//     the first MFMA is covered by the last group's MFMAs.  Within a stage the fragments of group
//     g+1 are read while group g is multiplied (two fragment sets).
#include "gemm_mfma_kernel.h"
#include <utility>
#include <mutex>
#include <map>

namespace dragon {
namespace {

constexpr int SK_MAX_TILES = 65536;   // arrival counters at the head of the workspace
constexpr size_t SK_MAX_WORKSPACES = 64;

// first unit of workgroup w: the first `rem` workgroups take q+1 units, the others q
__device__ __forceinline__ int sk_first_unit(int w, int q, int rem) { return w * q + (w < rem ? w : rem); }
// the workgroup that owns unit u
__device__ __forceinline__ int sk_owner(int u, int q, int rem) {
    const int big = rem * (q + 1);
    return u < big ? u / (q + 1) : rem + (u - big) / q;
}

// The hand-over of pieces between workgroups below is written for gfx950's memory system and for nothing else.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "the balanced kernel's piece hand-over relies on gfx950's cache behaviour (see store_partial)"
#endif

// Partial tile in the accumulators' own layout: block (i, j) of wavefront `wave`, element e, lane at
// float (((wave*TM + i)*TN + j)*16 + e)*64 + lane: a wavefront writes 256 contiguous bytes per store.
// The pieces travel between workgroups on different XCDs, each with an L2 of its own, inside one
// launch.  Every access to them is a relaxed atomic of device scope -- a store that writes through
// to memory, a load that does not take a stale line from the reader's L2 -- so that no cache has to be
// written back or invalidated as a whole (a device-scope fence does both to the XCD's L2, and with
// them went the operand reuse: 33 -> 110 us on 1000 x 777 x 1531).
// What the ordering rests on, instruction by instruction (gfx950; the formal memory model promises less):
//   * writer: the piece's stores carry the device-scope bit (sc1), i.e. they write through the XCD's L2
//     to memory and are acknowledged -- the wave's vmcnt counts them down -- only once they are there;
//     `s_waitcnt vmcnt(0)` after the run therefore means "every float of my pieces is in memory";
//   * the workgroup barrier behind it makes that true for all four wavefronts before thread 0 / 1 bumps the
//     tile's arrival counter with an atomic add that executes at the memory side (device scope as well);
//   * reader: the workgroup whose add returns the last count reads the pieces with device-scope loads
//     (sc1), which do not hit in its own L2, so a line of the workspace left there by an earlier launch is
//     never taken; its loads are issued after the add has returned and the workgroup has met at a barrier.
//   * the compiler keeps atomics of one address space in program order across the s_waitcnt builtin and the
//     barrier; the "memory" clobbers on the inline-assembly transfers pin the rest.
// The run-to-run bitwise test and the two-stream test in tests/test_gpu_streamk.py guard this.
template <int TM, int TN>
__device__ __forceinline__ void store_partial(const v16f (&acc)[TM][TN], float* slot, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            float* at = slot + (size_t)(((wave * TM + i) * TN + j) * 16) * 64 + lane;
#pragma unroll
            for (int e = 0; e < 16; e++)
                __hip_atomic_store(at + e * 64, acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
}

template <int TM, int TN>
__device__ __forceinline__ void add_partial(v16f (&acc)[TM][TN], const float* slot, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const float* at = slot + (size_t)(((wave * TM + i) * TN + j) * 16) * 64 + lane;
            float v[16];
#pragma unroll
            for (int e = 0; e < 16; e++) v[e] = __hip_atomic_load(at + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] += v[e];
        }
}

// N pieces at a time: the loads of all of them are on their way before the first is added (the order of the
// additions stays the order of the pieces).
template <int N, int TM, int TN>
__device__ __forceinline__ void add_partials(v16f (&acc)[TM][TN], const float* const (&slot)[N], int wave, int lane) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const size_t at = (size_t)(((wave * TM + i) * TN + j) * 16) * 64 + lane;
            float v[N][16];
#pragma unroll
            for (int k = 0; k < N; k++)
#pragma unroll
                for (int e = 0; e < 16; e++)
                    v[k][e] = __hip_atomic_load(slot[k] + at + e * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int k = 0; k < N; k++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][j][e] += v[k][e];
        }
}

template <bool A_KIN, bool B_KIN, int TM, int TN, int BM, int BN, int KT>
__device__ __forceinline__ void read_group(float (&fa)[TM][4], float (&fb)[TN][4], const float* as, const float* bs,
                                           int wm, int wn, int g, int r, int h) {
    if constexpr (A_KIN) read_frag_kinner<TM, KT>(fa, as, wm * TM * 32, g, r, h);
    else                 read_frag_kouter<TM, BM>(fa, as, wm * TM * 32, g, r, h);
    if constexpr (B_KIN) read_frag_kinner<TN, KT>(fb, bs, wn * TN * 32, g, r, h);
    else                 read_frag_kouter<TN, BN>(fb, bs, wn * TN * 32, g, r, h);
}

// The MFMAs of one group of 8 k, with `between(m)` placed after MFMA number m.  A wavefront issues one
// instruction every four cycles at best and an MFMA keeps the matrix pipe busy for 64: whatever else
// the wavefront has to do costs nothing while it sits BETWEEN two MFMAs (15 issue slots each) and
// costs its full issue time anywhere else -- and a workgroup alone on its compute unit has no other
// wavefront to fill the gap.  The order is pinned with scheduling barriers.
template <int NACC, int TM, int TN, typename Between>
__device__ __forceinline__ void mfma_group_with(v16f (&acc)[NACC][TM][TN], const float (&fa)[TM][4], const float (&fb)[TN][4],
                                                Between&& between) {
    static_for<4 * TM * TN>([&](auto mc) {
        constexpr int m = decltype(mc)::value;
        constexpr int q = m / (TM * TN), i = (m / TN) % TM, j = m % TN;
        // a single-block wavefront alternates between two accumulators: an MFMA that adds to the result
        // of the one just before it waits for that result
        constexpr int a = q % NACC;
        acc[a][i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q], acc[a][i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        between(mc);
        __builtin_amdgcn_sched_barrier(0);
    });
}

// The A operand of the forward convolution, gathered from the image X[N, IH, IW, IC] straight into LDS, for
// channel counts that are multiples of KT: a stage then lies inside one filter tap (fh, fw), which is the same
// for every lane.  off[s] is the lane's byte offset for tap (0, 0), channel 0, measured from cv_bias bytes BELOW
// X, so that a pixel above or left of the image -- which a later tap moves inside -- still has a non-negative
// one; bit f of vh[s] / vw[s] says whether filter row / column f reads inside the image for the lane's pixel.
// Per tap the lanes are left with a shift, an and and a select per transfer; the tap's own offset travels in
// the descriptor's base.
template <int R, int KT>
struct ConvDirect {
    static constexpr int CPR = KT / 4;
    static constexpr int RPP = NTHREADS / CPR;
    static constexpr int PASSES = R / RPP;
    static constexpr int LDS_FLOATS = R * KT;
    static_assert(R % RPP == 0 && PASSES >= 1, "tile does not divide over the workgroup");
    int off[PASSES];
    unsigned vh[PASSES], vw[PASSES];

    // bits [lo, hi) set, 0 <= lo, hi <= 32
    __device__ __forceinline__ static unsigned bit_range(int lo, int hi) {
        if (hi <= lo) return 0u;
        const unsigned upto_hi = hi >= 32 ? 0xffffffffu : ((1u << hi) - 1u);
        return upto_hi & ~((1u << lo) - 1u);
    }
    __device__ __forceinline__ void init_conv(int t, int row0, int gm, const GemmParams& p) {
        const int slot = t % CPR, r0 = t / CPR;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int rr = r0 + s * RPP;                       // LDS row = tile row
            const int c = slot ^ kin_swizzle<KT>(rr);          // the chunk that belongs at this LDS slot
            const int m = row0 + rr;
            const int q = div_by(m, p.cv_div_OW_mul, p.cv_div_OW_shift), ow = m - q * p.cv_OW;
            const int n = div_by(q, p.cv_div_OH_mul, p.cv_div_OH_shift), oh = q - n * p.cv_OH;
            const int ih0 = oh * p.cv_sh - p.cv_ph, iw0 = ow * p.cv_sw - p.cv_pw;
            off[s] = (((n * p.cv_IH + ih0) * p.cv_IW + iw0) * p.cv_IC + c * 4) * 4 + p.cv_bias;
            // filter row f reads image row ih0 + f: inside for max(0, -ih0) <= f < min(FH, IH - ih0)
            vh[s] = m < gm ? bit_range(max(0, -ih0), min(p.cv_FH, p.cv_IH - ih0)) : 0u;
            vw[s] = bit_range(max(0, -iw0), min(p.cv_FW, p.cv_IW - iw0));
        }
    }
    __device__ __forceinline__ int tap_offset(int s, int fh, int fw) const {
        return (((vh[s] >> fh) & (vw[s] >> fw)) & 1u) ? off[s] : OOB_OFFSET;
    }
    // the interface of the other loaders where the kernel's common code names it (never reached for a gather)
    __device__ __forceinline__ void init_dma(int, int, int, int) {}
    __device__ __forceinline__ int dma_offset(int s, int) const { return off[s]; }
    __device__ __forceinline__ static const float* tile_base(const float* X, int, int, int) { return X; }
    __device__ __forceinline__ static size_t k_advance(int) { return KT; }
};

// SPLIT: the tiles are (K slice, tile of C) pairs of a split-K launch; the tiles of the last slice, which takes
// the remainder of K, have their own stage count (they come last in the tile order), and a tile's K limits
// count from the slice's first k.
// CONV: A is gathered from an image (ConvDirect), B holds the filters K-inner, C is the output image.
// ZFILL: the launch also writes zeros over the caller's split-K partial buffers (a declined split).  A template
// flag and not a run-time test, so that the plain kernels carry none of it: the compiler's code for their stage
// loop has reacted to a few instructions added elsewhere in the kernel before.
template <bool A_KIN, bool B_KIN, int WM, int WN, int TM, int TN, int KT, int NS, int OCC, bool BIAS, bool SPLIT,
          bool CONV = false, bool ZFILL = false>
__global__ __launch_bounds__(NTHREADS, OCC)
void gemm_f32_mfma_streamk(const GemmParams p) {
    static_assert(!CONV || (A_KIN && B_KIN && !SPLIT), "the convolution is an A * B^T product, unsplit");
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    static_assert(NS == 3 || NS == 4, "stage buffers: 3 or 4 (deeper ones measured slower)");
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    using LoadA = typename std::conditional<CONV, ConvDirect<BM, KT>,
                  typename std::conditional<A_KIN, KInner<BM, KT>, KOuter<BM, KT>>::type>::type;
    using LoadB = typename std::conditional<B_KIN, KInner<BN, KT, TN>, KOuter<BN, KT>>::type;
    constexpr int STAGE_FLOATS = LoadA::LDS_FLOATS + LoadB::LDS_FLOATS;
    constexpr unsigned STAGE_BYTES = STAGE_FLOATS * 4;
    constexpr int PA = LoadA::PASSES, PB = LoadB::PASSES;
    constexpr int XFERS = PA + PB;                             // transfers per wave per stage
    constexpr int GR = KT / 8;                                 // k groups per stage
    constexpr int NM = 4 * TM * TN;                            // MFMAs per group
    static_assert(GR >= 2 && GR % 2 == 0, "an even number of k groups per stage (two fragment sets)");
    static_assert((NS - 2) * XFERS <= 63, "vmcnt holds 6 bits");
    static_assert(OCC * NS * STAGE_FLOATS * 4 <= 160 * 1024, "stage buffers exceed the LDS");

    __shared__ __attribute__((aligned(16))) float smem[NS * STAGE_FLOATS];
    __shared__ int sk_last[2];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    const unsigned long long a_step8 = (unsigned long long)LoadA::k_advance(p.lda) * 4;
    const unsigned long long b_step8 = (unsigned long long)LoadB::k_advance(p.ldb) * 4;

    if constexpr (ZFILL) {
        // A split-K call whose split was declined: this launch computes the whole product, and its workgroups
        // first write zeros over the partial buffers the caller will fold into C afterwards (16 bytes per
        // thread, the launch's threads side by side).  First of all, so that these stores are the oldest
        // vector-memory operations of the wave: the waits on the transfers below then never wait on them.
        static_assert(!SPLIT && !CONV && !BIAS, "only the plain unsplit product stands in for a split one");
        const long long n4 = p.zero_floats >> 2, step = (long long)gridDim.x * NTHREADS;
        v4f* z = (v4f*)p.zero_buf;
        for (long long i = (long long)blockIdx.x * NTHREADS + t; i < n4; i += step) z[i] = (v4f)(0.0f);
    }

    const int S = p.sk_S;
    // tile -> its stage count and first unit, unit -> tile (two regimes under SPLIT: the slices before the last
    // with S stages per tile, the sk_T1-th tile onwards with sk_S_last)
    auto stages_of = [&](int tile) __attribute__((always_inline)) -> int {
        if constexpr (SPLIT) return tile >= p.sk_T1 ? p.sk_S_last : S;
        else return S;
    };
    auto first_unit_of = [&](int tile) __attribute__((always_inline)) -> int {
        if constexpr (SPLIT) return tile >= p.sk_T1 ? p.sk_T1 * S + (tile - p.sk_T1) * p.sk_S_last : tile * S;
        else return tile * S;
    };
    auto tile_of = [&](int u) __attribute__((always_inline)) -> int {
        if constexpr (SPLIT) {
            const int u1 = p.sk_T1 * S;
            if (u >= u1) return p.sk_T1 + div_by(u - u1, p.sk_div_Sl_mul, p.sk_div_Sl_shift);
        }
        return div_by(u, p.sk_div_S_mul, p.sk_div_S_shift);
    };
    auto decode = [&](int tile) __attribute__((always_inline)) -> TileCtx {
        TileCtx c = decode_tile<A_KIN, B_KIN, BM, BN, KT, LoadA, LoadB>(p, tile + p.sk_tile_base);
        if constexpr (SPLIT) {   // K limits relative to the slice's first k, like the stage index
            c.ka_lim -= c.k0;
            c.kb_lim -= c.k0;
        }
        return c;
    };
    // neighbouring runs share a tile's operands: keep them on one XCD (one L2).  Where every tile is cut into the
    // same whole number of runs (few tiles, a very long K), a tile's runs share nothing -- but the runs of the
    // same k range of the tiles of a row read the same rows of A, those of a column the same of B: there the
    // workgroups of an XCD take neighbouring k ranges of all the tiles, and the L2 serves each operand row to
    // its tiles from one fetch.
    int w = xcd_contiguous_id(blockIdx.x, gridDim.x);
    if (p.sk_kmajor_rpt > 0) {
        const int k_range = w / p.sk_kmajor_tiles, tile = w - k_range * p.sk_kmajor_tiles;
        w = tile * p.sk_kmajor_rpt + k_range;
    }
    const int u0 = sk_first_unit(w, p.sk_q, p.sk_rem);
    const int n = p.sk_q + (w < p.sk_rem ? 1 : 0);             // >= 1: the grid never exceeds the unit count

    // ---- producer: the stage to fetch next ------------------------------------------------------
    // Kept as cheap as the hardware allows, because nothing a wavefront does beside its MFMAs is free
    // (see mfma_group_with): the descriptors point at the stage and move on by a scalar 64-bit add, the
    // LDS addresses are integers known at compile time up to the wave's base, and the lanes' offsets sit
    // ready in registers -- their K test is redone only for a stage that is not wholly inside K, and
    // what has to be looked at per stage is one countdown (f_until).
    const int first_tile = tile_of(u0);
    int f_tile = first_tile;
    int f_it = u0 - first_unit_of(first_tile);   // stage of its tile the producer fetches next, as of the last look
    int f_S = stages_of(first_tile);  // stages of the tile the producer is in
    int f_left = n;                   // stages of the run not yet fetched, as of the last look
    int f_span = 0, f_until = 0;      // stages until the next look, at the last look and now
    int f_interior = 0;               // stages of the tile that lie wholly inside K for both operands
    TileCtx ft = decode(f_tile);
    LoadA la;
    LoadB lb;
    if constexpr (CONV) la.init_conv(t, ft.row0, p.a_outer, p);
    else la.init_dma(t, ft.row0, A_KIN ? p.a_outer : p.a_inner, p.lda);
    lb.init_dma(t, ft.col0, B_KIN ? p.b_outer : p.b_inner, p.ldb);
    // CONV: the filter tap the producer is in and the stage inside it (cv_spt stages of KT channels per tap)
    int f_fh = 0, f_fw = 0, f_ic = 0;
    if constexpr (CONV) {
        const int tap = div_by(f_it, p.cv_div_spt_mul, p.cv_div_spt_shift);
        f_ic = f_it - tap * p.cv_spt;
        f_fh = div_by(tap, p.cv_div_FW_mul, p.cv_div_FW_shift);
        f_fw = tap - f_fh * p.cv_FW;
    }
    v4u rsrc_a = dma_descriptor(ft.a_ptr + (size_t)f_it * LoadA::k_advance(p.lda));
    v4u rsrc_b = dma_descriptor(ft.b_ptr + (size_t)f_it * LoadB::k_advance(p.ldb));
    int offa[PA], offb[PB];           // the lanes' offsets for the stage to fetch
    const unsigned lds_wave = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smem + wave * 1024;

    // decide how the following stages are fetched and for how many of them that holds
    auto look = [&]() __attribute__((always_inline)) {
        if (f_left <= 0) {            // past the end of the run: all-zero transfers, so that the count of
#pragma unroll                        // transfers in flight stays a constant
            for (int i = 0; i < PA; i++) offa[i] = OOB_OFFSET;
#pragma unroll
            for (int i = 0; i < PB; i++) offb[i] = OOB_OFFSET;
            f_span = 0x40000000;
        } else {
            if (f_it == f_S) {        // next tile
                f_tile++;
                if constexpr (SPLIT) f_S = stages_of(f_tile);
                ft = decode(f_tile);
                if constexpr (CONV) la.init_conv(t, ft.row0, p.a_outer, p);
                else la.init_dma(t, ft.row0, A_KIN ? p.a_outer : p.a_inner, p.lda);
                lb.init_dma(t, ft.col0, B_KIN ? p.b_outer : p.b_inner, p.ldb);
                rsrc_a = dma_descriptor(ft.a_ptr);
                rsrc_b = dma_descriptor(ft.b_ptr);
                f_it = 0;
                if constexpr (CONV) f_fh = f_fw = f_ic = 0;
            }
            f_interior = min(ft.ka_lim, ft.kb_lim) / KT;
            if (f_it < f_interior) {  // stages wholly inside K: no K test
                if constexpr (CONV) {
                    // the rest of the current tap: which lanes' pixels it reads, and where it starts
#pragma unroll
                    for (int i = 0; i < PA; i++) offa[i] = la.tap_offset(i, f_fh, f_fw);
                    rsrc_a = dma_descriptor(p.A + ((ptrdiff_t)(f_fh * p.cv_IW + f_fw) * p.cv_IC + f_ic * KT) - p.cv_bias / 4);
                } else {
#pragma unroll
                    for (int i = 0; i < PA; i++) offa[i] = la.off[i];
                }
#pragma unroll
                for (int i = 0; i < PB; i++) offb[i] = lb.off[i];
                f_span = min(f_interior - f_it, f_left);
                if constexpr (CONV) f_span = min(f_span, p.cv_spt - f_ic);
            } else {                  // a stage that reaches beyond K: tested lane by lane, one stage at a time
#pragma unroll
                for (int i = 0; i < PA; i++) offa[i] = la.dma_offset(i, ft.ka_lim - f_it * KT);
#pragma unroll
                for (int i = 0; i < PB; i++) offb[i] = lb.dma_offset(i, ft.kb_lim - f_it * KT);
                f_span = 1;
            }
        }
        f_until = f_span;
    };
    // transfer number i of the stage to fetch, into the stage buffer at LDS byte address stage_lds (+ the wave's part)
    auto xfer = [&](auto ic, unsigned stage_lds) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i < PA) dma_f4_lean<i * NTHREADS * 16>(rsrc_a, stage_lds, offa[i]);
        else dma_f4_lean<LoadA::LDS_FLOATS * 4 + (i - PA) * NTHREADS * 16>(rsrc_b, stage_lds, offb[i - PA]);
    };
    // after a stage's transfers
    auto advance = [&]() __attribute__((always_inline)) {
        dma_descriptor_advance(rsrc_a, a_step8);
        dma_descriptor_advance(rsrc_b, b_step8);
        if (--f_until == 0) {
            f_it += f_span;
            f_left -= f_span;
            if constexpr (CONV) {
                f_ic += f_span;
                if (f_ic == p.cv_spt) {   // next tap
                    f_ic = 0;
                    if (++f_fw == p.cv_FW) { f_fw = 0; f_fh++; }
                }
            }
            look();
        }
    };
    look();

    // ---- consumer: the tile being multiplied -------------------------------------------------------
    TileCtx cur = ft;
    int c_tile = first_tile, c_it = f_it;
    int left = n;                     // stages of the run not yet multiplied
    int rec_tile0 = 0, rec_tile1 = 0; // shared tiles this run has left a piece of
    int n_rec = 0;

    constexpr int NACC = 1;   // MFMAs that add to the same block issue back to back at the full rate (measured)
    v16f acc[NACC][TM][TN];
#pragma unroll
    for (int a = 0; a < NACC; a++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[a][i][j] = (v16f)(0.0f);

    float fa[2][TM][4], fb[2][TN][4];

    // prologue: NS-1 stages on their way, the first one landed and visible, its first fragments read
#pragma unroll
    for (int s = 0; s < NS - 1; s++) {
        static_for<XFERS>([&](auto ic) { xfer(ic, lds_wave + s * STAGE_BYTES); });
        advance();
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 2) * XFERS));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_group<A_KIN, B_KIN, TM, TN, BM, BN, KT>(fa[0], fb[0], smem, smem + LoadA::LDS_FLOATS, wm, wn, 0, r, h);

    // One stage, multiplied from stage buffer SLOT (a compile-time constant: every LDS address of the
    // stage is a lane's base register plus an immediate).
    auto stage = [&](auto slot_c) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_c)::value;
        const float* as = smem + SLOT * STAGE_FLOATS;
        const float* bs = as + LoadA::LDS_FLOATS;
        const float* nas = smem + ((SLOT + 1) % NS) * STAGE_FLOATS;
        const unsigned fetch_stage = lds_wave + ((SLOT + NS - 1) % NS) * STAGE_BYTES;   // the buffer of the stage before
        static_for<GR>([&](auto gc) {
            constexpr int g = decltype(gc)::value;
            if constexpr (g + 1 < GR) {
                // the fragments of the next group are read behind this group's first MFMA
                mfma_group_with<NACC, TM, TN>(acc, fa[g & 1], fb[g & 1], [&](auto mc) {
                    if constexpr (decltype(mc)::value == 0)
                        read_group<A_KIN, B_KIN, TM, TN, BM, BN, KT>(fa[(g + 1) & 1], fb[(g + 1) & 1], as, bs, wm, wn, g + 1, r, h);
                });
            } else {
                // Last group: every fragment of this stage is in registers.  Spread between its MFMAs:
                //   piece 0          own transfers of the next stage landed (vmcnt retires in order: at most
                //                    the younger stages may be outstanding; stores issued in between only
                //                    make this wait longer), then the barrier: everybody's part of that
                //                    stage is visible and nobody reads the buffer of the stage before any more
                //   pieces 1..XFERS  the transfers of the stage NS-1 ahead into that buffer
                //   then             the producer's bookkeeping; the next stage's first fragments
                constexpr int NP = XFERS + 3;
                mfma_group_with<NACC, TM, TN>(acc, fa[g & 1], fb[g & 1], [&](auto mc) {
                    constexpr int m = decltype(mc)::value;
                    constexpr int lo = m * NP / NM, hi = (m + 1) * NP / NM;
                    static_for<hi - lo>([&](auto pc) {
                        constexpr int piece = lo + decltype(pc)::value;
                        if constexpr (piece == 0) {
                            __builtin_amdgcn_s_waitcnt(waitcnt_vm((NS - 3) * XFERS));
                            __builtin_amdgcn_s_barrier();
                            asm volatile("" ::: "memory");
                        } else if constexpr (piece <= XFERS) {
                            xfer(std::integral_constant<int, piece - 1>{}, fetch_stage);
                        } else if constexpr (piece == XFERS + 1) {
                            advance();
                        } else {
                            read_group<A_KIN, B_KIN, TM, TN, BM, BN, KT>(fa[0], fb[0], nas, nas + LoadA::LDS_FLOATS, wm, wn, 0, r, h);
                        }
                    });
                });
            }
        });
    };

    // ---- the run, piece by piece: a piece = the stages of this run that belong to one tile ----
    // The stage buffers take turns in a fixed order, so the loop below is unrolled over them and always
    // entered at buffer 0; a piece may end behind any stage, and what then has to be done (store the tile
    // or the piece, move on to the next tile) stands behind each of the NS stages.  One loop, no way into
    // its middle: the accumulators stay in the registers they are in.
    int c_S = stages_of(first_tile);  // stages of the tile being multiplied (the producer may be a tile ahead)
    int piece_len = min(c_S - c_it, left);
    bool whole = c_it == 0 && piece_len == c_S;
    int todo = piece_len;
    // the piece of c_tile that this run holds has been multiplied; true when that was the run's last
    auto piece_end = [&]() __attribute__((always_inline)) -> bool {
        left -= piece_len;
        if (whole) {
            store_tile<A_KIN, B_KIN, TM, TN, BIAS>(acc[0], p, cur.row0, cur.col0, cur.c_ptr, wm, wn, r, h);
        } else {
            // A piece of a shared tile goes to the workspace: slot 2w for a piece of the tile the run starts
            // in, 2w+1 for a piece of a later tile.  It is counted at the end of the run.
            store_partial<TM, TN>(acc[0], p.sk_ws + (size_t)(2 * w + (c_tile != first_tile ? 1 : 0)) * (BM * BN), wave, lane);
            if (n_rec == 0) rec_tile0 = c_tile; else rec_tile1 = c_tile;
            n_rec++;
        }
        if (left == 0) return true;
        c_tile++;
        if constexpr (SPLIT) c_S = stages_of(c_tile);
        cur = decode(c_tile);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int jj = 0; jj < TN; jj++) acc[0][i][jj] = (v16f)(0.0f);
        piece_len = min(c_S, left);
        whole = piece_len == c_S;
        todo = piece_len;
        return false;
    };
    // one stage from buffer SLOT, then whatever the end of a piece asks for; true when the run is over
    auto step = [&](auto slot_c) __attribute__((always_inline)) -> bool {
        stage(slot_c);
        return --todo == 0 && piece_end();
    };
    // turn after turn through the buffers, until a step ends the run (written out: with the turn folded into
    // one expression the compiler's code was 8 % slower)
    for (;;) {
        if (step(std::integral_constant<int, 0>{})) break;
        if (step(std::integral_constant<int, 1>{})) break;
        if (step(std::integral_constant<int, 2>{})) break;
        if constexpr (NS == 4) {
            if (step(std::integral_constant<int, 3>{})) break;
        }
    }
    // nothing of this wave may still be on its way into LDS when the wave ends, and every piece it stored
    // has arrived in memory before the workgroup is counted
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    if (n_rec == 0) return;

    // ---- the shared tiles this run has left a piece of (at most two) ----
    // The pieces are counted per tile; whoever counts last adds up all the tile's pieces -- its own
    // included, read back like the others, in run order whatever the order of arrival -- and stores the
    // tile.  Nobody waits for anybody.  The last one also puts the counter back to zero for the next launch.
    __syncthreads();
    if (t < n_rec) {
        const int tile = t == 0 ? rec_tile0 : rec_tile1;
        const int wa = sk_owner(first_unit_of(tile), p.sk_q, p.sk_rem);
        const int wb = sk_owner(first_unit_of(tile) + stages_of(tile) - 1, p.sk_q, p.sk_rem);
        const int arrived = atomicAdd(p.sk_count + tile, 1);
        const int last = arrived == wb - wa;
        if (last) atomicExch(p.sk_count + tile, 0);
        sk_last[t] = last;
    }
    __syncthreads();
    for (int i = 0; i < n_rec; i++) {
        if (!sk_last[i]) continue;
        const int tile = i == 0 ? rec_tile0 : rec_tile1;
        const int wa = sk_owner(first_unit_of(tile), p.sk_q, p.sk_rem);
        const int wb = sk_owner(first_unit_of(tile) + stages_of(tile) - 1, p.sk_q, p.sk_rem);
#pragma unroll
        for (int ii = 0; ii < TM; ii++)
#pragma unroll
            for (int jj = 0; jj < TN; jj++) acc[0][ii][jj] = (v16f)(0.0f);
        auto piece_of = [&](int w2) __attribute__((always_inline)) -> const float* {
            const int w2_first_tile = tile_of(sk_first_unit(w2, p.sk_q, p.sk_rem));
            return p.sk_ws + (size_t)(2 * w2 + (w2_first_tile == tile ? 0 : 1)) * (BM * BN);
        };
        // two at a time (four at a time made the compiler's code of the 64 x 64 kernel's main loop 5 % slower)
        int w2 = wa;
        for (; w2 + 1 <= wb; w2 += 2) {
            const float* const two[2] = {piece_of(w2), piece_of(w2 + 1)};
            add_partials<2, TM, TN>(acc[0], two, wave, lane);
        }
        if (w2 <= wb) add_partial<TM, TN>(acc[0], piece_of(w2), wave, lane);
        const TileCtx c = decode(tile);
        store_tile<A_KIN, B_KIN, TM, TN, BIAS>(acc[0], p, c.row0, c.col0, c.c_ptr, wm, wn, r, h);
    }
}

template <bool A_KIN, bool B_KIN, int WM, int WN, int TM, int TN, int KT, int NS, int OCC = 1, bool CONV = false>
static hipError_t launch_streamk_cfg(GemmParams p, hipStream_t stream, float* ws, size_t ws_floats) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    // the bias row exists for the forward product and the convolution only (added where a tile is stored:
    // once, by whoever holds the whole sum)
    constexpr bool CAN_BIAS = (A_KIN && !B_KIN) || CONV;
    if (CONV && p.split) return hipErrorOutOfMemory;
    if (p.zero_floats > 0 && (CONV || p.split || p.bias != nullptr)) return hipErrorOutOfMemory;
    if (p.bias != nullptr && (!CAN_BIAS || p.split)) return hipErrorOutOfMemory;   // no balanced form: the caller falls back
    p.tiles_m = (p.rows + BM - 1) / BM;
    p.tiles_n = (p.cols + BN - 1) / BN;
    const long long all_tiles = (long long)p.tiles_m * p.tiles_n * p.nz;
    if (p.sk_tile_count > 0 && (p.split || CONV || p.zero_floats > 0 || p.sk_tile_base + (long long)p.sk_tile_count > all_tiles)) return hipErrorInvalidValue;
    const long long tiles = p.sk_tile_count > 0 ? p.sk_tile_count : all_tiles;
    // K slices: every slice but the last is k_slice long, the last takes the rest of K
    const long long k_first = p.split ? p.k_slice : p.k_total;
    const long long k_last = p.split ? (long long)p.k_total - (long long)(p.nz - 1) * p.k_slice : p.k_total;
    if (p.split && (p.k_slice < KT || k_last < KT)) return hipErrorOutOfMemory;   // slices shorter than a stage
    const long long S = (k_first + KT - 1) / KT, S_last = (k_last + KT - 1) / KT;
    const long long tiles_before = p.split ? (long long)p.tiles_m * p.tiles_n * (p.nz - 1) : tiles;
    const long long units = tiles_before * S + (tiles - tiles_before) * S_last;
    if (tiles <= 0 || S <= 0) return hipErrorInvalidValue;
    if (units > 0x3fffffffLL) return hipErrorOutOfMemory;
    gemm_fill_tile_divisors(p);
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const long long slots = (long long)num_cu * OCC;
    const long long grid = units < slots ? units : slots;
    if (ws == nullptr || tiles > SK_MAX_TILES || SK_MAX_TILES + (size_t)(2 * grid) * BM * BN > ws_floats)
        return hipErrorOutOfMemory;
    p.sk_count = (int*)ws;            // one arrival counter per tile, zero between launches
    p.sk_ws = ws + SK_MAX_TILES;
    p.sk_S = (int)S;
    gemm_magic_divisor((unsigned)S, p.sk_div_S_mul, p.sk_div_S_shift);
    p.sk_S_last = (int)S_last;
    p.sk_T1 = (int)tiles_before;
    gemm_magic_divisor((unsigned)S_last, p.sk_div_Sl_mul, p.sk_div_Sl_shift);
    p.sk_q = (int)(units / grid);
    p.sk_rem = (int)(units % grid);
    p.sk_kmajor_rpt = 0;
    p.sk_kmajor_tiles = (int)tiles;
    if (!CONV && !p.split && p.nz == 1 && tiles >= 2 && p.sk_rem == 0 && grid % tiles == 0 && grid / tiles >= 2 && S % (grid / tiles) == 0)
        p.sk_kmajor_rpt = (int)(grid / tiles);
    if constexpr (CAN_BIAS) {
        if (p.bias != nullptr) {
            hipLaunchKernelGGL((gemm_f32_mfma_streamk<A_KIN, B_KIN, WM, WN, TM, TN, KT, NS, OCC, true, false, CONV>),
                               dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
            return hipGetLastError();
        }
    }
    if constexpr (CONV) {
        hipLaunchKernelGGL((gemm_f32_mfma_streamk<A_KIN, B_KIN, WM, WN, TM, TN, KT, NS, OCC, false, false, true>),
                           dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
        return hipGetLastError();
    }
    if (p.split) {
        hipLaunchKernelGGL((gemm_f32_mfma_streamk<A_KIN, B_KIN, WM, WN, TM, TN, KT, NS, OCC, false, true>),
                           dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
        return hipGetLastError();
    }
    if constexpr (!CONV && !(WM == 4)) {   // every 2-D shape; the 256 x 64 tile is a batch's
        if (p.zero_floats > 0) {
            hipLaunchKernelGGL((gemm_f32_mfma_streamk<A_KIN, B_KIN, WM, WN, TM, TN, KT, NS, OCC, false, false, false, true>),
                               dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
            return hipGetLastError();
        }
    }
    if (p.zero_floats > 0) return hipErrorOutOfMemory;   // no zero-filling form of this shape: the caller keeps the split
    hipLaunchKernelGGL((gemm_f32_mfma_streamk<A_KIN, B_KIN, WM, WN, TM, TN, KT, NS, OCC, false, false>),
                       dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
    return hipGetLastError();
}

template <bool A_KIN, bool B_KIN>
static hipError_t launch_streamk_variant(const GemmParams& p, int tile, hipStream_t stream, float* ws, size_t ws_floats) {
    switch (tile) {
        case TILE_SK_64x64:     return launch_streamk_cfg<A_KIN, B_KIN, 2, 2, 1, 1, 32, 4, 1>(p, stream, ws, ws_floats);
        case TILE_SK_128x64:    return launch_streamk_cfg<A_KIN, B_KIN, 2, 2, 2, 1, 32, 4, 1>(p, stream, ws, ws_floats);
        case TILE_SK_64x128:    return launch_streamk_cfg<A_KIN, B_KIN, 2, 2, 1, 2, 32, 4, 1>(p, stream, ws, ws_floats);
        case TILE_SK_128x128:   return launch_streamk_cfg<A_KIN, B_KIN, 2, 2, 2, 2, 32, 4, 1>(p, stream, ws, ws_floats);
        case TILE_SK_64x64_O2:  return launch_streamk_cfg<A_KIN, B_KIN, 2, 2, 1, 1, 32, 4, 2>(p, stream, ws, ws_floats);
        case TILE_SK_128x64_O2: return launch_streamk_cfg<A_KIN, B_KIN, 2, 2, 2, 1, 32, 3, 2>(p, stream, ws, ws_floats);
        case TILE_SK_256x64:    return launch_streamk_cfg<A_KIN, B_KIN, 4, 1, 2, 2, 32, 3, 1>(p, stream, ws, ws_floats);
        default: return hipErrorInvalidValue;
    }
}

// ---- the workspace: one per (device, stream), made at the first balanced launch on that stream, released
// when the stream is deleted through the runtime bridge (or by gemm_streamk_release_workspaces) ----
struct Workspace { float* ptr; size_t floats; };
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Workspace> g_ws;
std::atomic<long long> g_ws_refused{0};   // balanced launches that found the table full and took another kernel

__global__ void sk_zero_counters_kernel(int* counters, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) counters[i] = 0;
}

// the device a stream belongs to (the current one for the null stream)
int device_of(hipStream_t stream) {
    int dev = 0;
    if (stream != nullptr) {
        hipDevice_t d = 0;
        if (hipStreamGetDevice(stream, &d) == hipSuccess) return (int)d;
        (void)hipGetLastError();
    }
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    return dev;
}

}  // namespace

size_t gemm_streamk_workspace_floats(int num_cu) { return SK_MAX_TILES + (size_t)2 * num_cu * 128 * 128; }
static_assert(GEMM_SK_WS_FLOATS_256CU == SK_MAX_TILES + (size_t)2 * 256 * 128 * 128, "the constant in the header");

float* gemm_streamk_workspace(hipStream_t stream, size_t* floats) {
    // Not under a stream capture: nothing may be allocated there, and a graph may later be launched on ANOTHER
    // stream, next to eager launches that use this stream's workspace -- two launches on one workspace at a
    // time would mix their pieces.  The caller takes the tile-per-workgroup kernel instead.
    // Nor on the per-thread default stream: one handle that stands for a different stream in every host thread,
    // whose launches may run side by side.
    if (stream == hipStreamPerThread) return nullptr;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;
    }
    const int dev = device_of(stream);
    if (dev < 0) return nullptr;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_ws.find({dev, stream});
    if (it != g_ws.end()) {
        *floats = it->second.floats;
        return it->second.ptr;
    }
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return nullptr;
    // a host that keeps making streams without deleting them does not make the library hold ever more memory
    if (g_ws.size() >= SK_MAX_WORKSPACES) {
        g_ws_refused.fetch_add(1, std::memory_order_relaxed);
        return nullptr;
    }
    Workspace w = {nullptr, gemm_streamk_workspace_floats(num_cu)};
    // Another host thread may be capturing a graph in the global mode, which forbids allocations from every
    // thread: for the length of the allocation this thread steps out of that rule (its own stream is not
    // capturing, checked above).
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    const hipError_t em = hipMalloc((void**)&w.ptr, w.floats * sizeof(float));
    if (swapped) (void)hipThreadExchangeStreamCaptureMode(&mode);
    if (em != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    // the arrival counters start at zero and every launch leaves them there.  Cleared by a kernel on the launch
    // stream itself: in order before the launch that follows, and no other stream is made to wait.
    hipLaunchKernelGGL(sk_zero_counters_kernel, dim3(SK_MAX_TILES / 256), dim3(256), 0, stream, (int*)w.ptr, SK_MAX_TILES);
    if (hipGetLastError() != hipSuccess) {
        (void)hipFree(w.ptr);
        return nullptr;
    }
    g_ws[{dev, stream}] = w;
    *floats = w.floats;
    return w.ptr;
}

void gemm_streamk_release_workspace(hipStream_t stream) {
    const int dev = device_of(stream);
    Workspace w = {nullptr, 0};
    {
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        auto it = g_ws.find({dev, stream});
        if (it == g_ws.end()) return;
        w = it->second;
        g_ws.erase(it);
    }
    // the stream's launches may still be using it
    (void)hipStreamSynchronize(stream);
    (void)hipFree(w.ptr);
}

int gemm_streamk_release_workspaces() {
    std::map<std::pair<int, hipStream_t>, Workspace> all;
    {
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        all.swap(g_ws);
    }
    int prev = -1;
    (void)hipGetDevice(&prev);
    for (auto& kv : all) {
        // a workspace is freed on its own device, after that device's work (the launches that use it) is done
        if (hipSetDevice(kv.first.first) != hipSuccess) continue;
        (void)hipDeviceSynchronize();
        (void)hipFree(kv.second.ptr);
    }
    if (prev >= 0) (void)hipSetDevice(prev);
    return (int)all.size();
}

int gemm_streamk_workspace_count() {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    return (int)g_ws.size();
}
long long gemm_streamk_workspaces_refused() { return g_ws_refused.load(std::memory_order_relaxed); }

namespace {
// The three fitted times for t64 tiles of 64 x 64 with S stages each on num_cu units (see below): tile per
// workgroup, balanced with one workgroup per unit, balanced with two (1e300 where its runs are not whole tiles).
struct FewTilesEstimate { double t_tiles, t_one, t_two; };
FewTilesEstimate few_tiles_estimate(long long t64, long long S, int num_cu, int variant) {
    const long long units = t64 * S;
    const long long run1 = (units + num_cu - 1) / num_cu;
    const bool whole1 = t64 % num_cu == 0;
    const double pieces = run1 < S ? (double)S / (double)run1 : 0.0;
    FewTilesEstimate e;
    e.t_one = (whole1 ? 3.0 : 7.5 + 0.4 * (pieces > 2.0 ? pieces - 2.0 : 0.0)) + 0.5 * (double)run1;
    const bool whole2 = t64 % (2LL * num_cu) == 0;
    e.t_two = whole2 ? 3.5 + 0.92 * (double)(units / (2LL * num_cu)) : 1e300;
    const double per_unit = (double)((t64 + num_cu - 1) / num_cu);
    e.t_tiles = 4.5 + (variant == GEMM_T1 ? 0.615 : 0.575) * (double)S * per_unit;
    return e;
}
}  // namespace

// Fitted to times measured on MI355X (256 ... 2048-wide squares and panels, 1000 x 780 x 1532, K from 64 to
// 131072, all three layouts), in microseconds, with S = 32-k stages per tile and `run` = stages per workgroup:
//   tile-per-workgroup kernels, at most two 64 x 64 tiles per compute unit: 4.5 + 0.575 S (0.615 for A^T*B) per
//                                                                           tile of the busiest unit;
//   balanced, one workgroup per unit: 0.5 per stage of a run (85 % of the matrix peak with every unit busy)
//     + 3 where every run is whole tiles, else 7.5 (the pieces cross the chip through memory, and the last
//     arriver adds them one after the other: 0.4 more for every piece of a tile beyond the second);
//   balanced, two workgroups per unit: behind the former except where its runs are whole tiles and the
//     former's are not (512 tiles on 256 units: 18.2 against 19.6).
// Products with fewer stages than two per unit stay with the tile-per-workgroup kernels (256^3: 7.9 against
// 9.7).  Measured gains where it is taken: 15 % at 1000 x 777 x 1531, 17 % at 1024^3 and 1536 x 1024 x 1024,
// 25 % at 512^3, 18 % at 2048 x 512 x 2048, 2.2 x at 128 x 128 x 4096, 17 x at 256 x 256 x 131072 (where it
// equals the host's split into 128 slices plus the fold: 138 us).
//
// LARGE products take the balanced kernel too, with 128 x 128 tiles: its stages carry no vector-ALU instruction
// (which would exclude MFMAs on the SIMD), so one workgroup per unit keeps the matrix pipes as busy as four of the
// tile-per-workgroup kernel do, and the equal runs leave no unit idle in a last, partial round of tiles.  Measured
// against the best tile-per-workgroup shape: 4096^3 918 against 934 us (95 % of the peak), 8192 x 4096 x 4096 1835 /
// 1882, 3584^3 636 / 721, 3072^3 404 / 425, 2560^3 241 / 283-299, 2048^3 119 / 128, 1024 x 8192 x 1024 121 / 128;
// level at K = 512 ... 768 (within +-5 % either way over ten shapes), so the rule starts at 768.  From K = 96 on
// one case is taken besides: 128 x 64 tiles that can be dealt whole, one to three each, to two workgroups per
// unit (2048^2 x 512: 33.2 / 35.9; 8192 x 1024 x 512: 63.5 / 67.4; 2048^2 x 256: 19.2 / 20.4; 6144 x 2048 x 256:
// 50.0 / 51.7; K = 96 ... 192: batch 64 of 256 x 256 x 128 11.5 / 12.8, batch 16 of 512 x 512 x 192 15.1 / 17.2,
// 2048^2 x 128 11.9 / 12.8, twelve such shapes 4 - 12 % ahead).  Between the two
// regimes (more than two 64 x 64 tiles per unit, fewer than one of 128 x 128) the tile is 128 x 64 or 64 x 128:
// 1536^3 61 against 74 us, 1792^3 92 / 111.
int gemm_choose_streamk(int rows, int cols, int nz, int k, int num_cu, int variant) {
    if (rows <= 0 || cols <= 0 || nz <= 0 || k <= 0 || num_cu <= 0) return -1;
    const long long t64 = (long long)((rows + 63) / 64) * ((cols + 63) / 64) * nz;
    if (k >= 96 && t64 > 2LL * num_cu) {
        const long long rm = (rows + 127) / 128, cn = (cols + 127) / 128, rm64 = (rows + 63) / 64, cn64 = (cols + 63) / 64;
        const double area = (double)rows * (double)cols;
        const long long t128 = rm * cn * nz;
        // A batch whose products are up to 64 columns wide and give exactly one 256 x 64 tile per unit: that shape
        // (the 128 x 128 tile's ratio of matrix work to LDS traffic) measured 0 - 5 % ahead of the 128 x 64 tiles
        // dealt two per unit on batches of 1024 / 2048 / 4096 x 64 x 1024 (68.4-70.9 against 72.2-73.0 us,
        // 67.1-67.4 / 67.5-68.0, 65.1-65.4 / 66.8-67.3), level at K = 2048, behind at K = 512 and for one product
        if (nz > 1 && cols > 32 && cols <= 64 && k >= 768 && k <= 1536 && rows % 256 == 0 &&
            (long long)(rows / 256) * nz == num_cu)
            return TILE_SK_256x64;
        if (k < 768) {
            // a shorter K: 128 x 64 tiles, two workgroups per unit, where that deals whole tiles, up to three each
            // (with four, 4096^2 x 512, the 128 x 128 tile-per-workgroup kernel is 1-2 % ahead again); other
            // shapes measured within +-5 % of the best tile-per-workgroup shape either way and stay there
            const long long th = rm * cn64 * nz;
            if (th % (2LL * num_cu) == 0 && th <= 6LL * num_cu && area >= 0.85 * (double)(rm * 128) * (double)(cn64 * 64))
                return TILE_SK_128x64_O2;
            return -1;
        }
        if (t128 >= num_cu && t128 <= SK_MAX_TILES && area >= 0.85 * (double)(rm * 128) * (double)(cn * 128))
            return TILE_SK_128x128;
        // the half-size tile that wastes less of C
        const bool tall = (double)(rm * 128) * (double)(cn64 * 64) <= (double)(rm64 * 64) * (double)(cn * 128);
        const long long th = (tall ? rm * cn64 : rm64 * cn) * nz;
        const double padded = tall ? (double)(rm * 128) * (double)(cn64 * 64) : (double)(rm64 * 64) * (double)(cn * 128);
        if (th >= num_cu && th <= SK_MAX_TILES && area >= 0.85 * padded) {
            // two workgroups per compute unit where that deals whole tiles
            if (tall && th % (2LL * num_cu) == 0) return TILE_SK_128x64_O2;
            return tall ? TILE_SK_128x64 : TILE_SK_64x128;
        }
        return -1;
    }
    if (t64 > 2LL * num_cu || t64 > SK_MAX_TILES) return -1;
    const long long S = ((long long)k + 31) / 32;
    const long long units = t64 * S;
    if (units < 2LL * num_cu) return -1;
    const bool whole1 = t64 % num_cu == 0;
    // Many tiles with a long K whose runs are not whole tiles: neighbouring workgroups then sit at different k of
    // the same operand panels, nothing is shared through the L2, and 64 x 64 tiles -- 16 FLOP per byte staged --
    // become bound by the fabric (1000 x 780 x 8192: 0.7 us per stage instead of 0.5).  The half-size tile stages
    // a third fewer bytes per FLOP: 148 -> 110 us there, 768^2 x 8192 90 -> 79, 1280^2 x 4096 119 -> 105; with
    // fewer tiles or a shorter K (640^2 x 4096, 512^2 x 16384, 1000 x 780 x 3072, 1536 x 768 x 2048) level or behind.
    if (!whole1 && t64 >= num_cu / 2 && S >= 128) {
        const long long rm = (rows + 127) / 128, cn = (cols + 127) / 128, rm64 = (rows + 63) / 64, cn64 = (cols + 63) / 64;
        const bool tall = (double)(rm * 128) * (double)(cn64 * 64) <= (double)(rm64 * 64) * (double)(cn * 128);
        return tall ? TILE_SK_128x64 : TILE_SK_64x128;
    }
    const FewTilesEstimate est = few_tiles_estimate(t64, S, num_cu, variant);
    const double t_balanced = est.t_two < est.t_one ? est.t_two : est.t_one;
    if (t_balanced > 0.97 * est.t_tiles) return -1;
    return est.t_two < est.t_one ? TILE_SK_64x64_O2 : TILE_SK_64x64;
}

double gemm_estimate_us(int rows, int cols, int nz, int k, int num_cu, int variant) {
    if (rows <= 0 || cols <= 0 || nz <= 0 || k <= 0 || num_cu <= 0) return 0.0;
    const long long rm64 = (rows + 63) / 64, cn64 = (cols + 63) / 64;
    const long long t64 = rm64 * cn64 * nz;
    const long long S = ((long long)k + 31) / 32;
    if (t64 <= 2LL * num_cu) {
        const FewTilesEstimate est = few_tiles_estimate(t64, S, num_cu, variant);
        double t = est.t_tiles;
        if (t64 * S >= 2LL * num_cu) {   // the balanced kernel's floor of two stages per unit
            if (est.t_one < t) t = est.t_one;
            if (est.t_two < t) t = est.t_two;
        }
        return t;
    }
    // more tiles: the matrix work of the padded tiles at 90 % of the chip's rate (256 FLOP per clock and unit,
    // 2400 clocks per microsecond) and what a launch of that size costs beside it
    const double flop = 2.0 * (double)(rm64 * 64) * (double)(cn64 * 64) * (double)nz * (double)k;
    return flop / (0.9 * 614400.0 * (double)num_cu) + 4.0;
}

bool gemm_split_loses(int variant, int rows, int cols, int gz, int k, int k_slice, int num_cu) {
    if (gz < 2 || k_slice < 32 || num_cu <= 0) return false;
    // only where the unsplit product takes the balanced kernel: the tile-per-workgroup kernels deal whole tiles,
    // and few of them leave units idle -- that is what the host's split is for
    if (gemm_choose_streamk(rows, cols, 1, k, num_cu, variant) < 0) return false;
    const long long t64 = (long long)((rows + 63) / 64) * ((cols + 63) / 64);
    // equal runs of 128-class tiles' stages: a split adds nothing there but its fold
    if (t64 > 2LL * num_cu) return true;
    // the fold: a launch, and gz + 1 passes over C at about 5.5 TB/s
    const double fold = 2.5 + 4.0 * (double)(gz + 1) * (double)rows * (double)cols / 5.5e6;
    // (the estimate of the slices runs 15 - 20 % under what they take once C has 128 Ki outputs or more -- 512^2 x 4096 in
    // 8: 22.4 estimated, 26.2 us measured; 384^2 x 16384 in 44: 45.1 / 53.8; 768^2 x 3072 in 4: 34.2 / 40.5 -- while it is
    // within 10 % on the small C of the long-K shapes that the split is for; the unsplit estimates are within 3 %)
    const double margin = (long long)rows * cols >= 131072 ? 1.15 : 1.0;
    return gemm_estimate_us(rows, cols, 1, k, num_cu, variant) <= margin * (gemm_estimate_us(rows, cols, gz, k_slice, num_cu, variant) + fold);
}

hipError_t gemm_launch_streamk_conv(const GemmParams& p0, int tile, hipStream_t stream) {
    GemmParams p = p0;
    // a stage of 32 channels inside one filter tap; the taps' validity bits in one register each; every byte
    // offset (the image's extent plus the bias that keeps offsets non-negative) below the out-of-range mark
    if (p.cv_IC <= 0 || (p.cv_IC & 31) != 0 || p.cv_FW <= 0 || p.cv_FW > 32 || p.split) return hipErrorOutOfMemory;
    const long long taps_k = (long long)p.cv_FW * p.cv_IC;
    if (p.k_total <= 0 || p.k_total % taps_k != 0) return hipErrorInvalidValue;
    p.cv_FH = (int)(p.k_total / taps_k);
    if (p.cv_FH > 32) return hipErrorOutOfMemory;
    const long long bias = ((long long)p.cv_ph * p.cv_IW + p.cv_pw) * p.cv_IC * 4;
    // the image as far as the lanes' rows can reach: rows beyond the last output pixel (tile padding) are
    // switched off by their validity bits, whatever their offset
    const long long n_images = ((long long)p.rows + (long long)p.cv_OH * p.cv_OW - 1) / ((long long)p.cv_OH * p.cv_OW);
    const long long extent = n_images * p.cv_IH * p.cv_IW * p.cv_IC * 4;
    if (extent + 2 * bias + 4096 >= (long long)OOB_OFFSET) return hipErrorOutOfMemory;
    p.cv_bias = (int)bias;
    p.cv_spt = p.cv_IC / 32;
    gemm_magic_divisor((unsigned)p.cv_OW, p.cv_div_OW_mul, p.cv_div_OW_shift);
    gemm_magic_divisor((unsigned)p.cv_OH, p.cv_div_OH_mul, p.cv_div_OH_shift);
    gemm_magic_divisor((unsigned)p.cv_spt, p.cv_div_spt_mul, p.cv_div_spt_shift);
    gemm_magic_divisor((unsigned)p.cv_FW, p.cv_div_FW_mul, p.cv_div_FW_shift);
    size_t floats = p.sk_ws_given_floats;
    float* ws = p.sk_ws_given != nullptr ? p.sk_ws_given : gemm_streamk_workspace(stream, &floats);
    if (ws == nullptr) return hipErrorOutOfMemory;
    switch (tile) {
        case TILE_SK_64x64:   return launch_streamk_cfg<true, true, 2, 2, 1, 1, 32, 4, 1, true>(p, stream, ws, floats);
        case TILE_SK_128x64:  return launch_streamk_cfg<true, true, 2, 2, 2, 1, 32, 4, 1, true>(p, stream, ws, floats);
        case TILE_SK_64x128:  return launch_streamk_cfg<true, true, 2, 2, 1, 2, 32, 4, 1, true>(p, stream, ws, floats);
        case TILE_SK_128x128: return launch_streamk_cfg<true, true, 2, 2, 2, 2, 32, 4, 1, true>(p, stream, ws, floats);
        case TILE_SK_256x64:  return launch_streamk_cfg<true, true, 4, 1, 2, 2, 32, 3, 1, true>(p, stream, ws, floats);
        default: return hipErrorOutOfMemory;   // the shapes with two workgroups per unit are not built for the gather
    }
}

static hipError_t launch_streamk_any(int variant, const GemmParams& p, int tile, hipStream_t stream, float* ws, size_t floats) {
    switch (variant) {
        case GEMM_NN: return launch_streamk_variant<true, false>(p, tile, stream, ws, floats);
        case GEMM_T1: return launch_streamk_variant<false, false>(p, tile, stream, ws, floats);
        case GEMM_T2: return launch_streamk_variant<true, true>(p, tile, stream, ws, floats);
        default: return hipErrorInvalidValue;
    }
}

// Many 128 x 128 tiles that do not divide among the workgroups (3072^3: 576 tiles for 256; 5120^3: 1600): dealt in
// equal runs, every workgroup starts inside a tile at a k of its own, neighbours on an XCD no longer read the same
// operand panels at the same time, and the L2 serves next to nothing (measured: 2 % and 1.3 % hits against 71 % at
// 4096^3, 24 x and 40 x the operands' bytes fetched through the fabric).  Such a product goes out as TWO launches:
// the largest multiple of the workgroup count as whole tiles (every workgroup the same number, in step, the band
// order's sharing intact), then the remaining tiles -- fewer than workgroups -- shared out in runs of stages, where
// the k ranges of all tiles sit together on an XCD (sk_kmajor_rpt) whenever the counts divide.
static bool streamk_two_launches(const GemmParams& p, int tile, long long& first_count, long long& all_tiles) {
    if (tile != TILE_SK_128x128 || p.split || p.zero_floats > 0 || p.sk_tile_count > 0) return false;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return false;
    all_tiles = (long long)((p.rows + 127) / 128) * ((p.cols + 127) / 128) * p.nz;
    first_count = all_tiles / num_cu * num_cu;
    const long long rest = all_tiles - first_count;
    // Worth a second launch from two whole tiles per workgroup on (with one it measured -2 ... +2 %) and a K of at
    // least 3072: 3072^3 414 -> 402 us, 5120^3 1871 -> 1800, 4096 x 11008 x 4096 2588 -> 2481; with K = 1024 ... 2048
    // (3072^2, 5120^2, 3584^2 x 1536, 2000 x 5000 x 1100) the launches' ends cost what the L2 gives back, -3 ... +1 %.
    return first_count >= 2LL * num_cu && rest > 0 && p.k_total >= 3072;
}

hipError_t gemm_launch_streamk(int variant, const GemmParams& p, int tile, hipStream_t stream) {
    size_t floats = p.sk_ws_given_floats;
    float* ws = p.sk_ws_given != nullptr ? p.sk_ws_given : gemm_streamk_workspace(stream, &floats);
    if (ws == nullptr) return hipErrorOutOfMemory;
    long long first_count = 0, all_tiles = 0;
    if (streamk_two_launches(p, tile, first_count, all_tiles)) {
        GemmParams q = p;
        q.sk_tile_base = 0;
        q.sk_tile_count = (int)first_count;
        const hipError_t e = launch_streamk_any(variant, q, tile, stream, ws, floats);
        if (e != hipSuccess) return e;
        q.sk_tile_base = (int)first_count;
        q.sk_tile_count = (int)(all_tiles - first_count);
        return launch_streamk_any(variant, q, tile, stream, ws, floats);
    }
    return launch_streamk_any(variant, p, tile, stream, ws, floats);
}

}  // namespace dragon
