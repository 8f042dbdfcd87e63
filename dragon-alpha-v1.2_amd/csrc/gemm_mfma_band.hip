// The products with a SHORT K (at most 64) and a large C: the score products of attention layers
// (Q*K^T, and its A^T*B twin in the backward pass), batch after batch of 1024 x 1024 x 64.
//
// Such a product writes 64 KiB of C for every 64 KiB of operands it reads and every 2048 MFMAs a
// compute unit issues: the matrix pipes and the memory's write path are needed at the same time, all
// the time, and a kernel that computes a tile and then stores it uses them in turns.  This one is
// built around four things:
//   * no K loop.  A stage holds the whole K, so a tile is ONE stage: one barrier per tile, no
//     pipeline to fill and drain;
//   * the A operand stays.  A workgroup takes a band of 128 rows and walks along its column tiles;
//     the band's rows of A go to LDS once per band (into the other of two buffers while the last
//     tile of the band before is multiplied), only B is fetched per tile (global -> LDS directly,
//     one tile ahead, into the other of two buffers);
//   * the stores of a tile leave during the NEXT tile.  Two accumulator sets take turns; while one
//     is multiplied into, the other -- the finished tile -- is stored a few rows at a time between
//     the MFMAs.  The write path sees an even stream instead of bursts of 64 KiB per workgroup, and
//     no wavefront ever waits for its own stores: the only vector-memory wait of a tile is for the
//     transfers of the next one, which were issued BEFORE the tile's stores, and the counter
//     retires in issue order;
//   * next to no vector-ALU instructions.  On this chip an MFMA and a vector-ALU instruction of
//     the same SIMD exclude each other: measured with MFMAs back to back, every v_add / v_mov /
//     v_cndmask put between them costs the matrix pipe 9-11 cycles with one wavefront on the SIMD
//     and 4-6 with four, while scalar instructions (up to ten per MFMA), LDS reads and writes,
//     buffer loads and stores and barriers cost nothing.  So: the LDS addresses of the fragment
//     reads are worked out once per launch and kept in registers; a store's row travels in its
//     scalar offset and the rows beyond C are cut off by the descriptor's size (the hardware
//     checks vector + scalar offset against it), columns by a lane offset that is out of range
//     from the start; the accumulators are stored as they lie (32-bit stores, 128 contiguous bytes
//     per row and half wavefront) rather than paired up with moves; a tile's first MFMA per
//     block takes a zero constant instead of cleared registers.  What is left per tile and
//     wavefront is a handful of selects in the last column tile of a band.
// Eight wavefronts of 32 x 64 share the 128 x 128 tile, two per SIMD (sixteen of 32 x 32 measured the same).
// LDS: two A bands and two B tiles of 32 KiB = 128 KiB, one workgroup per compute unit.
//
// The reference runs these shapes through its batched kernels tile by tile
// (BMM/batchMatMulT2_uernel.cuh:51-173); the result here is the same sum per element, k ascending
// within each lane half as in the other kernels.
#include "gemm_mfma_kernel.h"

namespace dragon {
namespace {

constexpr int BD_KT = 64, BD_THREADS = 512;
// Cache policy of the C stores: streaming (nt).  Measured on batch 64 of 1024 x 1024 x 64: 73 us, against 91-96 us
// with plain stores or with the scope bits alone (C's lines then stay in the L2 and compete with the operands).
constexpr int BD_STORE_AUX = 2;

// LDS addresses are kept as 32-bit integers and turned into LDS pointers where they are read (the host
// pass, for which every pointer has 64 bits, warns about that)
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"
typedef __attribute__((address_space(3))) const float* lds_f32;
typedef __attribute__((address_space(3))) const v4f* lds_v4f;

// A value the compiler may not work out again where it is used: it stays in the register it is in.
__device__ __forceinline__ unsigned pinned(unsigned v) {
    asm volatile("" : "+v"(v));
    return v;
}

// The lanes' part of a tile's transfers for a workgroup of NT threads: transfer s of thread t fills LDS
// chunk s * NT + t (the hardware puts lane l's 16 bytes at the wave's base + 16 * l), which in the
// layouts of gemm_mfma_kernel.h is
//   K-inner operand: LDS row (s * NT + t) / (KT / 4), chunk slot t % (KT / 4); the slot holds logical
//                    chunk slot ^ swizzle(row);
//   K-outer operand: k row (s * NT + t) / (R / 4), chunk t % (R / 4).
// An offset is out of range where its k lies beyond K (which is the same for every tile of a launch).
template <bool KIN, int R, int KT, int NT>
struct BandLanes {
    static constexpr int CPR = KIN ? KT / 4 : R / 4;     // chunks per LDS row
    static constexpr int RPP = NT / CPR;                 // LDS rows per transfer
    static constexpr int PASSES = (KIN ? R : KT) / RPP;
    static_assert(NT % CPR == 0 && (KIN ? R : KT) % RPP == 0 && PASSES >= 1, "tile does not divide over the workgroup");
    int off[PASSES];
    int first;   // K-outer: the lane's first column in the tile
    __device__ __forceinline__ void init(int t, int ld, int k_limit) {
        const int slot = t % CPR, r0 = t / CPR;
        first = slot * 4;
#pragma unroll
        for (int s = 0; s < PASSES; s++) {
            const int row = r0 + s * RPP;
            if constexpr (KIN) {
                const int c = slot ^ kin_swizzle<KT>(row);
                off[s] = (c * 4 < k_limit) ? (row * ld + c * 4) * 4 : OOB_OFFSET;
            } else {
                off[s] = (row < k_limit) ? (row * ld + slot * 4) * 4 : OOB_OFFSET;
            }
        }
    }
};

// Descriptor of an operand tile.  K-inner operand (a row of the tile per row of the matrix): the
// size is the bytes up to the last row that exists, so the hardware zeroes the rows beyond and the
// lanes' offsets never change from tile to tile.  K-outer operand (columns of the tile along a
// matrix row): the lane tests its own column.  rows <= 0 makes every lane out of range: a transfer
// that fetches nothing and fills its part of LDS with zeros.
template <bool KIN>
__device__ __forceinline__ v4u band_descriptor(const float* base, int rows, int tile_rows, int ld) {
    const unsigned long long b = (unsigned long long)base;
    rows = rows > tile_rows ? tile_rows : rows;
    const unsigned records = rows <= 0 ? 0u : KIN ? (unsigned)rows * (unsigned)ld * 4u : (unsigned)RSRC_RECORDS;
    const v4u rsrc = {(unsigned)b, (unsigned)(b >> 32) & 0xffffu, records, (unsigned)RSRC_FLAGS};
    return rsrc;
}

// BM x BN: 128 x 128 (bands of 128 rows), or 64 x 256 (bands of 64 rows under tiles of 256 columns: the stores of a
// tile then run along 1 KiB of a row of C instead of 512 bytes)
template <bool A_KIN, bool B_KIN, int BM, int BN>
__global__ __launch_bounds__(BD_THREADS, 1)
void gemm_f32_mfma_band(const GemmParams p) {
    constexpr int NT = BD_THREADS, TN = 2, WN = BN / (TN * 32), KT = BD_KT;
    static_assert(NT / 64 == (BM / 32) * WN && BN == WN * TN * 32, "the wavefronts cover the tile");
    constexpr int GR = KT / 8;                 // k groups per tile
    constexpr int NM = 4 * TN;                 // MFMAs per group: 4 k steps of TN blocks
    constexpr int NSTORE = 16 * TN;            // stores per wavefront and tile
    using LanesA = BandLanes<A_KIN, BM, KT, NT>;
    using LanesB = BandLanes<B_KIN, BN, KT, NT>;
    constexpr int PA = LanesA::PASSES, PB = LanesB::PASSES;
    constexpr int A_BYTES = BM * KT * 4, B_BYTES = BN * KT * 4;
    // where the pieces of a tile's side work sit among its GR * NM MFMAs (slot = number of the MFMA before)
    constexpr int SLOT_A = 1;                  // the next band's A, when the next tile starts a band
    constexpr int SLOT_B = 2;                  // PB transfers of the next tile's B, one per slot
    constexpr int STORE_EVERY = 3;
    constexpr int SLOT_STORE = SLOT_B + PB;    // then TN stores (element e of the TN blocks) behind every third MFMA
    constexpr int SLOT_SYNC = (GR - 1) * NM;   // own transfers landed + barrier
    static_assert(SLOT_B + PB <= SLOT_STORE, "the transfers are issued before the first store");
    static_assert(SLOT_STORE + STORE_EVERY * 15 < SLOT_SYNC, "the stores are issued before the barrier");
    static_assert(NSTORE <= 63, "vmcnt holds 6 bits");

    __shared__ __attribute__((aligned(16))) float smemA[2 * BM * KT];
    __shared__ __attribute__((aligned(16))) float smemB[2 * BN * KT];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    // ---- the lanes' part of every transfer: fixed for the whole launch ----
    LanesA la;
    LanesB lb;
    la.init(t, p.lda, min(p.k_total, A_KIN ? p.a_inner : p.a_outer));
    lb.init(t, p.ldb, min(p.k_total, B_KIN ? p.b_inner : p.b_outer));
    const unsigned lds_a0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smemA;
    const unsigned lds_b0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smemB;
    unsigned lds_wave_a = lds_a0 + wave * 1024;          // of the A buffer the NEXT band goes to
    const unsigned lds_wave_b = lds_b0 + wave * 1024;

    // ---- the lanes' LDS addresses of the fragment reads: fixed too (the A ones change buffer per band) ----
    // K-inner: the lane's row of the wavefront's first block, chunk (2g + h) ^ swizzle; block b is 32 rows on.
    // K-outer: k row 4h of group 0, the lane's column in the wavefront's first block; k step q of group g is
    //          8g + q rows on, block b 32 columns.
    unsigned a_rd[A_KIN ? GR : 1], b_rd[B_KIN ? GR : 1];
    if constexpr (A_KIN) {
#pragma unroll
        for (int g = 0; g < GR; g++) a_rd[g] = pinned(lds_a0 + ((wm * 32 + r) * KT + ((2 * g + h) ^ kin_swizzle<KT>(r)) * 4) * 4);
    } else {
        a_rd[0] = pinned(lds_a0 + (4 * h * BM + wm * 32 + r) * 4);
    }
    if constexpr (B_KIN) {
#pragma unroll
        for (int g = 0; g < GR; g++) b_rd[g] = pinned(lds_b0 + ((wn * TN * 32 + r) * KT + ((2 * g + h) ^ kin_swizzle<KT>(r)) * 4) * 4);
    } else {
        b_rd[0] = pinned(lds_b0 + (4 * h * BN + wn * TN * 32 + r) * 4);
    }
    float fa[2][4], fb[2][TN][4];
    // group g of the A band the addresses point at and of B buffer PB_
    auto read_group = [&](auto set_c, auto g_c, auto pb_c) __attribute__((always_inline)) {
        constexpr int set = decltype(set_c)::value, g = decltype(g_c)::value, PB_ = decltype(pb_c)::value;
        if constexpr (A_KIN) {
            const v4f v = *(lds_v4f)a_rd[g];
            fa[set][0] = v.x; fa[set][1] = v.y; fa[set][2] = v.z; fa[set][3] = v.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fa[set][q] = *(lds_f32)(a_rd[0] + (8 * g + q) * BM * 4);
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if constexpr (B_KIN) {
                const v4f v = *(lds_v4f)(b_rd[g] + PB_ * B_BYTES + j * 32 * KT * 4);
                fb[set][j][0] = v.x; fb[set][j][1] = v.y; fb[set][j][2] = v.z; fb[set][j][3] = v.w;
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) fb[set][j][q] = *(lds_f32)(b_rd[0] + PB_ * B_BYTES + ((8 * g + q) * BN + j * 32) * 4);
            }
        }
    };

    // ---- the lanes' part of every store: the lane's first row and column in the tile; block j is 32 columns on ----
    const int ldc4 = p.ldc * 4;
    const int c_lane = (int)pinned((unsigned)((wm * 32 + 4 * h) * ldc4 + (wn * TN * 32 + r) * 4));
    const int c_col = wn * TN * 32 + r;

    // ---- the workgroup's units: (batch, band of 128 rows, run of column tiles), every G-th one ----
    const int G = gridDim.x;
    const int U = p.nz * p.tiles_m * p.bd_chunks;
    int u = xcd_contiguous_id(blockIdx.x, G);   // G <= U
    int z, m, n, n_end;
    auto decode_unit = [&](int unit) __attribute__((always_inline)) {
        // the same for every lane; said explicitly, so that the values live in scalar registers
        const int per_z = p.tiles_m * p.bd_chunks;
        z = __builtin_amdgcn_readfirstlane(unit / per_z);
        const int rem = unit - z * per_z;
        m = __builtin_amdgcn_readfirstlane(rem / p.bd_chunks);
        n = (rem - m * p.bd_chunks) * p.bd_chunk_tiles;
        n_end = min(n + p.bd_chunk_tiles, p.tiles_n);
    };
    auto a_descriptor = [&]() __attribute__((always_inline)) {
        const float* base = p.A + (size_t)z * p.sA + (A_KIN ? (size_t)m * BM * p.lda : (size_t)m * BM);
        return band_descriptor<A_KIN>(base, (A_KIN ? p.a_outer : p.a_inner) - m * BM, BM, p.lda);
    };
    auto b_descriptor = [&](bool live) __attribute__((always_inline)) {
        const float* base = p.B + (size_t)z * p.sB + (B_KIN ? (size_t)n * BN * p.ldb : (size_t)n * BN);
        return band_descriptor<B_KIN>(base, live ? (B_KIN ? p.b_outer : p.b_inner) - n * BN : 0, BN, p.ldb);
    };
    auto issue_a = [&](const v4u& ra) __attribute__((always_inline)) {
        // a K-outer operand's lanes beyond the operand's row length fetch nothing (the last band only)
        const int left = p.a_inner - m * BM;
        if (!A_KIN && left < BM) {
            static_for<PA>([&](auto ic) {
                dma_f4_lean<decltype(ic)::value * NT * 16>(ra, lds_wave_a, la.first < left ? la.off[decltype(ic)::value] : OOB_OFFSET);
            });
        } else {
            static_for<PA>([&](auto ic) { dma_f4_lean<decltype(ic)::value * NT * 16>(ra, lds_wave_a, la.off[decltype(ic)::value]); });
        }
    };

    v16f acc[2][TN];

    // ---- prologue: the first band of A and its first tile of B; no finished tile yet ----
    decode_unit(u);
    {
        const v4u ra = a_descriptor(), rb = b_descriptor(true);
        issue_a(ra);
        const int left = p.b_inner - n * BN;
        static_for<PB>([&](auto ic) {
            dma_f4_lean<decltype(ic)::value * NT * 16>(rb, lds_wave_b, (B_KIN || lb.first < left) ? lb.off[decltype(ic)::value] : OOB_OFFSET);
        });
    }
    lds_wave_a ^= A_BYTES;
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_group(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});

    float* cur_c = p.C + (size_t)z * p.sC + (size_t)m * BM * p.ldc + (size_t)n * BN;   // origin of the tile being multiplied
    int cur_rows = p.rows - m * BM, cur_cols = p.cols - n * BN;                          // what C has from there on
    float* prev_c = p.C;                       // the finished tile on its way out
    int prev_rows = 0, prev_cols = 0;          // no rows: every store is dropped
    bool has_next = true;

    // One tile, multiplied from B buffer P into accumulator set P.
    auto tile = [&](auto pc) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value;
        // -- the tile after this one --
        bool new_band = false;
        if (++n == n_end) {
            u += G;
            if (u < U) {
                decode_unit(u);
                new_band = true;
            } else {
                has_next = false;
                n = 0;
            }
        }
        const v4u rb = b_descriptor(has_next);
        int offb_now[PB];
#pragma unroll
        for (int s = 0; s < PB; s++) offb_now[s] = lb.off[s];
        if constexpr (!B_KIN) {
            const int left = p.b_inner - n * BN;
            if (left < BN) {
#pragma unroll
                for (int s = 0; s < PB; s++) offb_now[s] = lb.first < left ? lb.off[s] : OOB_OFFSET;
            }
        }
        // -- the finished tile: rows beyond C are cut off by the descriptor, columns by the lane's offset --
        const unsigned long long pc_at = (unsigned long long)prev_c;
        const int prev_rows_in = prev_rows > BM ? BM : prev_rows;
        const unsigned out_lo = __builtin_amdgcn_readfirstlane((unsigned)pc_at), out_hi = __builtin_amdgcn_readfirstlane((unsigned)(pc_at >> 32));
        const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(((unsigned long long)out_hi << 32) | out_lo), 0,
            __builtin_amdgcn_readfirstlane(prev_rows_in > 0 ? prev_rows_in * ldc4 : 0), RSRC_FLAGS);
        int out_off[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) out_off[j] = c_lane + j * 128;
        if (prev_cols < BN) {
#pragma unroll
            for (int j = 0; j < TN; j++) out_off[j] = (c_col + j * 32 < prev_cols) ? c_lane + j * 128 : OOB_OFFSET;
        }

        static_for<GR>([&](auto gc) {
            constexpr int g = decltype(gc)::value;
            static_for<NM>([&](auto mc) {
                constexpr int mm = decltype(mc)::value;
                constexpr int slot = g * NM + mm;
                constexpr int q = mm / TN, j = mm % TN;
                if constexpr (g == 0 && q == 0)   // a tile's first MFMA per block starts from zero
                    acc[P][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[g & 1][q], fb[g & 1][j][q], (v16f)(0.0f), 0, 0, 0);
                else
                    acc[P][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[g & 1][q], fb[g & 1][j][q], acc[P][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                // the fragments of the next group, behind this group's first MFMA
                if constexpr (mm == 0 && g + 1 < GR)
                    read_group(std::integral_constant<int, (g + 1) & 1>{}, std::integral_constant<int, (g + 1 < GR ? g + 1 : 0)>{}, pc);
                if constexpr (slot == SLOT_A) {
                    if (new_band) {
                        const v4u ra = a_descriptor();
                        issue_a(ra);
                    }
                }
                if constexpr (slot >= SLOT_B && slot < SLOT_B + PB)
                    dma_f4_lean<(P ^ 1) * B_BYTES + (slot - SLOT_B) * NT * 16>(rb, lds_wave_b, offb_now[slot - SLOT_B]);
                if constexpr (slot >= SLOT_STORE && (slot - SLOT_STORE) % STORE_EVERY == 0 && (slot - SLOT_STORE) / STORE_EVERY < 16) {
                    // element e of both blocks: row 8 * (e / 4) + e % 4 below the lane's first, in the scalar offset
                    constexpr int e = (slot - SLOT_STORE) / STORE_EVERY;
                    const int row_off = (8 * (e / 4) + e % 4) * ldc4;
#pragma unroll
                    for (int jj = 0; jj < TN; jj++) {
                        const float value = acc[P ^ 1][jj][e];
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), out_rsrc, out_off[jj],
                                                              row_off, BD_STORE_AUX);
                    }
                }
                if constexpr (slot == SLOT_SYNC) {
                    // Every fragment of this tile is in registers.  The transfers of the next tile are older
                    // than every store of this one, and vector-memory operations retire in issue order: once
                    // at most this tile's stores are outstanding, the transfers have landed.  The barrier then
                    // makes every wavefront's part visible, and tells that nobody reads this tile's B (and, at
                    // the end of a band, its A) any more.
                    __builtin_amdgcn_s_waitcnt(waitcnt_vm(NSTORE));
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                }
                if constexpr (slot == SLOT_SYNC + 1) {
                    if (new_band) {   // the next band's A lies in the other buffer: the read addresses move there
                        if constexpr (A_KIN) {
#pragma unroll
                            for (int gg = 0; gg < GR; gg++) a_rd[gg] ^= A_BYTES;
                        } else {
                            a_rd[0] ^= A_BYTES;
                        }
                        lds_wave_a ^= A_BYTES;
                    }
                    read_group(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, P ^ 1>{});
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        prev_c = cur_c; prev_rows = cur_rows; prev_cols = cur_cols;
        cur_c = p.C + (size_t)z * p.sC + (size_t)m * BM * p.ldc + (size_t)n * BN;
        cur_rows = p.rows - m * BM; cur_cols = p.cols - n * BN;
    };

    // the last tile leaves in one go
    auto last_out = [&](auto pc) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value;
        const unsigned long long pc_at = (unsigned long long)prev_c;
        const int rows_in = prev_rows > BM ? BM : prev_rows;
        const unsigned out_lo = __builtin_amdgcn_readfirstlane((unsigned)pc_at), out_hi = __builtin_amdgcn_readfirstlane((unsigned)(pc_at >> 32));
        const __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(((unsigned long long)out_hi << 32) | out_lo), 0,
            __builtin_amdgcn_readfirstlane(rows_in > 0 ? rows_in * ldc4 : 0), RSRC_FLAGS);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int off = (c_col + j * 32 < prev_cols) ? c_lane + j * 128 : OOB_OFFSET;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const float value = acc[P][j][e];
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), out_rsrc, off,
                                                      (8 * (e / 4) + e % 4) * ldc4, BD_STORE_AUX);
            }
        }
    };
    for (;;) {
        tile(std::integral_constant<int, 0>{});
        if (!has_next) {
            last_out(std::integral_constant<int, 0>{});
            break;
        }
        tile(std::integral_constant<int, 1>{});
        if (!has_next) {
            last_out(std::integral_constant<int, 1>{});
            break;
        }
    }
}

// ---- the band's rows of A in registers ----
// With K <= 64 a wavefront's share of A -- 64 rows x 64 k -- is 64 floats a lane: it is read from memory once per
// band straight into registers (lane half h takes the k of [32h, 32h + 32), so a lane's floats of a row are
// contiguous) and stays there while the workgroup walks the band's column tiles.  LDS then holds only the two
// B tiles (64 KiB), a workgroup is four wavefronts of 64 x 64 (half the LDS reads per MFMA of the 32 x 64 share
// above) with about 170 registers, and TWO workgroups fit a compute unit: while one waits at its barrier, reads
// its fragments or loads a band, the other one's MFMAs keep the pipes busy.  A tile is multiplied block after
// block (32 x 32 outputs, the whole K: 32 MFMAs in a row into one accumulator): a finished block's 16 stores go
// out between the MFMAs of the next block, so one accumulator set is enough and the write path sees an even
// stream; a lane's B values of a column block (32 floats) are read from LDS as the values before them have had
// their last use.
template <bool A_KIN, bool B_KIN>
__global__ __launch_bounds__(256, 2)
void gemm_f32_mfma_band_regs(const GemmParams p) {
    constexpr int NT = 256, BM = 128, BN = 128, KT = BD_KT, TM = 2, TN = 2;
    constexpr int GR = KT / 8;                 // groups of 4 k steps (a step = one MFMA's two k: s and 32 + s)
    using LanesB = BandLanes<B_KIN, BN, KT, NT>;
    constexpr int PB = LanesB::PASSES, B_BYTES = BN * KT * 4;
    __shared__ __attribute__((aligned(16))) float smemB[2 * BN * KT];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;
    const int k_a = min(p.k_total, A_KIN ? p.a_inner : p.a_outer), k_b = min(p.k_total, B_KIN ? p.b_inner : p.b_outer);

    LanesB lb;
    lb.init(t, p.ldb, k_b);
    const unsigned lds_b0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smemB;
    const unsigned lds_wave_b = lds_b0 + wave * 1024;

    // B fragments of step group g (steps 4g .. 4g + 3: k = 32h + 4g + q): K-inner logical chunk 8h + g of the lane's
    // column; K-outer k row 32h + 4g + q, the lane's column.  Block j is 32 columns on.
    unsigned b_rd[B_KIN ? GR : 1];
    if constexpr (B_KIN) {
#pragma unroll
        for (int g = 0; g < GR; g++) b_rd[g] = pinned(lds_b0 + ((wn * 64 + r) * KT + ((8 * h + g) ^ kin_swizzle<KT>(r)) * 4) * 4);
    } else {
        b_rd[0] = pinned(lds_b0 + (32 * h * BN + wn * 64 + r) * 4);
    }
    // the lane's B values of one 32-column block for the whole K: fb[s] = B(k = 32 h + s, the lane's column)
    float fb[32];
    // steps 4g .. 4g + 3 of block j from B buffer PB_
    auto read_group = [&](auto g_c, auto j_c, auto pb_c) __attribute__((always_inline)) {
        constexpr int g = decltype(g_c)::value, j = decltype(j_c)::value, PB_ = decltype(pb_c)::value;
        if constexpr (B_KIN) {
            const v4f v = *(lds_v4f)(b_rd[g] + PB_ * B_BYTES + j * 32 * KT * 4);
            fb[4 * g] = v.x; fb[4 * g + 1] = v.y; fb[4 * g + 2] = v.z; fb[4 * g + 3] = v.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fb[4 * g + q] = *(lds_f32)(b_rd[0] + PB_ * B_BYTES + ((4 * g + q) * BN + j * 32) * 4);
        }
    };

    const int ldc4 = p.ldc * 4;
    const int c_lane = (int)pinned((unsigned)((wm * 64 + 4 * h) * ldc4 + (wn * 64 + r) * 4));
    const int c_col = wn * 64 + r;

    const int G = gridDim.x;
    const int U = p.nz * p.tiles_m * p.bd_chunks;
    int u = xcd_contiguous_id(blockIdx.x, G);   // G <= U
    int z, m, n, n_end;
    auto decode_unit = [&](int unit) __attribute__((always_inline)) {
        const int per_z = p.tiles_m * p.bd_chunks;
        z = __builtin_amdgcn_readfirstlane(unit / per_z);
        const int rem = unit - z * per_z;
        m = __builtin_amdgcn_readfirstlane(rem / p.bd_chunks);
        n = (rem - m * p.bd_chunks) * p.bd_chunk_tiles;
        n_end = min(n + p.bd_chunk_tiles, p.tiles_n);
    };
    auto b_descriptor = [&](bool live) __attribute__((always_inline)) {
        const float* base = p.B + (size_t)z * p.sB + (B_KIN ? (size_t)n * BN * p.ldb : (size_t)n * BN);
        return band_descriptor<B_KIN>(base, live ? (B_KIN ? p.b_outer : p.b_inner) - n * BN : 0, BN, p.ldb);
    };

    // ---- the band's A: a[i][s] = A(row 64 wm + 32 i + r of the band, k = 32 h + s); zero beyond the operand ----
    float a[TM][32];
    auto load_a = [&]() __attribute__((always_inline)) {
        if constexpr (A_KIN) {
            const int rows_left = p.a_outer - m * BM;
            const float* base = p.A + (size_t)z * p.sA + (size_t)m * BM * p.lda;
            const int rows = rows_left > BM ? BM : rows_left;
            const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, rows > 0 ? rows * p.lda * 4 : 0, RSRC_FLAGS);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int c = 0; c < 8; c++) {
                    const int k = 32 * h + 4 * c;
                    const int off = k < k_a ? ((wm * 64 + 32 * i + r) * p.lda + k) * 4 : OOB_OFFSET;
                    const v4f v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(ra, off, 0, 0));
                    a[i][4 * c] = v.x; a[i][4 * c + 1] = v.y; a[i][4 * c + 2] = v.z; a[i][4 * c + 3] = v.w;
                }
        } else {
            const float* base = p.A + (size_t)z * p.sA + (size_t)m * BM;
            const int cols_left = p.a_inner - m * BM;
            const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, RSRC_RECORDS, RSRC_FLAGS);
#pragma unroll
            for (int i = 0; i < TM; i++) {
                const int col = wm * 64 + 32 * i + r;
#pragma unroll
                for (int s2 = 0; s2 < 32; s2++) {
                    const int k = 32 * h + s2;     // differs between the lane halves: it travels in the lanes' offset
                    const int off = (col < cols_left && k < k_a) ? (k * p.lda + col) * 4 : OOB_OFFSET;
                    a[i][s2] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ra, off, 0, 0));
                }
            }
        }
    };
    auto issue_b = [&](auto pc, const v4u& rb) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value;
        const int left = p.b_inner - n * BN;
        static_for<PB>([&](auto ic) {
            constexpr int s2 = decltype(ic)::value;
            dma_f4_lean<P * B_BYTES + s2 * NT * 16>(rb, lds_wave_b, (B_KIN || lb.first < left) ? lb.off[s2] : OOB_OFFSET);
        });
    };

    v16f acc[TM][TN];

    // ---- prologue ----
    decode_unit(u);
    load_a();
    issue_b(std::integral_constant<int, 0>{}, b_descriptor(true));
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    static_for<GR>([&](auto gc) { read_group(gc, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}); });
    bool has_next = true;
    // the block on its way out: the descriptor of its tile (no rows before the first tile: every store is dropped)
    __amdgpu_buffer_rsrc_t out_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.C, 0, 0, RSRC_FLAGS);
    int out_off[TN] = {OOB_OFFSET, OOB_OFFSET};

    // 16 stores of block (I, J), one behind every second MFMA of the block that follows it
    auto store_e = [&](auto ic, auto jc, auto ec) __attribute__((always_inline)) {
        constexpr int I = decltype(ic)::value, J = decltype(jc)::value, e = decltype(ec)::value;
        const float value = acc[I][J][e];
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), out_rsrc, out_off[J],
                                              (32 * I + 8 * (e / 4) + e % 4) * ldc4, BD_STORE_AUX);
    };
    // One block: 32 dependent MFMAs into acc[I][J] from a[I] and fb, with the stores of block (SI, SJ) between them
    // and, where NEXT_J >= 0, fb's next contents read group by group as the values there have had their last use
    // (block NEXT_J of B buffer NEXT_P).
    auto block = [&](auto ic, auto jc, auto sic, auto sjc, auto njc, auto npc) __attribute__((always_inline)) {
        constexpr int I = decltype(ic)::value, J = decltype(jc)::value;
        constexpr int NEXT_J = decltype(njc)::value;
        static_for<32>([&](auto sc) {
            constexpr int s2 = decltype(sc)::value;
            if constexpr (s2 == 0)
                acc[I][J] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[I][s2], fb[s2], (v16f)(0.0f), 0, 0, 0);
            else
                acc[I][J] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[I][s2], fb[s2], acc[I][J], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (s2 % 2 == 1) store_e(sic, sjc, std::integral_constant<int, s2 / 2>{});
            if constexpr (NEXT_J >= 0 && s2 % 4 == 3)
                read_group(std::integral_constant<int, s2 / 4>{}, std::integral_constant<int, (NEXT_J >= 0 ? NEXT_J : 0)>{}, npc);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using CN = std::integral_constant<int, -1>;

    // One tile from B buffer P, block after block: (0,0) (1,0) (0,1) (1,1).
    auto tile = [&](auto pc) __attribute__((always_inline)) {
        constexpr int P = decltype(pc)::value;
        float* const cur_c = p.C + (size_t)z * p.sC + (size_t)m * BM * p.ldc + (size_t)n * BN;
        const int cur_rows = p.rows - m * BM, cur_cols = p.cols - n * BN;
        // -- the tile after this one: its B goes to the other buffer now --
        bool new_band = false;
        if (++n == n_end) {
            u += G;
            if (u < U) {
                decode_unit(u);
                new_band = true;
            } else {
                has_next = false;
                n = 0;
            }
        }
        issue_b(std::integral_constant<int, P ^ 1>{}, b_descriptor(has_next));
        __builtin_amdgcn_sched_barrier(0);

        // block (0,0), with the last block of the tile before on its way out
        block(C0{}, C0{}, C1{}, C1{}, CN{}, C0{});
        // from here on the stores are this tile's: rows beyond C are cut off by the descriptor, columns by the offsets
        {
            const unsigned long long pc_at = (unsigned long long)cur_c;
            const int rows_in = cur_rows > BM ? BM : cur_rows;
            const unsigned out_lo = __builtin_amdgcn_readfirstlane((unsigned)pc_at), out_hi = __builtin_amdgcn_readfirstlane((unsigned)(pc_at >> 32));
            out_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(((unsigned long long)out_hi << 32) | out_lo), 0,
                                                         __builtin_amdgcn_readfirstlane(rows_in > 0 ? rows_in * ldc4 : 0), RSRC_FLAGS);
#pragma unroll
            for (int j = 0; j < TN; j++) out_off[j] = (c_col + j * 32 < cur_cols) ? c_lane + j * 128 : OOB_OFFSET;
        }
        // block (1,0): fb's values have their last use for column block 0; block 1's come in behind them
        block(C1{}, C0{}, C0{}, C0{}, C1{}, pc);
        block(C0{}, C1{}, C1{}, C0{}, CN{}, C0{});
        // The next tile's B was requested before this tile's 48 stores so far, and vector-memory operations retire
        // in issue order: with at most those outstanding it has landed.  The barrier makes every wavefront's part
        // visible; everybody has read the last of this tile's B (block 1's values) before its block (0,1) ended.
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(48));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // block (1,1): the next tile's column block 0 comes in behind fb's last uses
        block(C1{}, C1{}, C0{}, C1{}, C0{}, std::integral_constant<int, P ^ 1>{});
        // the next band's A replaces this one's (every MFMA that read it has been issued)
        if (new_band) {
            load_a();
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    for (;;) {
        tile(std::integral_constant<int, 0>{});
        if (!has_next) break;
        tile(std::integral_constant<int, 1>{});
        if (!has_next) break;
    }
    // the last block of the last tile
    static_for<16>([&](auto ec) { store_e(C1{}, C1{}, ec); });
}

template <bool A_KIN, bool B_KIN>
static hipError_t launch_band_regs_cfg(GemmParams p, hipStream_t stream) {
    if (p.split || p.bias != nullptr || p.k_total > BD_KT) return hipErrorOutOfMemory;   // the caller falls back
    p.tiles_m = (p.rows + 127) / 128;
    p.tiles_n = (p.cols + 127) / 128;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const long long bands = (long long)p.tiles_m * p.nz;
    if (bands <= 0 || bands * p.tiles_n > 0x3fffffffLL) return hipErrorOutOfMemory;
    gemm_band_split(bands, p.tiles_n, 2 * num_cu, p.bd_chunks, p.bd_chunk_tiles);    // two workgroups per unit
    const long long units = bands * p.bd_chunks;
    const long long grid = units < 2LL * num_cu ? units : 2LL * num_cu;
    hipLaunchKernelGGL((gemm_f32_mfma_band_regs<A_KIN, B_KIN>), dim3((unsigned)grid), dim3(256), 0, stream, p);
    return hipGetLastError();
}

template <bool A_KIN, bool B_KIN, int BD_BM, int BD_BN>
static hipError_t launch_band_cfg(GemmParams p, hipStream_t stream) {
    if (p.split || p.bias != nullptr || p.k_total > BD_KT) return hipErrorOutOfMemory;   // the caller falls back
    p.tiles_m = (p.rows + BD_BM - 1) / BD_BM;
    p.tiles_n = (p.cols + BD_BN - 1) / BD_BN;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const long long bands = (long long)p.tiles_m * p.nz;
    if (bands <= 0 || bands * p.tiles_n > 0x3fffffffLL) return hipErrorOutOfMemory;
    gemm_band_split(bands, p.tiles_n, num_cu, p.bd_chunks, p.bd_chunk_tiles);
    const long long units = bands * p.bd_chunks;
    const long long grid = units < num_cu ? units : num_cu;
    hipLaunchKernelGGL((gemm_f32_mfma_band<A_KIN, B_KIN, BD_BM, BD_BN>), dim3((unsigned)grid), dim3(BD_THREADS), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

// A band's column tiles are dealt to `chunks` workgroups in runs of `chunk_tiles`: one run per band when
// the bands alone fill the compute units evenly, more where that leaves units idle in the last round.
void gemm_band_split(long long bands, int tiles_n, int num_cu, int& chunks, int& chunk_tiles) {
    chunks = 1;
    chunk_tiles = tiles_n;
    double best = 1e300;
    for (int c = 1; c <= 8 && c <= tiles_n; c *= 2) {
        const int ct = (tiles_n + c - 1) / c;
        const int real = (tiles_n + ct - 1) / ct;              // runs that are not empty
        const long long units = bands * real;
        const long long g = units < num_cu ? units : num_cu;
        const long long rounds = (units + g - 1) / g;
        // the busiest workgroup's tiles; every run pays about half a tile's time for its band of A
        const double cost = (double)rounds * (ct + 0.5);
        if (cost < best * 0.98) { best = cost; chunks = real; chunk_tiles = ct; }
    }
}

// The band kernel's shapes, from measurements against the tile-per-workgroup kernels on batches of
// 256 ... 2048 x 256 ... 2048 and single products up to 8192 x 8192: with K = 57 ... 64 it is level or ahead
// (5-15 % on most) from two tiles per compute unit on; a K of 48 or less leaves its one stage of 64 k too
// empty; rows of C that do not start on 128-byte lines split its 128-byte store runs.
int gemm_choose_band(int rows, int cols, int nz, int k, int num_cu, int variant) {
    if (rows <= 0 || cols <= 0 || nz <= 0 || k <= 0 || num_cu <= 0) return -1;
    if (k > BD_KT || k <= BD_KT - 8) return -1;
    if (cols % 32 != 0) return -1;
    constexpr int BD_BM = 128, BD_BN = 128;
    const long long tiles_m = (rows + BD_BM - 1) / BD_BM, tiles_n = (cols + BD_BN - 1) / BD_BN;
    if (tiles_n < 2 || tiles_m * nz * tiles_n < 2LL * num_cu) return -1;
    // rows and columns that fill their tiles: the padded part of a ragged C is multiplied too
    if ((double)rows * cols < 0.85 * (double)(tiles_m * BD_BM) * (double)(tiles_n * BD_BN)) return -1;
    return TILE_BAND_128x128;
}

hipError_t gemm_launch_band(int variant, const GemmParams& p, hipStream_t stream, bool wide, bool regs) {
    if (regs) {
        switch (variant) {
            case GEMM_NN: return launch_band_regs_cfg<true, false>(p, stream);
            case GEMM_T1: return launch_band_regs_cfg<false, false>(p, stream);
            case GEMM_T2: return launch_band_regs_cfg<true, true>(p, stream);
            default: return hipErrorInvalidValue;
        }
    }
    if (wide) {
        switch (variant) {
            case GEMM_NN: return launch_band_cfg<true, false, 64, 256>(p, stream);
            case GEMM_T1: return launch_band_cfg<false, false, 64, 256>(p, stream);
            case GEMM_T2: return launch_band_cfg<true, true, 64, 256>(p, stream);
            default: return hipErrorInvalidValue;
        }
    }
    switch (variant) {
        case GEMM_NN: return launch_band_cfg<true, false, 128, 128>(p, stream);
        case GEMM_T1: return launch_band_cfg<false, false, 128, 128>(p, stream);
        case GEMM_T2: return launch_band_cfg<true, true, 128, 128>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace dragon
