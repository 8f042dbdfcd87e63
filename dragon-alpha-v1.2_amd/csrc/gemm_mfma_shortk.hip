// The products with a K of 89 ... 144 and a RAGGED C, batch after batch: 257 x 385 outputs of 129 products each
// (the reference's kernels for these are the padded and texture forms with a ceil-div grid,
// BMM/batchMatMul_kernel_padding.cuh:20-42, BMM/batchMatMulT2_kernel_padding.cuh:23-45, and the carving of C's
// edges down to tiles of 4, MM/matMul.cuh:24-43).
//
// Such a product is a few thousand 32 x 32 blocks of ~65 MFMAs each: 3 to 4 of them per SIMD of the chip, done in
// a handful of microseconds.  What a kernel spends beside the MFMAs decides its time:
//   * the whole K of a tile is resident.  A tile's operands go global -> LDS in one piece (nine panels of 16 k,
//     each in the layout of the 16-k stages of gemm_mfma_kernel.h), while the tile before is multiplied: one
//     barrier per tile, no stage pipeline to fill and drain per tile;
//   * one persistent workgroup per compute unit walks a run of the tiles (tiles of several batches), the runs
//     of equal cost; the finished tile is stored between the MFMAs of the next one (as in gemm_mfma_band.hip);
//   * every lane's part of the transfers, of the fragment reads and of the stores is worked out once per launch;
//     per tile the scalar unit moves descriptors along (a piece behind each of the tile's first MFMAs), the
//     vector ALU has next to nothing to do;
//   * the rim.  A C that is 1 ... 4 rows and / or columns past a multiple of 64 (257 x 388) would cost a whole
//     extra row and column of tiles (35 instead of 24).  The tiles cover the multiple; the workgroup that has a
//     tile of the last tile row (column) in LDS also fetches the few rim rows of A (columns of B) and computes
//     the strip of C below (beside) its tile with v_mfma_f32_4x4x1_16B_f32: sixteen independent 4 x 4 x 1
//     products per instruction -- four groups of 4 outputs across times four different k -- so a wavefront
//     covers 16 outputs along the strip x 4 across with no padded work, adds its four k classes with two lane
//     exchanges and stores; nothing meets in LDS and no extra barrier is needed.
// Measured on MI355X (cycle counters read inside the kernel, batch 36 of 257 x 388 x 129): a workgroup takes
// 5300 cycles before and after its tiles (4300 of them until the first tile's operands are in LDS), 5500 per
// tile (68 MFMAs: 4350 at the pipe's rate) and 1550 per strip.
// The sum of an output element runs k-ascending within each lane half like in the other kernels (same bits as
// theirs on the tiles); a strip's element is the sum of four interleaved k classes, inside the same error bound.
#include "gemm_mfma_kernel.h"

namespace dragon {
namespace {

constexpr int SHK_PANELS = 9;                       // panels of 16 k: K <= 144
constexpr int SHK_PANEL_BYTES = 4096;               // 64 rows (or columns) x 16 k floats
constexpr int SHK_TILE_FLOATS = SHK_PANELS * 1024;  // one operand of one tile
constexpr int SHK_TILE_BYTES = SHK_TILE_FLOATS * 4;
constexpr int SHK_RIM_FLOATS = 768;                 // 4 rim lines x up to 192 k
constexpr int SHK_RIM_BYTES = SHK_RIM_FLOATS * 4;
constexpr int SHK_MAX_K = SHK_PANELS * 16;
constexpr int SHK_STRIP_COST = 3;                   // what a strip of the rim costs, a tile being 10 (measured)
constexpr int SHK_STORE_AUX = 2;                    // streaming stores: C is not read back here

#pragma clang diagnostic ignored "-Wint-to-pointer-cast"
typedef __attribute__((address_space(3))) const float* shk_lds_f32;
typedef __attribute__((address_space(3))) const v4f* shk_lds_v4f;

__device__ __forceinline__ unsigned shk_pinned(unsigned v) {
    asm volatile("" : "+v"(v));
    return v;
}

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// 16 bytes per lane, global -> LDS, with a wave-uniform byte offset on top of the lane's (the hardware checks
// their sum against the descriptor's size).  lds = wave's LDS base + LDS_IMM.
template <int LDS_IMM>
__device__ __forceinline__ void shk_dma(v4u rsrc, unsigned lds_wave_base, int lane_offset, int wave_offset) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %4 offen lds"
                 :
                 : "s"(lds_wave_base), "v"(lane_offset), "s"(rsrc), "n"(LDS_IMM), "s"(wave_offset)
                 : "memory", "m0", "scc");
}
#pragma clang diagnostic pop

__device__ __forceinline__ v4u shk_descriptor(const float* base, unsigned bytes) {
    const unsigned long long b = (unsigned long long)base;
    const v4u rsrc = {(unsigned)__builtin_amdgcn_readfirstlane((unsigned)b),
                      (unsigned)__builtin_amdgcn_readfirstlane((unsigned)(b >> 32) & 0xffffu),
                      (unsigned)__builtin_amdgcn_readfirstlane(bytes), (unsigned)RSRC_FLAGS};
    return rsrc;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t shk_out_descriptor(float* base, int bytes) {
    const unsigned long long at = (unsigned long long)base;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)at), hi = __builtin_amdgcn_readfirstlane((unsigned)(at >> 32));
    return __builtin_amdgcn_make_buffer_rsrc((void*)(((unsigned long long)hi << 32) | lo), 0,
                                             __builtin_amdgcn_readfirstlane(bytes > 0 ? bytes : 0), RSRC_FLAGS);
}

// One job of a workgroup: a tile of C, and which strips of the rim hang on it.
struct ShkJob {
    int z, m, n;            // batch, tile row, tile column
    const float* a_z;       // the batch's operands and result
    const float* b_z;
    float* c_z;
    bool row_strip;         // the tile lies in the last tile row and C has rim rows
    bool col_strip;         // the tile lies in the last tile column and C has rim columns
};

// MINB: the first MINB groups of 8 k exist in every tile this instantiation runs (K > 8 * MINB), so that the
// side work placed between their MFMAs -- the next tile's transfers, the last tile's stores -- needs no test.
template <bool A_KIN, bool B_KIN, int MINB>
__global__ __launch_bounds__(NTHREADS, 1)
void gemm_f32_mfma_shortk(const GemmParams p) {
    constexpr int GMAX = SHK_PANELS * 2;                 // groups of 8 k at most
    constexpr int NBODY = GMAX - 2;                      // groups before the last two
    constexpr int SLOTS = 4 * MINB;                      // MFMA slots that always exist
    constexpr int NXFER = 2 * SHK_PANELS + 2;            // transfers per tile: panels of A and B, the two rim panels
    // what stands behind which of a tile's first MFMAs: the next tile's place and descriptors (scalar work, a
    // piece per slot so that no MFMA waits for it), its transfers, the last tile's stores
    constexpr int SLOT_XFER = 6, SLOT_STORE = SLOT_XFER + NXFER;   // the stores two to a slot
    static_assert(SLOT_STORE + 8 <= SLOTS, "transfers and stores fit between the MFMAs that always exist");

    __shared__ __attribute__((aligned(16))) float smA[2 * SHK_TILE_FLOATS];
    __shared__ __attribute__((aligned(16))) float smB[2 * SHK_TILE_FLOATS];
    __shared__ __attribute__((aligned(16))) float smRA[2 * SHK_RIM_FLOATS];
    __shared__ __attribute__((aligned(16))) float smRB[2 * SHK_RIM_FLOATS];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- the shape: the same for every tile ----
    const int klimA = min(p.k_total, A_KIN ? p.a_inner : p.a_outer);
    const int klimB = min(p.k_total, B_KIN ? p.b_inner : p.b_outer);
    const int K = min(klimA, klimB);                     // 8 * (MINB + 1) < K <= 144, checked by the launcher
    const int ng = (K + 7) >> 3;                         // groups of 8 k
    const int tail_steps = min(4, K - 8 * (ng - 1));     // MFMAs of the last group
    // (Where the unrolled code below tests one of these per panel or group, the value goes through fresh(): the
    // test is then made where it stands -- a compare and a branch of the scalar unit -- instead of being worked out
    // for every panel and group ahead of the tile loop and kept in a register pair each, which the scalar
    // registers do not have room for.)
    const int rr = p.rim_rows, rc = p.rim_cols;
    const int R0 = p.rows - rr, C0 = p.cols - rc;        // the tiles' part of C
    const int tm = p.tiles_m, tn = p.tiles_n;

    const unsigned ldsA = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smA;
    const unsigned ldsB = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smB;
    const unsigned ldsRA = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smRA;
    const unsigned ldsRB = (unsigned)(unsigned long long)(__attribute__((address_space(3))) float*)smRB;
    const unsigned lds_waveA = ldsA + wave * 1024, lds_waveB = ldsB + wave * 1024;
    const unsigned lds_waveRA = ldsRA + wave * 1024, lds_waveRB = ldsRB + wave * 1024;

    // ---- the lanes' part of the transfers: one byte offset per panel, from the tile's origin ----
    // K-inner panel [64 rows][16 k], chunks swizzled: wave w fills rows 16w .. 16w+15, lane l the slot l & 3 of row
    // 16w + l / 4 with logical chunk slot ^ swizzle(row).  K-outer panel [16 k][64]: wave w fills k rows 4w .. 4w+3.
    // A chunk or k row at or beyond the operand's K is out of range (the transfer writes zeros) -- K is the same
    // for every tile, so the offsets never change.  Rows (K-inner) beyond the operand's last lie beyond the
    // descriptor's end; a K-outer operand's columns beyond its row length belong to outputs that are not stored.
    // (Worked out in the prologue, panel by panel between the first tile's transfers.)
    int offA[SHK_PANELS], offB[SHK_PANELS];
    auto panel_lanes = [&](bool kin, int ld, int klim, int pn) __attribute__((always_inline)) -> int {
        if (kin) {
            const int row = 16 * wave + (lane >> 2), c = (lane & 3) ^ kin_swizzle<16>(row);
            return (16 * pn + 4 * c < klim) ? (row * ld + 16 * pn + c * 4) * 4 : OOB_OFFSET;
        }
        const int k = 16 * pn + 4 * wave + (lane >> 4);
        return (k < klim) ? (k * ld + (lane & 15) * 4) * 4 : OOB_OFFSET;
    };
    // rim panels.  K-inner lines [4 lines][k]: wave u < 3 fetches k 64u .. 64u+63 of the four lines, lane l chunk
    // l & 15 of line l / 16; K-outer [k][4 lines]: lane l of wave u fetches the 16 bytes of k row 64u + l.
    auto rim_lanes = [&](bool kin, int ld, int klim) -> int {
        if (wave >= 3) return OOB_OFFSET;
        if (kin) {
            const int k = 64 * wave + (lane & 15) * 4;
            return k < klim ? ((lane >> 4) * ld + k) * 4 : OOB_OFFSET;
        }
        return (64 * wave + lane) * ld * 4;          // rows beyond K lie beyond the descriptor's end
    };
    const int offRA = rim_lanes(A_KIN, p.lda, klimA), offRB = rim_lanes(B_KIN, p.ldb, klimB);

    // ---- the workgroup's share of the tiles: tiles numbered (batch, tile row, tile column), dealt in runs of
    // equal COST -- a tile counts 10, each strip that hangs on it 3 (a tile with both also computes the corner:
    // 3 more), as measured: the workgroups that get the last tile row and column of a batch get fewer tiles.
    // Workgroup w starts at the first tile whose middle lies at or behind w's share of the cost (a tile goes to the
    // workgroup that most of it falls to).  The launcher made the divisors' multiply-and-shift pairs. ----
    const int G = gridDim.x;
    const int wg = xcd_contiguous_id(blockIdx.x, G);
    const int cost_r = rr > 0 ? SHK_STRIP_COST : 0, cost_c = rc > 0 ? SHK_STRIP_COST : 0, cost_x = (rr > 0 && rc > 0) ? SHK_STRIP_COST : 0;
    const int row_plain = 10 * tn + cost_c, row_last = (10 + cost_r) * tn + cost_c + cost_x;
    const int batch_cost = (tm - 1) * row_plain + row_last;              // p.sk_S, as the launcher has it
    const int cost_q = p.sk_q, cost_rem = p.sk_rem;                      // the cost of all tiles over G, and the rest
    // the first tile whose cost prefix (the cost of every tile before it) reaches `target`, as (z, m, n)
    auto tile_at = [&](int target, int& z, int& m, int& n) {
        z = div_by(target, p.div_tiles_mul, p.div_tiles_shift);          // / batch_cost
        int rest = target - z * batch_cost;
        bool last = true;
        m = tm - 1;
        if (rest < (tm - 1) * row_plain) {
            m = div_by(rest, p.div_band_mul, p.div_band_shift);          // / row_plain
            rest -= m * row_plain;
            last = false;
        } else {
            rest -= (tm - 1) * row_plain;
        }
        n = (last && rr > 0) ? (rest + 9 + SHK_STRIP_COST) / (10 + SHK_STRIP_COST) : (rest + 9) / 10;
        if (n >= tn) {
            n = 0;
            if (++m == tm) { m = 0; z++; }
        }
    };
    int z0, m0, n0, z1, m1, n1;
    tile_at(max(wg * cost_q + min(wg, cost_rem) - 5, 0), z0, m0, n0);
    tile_at((wg + 1) * cost_q + min(wg + 1, cost_rem) - 5, z1, m1, n1);
    int left = __builtin_amdgcn_readfirstlane(((z1 * tm + m1) * tn + n1) - ((z0 * tm + m0) * tn + n0));
    if (left <= 0) return;   // a run that no tile starts in (possible only where tiles are about as many as workgroups)

    ShkJob cur, nxt;
    cur.z = __builtin_amdgcn_readfirstlane(z0);
    cur.m = __builtin_amdgcn_readfirstlane(m0);
    cur.n = __builtin_amdgcn_readfirstlane(n0);
    cur.row_strip = rr > 0 && cur.m == tm - 1;
    cur.col_strip = rc > 0 && cur.n == tn - 1;
    cur.a_z = p.A + (size_t)cur.z * p.sA;
    cur.b_z = p.B + (size_t)cur.z * p.sB;
    cur.c_z = p.C + (size_t)cur.z * p.sC;
    auto advance = [&](const ShkJob& j) __attribute__((always_inline)) -> ShkJob {
        ShkJob o = j;
        if (++o.n == tn) {
            o.n = 0;
            if (++o.m == tm) {
                o.m = 0;
                o.z++;
                o.a_z += p.sA; o.b_z += p.sB; o.c_z += p.sC;
            }
        }
        o.row_strip = rr > 0 && o.m == tm - 1;
        o.col_strip = rc > 0 && o.n == tn - 1;
        return o;
    };

    // Descriptors of a job's operand tiles, based at the tile's origin.  K-inner (a row of the tile per row of the
    // matrix): the size ends behind the last row that exists, the hardware zeroes the rows beyond.  K-outer: the
    // size ends in the operand's last k row, behind the last column the operand has in this tile (a column beyond
    // it in an earlier k row is the next row's data: it only reaches outputs that are not stored).
    // live == false: every lane out of range.
    const unsigned a_pitch = (unsigned)p.lda * 4u, b_pitch = (unsigned)p.ldb * 4u;
    auto a_desc = [&](const ShkJob& j, bool live) __attribute__((always_inline)) {
        const float* base = j.a_z + (A_KIN ? (size_t)(j.m * 64) * p.lda : (size_t)(j.m * 64));
        const int lines = min((A_KIN ? p.a_outer : p.a_inner) - j.m * 64, 64);
        const unsigned bytes = A_KIN ? (unsigned)lines * a_pitch : (unsigned)(klimA - 1) * a_pitch + (unsigned)lines * 4u;
        return shk_descriptor(base, live && lines > 0 ? bytes : 0u);
    };
    auto b_desc = [&](const ShkJob& j, bool live) __attribute__((always_inline)) {
        const float* base = j.b_z + (B_KIN ? (size_t)(j.n * 64) * p.ldb : (size_t)(j.n * 64));
        const int lines = min((B_KIN ? p.b_outer : p.b_inner) - j.n * 64, 64);
        const unsigned bytes = B_KIN ? (unsigned)lines * b_pitch : (unsigned)(klimB - 1) * b_pitch + (unsigned)lines * 4u;
        return shk_descriptor(base, live && lines > 0 ? bytes : 0u);
    };
    // rim lines: rows R0 .. of A (for the strip below the tiles), columns C0 .. of B (for the strip beside them)
    const int linesRA = min((A_KIN ? p.a_outer : p.a_inner) - R0, 4), linesRB = min((B_KIN ? p.b_outer : p.b_inner) - C0, 4);
    const unsigned bytesRA = linesRA <= 0 ? 0u : A_KIN ? (unsigned)linesRA * a_pitch : (unsigned)(klimA - 1) * a_pitch + 16u;
    const unsigned bytesRB = linesRB <= 0 ? 0u : B_KIN ? (unsigned)linesRB * b_pitch : (unsigned)(klimB - 1) * b_pitch + 16u;
    const size_t atRA = A_KIN ? (size_t)R0 * p.lda : (size_t)R0, atRB = B_KIN ? (size_t)C0 * p.ldb : (size_t)C0;
    auto ra_desc = [&](const ShkJob& j, bool live) __attribute__((always_inline)) { return shk_descriptor(j.a_z + atRA, live ? bytesRA : 0u); };
    auto rb_desc = [&](const ShkJob& j, bool live) __attribute__((always_inline)) { return shk_descriptor(j.b_z + atRB, live ? bytesRB : 0u); };
    // transfer number i of job `j` into buffer BUF: panels of A and B in turns, then the two rim panels
    v4u dA, dB, dRA, dRB;
    auto transfer = [&](auto i_c, auto buf_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value, BUF = decltype(buf_c)::value;
        if constexpr (i < 2 * SHK_PANELS) {
            constexpr int pn = i >> 1;
            if constexpr ((i & 1) == 0) shk_dma<BUF * SHK_TILE_BYTES + pn * SHK_PANEL_BYTES>(dA, lds_waveA, offA[pn], 0);
            else shk_dma<BUF * SHK_TILE_BYTES + pn * SHK_PANEL_BYTES>(dB, lds_waveB, offB[pn], 0);
        } else if constexpr (i == 2 * SHK_PANELS) {   // three wavefronts fill a rim panel of 3 KiB
            if (rr > 0 && wave < 3) shk_dma<BUF * SHK_RIM_BYTES>(dRA, lds_waveRA, offRA, 0);
        } else {
            if (rc > 0 && wave < 3) shk_dma<BUF * SHK_RIM_BYTES>(dRB, lds_waveRB, offRB, 0);
        }
    };

    v16f acc[2];

    // ---- prologue: the first tile's operands; no finished tile yet ----
    dA = a_desc(cur, true);
    dB = b_desc(cur, true);
    dRA = ra_desc(cur, cur.row_strip);
    dRB = rb_desc(cur, cur.col_strip);
    static_for<NXFER>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i < 2 * SHK_PANELS) {
            if constexpr ((i & 1) == 0) offA[i >> 1] = panel_lanes(A_KIN, p.lda, klimA, i >> 1);
            else offB[i >> 1] = panel_lanes(B_KIN, p.ldb, klimB, i >> 1);
        }
        transfer(ic, std::integral_constant<int, 0>{});
        __builtin_amdgcn_sched_barrier(0);
    });
    // (the first tile's operands are on their way; what follows is worked out while they travel)
    __builtin_amdgcn_sched_barrier(0);

    // ---- the lanes' LDS addresses of the fragment reads (buffer 0, panel 0) ----
    // K-inner: row of the wavefront's block, chunk (2 * (g & 1) + h) ^ swizzle; K-outer: k row 4h of an even group,
    // the lane's column; group g is (g >> 1) panels and (g & 1) * 8 k rows on, step q one more row.
    unsigned a_rd0, a_rd1 = 0, b_rd0, b_rd1 = 0;
    if constexpr (A_KIN) {
        a_rd0 = shk_pinned(ldsA + ((wm * 32 + r) * 16 + ((0 + h) ^ kin_swizzle<16>(r)) * 4) * 4);
        a_rd1 = shk_pinned(ldsA + ((wm * 32 + r) * 16 + ((2 + h) ^ kin_swizzle<16>(r)) * 4) * 4);
    } else {
        a_rd0 = shk_pinned(ldsA + (4 * h * 64 + wm * 32 + r) * 4);
    }
    if constexpr (B_KIN) {
        b_rd0 = shk_pinned(ldsB + ((wn * 32 + r) * 16 + ((0 + h) ^ kin_swizzle<16>(r)) * 4) * 4);
        b_rd1 = shk_pinned(ldsB + ((wn * 32 + r) * 16 + ((2 + h) ^ kin_swizzle<16>(r)) * 4) * 4);
    } else {
        b_rd0 = shk_pinned(ldsB + (4 * h * 64 + wn * 32 + r) * 4);
    }
    // fragment sets: F for a tile's first group (read during the tile before), L1 and L2 for its last two (read at
    // the tile's start: their place in LDS depends on K, which the launch fixes, so the lanes keep the addresses),
    // 0 / 1 / 2 in turns between, each read two groups (eight MFMAs) before it is multiplied: with one block per
    // wavefront a group is only four MFMAs long, which does not cover an LDS read.  Which set a read goes to is fixed in the code: a set chosen at run time would be a select per
    // operand register in front of every MFMA.
    float fa[6][4], fb[6][4];
    constexpr int SET_F = 3, SET_L1 = 4, SET_L2 = 5;
    auto read_group = [&](auto set_c, auto g_c, auto buf_c) __attribute__((always_inline)) {
        constexpr int set = decltype(set_c)::value, g = decltype(g_c)::value, buf = decltype(buf_c)::value;
        constexpr int at = buf * SHK_TILE_BYTES + (g >> 1) * SHK_PANEL_BYTES;
        if constexpr (A_KIN) {
            const v4f v = *(shk_lds_v4f)(((g & 1) ? a_rd1 : a_rd0) + at);
            fa[set][0] = v.x; fa[set][1] = v.y; fa[set][2] = v.z; fa[set][3] = v.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fa[set][q] = *(shk_lds_f32)(a_rd0 + at + ((g & 1) * 8 + q) * 256);
        }
        if constexpr (B_KIN) {
            const v4f v = *(shk_lds_v4f)(((g & 1) ? b_rd1 : b_rd0) + at);
            fb[set][0] = v.x; fb[set][1] = v.y; fb[set][2] = v.z; fb[set][3] = v.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fb[set][q] = *(shk_lds_f32)(b_rd0 + at + ((g & 1) * 8 + q) * 256);
        }
    };
    // the last two groups (numbers ng - 2 and ng - 1), buffer 0: read into sets of their own at the tile's start
    auto group_address = [&](bool kin, unsigned rd0, unsigned rd1, int g) -> unsigned {
        return (kin ? ((g & 1) ? rd1 : rd0) : rd0 + (g & 1) * 8 * 256) + (g >> 1) * SHK_PANEL_BYTES;
    };
    const unsigned a_rdl1 = shk_pinned(group_address(A_KIN, a_rd0, a_rd1, ng - 2)), a_rdl2 = shk_pinned(group_address(A_KIN, a_rd0, a_rd1, ng - 1));
    const unsigned b_rdl1 = shk_pinned(group_address(B_KIN, b_rd0, b_rd1, ng - 2)), b_rdl2 = shk_pinned(group_address(B_KIN, b_rd0, b_rd1, ng - 1));
    auto read_at = [&](auto set_c, unsigned a_at, unsigned b_at, auto buf_c) __attribute__((always_inline)) {
        constexpr int set = decltype(set_c)::value, at = decltype(buf_c)::value * SHK_TILE_BYTES;
        if constexpr (A_KIN) {
            const v4f v = *(shk_lds_v4f)(a_at + at);
            fa[set][0] = v.x; fa[set][1] = v.y; fa[set][2] = v.z; fa[set][3] = v.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fa[set][q] = *(shk_lds_f32)(a_at + at + q * 256);
        }
        if constexpr (B_KIN) {
            const v4f v = *(shk_lds_v4f)(b_at + at);
            fb[set][0] = v.x; fb[set][1] = v.y; fb[set][2] = v.z; fb[set][3] = v.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) fb[set][q] = *(shk_lds_f32)(b_at + at + q * 256);
        }
    };

    // ---- the lanes' part of a tile's stores: first row and column of the wavefront's block ----
    const int ldc4 = p.ldc * 4;
    const int c_lane = (int)shk_pinned((unsigned)((wm * 32 + 4 * h) * ldc4 + (wn * 32 + r) * 4));
    const int c_col = wn * 32 + r;

    // ---- the strips' lanes.  Lane l: x = l & 3 (line across the strip), a = (l >> 2) & 3 (group of 4 along it),
    // kk = l >> 4 (k class: k = 16 T + 4 kk + q in panel T).  line = 16 * wave + (l & 15) along the strip. ----
    const int s_line = 16 * wave + (lane & 15), s_x = lane & 3, s_kk = lane >> 4;
    // the tile operand's element (line, 16 T + 4 kk + q): K-inner chunk kk of the line, K-outer k row 4 kk + q
    const unsigned sa_rd = shk_pinned(A_KIN ? ldsA + (s_line * 16 + (s_kk ^ kin_swizzle<16>(s_line)) * 4) * 4 : ldsA + (4 * s_kk * 64 + s_line) * 4);
    const unsigned sb_rd = shk_pinned(B_KIN ? ldsB + (s_line * 16 + (s_kk ^ kin_swizzle<16>(s_line)) * 4) * 4 : ldsB + (4 * s_kk * 64 + s_line) * 4);
    // the rim panel's element (line x, k): K-inner [k / 64][x][k % 64], K-outer [k][x]
    const unsigned ra_rd = shk_pinned(A_KIN ? ldsRA + s_x * 256 + s_kk * 16 : ldsRA + s_x * 4 + s_kk * 64);
    const unsigned rb_rd = shk_pinned(B_KIN ? ldsRB + s_x * 256 + s_kk * 16 : ldsRB + s_x * 4 + s_kk * 64);
    // four values (q = 0 .. 3) of panel T from a tile operand / a rim panel in buffer `buf`
    auto strip_tile4 = [&](float (&v)[4], bool kin_c, unsigned rd, int T, int buf) __attribute__((always_inline)) {
        const unsigned at = rd + buf * SHK_TILE_BYTES + T * SHK_PANEL_BYTES;
        if (kin_c) {
            const v4f w = *(shk_lds_v4f)at;
            v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) v[q] = *(shk_lds_f32)(at + q * 256);
        }
    };
    auto strip_rim4 = [&](float (&v)[4], bool kin_c, unsigned rd, int T, int buf) __attribute__((always_inline)) {
        if (kin_c) {
            const v4f w = *(shk_lds_v4f)(rd + buf * SHK_RIM_BYTES + (T >> 2) * 1024 + (T & 3) * 64);
            v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w;
        } else {
#pragma unroll
            for (int q = 0; q < 4; q++) v[q] = *(shk_lds_f32)(rd + buf * SHK_RIM_BYTES + T * 256 + q * 16);
        }
    };
    // the four k classes of a strip's sums meet: lanes l, l ^ 16, l ^ 32, l ^ 48 hold the same outputs
    auto meet = [&](v4f& d) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            d[i] += __shfl_xor(d[i], 16);
            d[i] += __shfl_xor(d[i], 32);
        }
    };

    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_group(std::integral_constant<int, SET_F>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});

    float* prev_c = p.C;
    int prev_rows = 0, prev_cols = 0;                    // no rows: every store is dropped
    bool has_next = true;

    // A strip of 4 x 4 blocks: every panel's operand values first (those beyond K too: they hold zeros), then the
    // MFMAs in one go, into two sums in turns so that none waits for the one before it.
    // KIND 0: the tile's rows x the rim's columns; 1: the rim's rows x the tile's columns; 2: the corner.
    auto strip = [&](auto kind_c, auto buf_c) __attribute__((always_inline)) -> v4f {
        constexpr int KIND = decltype(kind_c)::value, BUF = decltype(buf_c)::value;
        float va[SHK_PANELS][4], vb[SHK_PANELS][4];
#pragma unroll
        for (int T = 0; T < SHK_PANELS; T++) {
            if constexpr (KIND == 0) strip_tile4(va[T], A_KIN, sa_rd, T, BUF); else strip_rim4(va[T], A_KIN, ra_rd, T, BUF);
            if constexpr (KIND == 1) strip_tile4(vb[T], B_KIN, sb_rd, T, BUF); else strip_rim4(vb[T], B_KIN, rb_rd, T, BUF);
        }
        __builtin_amdgcn_sched_barrier(0);
        v4f d = {0.0f, 0.0f, 0.0f, 0.0f}, d2 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int T = 0; T < SHK_PANELS; T++) {
            d = __builtin_amdgcn_mfma_f32_4x4x1f32(va[T][0], vb[T][0], d, 0, 0, 0);
            d2 = __builtin_amdgcn_mfma_f32_4x4x1f32(va[T][1], vb[T][1], d2, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_4x4x1f32(va[T][2], vb[T][2], d, 0, 0, 0);
            d2 = __builtin_amdgcn_mfma_f32_4x4x1f32(va[T][3], vb[T][3], d2, 0, 0, 0);
        }
        d += d2;
        meet(d);
        return d;
    };
    auto strip_store = [&](const v4f& d, const __amdgpu_buffer_rsrc_t& rs, int off) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float value = d[i];   // (a bit_cast of the vector's element itself reads element 0)
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), rs, off, i * ldc4, SHK_STORE_AUX);
        }
    };

    // One tile, multiplied from buffer PB into accumulator PB; the tile before leaves from accumulator PB ^ 1.
    auto tile = [&](auto pb_c) __attribute__((always_inline)) {
        constexpr int PB = decltype(pb_c)::value;
        using BUF = std::integral_constant<int, PB>;
        using NBUF = std::integral_constant<int, PB ^ 1>;
        __amdgpu_buffer_rsrc_t out_rsrc = shk_out_descriptor(p.C, 0);
        int out_off = OOB_OFFSET;

        // -- the groups before the last two: MFMAs with the side work between them --
        bool done = false;
        static_for<NBODY>([&](auto gc) {
            constexpr int g = decltype(gc)::value;
            constexpr int set = g == 0 ? SET_F : (g % 3);
            if constexpr (g >= MINB) {
                if (g >= fresh(ng) - 2) done = true;
            }
            if (g < MINB || !done) {
                static_for<4>([&](auto qc) {
                    constexpr int q = decltype(qc)::value;
                    constexpr int slot = 4 * g + q;
                    if constexpr (slot == 0)
                        acc[PB] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[set][q], fb[set][q], (v16f)(0.0f), 0, 0, 0);
                    else
                        acc[PB] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[set][q], fb[set][q], acc[PB], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (q == 0) {
                        // the fragments of the group after the next, behind this group's first MFMA (if that group
                        // is one of the last two, which have sets of their own, the read is for nothing); behind
                        // the tile's first MFMA also the next group's and the last two's
                        if constexpr (g == 0) {
                            read_group(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{}, BUF{});
                            read_at(std::integral_constant<int, SET_L1>{}, a_rdl1, b_rdl1, BUF{});
                            read_at(std::integral_constant<int, SET_L2>{}, a_rdl2, b_rdl2, BUF{});
                        }
                        if constexpr (g + 2 < GMAX)
                            read_group(std::integral_constant<int, (g + 2) % 3>{}, std::integral_constant<int, g + 2>{}, BUF{});
                    }
                    // the tile after this one and the finished one before it: scalar work, behind the first MFMAs
                    if constexpr (slot == 0) {
                        has_next = --left > 0;
                        nxt = advance(cur);
                    }
                    // (a dozen scalar instructions fit behind an MFMA for nothing; more than that delay the next
                    // one -- hence a piece per slot)
                    if constexpr (slot == 1) dA = a_desc(nxt, has_next);
                    if constexpr (slot == 2) dB = b_desc(nxt, has_next);
                    if constexpr (slot == 3) dRA = ra_desc(nxt, has_next && nxt.row_strip);
                    if constexpr (slot == 4) dRB = rb_desc(nxt, has_next && nxt.col_strip);
                    if constexpr (slot == 5) {
                        // rows beyond C are cut off by the descriptor, columns by the lane's offset
                        out_rsrc = shk_out_descriptor(prev_c, min(prev_rows, 64) * ldc4);
                        out_off = (prev_cols >= 64 || c_col < prev_cols) ? c_lane : OOB_OFFSET;
                    }
                    if constexpr (slot >= SLOT_XFER && slot < SLOT_XFER + NXFER)
                        transfer(std::integral_constant<int, slot - SLOT_XFER>{}, NBUF{});
                    if constexpr (slot >= SLOT_STORE && slot < SLOT_STORE + 8) {
#pragma unroll
                        for (int e = 2 * (slot - SLOT_STORE); e < 2 * (slot - SLOT_STORE) + 2; e++) {
                            const float value = acc[PB ^ 1][e];
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), out_rsrc, out_off,
                                                                  (8 * (e / 4) + e % 4) * ldc4, SHK_STORE_AUX);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            }
        });

        // -- the strips of the rim that hang on this tile; every wavefront issues the same number of stores --
        int strip_stores = 0;
        float* c_z = cur.c_z;
        if (cur.col_strip) {
            const v4f d = strip(std::integral_constant<int, 0>{}, BUF{});
            // lane l < 16 (k class 0): rows 16 * wave + 4 a + i, column C0 + x
            const int rows_here = min(R0 - cur.m * 64, 64);
            const __amdgpu_buffer_rsrc_t rs = shk_out_descriptor(c_z + (size_t)cur.m * 64 * p.ldc + C0, rows_here * ldc4);
            strip_store(d, rs, (lane < 16 && s_x < rc) ? ((16 * wave + (lane & 12)) * ldc4 + s_x * 4) : OOB_OFFSET);
            strip_stores += 4;
        }
        if (cur.row_strip) {
            const v4f d = strip(std::integral_constant<int, 1>{}, BUF{});
            // lane l < 16: row R0 + i, column 64 n + 16 * wave + l
            const __amdgpu_buffer_rsrc_t rs = shk_out_descriptor(c_z + (size_t)R0 * p.ldc + (size_t)cur.n * 64, rr * ldc4);
            strip_store(d, rs, (lane < 16 && s_line < C0 - cur.n * 64) ? s_line * 4 : OOB_OFFSET);
            strip_stores += 4;
        }
        if (cur.row_strip && cur.col_strip) {
            // the corner: the rim's rows x the rim's columns; the last wavefront stores it
            const v4f d = strip(std::integral_constant<int, 2>{}, BUF{});
            const __amdgpu_buffer_rsrc_t rs = shk_out_descriptor(c_z + (size_t)R0 * p.ldc + C0, rr * ldc4);
            strip_store(d, rs, (wave == 3 && lane < 4 && s_x < rc) ? s_x * 4 : OOB_OFFSET);
            strip_stores += 4;
        }

        // -- every fragment of this tile is in registers, and its strips are done: nobody reads this buffer any
        // more.  The next tile's transfers are older than this tile's stores and vector-memory operations retire
        // in issue order: with at most the stores outstanding the transfers have landed; the barrier makes every
        // wavefront's part visible. --
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the LDS reads above have returned
        if (strip_stores == 0) __builtin_amdgcn_s_waitcnt(waitcnt_vm(16));
        else if (strip_stores == 4) __builtin_amdgcn_s_waitcnt(waitcnt_vm(20));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm(28));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (has_next) read_group(std::integral_constant<int, SET_F>{}, std::integral_constant<int, 0>{}, NBUF{});
        __builtin_amdgcn_sched_barrier(0);
        // -- the last two groups, the very last with only the k that exist --
        static_for<4>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            acc[PB] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[SET_L1][q], fb[SET_L1][q], acc[PB], 0, 0, 0);
        });
        static_for<4>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            if (q < fresh(tail_steps)) acc[PB] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[SET_L2][q], fb[SET_L2][q], acc[PB], 0, 0, 0);
        });

        prev_c = c_z + (size_t)cur.m * 64 * p.ldc + (size_t)cur.n * 64;
        prev_rows = R0 - cur.m * 64;
        prev_cols = C0 - cur.n * 64;
        cur = nxt;
    };

    // the last tile leaves in one go
    auto last_out = [&](auto pb_c) __attribute__((always_inline)) {
        constexpr int PB = decltype(pb_c)::value;
        const __amdgpu_buffer_rsrc_t out_rsrc = shk_out_descriptor(prev_c, min(prev_rows, 64) * ldc4);
        const int out_off = (prev_cols >= 64 || c_col < prev_cols) ? c_lane : OOB_OFFSET;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const float value = acc[PB][e];
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), out_rsrc, out_off,
                                                  (8 * (e / 4) + e % 4) * ldc4, SHK_STORE_AUX);
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
    // nothing of this wave may still be on its way into LDS when the wave ends
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
}

template <bool A_KIN, bool B_KIN>
static hipError_t launch_shortk_cfg(GemmParams p, hipStream_t stream) {
    if (p.split || p.bias != nullptr) return hipErrorOutOfMemory;   // the caller falls back
    const int klimA = p.k_total < (A_KIN ? p.a_inner : p.a_outer) ? p.k_total : (A_KIN ? p.a_inner : p.a_outer);
    const int klimB = p.k_total < (B_KIN ? p.b_inner : p.b_outer) ? p.k_total : (B_KIN ? p.b_inner : p.b_outer);
    const int K = klimA < klimB ? klimA : klimB;
    if (K <= 88 || K > SHK_MAX_K) return hipErrorOutOfMemory;
    // a K-outer operand's panels are reached by 32-bit byte offsets of up to 144 rows
    if ((!A_KIN && (long long)p.lda * 4 * SHK_MAX_K >= 0x40000000LL) || (!B_KIN && (long long)p.ldb * 4 * SHK_MAX_K >= 0x40000000LL))
        return hipErrorOutOfMemory;
    // the rim: 1 ... 4 rows / columns past a multiple of 64 go to strips, the tiles cover the rest
    const int rr = p.rows % 64, rc = p.cols % 64;
    p.rim_rows = (rr >= 1 && rr <= 4 && p.rows > 64) ? rr : 0;
    p.rim_cols = (rc >= 1 && rc <= 4 && p.cols > 64) ? rc : 0;
    p.tiles_m = (p.rows - p.rim_rows + 63) / 64;
    p.tiles_n = (p.cols - p.rim_cols + 63) / 64;
    const long long total = (long long)p.tiles_m * p.tiles_n * p.nz;
    if (total <= 0 || total > (1LL << 26)) return hipErrorOutOfMemory;
    const int num_cu = gemm_device_num_cu();
    if (num_cu <= 0) return hipErrorNoDevice;
    const long long grid = total < num_cu ? total : num_cu;
    {   // the tiles' costs, as the kernel counts them
        const int cr = p.rim_rows > 0 ? SHK_STRIP_COST : 0, cc = p.rim_cols > 0 ? SHK_STRIP_COST : 0, cx = (cr && cc) ? SHK_STRIP_COST : 0;
        const int row_plain = 10 * p.tiles_n + cc, row_last = (10 + cr) * p.tiles_n + cc + cx;
        const long long batch_cost = (long long)(p.tiles_m - 1) * row_plain + row_last;
        const long long all_cost = batch_cost * p.nz;
        if (all_cost >= 0x7fffffffLL) return hipErrorOutOfMemory;
        p.sk_S = (int)batch_cost;
        p.sk_q = (int)(all_cost / grid);
        p.sk_rem = (int)(all_cost % grid);
        gemm_magic_divisor((unsigned)batch_cost, p.div_tiles_mul, p.div_tiles_shift);
        gemm_magic_divisor((unsigned)row_plain, p.div_band_mul, p.div_band_shift);
    }
    hipLaunchKernelGGL((gemm_f32_mfma_shortk<A_KIN, B_KIN, 10>), dim3((unsigned)grid), dim3(NTHREADS), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

// Where the resident-K kernel is taken: a K of 89 ... 144, at least two 64 x 64 tiles per compute unit, and a C that
// the larger tiles of the other kernels would leave ragged (their shapes measured level or ahead on a C that fills
// them: batch 64 of 256 x 256 x 128 through 128 x 64 tiles dealt whole).
int gemm_choose_shortk(int rows, int cols, int nz, int k, int num_cu, int variant) {
    if (rows <= 0 || cols <= 0 || nz <= 0 || num_cu <= 0) return -1;
    if (k <= 88 || k > SHK_MAX_K) return -1;
    const int rr = rows % 64, rc = cols % 64;
    const bool rim = (rr >= 1 && rr <= 4 && rows > 64) || (rc >= 1 && rc <= 4 && cols > 64);
    if (!rim) return -1;
    const long long tiles = (long long)((rows - (rr <= 4 ? rr : 0) + 63) / 64) * ((cols - (rc <= 4 ? rc : 0) + 63) / 64) * nz;
    if (tiles < 2LL * num_cu) return -1;
    return TILE_SHORTK_64x64;
}

hipError_t gemm_launch_shortk(int variant, const GemmParams& p, hipStream_t stream) {
    switch (variant) {
        case GEMM_NN: return launch_shortk_cfg<true, false>(p, stream);
        case GEMM_T1: return launch_shortk_cfg<false, false>(p, stream);
        case GEMM_T2: return launch_shortk_cfg<true, true>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace dragon
