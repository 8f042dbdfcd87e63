// Tile choice and dispatch of the FP32 GEMM kernel (gemm_mfma_kernel.h); instantiates the
// plain products C = A*B, A^T*B, A*B^T in every tile shape.
#include "gemm_mfma_kernel.h"
#include <atomic>

namespace dragon {

int gemm_device_num_cu() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            return 0;   // no answer: the callers fail the launch rather than guess a grid
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// n / d == mulhi(2n, mul) >> shift for every 0 <= n < 2^31: mul = ceil(2^(31 + shift) / d) with
// shift = ceil(log2 d) lies in [2^31, 2^32), and the error n * (mul * d - 2^(31+shift)) stays below 2^(31+shift).
void gemm_magic_divisor(unsigned d, unsigned& mul, unsigned& shift) {
    if (d == 0) d = 1;
    unsigned l = 0;
    while ((1ull << l) < d) l++;
    const unsigned long long two = 1ull << (31 + l);
    mul = (unsigned)((two + d - 1) / d);
    shift = l;
}

void gemm_fill_tile_divisors(GemmParams& p) {
    gemm_magic_divisor((unsigned)(p.tiles_m * p.tiles_n), p.div_tiles_mul, p.div_tiles_shift);
    gemm_magic_divisor((unsigned)(8 * p.tiles_n), p.div_band_mul, p.div_band_shift);
    const int last = p.tiles_m % 8;
    gemm_magic_divisor((unsigned)(last ? last : 8), p.div_last_mul, p.div_last_shift);
}

bool gemm_pitches_addressable(const GemmParams& p) {
    constexpr long long MAX_PITCH = (OOB_OFFSET / 4 - 256) / 256;   // floats
    return p.lda <= MAX_PITCH && p.ldb <= MAX_PITCH && p.ldc <= MAX_PITCH;
}

bool gemm_paired_form_fits(bool a_k_inner, bool b_k_inner, const GemmParams& p) {
    long long kext = p.k_total;
    if (p.split) {   // the last slice takes the remainder
        const long long last = (long long)p.k_total - (long long)(p.nz - 1) * p.k_slice;
        kext = last > p.k_slice ? last : p.k_slice;
    }
    const long long a_span = kext * 4 * (a_k_inner ? 1 : p.lda), b_span = kext * 4 * (b_k_inner ? 1 : p.ldb);
    return a_span < 0x7fffffffLL && b_span < 0x7fffffffLL;
}

bool gemm_rim_applies(GemmParams& p) {
    p.rim_rows = p.rim_cols = p.rim_wgs = 0;
    if (p.split || p.k_total > 256) return false;
    const int rr = p.rows % 64, rc = p.cols % 64;
    const bool use_r = rr >= 1 && rr <= 4 && p.rows > 64, use_c = rc >= 1 && rc <= 4 && p.cols > 64;
    if (!use_r && !use_c) return false;
    const long long before = (long long)((p.rows + 63) / 64) * ((p.cols + 63) / 64);
    const long long after = (long long)((p.rows - (use_r ? rr : 0) + 63) / 64) * ((p.cols - (use_c ? rc : 0) + 63) / 64);
    if (after * 8 > before * 7) return false;
    p.rim_rows = use_r ? rr : 0;
    p.rim_cols = use_c ? rc : 0;
    return true;
}

// a test and tuning hook: a setting of the calling thread only
static thread_local int t_forced_tile = TILE_AUTO;
void gemm_force_tile(int tile) { t_forced_tile = tile; }
int gemm_forced_tile() { return t_forced_tile; }

// What the tile shapes are worth, measured on MI355X (fractions of a compute unit's
// FP32 matrix peak): `alone` is what one resident workgroup sustains by itself (its
// global-load latency is exposed), `cap` what a full compute unit reaches with
// `resident` workgroups sharing it.  The caps and the rules below were last fitted to the times
// of 23 shapes of each of 26 problem sizes x 3 layouts (768^3 ... 5120^3, K from 128 to 8192, panels):
// the choice is on average 0.7 % slower than the best shape, 5 % at worst.
struct TileTraits { int bm, bn, kt, resident; float alone, cap; };
static const TileTraits kTiles[TILE_ALL_COUNT] = {
    /* TILE_128x128     */ {128, 128, 16, 4, 0.62f, 0.91f},
    /* TILE_64x64       */ { 64,  64, 16, 8, 0.35f, 0.82f},
    /* TILE_256x64      */ {256,  64, 16, 4, 0.62f, 0.88f},
    /* TILE_64x256      */ { 64, 256, 16, 4, 0.62f, 0.88f},
    /* TILE_128x64      */ {128,  64, 16, 6, 0.48f, 0.83f},
    /* TILE_64x128      */ { 64, 128, 16, 6, 0.48f, 0.83f},
    /* TILE_128x128_K32 */ {128, 128, 32, 2, 0.65f, 0.90f},
    /* TILE_64x64_K32   */ { 64,  64, 32, 5, 0.42f, 0.82f},
    /* TILE_128x64_K32  */ {128,  64, 32, 3, 0.52f, 0.84f},
    /* TILE_64x128_K32  */ { 64, 128, 32, 3, 0.52f, 0.84f},
    /* TILE_64x64_K64   */ { 64,  64, 64, 2, 0.55f, 0.80f},
    /* TILE_64x64_K128  */ { 64,  64, 128, 1, 0.65f, 0.65f},
    /* TILE_128x128_K64 */ {128, 128, 64, 1, 0.80f, 0.80f},
    /* TILE_128x64_K64  */ {128,  64, 64, 1, 0.70f, 0.70f},
    /* TILE_64x128_K64  */ { 64, 128, 64, 1, 0.70f, 0.70f},
    // direct-to-LDS staging, three stages in flight: the best a lone workgroup does; with company
    // its larger LDS footprint (fewer resident workgroups) loses to the register-staged shapes
    /* TILE_DMA_128x128_S4   */ {128, 128, 16, 2, 0.60f, 0.86f},
    /* TILE_DMA_64x64_S4     */ { 64,  64, 16, 5, 0.40f, 0.78f},
    /* TILE_DMA_64x64_K32_S4 */ { 64,  64, 32, 2, 0.69f, 0.78f},
};

// Pick the tile shape with the lowest estimated time: the matrix work of the busiest
// compute unit (padded tiles, k rounded up to the stage), divided by what that unit
// sustains with the workgroups it gets.
int gemm_choose_tile(int rows, int cols, int nz, int k, int num_cu, int variant) {
    const int forced = gemm_forced_tile();
    if (forced != TILE_AUTO) return forced;
    const int skinny = gemm_choose_skinny(rows, cols, nz, k, variant, num_cu);
    if (skinny >= 0) return skinny;
    const int band = gemm_choose_band(rows, cols, nz, k, num_cu, variant);
    if (band >= 0) return band;
    const int shortk = gemm_choose_shortk(rows, cols, nz, k, num_cu, variant);
    if (shortk >= 0) return shortk;
    const int balanced = gemm_choose_streamk(rows, cols, nz, k, num_cu, variant);
    return balanced >= 0 ? balanced : gemm_choose_tile_per_workgroup(rows, cols, nz, k, num_cu, variant);
}

int gemm_choose_tile_per_workgroup(int rows, int cols, int nz, int k, int num_cu, int variant) {
    int best = TILE_128x128;
    double best_cost = 1e300;
    for (int tile = 0; tile < TILE_ALL_COUNT; tile++) {
        const TileTraits& tt = kTiles[tile];
        const long long tm = (rows + tt.bm - 1) / tt.bm, tn = (cols + tt.bn - 1) / tt.bn;
        const long long total = tm * tn * nz;
        const long long per_cu = (total + num_cu - 1) / num_cu;       // tiles on the busiest unit
        const long long together = per_cu < tt.resident ? per_cu : tt.resident;
        double eff = together * (double)tt.alone;
        if (eff > tt.cap) eff = tt.cap;
        const long long kp = ((long long)k + tt.kt - 1) / tt.kt * tt.kt;
        // a short tile pays for filling and draining its pipeline: about two stages' worth
        const double work = (double)per_cu * tt.bm * tt.bn * (double)(kp + 2 * tt.kt);
        const double cost = work / eff;
        if (cost < best_cost * 0.98) { best_cost = cost; best = tile; }
    }
    // Measured, and beyond the model's resolution: with at most two 128 x 128 tiles per compute unit the
    // stages of 32 k (which fit two workgroups to a unit) run 1.5-3 % faster than those of 16 k.
    if (best == TILE_128x128 && k >= 256) {
        const long long total = (long long)((rows + 127) / 128) * ((cols + 127) / 128) * nz;
        if ((total + num_cu - 1) / num_cu <= 2) best = TILE_128x128_K32;
    }

    // The same for the 8192-element shapes, of which three workgroups with 32-k stages fit a unit: 2-4 %
    // faster up to three tiles per unit -- except 64 x 128 with both operands K-outer (A^T * B), where the
    // 32-k stages lose.
    if ((best == TILE_128x64 || (best == TILE_64x128 && variant != GEMM_T1)) && k >= 256) {
        const int bm = best == TILE_128x64 ? 128 : 64, bn = best == TILE_128x64 ? 64 : 128;
        const long long total = (long long)((rows + bm - 1) / bm) * ((cols + bn - 1) / bn) * nz;
        if ((total + num_cu - 1) / num_cu <= 3) best = best == TILE_128x64 ? TILE_128x64_K32 : TILE_64x128_K32;
    }
    // and for 64 x 64, of which five workgroups with 32-k stages fit a unit: 4-10 % faster, and with
    // the paired form still ahead at nine tiles per unit (3072^3: 8 %)
    if (best == TILE_64x64 && k >= 256) {
        const long long total = (long long)((rows + 63) / 64) * ((cols + 63) / 64) * nz;
        if ((total + num_cu - 1) / num_cu <= 9) best = TILE_64x64_K32;
    }
    // A C that is a single 64-column tile wide and has rows to spare: the 128-row tile halves the re-reads
    // of B at the same stage depth (batch 64 of 1024x1024 . 1024x64: 75.3 against 76.6 us).
    // (not where the rows do not fill it: batch 1024 of 64 x 64 x 64 takes 8.2 us in 64 x 64 tiles, 12.9 in 128 x 64)
    if ((best == TILE_64x64 || best == TILE_64x64_K32) && cols <= 64 && (rows + 127) / 128 * 128 <= (rows + 63) / 64 * 64 + rows / 8) {
        const long long total = (long long)((rows + 127) / 128) * nz;
        const long long per_cu = (total + num_cu - 1) / num_cu;
        if (per_cu >= 2) best = (k >= 256 && per_cu <= 3) ? TILE_128x64_K32 : TILE_128x64;
    }
    // One tile per compute unit or fewer: the direct-to-LDS kernel was the best a lone workgroup did until
    // the paired form, which beats it by 2-9 % wherever an operand is K-inner (A*B, A*B^T; measured on
    // 1000x777x1531, 768^3, 1024^3, 1024x1024x4096, 512x512x8192) and loses 0-5 % on A^T*B.
    if (best == TILE_DMA_64x64_K32_S4 && variant != GEMM_T1 && k >= 512) best = TILE_64x64_K32;
    // The paired-stage form of the kernel, measured over 2048..4096 x 2048..4096 x K in all layouts: equal
    // at K = 256, 2-5 % faster at 512..1024, 3.5-8 % at 4096; slower on a short K (8 % at K = 64).  The two
    // 256-row shapes spill in it and gain only from K = 2048 on.  With 128 x 128 tiles of 16 k it is ahead from
    // K = 256 on wherever C is large (1.5 - 3.5 % on 4096^2 ... 131072 x 256 under K = 256 ... 448).
    if (best <= TILE_64x128_K32 && k >= ((best == TILE_256x64 || best == TILE_64x256) ? 2048 : best == TILE_128x128 ? 256 : 512))
        best |= TILE_PAIRED;
    return best;
}

hipError_t gemm_launch(int variant, const GemmParams& p, int tile, hipStream_t stream) {
    if (!gemm_pitches_addressable(p)) return hipErrorInvalidValue;
    if (gemm_tile_is_streamk(tile) || gemm_tile_is_band(tile) || gemm_tile_is_shortk(tile) || gemm_tile_is_skinny(tile)) {
        // where the product cannot take the balanced kernel (K slices shorter than a stage; a capturing
        // stream that has no workspace yet; a bias row on a transposed product) or the band kernel (a K beyond one stage, K slices, a
        // bias row) a tile-per-workgroup kernel takes over
        const hipError_t e = gemm_tile_is_skinny(tile)   ? gemm_launch_skinny(variant, p, stream)
                             : gemm_tile_is_band(tile)   ? gemm_launch_band(variant, p, stream, tile == TILE_BAND_64x256, tile == TILE_BAND_REGS)
                             : gemm_tile_is_shortk(tile) ? gemm_launch_shortk(variant, p, stream)
                                                         : gemm_launch_streamk(variant, p, tile, stream);
        if (e != hipErrorOutOfMemory) return e;
        (void)hipGetLastError();
        const int k = p.split ? (p.k_slice > 0 ? p.k_slice : p.k_total) : p.k_total;
        const int num_cu = gemm_device_num_cu();
        if (num_cu <= 0) return hipErrorNoDevice;
        tile = gemm_choose_tile_per_workgroup(p.rows, p.cols, p.nz, k, num_cu, variant);
    }
    if (p.bias != nullptr)   // the bias row exists for the forward product only
        return variant == GEMM_NN ? gemm_launch_nn_biased(p, tile, stream) : hipErrorInvalidValue;
    if (gemm_tile_is_dma(tile)) return gemm_launch_dma(variant, p, tile, stream);
    switch (variant) {
        case GEMM_NN: return launch_variant<true, false, false>(p, tile, stream);
        case GEMM_T1: return launch_variant<false, false, false>(p, tile, stream);
        case GEMM_T2: return launch_variant<true, true, false>(p, tile, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace dragon
