// Internal interface between the C-ABI entry points and the gfx950 GEMM kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace dragon {

enum GemmVariant { GEMM_NN = 0, GEMM_T1 = 1, GEMM_T2 = 2 };

enum GemmTile {
    TILE_AUTO = -1,
    TILE_128x128 = 0,
    TILE_64x64 = 1,
    TILE_256x64 = 2,
    TILE_64x256 = 3,
    TILE_128x64 = 4,
    TILE_64x128 = 5,
    TILE_128x128_K32 = 6,   // the same shapes with 32 k per LDS stage
    TILE_64x64_K32 = 7,
    TILE_128x64_K32 = 8,
    TILE_64x128_K32 = 9,
    TILE_64x64_K64 = 10,    // long stages: one workgroup per compute unit still covers its load latency
    TILE_64x64_K128 = 11,
    TILE_128x128_K64 = 12,
    TILE_128x64_K64 = 13,
    TILE_64x128_K64 = 14,
    TILE_COUNT = 15,        // the shapes above use register-staged double buffering
    // direct global->LDS staging through 4 stage buffers
    TILE_DMA_128x128_S4 = 15,
    TILE_DMA_64x64_S4 = 16,
    TILE_DMA_64x64_K32_S4 = 17,
    TILE_ALL_COUNT = 18,
    // Few tiles, long K: persistent workgroups that share the work in equal runs of LDS stages rather than in
    // whole tiles (gemm_mfma_streamk.hip); 32 k per stage, direct global->LDS staging
    TILE_SK_64x64 = 18,        // one workgroup per compute unit, 4 stage buffers
    TILE_SK_128x64 = 19,
    TILE_SK_64x128 = 20,
    TILE_SK_128x128 = 21,
    TILE_SK_64x64_O2 = 22,     // two workgroups per compute unit, 4 stage buffers
    TILE_SK_128x64_O2 = 23,    // two workgroups per compute unit, 3 stage buffers
    TILE_SK_END = 24,
    // Short K (at most 64), large C: a workgroup keeps a band of 128 rows of A in LDS, walks along its
    // column tiles with the whole K in one stage and stores a tile while it multiplies the next
    // (gemm_mfma_band.hip)
    TILE_BAND_128x128 = 24,
    // one more balanced shape: 256 x 64, four wavefronts of 64 x 64 one above the other, 3 stage buffers -- for a
    // C of 64 columns, where it has the 128 x 128 tile's ratio of matrix work to LDS traffic
    TILE_SK_256x64 = 25,
    // A K of 89 ... 144 under a ragged C, batch after batch: 64 x 64 tiles with the whole K of a tile resident in
    // LDS, one persistent workgroup per compute unit, the rim of C (1 ... 4 rows / columns past a multiple of 64)
    // as strips of 4 x 4 MFMA blocks beside the tiles (gemm_mfma_shortk.hip)
    TILE_SHORTK_64x64 = 26,
    // A C of 4 ... 16 columns (or rows) under a long other side: wavefronts stream the long operand from memory into
    // 4 x 4 x 1 MFMA blocks, no tiles and no LDS staging (gemm_skinny.hip)
    TILE_SKINNY = 27,
    // the band kernel with bands of 64 rows under tiles of 256 columns
    TILE_BAND_64x256 = 28,
    // the band kernel with the band's rows of A in registers: 128 x 128 tiles, four wavefronts, two workgroups per unit
    TILE_BAND_REGS = 29,
    // Flag on the ids 0..9: the stages of a long K run two by two, with the LDS buffer known at compile
    // time and without the per-lane K test (see the kernel).  Faster from about K = 512 on, slower on a
    // short K; gemm_choose_tile sets it.
    TILE_PAIRED = 0x100
};
inline bool gemm_tile_is_streamk(int tile) { return (tile >= TILE_SK_64x64 && tile < TILE_SK_END) || tile == TILE_SK_256x64; }
inline bool gemm_tile_is_band(int tile) { return tile == TILE_BAND_128x128 || tile == TILE_BAND_64x256 || tile == TILE_BAND_REGS; }
inline bool gemm_tile_is_shortk(int tile) { return tile == TILE_SHORTK_64x64; }
inline bool gemm_tile_is_skinny(int tile) { return tile == TILE_SKINNY; }
inline bool gemm_tile_is_dma(int tile) { return tile >= TILE_DMA_128x128_S4 && tile <= TILE_DMA_64x64_K32_S4; }

// One product C[z] = op(A[z]) * op(B[z]) or one K slice of it.
//   K-inner operand (k contiguous): outer bound = number of rows that exist (exact),
//                                   inner bound = k extent (multiple of 4).
//   K-outer operand (k is the row): outer bound = number of k rows that exist (exact),
//                                   inner bound = row length (multiple of 4).
struct GemmParams {
    const float* A;
    const float* B;
    float* C;
    float* Cbuf;            // split-K partials: slice z >= 1 goes to Cbuf + (z-1)*sizeC
    int rows, cols;         // stored extent of C: rows exact, cols a multiple of 4
    int k_total;            // contraction length
    int lda, ldb, ldc;      // leading strides in floats (multiples of 4)
    int a_outer, a_inner;
    int b_outer, b_inner;
    long long sA, sB, sC;   // batch strides in floats
    int nz;                 // grid depth: batches, or K slices when split is set
    int split;              // non-zero selects split-K
    int k_slice;            // slice z covers [z*k_slice, (z+1)*k_slice), the last runs to k_total
    long long sizeC;        // floats per split-K partial
    // implicit-GEMM convolution (gemm_launch_conv): A is gathered from X[N, IH, IW, IC]; rows = N*OH*OW,
    // k_total = FH*FW*IC, B = W[OC, FH*FW*IC], C = Y[N*OH*OW, OC]
    int cv_IH, cv_IW, cv_IC, cv_FW, cv_OH, cv_OW, cv_sh, cv_sw, cv_ph, cv_pw;
    float cv_rcp_IC, cv_rcp_FW;
    int cv_walk;          // 1: visit the K chunks filter-column fastest (see the kernel), 0: in storage order
    // filled by the launcher of the balanced kernel's convolution form (gemm_launch_streamk_conv): filter rows,
    // LDS stages per filter tap (IC / 32), the bytes the lanes' offsets are raised by so that a pixel above or left
    // of the image still has a non-negative one, and multiply-and-shift pairs for OW, OH, cv_spt and FW
    int cv_FH, cv_spt, cv_bias;
    unsigned cv_div_OW_mul, cv_div_OW_shift, cv_div_OH_mul, cv_div_OH_shift;
    unsigned cv_div_spt_mul, cv_div_spt_shift, cv_div_FW_mul, cv_div_FW_shift;
    const float* bias;      // optional row vector added to C[i][j] for i < bias_rows, j < bias_width
    int bias_rows, bias_width;
    int tiles_m, tiles_n;   // filled by the launcher
    // filled by the launcher (gemm_fill_tile_divisors): the divisors of the tile-index decode as
    // multiply-and-shift pairs, n / d == mulhi(2 * n, mul) >> shift for 0 <= n < 2^31
    unsigned div_tiles_mul, div_tiles_shift;   // d = tiles_m * tiles_n
    unsigned div_band_mul, div_band_shift;     // d = 8 * tiles_n (a band of 8 tile rows)
    unsigned div_last_mul, div_last_shift;     // d = tile rows of the last, shorter band (tiles_m % 8, or 8)
    // filled by the launcher of the balanced kernel (gemm_launch_streamk): a tile has sk_S stages, workgroup w
    // takes sk_q stages (one more for w < sk_rem) of the tiles' stages numbered tile by tile; pieces of shared
    // tiles go to sk_ws
    float* sk_ws;
    int* sk_count;
    int sk_S, sk_q, sk_rem;
    unsigned sk_div_S_mul, sk_div_S_shift;
    // set by a caller that may not allocate: a workspace of its own for the balanced kernel (arrival counters
    // zero) instead of the stream's
    float* sk_ws_given;
    size_t sk_ws_given_floats;
    // few tiles under a very long K, dealt in whole runs per tile: sk_kmajor_rpt runs per tile (0: off) of
    // sk_kmajor_tiles tiles; the workgroups that share an XCD then take the same k ranges of different tiles
    int sk_kmajor_rpt, sk_kmajor_tiles;
    // a launch of the balanced kernel over the tiles sk_tile_base ... sk_tile_base + sk_tile_count - 1 only
    // (sk_tile_count 0: all of them): see gemm_launch_streamk
    int sk_tile_base, sk_tile_count;
    // K slices: the tiles from number sk_T1 on (the last slice's) have sk_S_last stages
    int sk_S_last, sk_T1;
    unsigned sk_div_Sl_mul, sk_div_Sl_shift;
    // a split-K call whose split was declined (gemm_split_loses): the whole product goes to C and the balanced
    // kernel's workgroups write zeros over the zero_floats floats (a multiple of 4) of the caller's partial buffers
    float* zero_buf;
    long long zero_floats;
    // filled by the launcher of the band kernel (gemm_launch_band): a band's tiles_n column tiles are dealt
    // out in bd_chunks runs of bd_chunk_tiles
    int bd_chunks, bd_chunk_tiles;
    // filled by gemm_rim_applies for the 64 x 64 kernels with a rim (see rim_job in gemm_mfma_kernel.h): the last
    // rim_rows rows and rim_cols columns of C (0..4 each) are computed by the launch's first rim_wgs workgroups,
    // the tiles cover the rest
    int rim_rows, rim_cols, rim_wgs;
};
void gemm_fill_tile_divisors(GemmParams& p);
void gemm_magic_divisor(unsigned d, unsigned& mul, unsigned& shift);

// Compute units of the current device, cached per device; 0 when no device answers (the launchers then
// return hipErrorNoDevice).
int gemm_device_num_cu();
// True where C's extent is 1..4 rows and / or columns past a multiple of 64 and leaving those to the rim's
// workgroups saves at least an eighth of the 64 x 64 tiles (and K is short enough for the rim's serial
// walk along it); fills p.rim_rows / p.rim_cols.
bool gemm_rim_applies(GemmParams& p);
// The kernels address an operand tile with 32-bit byte offsets from the tile's origin: up to 256 rows
// (or k) of pitch.  False when a leading stride is too long for that; the entry points reject such calls.
bool gemm_pitches_addressable(const GemmParams& p);
// The paired form addresses a tile's stages by 32-bit scalar byte offsets from its first stage: K-inner
// operands advance 4 bytes per k, K-outer ones a whole row.  False where the longest K range of a tile
// does not fit 31 bits; the launcher then runs the plain form (advancing 64-bit pointers) instead.
bool gemm_paired_form_fits(bool a_k_inner, bool b_k_inner, const GemmParams& p);
int gemm_choose_tile(int rows, int cols, int nz, int k, int num_cu, int variant = -1);   // variant: GEMM_* or -1
// the same without the balanced kernel's shapes
int gemm_choose_tile_per_workgroup(int rows, int cols, int nz, int k, int num_cu, int variant = -1);
void gemm_force_tile(int tile);
int gemm_forced_tile();   // TILE_AUTO when the choice is left to gemm_choose_tile
hipError_t gemm_launch(int variant, const GemmParams& p, int tile, hipStream_t stream);
// The resident-K kernel (tile id TILE_SHORTK_64x64) for the three products, batched too, with 88 < K <= 144.
// hipErrorOutOfMemory says that the product cannot go this way (another K, K slices, a bias row) and the caller
// takes a tile-per-workgroup kernel instead.
hipError_t gemm_launch_shortk(int variant, const GemmParams& p, hipStream_t stream);
// TILE_SHORTK_64x64 where that kernel is the better choice, else -1
int gemm_choose_shortk(int rows, int cols, int nz, int k, int num_cu, int variant = -1);
// The skinny kernel (tile id TILE_SKINNY) for the three 2-D products whose C has 4, 8, ... 32 columns under at
// least 256 rows, or as many rows over at least 256 columns.  hipErrorOutOfMemory says that the product cannot go this way
// (another shape, a batch, K slices, a bias row) and the caller takes a tile-per-workgroup kernel instead.
hipError_t gemm_launch_skinny(int variant, const GemmParams& p, hipStream_t stream);
// TILE_SKINNY for such a shape, else -1
int gemm_choose_skinny(int rows, int cols, int nz, int k, int variant, int num_cu);
// force one of the kernel's forms (0..11, see gemm_skinny.hip) for the calling thread's launches; -1 = automatic
void gemm_skinny_form(int form);
// the three products through the direct-to-LDS kernel (tile ids TILE_DMA_*)
hipError_t gemm_launch_dma(int variant, const GemmParams& p, int tile, hipStream_t stream);
// the three products (batched too) through the balanced kernel (tile ids TILE_SK_*).  It needs the stream's
// workspace (or the one in p.sk_ws_given); hipErrorOutOfMemory says that the product cannot go this way (no
// workspace and none may be made now, sizes beyond its counters, K slices shorter than a stage) and the caller
// takes a tile-per-workgroup kernel instead.
hipError_t gemm_launch_streamk(int variant, const GemmParams& p, int tile, hipStream_t stream);
// The balanced kernel's tile for this product, or -1 where the tile-per-workgroup kernels do as well or
// better (an estimate fitted to measurements: at most two 64 x 64 tiles per compute unit, and K long enough
// to carry the balanced kernel's larger fixed time).
int gemm_choose_streamk(int rows, int cols, int nz, int k, int num_cu, int variant = -1);
// The fitted estimate behind that choice, in microseconds: what the product takes through the kernel
// gemm_choose_tile names (few 64 x 64 tiles: the measured per-stage and per-launch costs of the balanced and the
// tile-per-workgroup kernels; more tiles: the padded matrix work at the rate the large kernels sustain).
double gemm_estimate_us(int rows, int cols, int nz, int k, int num_cu, int variant = -1);
// True where cutting K into gz slices (k_slice each, partials folded by SKbuf_summary afterwards) is estimated
// to take longer than the unsplit product through the balanced kernel, which deals equal runs of stages to the
// compute units by itself: the split-K entry points then run the unsplit product and zero the partial buffers.
bool gemm_split_loses(int variant, int rows, int cols, int gz, int k, int k_slice, int num_cu);
// Floats of a balanced-kernel workspace for a device of num_cu compute units (GEMM_SK_WS_FLOATS_256CU: the
// same for 256 units, as a constant for static storage)
size_t gemm_streamk_workspace_floats(int num_cu);
constexpr size_t GEMM_SK_WS_FLOATS_256CU = 65536 + (size_t)2 * 256 * 128 * 128;
// The forward convolution (A gathered from the image, see ConvDirect) through the balanced kernel, for channel
// counts that are multiples of 32 and filters of at most 32 x 32; hipErrorOutOfMemory as above (then
// gemm_launch_conv takes over).
hipError_t gemm_launch_streamk_conv(const GemmParams& p, int tile, hipStream_t stream);
// The workspace of `stream` on the stream's device: arrival counters and the slots for pieces of shared tiles.
// Made at the first balanced launch on that stream (a device allocation, and a small kernel on that stream that
// clears the counters) and kept for later launches on the same handle until the stream is deleted through the
// runtime bridge or the workspaces are released; nullptr while the stream is capturing (a graph's launches may
// run next to the stream's own) and when the library already holds its maximum number of workspaces.
float* gemm_streamk_workspace(hipStream_t stream, size_t* floats);
// Gives the stream's workspace back (after the stream's work is done); the runtime bridge calls it before it
// destroys a stream.  Nothing happens for a stream that has none.
void gemm_streamk_release_workspace(hipStream_t stream);
// The same for every workspace the library holds, on every device (each device is synchronised first);
// returns how many there were.  Streams that launch the balanced kernel again get a new one.
int gemm_streamk_release_workspaces();
int gemm_streamk_workspace_count();               // workspaces held now
long long gemm_streamk_workspaces_refused();      // balanced launches that found the table full and took another kernel
// The band kernel (tile ids TILE_BAND_128x128, and TILE_BAND_64x256 with `wide`) for the three products, batched
// too, with K <= 64.  hipErrorOutOfMemory says that the product cannot go this way (a longer K, K slices, a bias
// row) and the caller takes a tile-per-workgroup kernel instead.
hipError_t gemm_launch_band(int variant, const GemmParams& p, hipStream_t stream, bool wide = false, bool regs = false);
// TILE_BAND_128x128 where the band kernel is the better choice, else -1
int gemm_choose_band(int rows, int cols, int nz, int k, int num_cu, int variant = -1);
// how the band kernel deals a band's column tiles to workgroups
void gemm_band_split(long long bands, int tiles_n, int num_cu, int& chunks, int& chunk_tiles);
// Y = conv(X, W) [+ bias row over OC] as an implicit GEMM (the A * B^T kernel with a gathered A);
// classic tile ids only
hipError_t gemm_launch_conv(const GemmParams& p, int tile, hipStream_t stream);
// the GEMM_NN product with p.bias added in the epilogue (what gemm_launch forwards to when p.bias is set)
hipError_t gemm_launch_nn_biased(const GemmParams& p, int tile, hipStream_t stream);
// the GEMM_T2 product with p.bias added in the epilogue, tile-per-workgroup shapes 0 .. TILE_64x128_K32 (+ TILE_PAIRED)
hipError_t gemm_launch_t2_biased(const GemmParams& p, int tile, hipStream_t stream);

// Y[i] = alpha*X1[i] + beta*X2[i % row_lengthv] + gamma over lengthv floats laid out in rows of
// `stride`, elements at or beyond `width` in a row written as zero.
hipError_t linear_dual2D_row_launch(hipStream_t stream, const float* X1, const float* X2, int row_lengthv,
                                    float alpha, float beta, float gamma, float* Y, int lengthv,
                                    int width, int stride);

// C[i] += sum_p Cbuf[p*sizeC + i], Kahan-compensated, p ascending.
hipError_t skbuf_summary_launch(hipStream_t stream, const float* Cbuf, float* C, int part, int sizeC);

}  // namespace dragon
