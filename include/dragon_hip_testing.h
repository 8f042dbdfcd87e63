/*
 * dragon_hip_testing.h -- inspection and test hooks of libdragon_hip.so.
 *
 * NOT part of the drop-in boundary: nothing here has a counterpart in the reference and no host
 * needs it to run the engine.  The hooks exist so that tests and benchmarks can sweep the kernel
 * variants, check host arithmetic without a device, and calibrate profiler byte counters.
 */
#ifndef DRAGON_HIP_TESTING_H
#define DRAGON_HIP_TESTING_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Force one tile shape for the following launches OF THE CALLING THREAD (the setting is
 * thread-local: no other thread's kernel choice changes); -1 restores the automatic choice.
 * Shapes: 0 = 128x128, 1 = 64x64, 2 = 256x64, 3 = 64x256, 4 = 128x64, 5 = 64x128 (16 k per
 * LDS stage); 6 = 128x128, 7 = 64x64, 8 = 128x64, 9 = 64x128 with 32 k per stage; 10 = 64x64
 * with 64 k, 11 = 64x64 with 128 k, 12 = 128x128, 13 = 128x64, 14 = 64x128 with 64 k per stage;
 * 15 = 128x128 and 16 = 64x64 with 16 k, 17 = 64x64 with 32 k per stage, staged global -> LDS
 * directly through four stage buffers.  Adding 256 to a shape 0..9 selects its paired-stage form
 * (stages run two by two with compile-time LDS buffers; what the automatic choice takes from
 * K = 512 on, 256 for shape 0).  18..23 and 25: the balanced kernel (workgroups share the work in equal runs of LDS
 * stages; taken for few tiles and a long K, for large products, their K slices and large
 * convolutions): 18 = 64x64, 19 = 128x64, 20 = 64x128, 21 = 128x128 with one workgroup per
 * compute unit, 22 = 64x64 and 23 = 128x64 with two, 25 = 256x64 with one.  24: the band kernel
 * for a K of at most 64 under a large C (a band of 128 rows of A stays in LDS; a longer K falls
 * back to the automatic choice).  26: the resident-K kernel for a K of 89 ... 144 (64x64 tiles whose whole K
 * sits in LDS, the rim of C -- 1 ... 4 rows / columns past a multiple of 64 -- as strips of 4x4 MFMA blocks;
 * another K falls back to the automatic choice).  27: the skinny kernel for a 2-D product whose C has 4, 8, ... 32
 * columns under at least 256 rows, or as many rows over at least 256 columns (wavefronts stream the long operand into 4x4x1
 * or 16x16x4 MFMA blocks; what the automatic choice takes there; another shape falls back to the automatic choice).  28: the band
 * kernel with bands of 64 rows under tiles of 256 columns, 29: the band kernel with the band's rows of A in registers
 * (four wavefronts, two workgroups per compute unit, a tile multiplied block after block); neither is chosen
 * automatically: both measure level with 24. */
void dragon_gemm_force_tile(int32_t tile);
/* Force a form of the skinny kernel for the following launches OF THE CALLING THREAD: 0 = a wavefront per run of
 * lines of the long operand (64 lines where k is its row index, 16 where k is contiguous) with the whole K, 1 = the
 * four wavefronts of a workgroup share a run and split K, 2 = sixteen wavefronts do, 3 and 4 = as 0 and 1 with runs
 * four (two) times as long, 5 and 6 = as 2 with runs of 32 and 16 lines (k the row index; else as 2), 7 = as 1 with K
 * cut across workgroups as well, two workgroups per compute unit (100 + c: c cuts, at most 8; needs the stream's
 * workspace); 8 ... 11 = 16x16x4 MFMA blocks (16 lines against all short lines per instruction; what the automatic
 * choice takes for 12 or 16 short lines and for most products with 8): 8 = a wavefront per run of 64 lines with the
 * whole K, 9 = the four wavefronts of a workgroup share a run, 10 and 11 = as 8 and 9 with runs of 32 lines
 * (200 + c: as 11 with K cut across c workgroups per run, at most 16; needs the stream's workspace);
 * -1 restores the automatic choice.  Adding 1000 makes the long forms (3, 4, 8, 9) read the long operand with
 * non-temporal loads, adding 2000 with ordinary ones (automatic: non-temporal from 320 MiB on); 1999 and 2999 are
 * the automatic form with that policy. */
void dragon_gemm_skinny_form(int32_t form);
/* 1 if the paired-stage form can address the 2-D product (variant 0 = A*B, 1 = A^T*B, 2 = A*B^T, cut into
 * GridZ K slices): it reaches a tile's stages by 32-bit byte offsets, so the longest K range times the
 * operand's advance per k (4 bytes, or a row of a K-outer operand) must stay below 2^31; 0 if not (the
 * launch then runs the plain form), -1 on bad arguments.  Host arithmetic only. */
int32_t dragon_gemm_paired_form_fits(int32_t variant, int32_t GridZ, int32_t N, int32_t M, int32_t K);
/* The multiply-and-shift pair the kernels divide a tile index by d with: n / d == (((2n) * mul) >> 32) >> shift
 * for every 0 <= n < 2^31 (the launcher makes the pairs, the kernels only multiply).  Host arithmetic. */
void dragon_gemm_tile_divisor(uint32_t d, uint32_t* mul, uint32_t* shift);
/* The shape the automatic choice takes for a product of `rows` x `cols` outputs, depth `nz` (batch or
 * K slices), `k` per output, on `num_cu` compute units; variant 0 = A*B, 1 = A^T*B, 2 = A*B^T, -1 = unknown.
 * Pure host arithmetic (no device needed); returns the forced shape while the calling thread forces one,
 * -1 on bad arguments. */
int32_t dragon_gemm_choose_tile(int32_t variant, int32_t rows, int32_t cols, int32_t nz, int32_t k, int32_t num_cu);
/* How the split-K entry points (matMulSK, matMulT1SK, matMulT2SK, matMulSK_static) treat the caller's GridZ,
 * for the following calls OF THE CALLING THREAD: -1 (default) the library's estimate decides -- where the
 * unsplit product through the balanced kernel is estimated to beat the slices plus their fold, the whole
 * product goes to C and the partial buffers get exact zeros; 0 the K slices always as asked; 1 declined
 * wherever the unsplit product can take the balanced kernel.  A forced tile shape always honours the split. */
void dragon_gemm_split_policy(int32_t mode);
/* 0: SKbuf_summary always launches its kernel; 1 (default): the fold that follows a declined split with the
 * same stream, Cbuf, C, part and sizeC -- which would add zeros -- returns without launching (see
 * dragon_hip_gemm.h).  Process-wide.  And the number of folds elided so far. */
void dragon_gemm_fold_skip(int32_t on);
int64_t dragon_gemm_folds_skipped(void);
/* Split-K calls of this process that ran unsplit (with zeroed partial buffers) so far. */
int64_t dragon_gemm_declined_splits(void);
/* 1 if the estimate declines GridZ slices of the 2-D product N x M x K (all multiples of 4) on num_cu compute
 * units, 0 if it honours them, -1 on bad arguments; and the estimate itself in microseconds for `nz` products
 * (or K slices) of rows x cols x k.  Host arithmetic only. */
int32_t dragon_gemm_split_loses(int32_t variant, int32_t N, int32_t M, int32_t GridZ, int32_t K, int32_t num_cu);
double dragon_gemm_estimate_us(int32_t variant, int32_t rows, int32_t cols, int32_t nz, int32_t k, int32_t num_cu);
/* The balanced kernel's per-stream workspaces (device memory the library owns, see dragon_hip_gemm.h):
 * how many it holds now, and how many balanced launches found the table of 64 full and took a
 * tile-per-workgroup kernel instead. */
int32_t dragon_gemm_workspace_count(void);
int64_t dragon_gemm_workspaces_refused(void);
/* Free and total device memory of the current device in bytes (hipMemGetInfo). */
int dragon_test_mem_get_info(int64_t* free_bytes, int64_t* total_bytes);
/* Device-to-device copy of `length` floats (a multiple of 4, 16-byte aligned) done by an ordinary
 * kernel rather than the copy engine: the known-size copy that hardware byte counters are
 * calibrated against when profiling. */
int dragon_test_copy1D_kernel(int64_t stream, int64_t dst, int64_t src, int64_t length);

#ifdef __cplusplus
}
#endif
#endif /* DRAGON_HIP_TESTING_H */
