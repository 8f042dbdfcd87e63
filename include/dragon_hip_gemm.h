/*
 * dragon_hip_gemm.h -- C ABI of the gfx950 FP32 matrix-multiplication engine.
 *
 * Each entry point takes exactly the argument list of one `static native` method of
 * the reference's z.dragon.engine.cuda.impl.math.Cuda_matMul / Cuda_batchMatMul
 * classes, i.e. of one JNI function of Cuda_matMul.dll / Cuda_batchMatMul.dll, minus
 * the (JNIEnv*, jclass) pair:  jlong -> int64_t (a raw device address or a stream
 * handle), jint -> int32_t, jlongArray -> const int64_t*.  Where the JNI functions
 * return void and throw z.dragon.engine.cuda.impl.CudaException(int), these return
 * the hipError_t value as int (0 = success); a JNI shim turns a non-zero value into
 * the exception.
 *
 * Reference paths below are relative to source/ of the reference tree:
 *   MM  = engine-cuda-base/Cuda_matMul/Cuda_matMul
 *   BMM = engine-cuda-base/Cuda_batchMatMul/Cuda_batchMatMul
 *   JM  = alpha-Dragon-v1.2/src/z/dragon/engine/cuda/impl/math
 *
 * Conventions shared by all entry points (same as the reference):
 *   - Letters follow the reference: N = rows of C, M = columns of C, K = contraction.
 *   - Row-major FP32.  Addresses are device pointers owned by the caller, 16-byte
 *     aligned; no caller memory is freed or retained here.  The one thing the library allocates:
 *     for large products (K from 768 on), for products with few tiles and a long K (at most two
 *     64 x 64 tiles of C per compute unit) and for their split-K forms the first call on a stream
 *     makes a 32 MiB workspace (one hipMalloc, and a small kernel on that stream that clears its
 *     counters; nothing waits and no other stream is touched) that later calls on the same stream
 *     handle reuse (partial tiles of workgroups that share the K range of a tile pass through it).
 *     The workspace belongs to the stream: dragon_Cuda_deleteStream / deleteStreams give it back,
 *     dragon_gemm_release_workspaces() below gives all of them back.  At most 64 exist at a time
 *     (a launch on a 65th stream runs the ordinary kernel), and none is made or used while the
 *     stream is being captured into a graph -- such a call runs the ordinary kernel instead, as
 *     does every call when the allocation fails.
 *   - C is overwritten (no alpha/beta).  Padded rows/columns of C receive exact zeros.
 *   - streams[0..length) are valid stream handles, 1 <= length <= 10.  Work is issued
 *     asynchronously on streams[0]; the other handles are left idle (the caller joins
 *     all of them into streams[0] anyway).  The call returns without waiting.
 *   - Callable from any host thread; the only host-side state is the table of those
 *     workspaces (behind a mutex) and per-kernel occupancy figures cached on first use.
 *   - Errors: hipErrorInvalidValue (1) for a null address, a non-positive dimension, a
 *     stream count outside 1..10, a dimension that violates the x4 padding contract, or
 *     a misaligned address, or a size beyond the limits below; otherwise the launch
 *     status.
 *   - Limits: a 2-D C holds at most 2^31-1 floats, and no row pitch (K, M, N, AK, AN,
 *     CM as the layout has them) exceeds 2 097 150 floats: inside a tile the kernels
 *     address with 32-bit byte offsets, 256 rows of pitch at most.
 */
#ifndef DRAGON_HIP_GEMM_H
#define DRAGON_HIP_GEMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- 2-D products: N, M, K are multiples of 4 (caller-padded with zeros) -------- */

/* C[N,M] = A[N,K] * B[K,M].
 * Replaces Java_z_dragon_engine_cuda_impl_math_Cuda_1matMul_matMul (MM/A.cu:41-56,
 * declared JM/Cuda_matMul.java:109) and its dispatcher matMul4x (MM/matMul.cuh:47-119). */
int dragon_Cuda_matMul_matMul(const int64_t* streams, int32_t length,
                              int64_t dA, int64_t dB, int64_t dC,
                              int32_t N, int32_t M, int32_t K);

/* C[N,M] = A[K,N]^T * B[K,M].
 * Replaces ..._Cuda_1matMul_matMulT1 (MM/A.cu:90-105, JM/Cuda_matMul.java:206,
 * dispatcher MM/matMulT1.cuh:42-89). */
int dragon_Cuda_matMul_matMulT1(const int64_t* streams, int32_t length,
                                int64_t dA, int64_t dB, int64_t dC,
                                int32_t N, int32_t M, int32_t K);

/* C[N,M] = A[N,K] * B[M,K]^T.
 * Replaces ..._Cuda_1matMul_matMulT2 (MM/A.cu:139-154, JM/Cuda_matMul.java:315,
 * dispatcher MM/matMulT2.cuh:44-107). */
int dragon_Cuda_matMul_matMulT2(const int64_t* streams, int32_t length,
                                int64_t dA, int64_t dB, int64_t dC,
                                int32_t N, int32_t M, int32_t K);

/* ---- split-K stage 1: K is cut into GridZ slices of K_slice = (K/GridZ)>>3<<3, the
 * last slice takes the remainder; slice 0 is written to C, slice z >= 1 to
 * Cbuf + (z-1)*N*M.  Cbuf holds (GridZ-1)*N*M floats.  GridZ >= 1.
 * What the caller may rely on is the SUM: C + sum over the GridZ-1 partials of Cbuf is the
 * product, and every float of C and Cbuf is written.  Where the library estimates that the
 * unsplit product is faster than the slices plus their fold (its balanced kernel deals equal
 * shares of K to the compute units by itself; e.g. 1000 x 780 x 1532 with GridZ 2), it declines
 * the split: the whole product goes to C and Cbuf gets exact zeros, in the same launch, so that
 * SKbuf_summary afterwards leaves C as it is.  The same goes for a product whose C has at most 32
 * rows or columns beside a long other side (8 x 4096 x 4096 with GridZ 16): the kernels for such
 * shapes share K among their wavefronts and workgroups themselves.  Where the split wins (256 x 256 x 131072 in 128 slices) the slices are
 * computed as asked.
 * The library remembers a declined call (stream, Cbuf, C, GridZ-1, N*M): the SKbuf_summary call
 * with exactly these arguments on streams[0] -- the one the reference's host issues next,
 * CudaFloat32EngineBase.java:1565-1588 -- would add zeros and returns without launching
 * anything.  The memory is forgotten at its first use, when any entry point of this library
 * writes to or frees memory that overlaps that C or Cbuf, and when 64 later declined calls
 * exist; a fold with other arguments, or after the entry is gone, runs as usual and finds the
 * zeros.  Only writes that bypass this library (another library's kernels writing into Cbuf
 * between the two calls) are invisible to it: a host that does that must not rely on the fold.
 * Replace ..._Cuda_1matMul_matMulSK / matMulT1SK / matMulT2SK (MM/A.cu:59-79, 108-128,
 * 157-178; JM/Cuda_matMul.java:137, 251, 343; slice rule MM/micro.cuh:92 and
 * MM/matMulSK_kernel.cuh:124-131). */
int dragon_Cuda_matMul_matMulSK(const int64_t* streams, int32_t length, int32_t GridZ,
                                int64_t dA, int64_t dB, int64_t dC, int64_t dCbuf,
                                int32_t N, int32_t M, int32_t K);
int dragon_Cuda_matMul_matMulT1SK(const int64_t* streams, int32_t length, int32_t GridZ,
                                  int64_t dA, int64_t dB, int64_t dC, int64_t dCbuf,
                                  int32_t N, int32_t M, int32_t K);
int dragon_Cuda_matMul_matMulT2SK(const int64_t* streams, int32_t length, int32_t GridZ,
                                  int64_t dA, int64_t dB, int64_t dC, int64_t dCbuf,
                                  int32_t N, int32_t M, int32_t K);

/* ---- split-K stage 2: C[i] += sum_{p < part} Cbuf[p*sizeC + i], Kahan-compensated,
 * p ascending, starting from the value already in C.  sizeC is a multiple of 4.
 * Bit-identical to the reference's operation order.
 * Replaces ..._Cuda_1matMul_SKbuf_1summary (MM/A.cu:20-30, JM/Cuda_matMul.java:69,
 * kernel MM/SKbufsum.cuh:29-81). */
int dragon_Cuda_matMul_SKbuf_summary(int64_t stream, int64_t dCbuf, int64_t dC,
                                     int32_t part, int32_t sizeC);

/* Gives back every per-stream workspace the library holds (see the conventions above), on every
 * device, after synchronising that device; returns how many there were.  For hosts that keep their
 * streams for the life of the process and want the memory back in between; streams that run a large or
 * few-tile product again get a new workspace.  No counterpart in the reference, whose natives own no
 * device memory (engine-cuda-base/Cuda/Cuda/Cuda_Stream.cuh:55-75 destroys a stream and that is all). */
int32_t dragon_gemm_release_workspaces(void);

/* ---- the complete split-K product without any allocation: stage 1 as above (variant 0 = A*B,
 * 1 = A^T*B, 2 = A*B^T), the GridZ-1 partial products in a workspace that is part of the library's
 * device image instead of a caller's Cbuf, then the Kahan fold of stage 2 into C, all on streams[0].
 * Every bit of C equals what matMulSK / matMulT1SK / matMulT2SK + SKbuf_summary leave.
 * No counterpart in the reference (whose Java side allocates Cbuf per call,
 * CudaFloat32EngineBase.java:1565-1583); it is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid device allocation.  Neither this call nor anything
 * it runs allocates or frees memory, and it enqueues kernels only (no memset).
 * Limit: (GridZ-1)*N*M <= 8 388 608 floats (32 MiB); beyond it the call returns hipErrorOutOfMemory (2)
 * and says so on stderr, without launching anything.  The same array holds, behind the partials, the
 * 32 MiB of arrival counters and pieces of shared tiles that the balanced kernel needs (the other entry
 * points keep those per stream in allocated memory), so that this call runs the very kernels they run:
 * 64 MiB in all, held once per GPU until the process ends.
 * All calls on one GPU share that workspace, which keeps the last call's partials: two calls that
 * overlap in time on one GPU (different streams or threads) race and must be ordered by the caller.
 * The first call on a device looks up the workspace's address (which may load the library's device
 * code); make that call outside a graph capture. */
int dragon_Cuda_matMul_matMulSK_static(const int64_t* streams, int32_t length, int32_t variant,
                                       int32_t GridZ, int64_t dA, int64_t dB, int64_t dC,
                                       int32_t N, int32_t M, int32_t K);

/* ---- bias row -------------------------------------------------------------------- */

/* Y[i] = alpha*X1[i] + beta*X2[i % row_lengthv] + gamma for i < lengthv, then elements whose
 * column (i % stride) is >= width are multiplied by zero.  X2 is a row vector of row_lengthv
 * floats broadcast over the rows of X1; Y may alias X1.  lengthv, row_lengthv and stride are
 * multiples of 4, row_lengthv a multiple of stride, lengthv a multiple of row_lengthv.
 * Issued on `stream`.  With (alpha, beta, gamma) = (1, 1, 0) this is the bias addition of
 * matMul_biased / fullconnect_biased
 * (alpha-Dragon-v1.2/src/z/dragon/engine/cuda/CudaFloat32EngineBase.java:1626-1634, 1676-1680).
 * Replaces Java_z_dragon_engine_cuda_impl_math_Cuda_1function_linear_1dual2D_1row
 * (engine-cuda-base/Cuda_function/Cuda_function/A.cu:287-303, declared JM/Cuda_function.java:489,
 * kernel .../type1_linear_dual2D_row.cuh:43-84). */
int dragon_Cuda_function_linear_dual2D_row(int64_t stream, int64_t dX1, int64_t dX2,
                                           int32_t row_lengthv, float alpha, float beta,
                                           float gamma, int64_t dY, int32_t lengthv,
                                           int32_t width, int32_t stride);

/* C[N,M] = A[N,K] * B[K,M], then C[i][j] += Bias[j] for the first lengthv/M rows and j < width,
 * in one launch: the bias row is added to the accumulators before they are stored.  Every bit
 * of C equals what dragon_Cuda_matMul_matMul followed by
 * dragon_Cuda_function_linear_dual2D_row(streams[0], C, Bias, M, 1, 1, 0, C, lengthv, width, M)
 * leaves.  lengthv is a multiple of M with lengthv/M <= N (the unpadded row count), width <= M.
 * No native counterpart in the reference, which issues the two launches above from Java
 * (CudaFloat32EngineBase.java:1594-1638); a host that owns that method calls this instead. */
int dragon_Cuda_matMul_matMul_biased(const int64_t* streams, int32_t length,
                                     int64_t dA, int64_t dB, int64_t dC, int64_t dBias,
                                     int32_t N, int32_t M, int32_t K,
                                     int32_t lengthv, int32_t width);

/* ---- dimension swap (the layout step either side of the batched products) ---------
 * Y = X with dimensions dimIndex1 and dimIndex2 exchanged.  Tensors are row-major with the last
 * dimension stored at strideX / strideY floats (the width rounded up to 4, pad zero); `length` is
 * the number of logical elements; Xdim0 = length / (the other X dims).  When the swap leaves the
 * last dimension alone strideX == strideY and whole padded rows move; otherwise Y's pad columns
 * are written as zeros.  X and Y must not overlap.  Issued on `stream`.
 * Replace Java_z_dragon_engine_cuda_impl_Cuda_1expk2_transpose2D / 3D / 4D
 * (engine-cuda-base/Cuda_expk2/Cuda_expk2/Cuda_transpose.cuh:13-75), called from
 * CudaFloat32EngineBase.transpose (alpha-Dragon-v1.2/src/z/dragon/engine/cuda/CudaFloat32EngineBase.java:1343-1375). */
int dragon_Cuda_expk2_transpose2D(int64_t stream, int64_t dX, int64_t dY,
                                  int32_t Xdim1, int32_t Ydim1,
                                  int32_t strideX, int32_t strideY, int32_t length);
int dragon_Cuda_expk2_transpose3D(int64_t stream, int64_t dX, int64_t dY,
                                  int32_t Xdim1, int32_t Xdim2, int32_t Ydim1, int32_t Ydim2,
                                  int32_t dimIndex1, int32_t dimIndex2,
                                  int32_t strideX, int32_t strideY, int32_t length);
int dragon_Cuda_expk2_transpose4D(int64_t stream, int64_t dX, int64_t dY,
                                  int32_t Xdim1, int32_t Xdim2, int32_t Xdim3,
                                  int32_t Ydim1, int32_t Ydim2, int32_t Ydim3,
                                  int32_t dimIndex1, int32_t dimIndex2,
                                  int32_t strideX, int32_t strideY, int32_t length);

/* ---- between the two batched products of an attention block ------------------------ */

/* Y[i] = alpha*X[i] + beta for i < lengthv, elements whose column (i % stride) is >= width
 * multiplied by zero.  Y may alias X.  Engine.linear / Engine.sdiv (X / C = linear(1/C, X, 0)).
 * Replaces Java_z_dragon_engine_cuda_impl_math_Cuda_1function_linear2D
 * (engine-cuda-base/Cuda_function/Cuda_function/A.cu:170-183). */
int dragon_Cuda_function_linear2D(int64_t stream, float alpha, int64_t dX, float beta, int64_t dY,
                                  int32_t lengthv, int32_t width, int32_t stride);

/* Y = softmax(scale * X) over each of the field_length fields of row_lengthv floats (a multiple
 * of stride; only columns < width of every memory row take part, the pad of Y gets zeros):
 * y = exp(s*x - max) / sum(exp(s*x - max)).  Y may alias X.  One launch; scale = 1 gives
 * Engine.softmax, scale = 1/C folds the sdiv that precedes it in an attention block.
 * No native of this shape in the reference, which runs Cuda_reduce.row_max, Cuda_reduce.row_softmax
 * and Cuda_function.div2D_field with two temporary buffers
 * (alpha-Dragon-v1.2/src/z/dragon/engine/cuda/CudaFloat32EngineBase.java:5738-5774); a host that owns
 * that method calls this instead. */
int dragon_Cuda_reduce_softmax2D(int64_t stream, int64_t dX, int64_t dY, int32_t field_length,
                                 int32_t row_lengthv, int32_t width, int32_t stride, float scale);

/* The attention block in one launch: per (image n, head h)
 *     Y[n, h, i, :] = sum_j softmax_j(scale * <Q[n, h, i, :], K[n, h, j, :]>) * V[n, h, j, :]
 * for QL queries and VL keys, head dimensions dK4 (Q, K) and dV4 (V, Y), both multiples of 4 and at
 * most 256 (pad columns of Q, K, V zero, as everywhere; the pad columns of Y get zeros).  Above 128 a
 * query's registers fill the register file and one workgroup runs per compute unit: there the call is
 * level with the three-launch chain (batchMatMulT2, softmax2D with the scale, batchMatMul) at 256 and
 * 10 - 20 % ahead of it at 160 ... 224 (only the 32-wide blocks of the head dimension that hold anything
 * are multiplied), and saves that chain's score matrix; up to 128 it is 1.4 - 1.9 times faster than the chain.
 * head_inner = 0: tensors laid out [N, head, L, d4] -- the operands of the reference's
 *                 batchMatMulT2 / batchMatMul after its transpose(1, 2);
 * head_inner = 1: tensors laid out [N, L, head, d4] (= [N, L, head*d4]) -- as the layer holds them
 *                 before that transpose; Y comes out in the layout the block returns, so the four
 *                 transposes of the block are not needed either.
 * The score matrix is never stored.  No native of this shape in the reference, which runs
 * batchMatMulT2, linear2D (sdiv), row_max, row_softmax, div2D_field, batchMatMul and four transposes
 * (alpha-Dragon-v1.2/src/z/dragon/nn/unit/complex/block/ChannelMHA.java:66-83); a host that owns that
 * block calls this instead when the head dimensions fit (and the next entry when a mask is set).  Work goes
 * to streams[0]. */
int dragon_Cuda_attention_forward(const int64_t* streams, int32_t length, int64_t dQ, int64_t dK, int64_t dV,
                                  int64_t dY, int32_t N, int32_t head, int32_t QL, int32_t VL, int32_t dK4,
                                  int32_t dV4, int32_t head_inner, float scale);

/* The same with the block's mask: the probabilities are multiplied by a tensor AFTER the softmax,
 *     Y[n, h, i, :] = sum_j softmax_j(...)[j] * M[.., i, j] * V[n, h, j, :]
 * which is what `if (mask != null) P = mask.forward(P)` does for a mask unit that multiplies element by
 * element (a dropout pattern, a causal 0/1 pattern; ChannelMHA.java:75-76).  dMask: rows of mask_pitch floats
 * (a multiple of 4, >= VL), QL rows per slice; mask_per_head = 0: one [QL, mask_pitch] mask for every
 * (image, head), 1: [N, head, QL, mask_pitch].  Every other argument as above. */
int dragon_Cuda_attention_forward_masked(const int64_t* streams, int32_t length, int64_t dQ, int64_t dK, int64_t dV,
                                         int64_t dMask, int64_t dY, int32_t N, int32_t head, int32_t QL, int32_t VL,
                                         int32_t dK4, int32_t dV4, int32_t head_inner, float scale,
                                         int32_t mask_pitch, int32_t mask_per_head);

/* ---- batched products (grid depth = Batch) --------------------------------------- */

/* C[b][N,M] = A[b][N,AK] * B[b][BK,M], k < BK.  M and AK are multiples of 4, N and BK
 * are arbitrary; batch strides N*AK, BK*M, N*M.  Rows of B from BK on are never read and columns
 * of A from the multiple of 4 at or above BK on neither; the up to three columns of A between BK and
 * that multiple are read and multiplied by zeros, so they must hold finite values (they are zeros in
 * the engine's layout).
 * Replaces ..._Cuda_1batchMatMul_batchMatMul and batchMatMul_texture (BMM/A.cu:20-62,
 * JM/Cuda_batchMatMul.java:90,137, dispatcher BMM/batchMatMul.cuh:48-254).  The texture
 * entry is the same computation (textures only served the reference's edge tiles). */
int dragon_Cuda_batchMatMul_batchMatMul(const int64_t* streams, int32_t length,
                                        int64_t dA, int64_t dB, int64_t dC,
                                        int32_t Batch, int32_t N, int32_t M,
                                        int32_t BK, int32_t AK);
int dragon_Cuda_batchMatMul_batchMatMul_texture(const int64_t* streams, int32_t length,
                                                int64_t dA, int64_t dB, int64_t dC,
                                                int32_t Batch, int32_t N, int32_t M,
                                                int32_t BK, int32_t AK);

/* C[b][CN,M] = A[b][K,AN]^T * B[b][K,M].  AN and M are multiples of 4, CN <= AN and K
 * are arbitrary; batch strides K*AN, K*M, CN*M.
 * Replaces ..._Cuda_1batchMatMul_batchMatMulT1 (BMM/A.cu:71-89,
 * JM/Cuda_batchMatMul.java:209, dispatcher BMM/batchMatMulT1.cuh:45-155). */
int dragon_Cuda_batchMatMul_batchMatMulT1(const int64_t* streams, int32_t length,
                                          int64_t dA, int64_t dB, int64_t dC,
                                          int32_t Batch, int32_t CN, int32_t AN,
                                          int32_t M, int32_t K);

/* C[b][N,CM] = A[b][N,K] * B[b][BM,K]^T.  CM and K are multiples of 4, N and BM <= CM
 * are arbitrary; columns BM..CM-1 of C are written as zeros; batch strides N*K, BM*K,
 * N*CM.
 * Replaces ..._Cuda_1batchMatMul_batchMatMulT2 and batchMatMulT2_texture
 * (BMM/A.cu:98-143, JM/Cuda_batchMatMul.java:283,327, dispatcher
 * BMM/batchMatMulT2.cuh:48-248). */
int dragon_Cuda_batchMatMul_batchMatMulT2(const int64_t* streams, int32_t length,
                                          int64_t dA, int64_t dB, int64_t dC,
                                          int32_t Batch, int32_t N, int32_t CM,
                                          int32_t BM, int32_t K);
int dragon_Cuda_batchMatMul_batchMatMulT2_texture(const int64_t* streams, int32_t length,
                                                  int64_t dA, int64_t dB, int64_t dC,
                                                  int32_t Batch, int32_t N, int32_t CM,
                                                  int32_t BM, int32_t K);

/* ---- *_mma entries: the reference declares TF32 tensor-core variants
 * (JM/Cuda_matMul.java:163,278,369; JM/Cuda_batchMatMul.java:166,236,355) whose native
 * source is not published and which are off by default.  gfx950 has no reduced-precision
 * FP32 matrix instruction, so these forward to the FP32 path above (results are at least
 * as accurate as TF32). */
int dragon_Cuda_matMul_matMul_mma(const int64_t* streams, int32_t length,
                                  int64_t dA, int64_t dB, int64_t dC,
                                  int32_t N, int32_t M, int32_t K);
int dragon_Cuda_matMul_matMulT1_mma(const int64_t* streams, int32_t length,
                                    int64_t dA, int64_t dB, int64_t dC,
                                    int32_t N, int32_t M, int32_t K);
int dragon_Cuda_matMul_matMulT2_mma(const int64_t* streams, int32_t length,
                                    int64_t dA, int64_t dB, int64_t dC,
                                    int32_t N, int32_t M, int32_t K);
int dragon_Cuda_batchMatMul_batchMatMul_mma(int32_t useTexture,
                                            const int64_t* streams, int32_t length,
                                            int64_t dA, int64_t dB, int64_t dC,
                                            int32_t Batch, int32_t N, int32_t M,
                                            int32_t BK, int32_t AK);
int dragon_Cuda_batchMatMul_batchMatMulT1_mma(const int64_t* streams, int32_t length,
                                              int64_t dA, int64_t dB, int64_t dC,
                                              int32_t Batch, int32_t CN, int32_t AN,
                                              int32_t M, int32_t K);
int dragon_Cuda_batchMatMul_batchMatMulT2_mma(int32_t useTexture,
                                              const int64_t* streams, int32_t length,
                                              int64_t dA, int64_t dB, int64_t dC,
                                              int32_t Batch, int32_t N, int32_t CM,
                                              int32_t BM, int32_t K);

/* ---- host heuristics the Java side keeps as static methods; exported so a non-Java
 * host can reproduce its decisions.
 * blockNum: JM/Cuda_matMul.java:18-38; nstream: JM/Cuda_matMul.java:41-65;
 * streamSize: JM/Cuda_batchMatMul.java:18-42. */
int32_t dragon_Cuda_matMul_blockNum(int32_t N, int32_t M);
int32_t dragon_Cuda_matMul_nstream(int32_t N, int32_t M);
int32_t dragon_Cuda_batchMatMul_streamSize(int32_t N, int32_t M);

#ifdef __cplusplus
}
#endif
#endif /* DRAGON_HIP_GEMM_H */
