/*
 * dragon_hip_engine.h -- C access to the host-side engine mirror (C++ classes named after
 * the reference's Java classes: Engine, EngineCore, CudaFloat32EngineBase, Tensor, Syncer).
 *
 * This is NOT the drop-in boundary (that is dragon_hip_gemm.h / dragon_hip_runtime.h, the
 * level of the reference's JNI functions).  It exposes the layer above it -- the logic the
 * reference keeps in Java -- to hosts without a JVM: tests, benchmarks, C programs.
 * Reference: source/alpha-Dragon-v1.2/src/z/dragon/engine/Engine.java:522-551, 671-676,
 * 824-837, 908-914, 955-1312; EngineCore.java:693-811; cuda/CudaFloat32EngineBase.java:70-92,
 * 649-694, 1008-1054, 1471-2020; Tensor.java:206-239.
 *
 * Errors: functions returning int give 0 on success, else DRAGON_E_*; functions returning a
 * pointer give NULL on failure.  dragon_engine_last_error() describes the last failure of
 * the calling thread; for DRAGON_E_CUDA dragon_engine_last_cuda_code() holds the runtime code.
 */
#ifndef DRAGON_HIP_ENGINE_H
#define DRAGON_HIP_ENGINE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dragon_engine dragon_engine;   /* z.dragon.engine.Engine over CudaFloat32EngineBase */
typedef struct dragon_tensor dragon_tensor;   /* z.dragon.engine.Tensor */

enum {
    DRAGON_OK = 0,
    DRAGON_E_NULL_POINTER = 1,       /* java.lang.NullPointerException */
    DRAGON_E_ILLEGAL_ARGUMENT = 2,   /* java.lang.IllegalArgumentException */
    DRAGON_E_CUDA = 3,               /* z.dragon.engine.cuda.impl.CudaException */
    DRAGON_E_OTHER = 4
};
const char* dragon_engine_last_error(void);
int32_t dragon_engine_last_cuda_code(void);
/* status (DRAGON_OK or DRAGON_E_*) of the calling thread's last engine call: tells the kind of failure of
 * the functions that return a handle (NULL on failure) */
int32_t dragon_engine_last_status(void);

/* alpha.engine.cuda_float32(deviceId, ...) with a stream pool of the given size (32 in the
 * reference's default constructor). */
dragon_engine* dragon_engine_cuda_float32(int32_t device_id, int32_t stream_pool_size);
/* the same with a pinned staging pool of max_trans_buf_size bytes for tensor upload / download
 * (alpha.engine.cuda_float32(deviceId, streamPool, mempool, max_trans_buf_size, check),
 * Alpha.java:770-790; PinnedMempool.java) */
dragon_engine* dragon_engine_cuda_float32_buffered(int32_t device_id, int32_t stream_pool_size,
                                                   int64_t max_trans_buf_size);
/* the same with a device memory pool of max_mem_size bytes behind every tensor and every split-K
 * partial buffer (alpha.engine.cuda_float32(deviceId, alpha.engine.memp1(max_mem_size), max_trans_buf_size),
 * Alpha.java:792-805; engine/memp/Mempool.java, Memp1.java): blocks are recycled by size instead of
 * being allocated and freed on the device per operation.  max_trans_buf_size may be 0. */
dragon_engine* dragon_engine_cuda_float32_pooled(int32_t device_id, int32_t stream_pool_size,
                                                 int64_t max_mem_size, int64_t max_trans_buf_size);
void dragon_engine_delete(dragon_engine* eg);
int dragon_engine_check(dragon_engine* eg, int32_t flag);   /* Engine.check(boolean) */
int dragon_engine_sync(dragon_engine* eg, int32_t flag);    /* Engine.sync(boolean)  */

/* knobs of CudaFloat32EngineBase; names as in Java: "matMul_splitK_threshold",
 * "matMul_splitK_maxPart", "matMulT1_splitK_threshold", "matMulT1_maxPart",
 * "matMulT2_splitK_threshold", "matMulT2_splitK_maxPart", "tf32", "batchMatMul_useTexture",
 * "batchMatMulT2_useTexture", and "multiProcessorCount" (test hook: pretend another unit
 * count and recompute maxPart from it). */
int dragon_engine_set_param(dragon_engine* eg, const char* name, int32_t value);
int32_t dragon_engine_get_param(dragon_engine* eg, const char* name);   /* also "last_gridZ",
    "last_stream_count", "live_blocks", "stream_pool_size", and of the staging pool
    "buf_physical_blocks", "buf_buffered_blocks", "buf_used_mem_size", "buf_total_mem_size_MB"
    (-1 without a pool), and of the device pool "memp_physical_blocks", "memp_buffered_blocks",
    "memp_used_mem_size_KB", "memp_total_mem_size_KB" (-1 without a pool) */

/* split-K decision for padded dims; kind 0 matMul, 1 matMulT1, 2 matMulT2, 3 matMul_biased;
 * 1 = no split */
int32_t dragon_engine_gridZ(dragon_engine* eg, int32_t kind, int32_t N, int32_t M, int32_t K);
/* the same decision as a pure function of the unit count, with the default knobs
 * (threshold 512, maxPart smooth(SM), minBlock 1.2 / 1.14, maxBlock 4.0); needs no device */
int32_t dragon_policy_gridZ(int32_t kind, int32_t N, int32_t M, int32_t K, int32_t SM);
int32_t dragon_policy_smooth_maxPart(int32_t x);

/* tensors */
dragon_tensor* dragon_engine_empty(dragon_engine* eg, const int32_t* dim, int32_t ndim);
dragon_tensor* dragon_engine_zeros(dragon_engine* eg, const int32_t* dim, int32_t ndim);
dragon_tensor* dragon_engine_tensor(dragon_engine* eg, const float* value, int32_t value_length,
                                    const int32_t* dim, int32_t ndim);
int dragon_engine_set(dragon_engine* eg, dragon_tensor* X, const float* value, int32_t value_length);
int dragon_engine_valueOf(dragon_engine* eg, dragon_tensor* ts, float* out, int32_t out_length);
int dragon_engine_delete_tensor(dragon_engine* eg, dragon_tensor* ts);
int dragon_tensor_c(dragon_tensor* ts);                      /* Tensor.c(): wait for its producer */
int32_t dragon_tensor_ndim(const dragon_tensor* ts);
int32_t dragon_tensor_dim(const dragon_tensor* ts, int32_t i);
int32_t dragon_tensor_length(const dragon_tensor* ts);
int32_t dragon_tensor_lengthv(const dragon_tensor* ts);
int32_t dragon_tensor_length_4x(const dragon_tensor* ts);
int64_t dragon_tensor_address(const dragon_tensor* ts);

/* products: op 0 matMul, 1 matMulT1, 2 matMulT2, 3 batchMatMul, 4 batchMatMulT1,
 * 5 batchMatMulT2.  The first form allocates C (likeA picks whose leading dims C copies in
 * the batched forms), the second writes into an existing C. */
dragon_tensor* dragon_engine_product(dragon_engine* eg, int32_t op, int32_t likeA,
                                     dragon_tensor* A, dragon_tensor* B);
int dragon_engine_product_into(dragon_engine* eg, int32_t op, dragon_tensor* C,
                               dragon_tensor* A, dragon_tensor* B);

/* fully connected layer over the last dimension (Engine.java:1315-1470) and the biased
 * 2-D product (Engine.java:998-1039):
 *   op 0 fullconnect(X, W)            Y = X * W                  Bias ignored
 *   op 1 fullconnect_biased(X, W, B)  Y = X * W + B
 *   op 2 fullconnect_deltaX(dY, W)    dX = dY * W^T              X is deltaY, Bias ignored
 *   op 3 fullconnect_deltaW(X, dY)    dW = X^T * dY              W is deltaY, Bias ignored
 *   op 4 matMul_biased(A, B, Bias)    C = A * B + Bias, 2-D only
 * The into-form takes ops 0, 1 and 4. */
dragon_tensor* dragon_engine_fullconnect(dragon_engine* eg, int32_t op, dragon_tensor* X,
                                         dragon_tensor* W, dragon_tensor* Bias);
int dragon_engine_fullconnect_into(dragon_engine* eg, int32_t op, dragon_tensor* Y,
                                   dragon_tensor* X, dragon_tensor* W, dragon_tensor* Bias);

/* Engine.conv3D / conv3D_biased (Engine.java:2076-2204) over NHWC tensors X[N, IH, IW, IC],
 * W[OC, FH, FW, IC] -> Y[N, OH, OW, OC]; Bias (NULL = none) is added to every output pixel.
 * dragon_engine_conv3D creates Y: OH / OW = -1 derive the output size from the padding (rounded down).
 * dragon_engine_conv3D_into writes into Y: ph / pw = -1 derive the padding from the shapes (rounded up).
 * Parameters "conv3D_remode" (default 0 here; the Java default is 1) and "conv3D_biased_fused" (default
 * 1; not a Java field) choose between one launch and the reference's launch sequences. */
dragon_tensor* dragon_engine_conv3D(dragon_engine* eg, dragon_tensor* X, dragon_tensor* W, int32_t OH,
                                    int32_t OW, int32_t sh, int32_t sw, int32_t ph, int32_t pw,
                                    dragon_tensor* Bias);
int dragon_engine_conv3D_into(dragon_engine* eg, dragon_tensor* Y, dragon_tensor* X, dragon_tensor* W,
                              int32_t sh, int32_t sw, int32_t ph, int32_t pw, dragon_tensor* Bias);
/* Cuda_conv3D.GEMM_nstream(GM, OC) (Cuda_conv3D.java:264-285): how many streams the engine checks out */
int32_t dragon_policy_conv3D_GEMM_nstream(int32_t GM, int32_t OC);

/* The attention block of nn/unit/complex/block/ChannelMHA.java:66-83 in one launch: Q[N, QL, KC],
 * K[N, VL, KC], V[N, VL, VC] with `head` heads side by side in the last dimension ->
 * Y[N, QL, VC] = per head softmax(scale * Q.K^T).V; scale = 0 selects the block's 1/sqrt(KC).
 * KC/head and VC/head must be <= 256 and, with several heads, multiples of 4 (IllegalArgumentException
 * otherwise: such shapes take the operator chain).  Not a Java method. */
dragon_tensor* dragon_engine_attention(dragon_engine* eg, dragon_tensor* Q, dragon_tensor* K, dragon_tensor* V,
                                       int32_t head, float scale);
/* The same with the block's mask (ChannelMHA.java:75-76, `P = mask.forward(P)` between the softmax and the second
 * product) for a mask unit that multiplies element by element: Mask[QL, VL] for every image and head, or
 * Mask[N, head, QL, VL]. */
dragon_tensor* dragon_engine_attention_masked(dragon_engine* eg, dragon_tensor* Q, dragon_tensor* K, dragon_tensor* V,
                                              dragon_tensor* Mask, int32_t head, float scale);

/* Engine.linear(inplace, alpha, X, beta): Y = alpha*X + beta (Engine.java:4005-4013); Engine.sdiv(X, C)
 * is linear(1/C, X, 0).  inplace != 0 writes into X and returns X itself. */
dragon_tensor* dragon_engine_linear(dragon_engine* eg, int32_t inplace, float alpha, dragon_tensor* X,
                                    float beta);
/* Engine.softmax(inplace, X, features) (Engine.java:6082-6100): softmax over groups of `features`
 * elements, -1 = the last dimension.  scale = 1 is the Java method; another value computes
 * softmax(scale * X) in the same launch. */
dragon_tensor* dragon_engine_softmax(dragon_engine* eg, int32_t inplace, dragon_tensor* X, int32_t features,
                                     float scale);

/* Engine.transpose(inplace, X, dimIdx1, dimIdx2) (Engine.java:1797-1831): exchange of two dimensions
 * of a 2-D .. 4-D tensor, negative indices count from the end.  inplace != 0 gives X the new shape
 * and memory and returns X itself; equal indices return X (inplace) or a copy. */
dragon_tensor* dragon_engine_transpose(dragon_engine* eg, int32_t inplace, dragon_tensor* X,
                                       int32_t dimIdx1, int32_t dimIdx2);

/* linear2_row / add_row (Engine.java:4185-4207): Y = alpha*X1 + beta*X2 + gamma, the row vector
 * X2 broadcast over the rows of X1.  inplace != 0 writes into X1 and returns X1 itself. */
dragon_tensor* dragon_engine_linear2_row(dragon_engine* eg, int32_t inplace, dragon_tensor* X1,
                                         dragon_tensor* X2, float alpha, float beta, float gamma);

#ifdef __cplusplus
}
#endif
#endif /* DRAGON_HIP_ENGINE_H */
