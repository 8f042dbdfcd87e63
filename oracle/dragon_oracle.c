/*
 * dragon_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the arithmetic and host heuristics of Dragon-Alpha's FP32
 * matrix-multiplication path.  It is the checker for the HIP kernels: only the
 * test-suite, the smoke check and the benchmark's CPU-baseline leg may load it.
 * Nothing in the shipped library links, loads or falls back to this file.
 *
 * Every function cites the reference file:line it restates (paths relative to
 * source/ in the reference tree; MM = engine-cuda-base/Cuda_matMul/Cuda_matMul,
 * BMM = engine-cuda-base/Cuda_batchMatMul/Cuda_batchMatMul,
 * AJ = alpha-Dragon-v1.2/src/z/dragon).
 *
 * Arithmetic contract of the reference's CPU matmul: every output element
 * accumulates k = 0..K-1 in ascending order in FP32, the multiply and the add
 * rounded separately (C `float` without contraction, Java `float`).  The file
 * must be compiled with -ffp-contract=off and without -ffast-math.  Any loop
 * order that keeps "k ascending per element" is bit-identical to the literal
 * k,i,j loops, which is what the *_fast variants exploit.
 *
 * Pinning status (what checks each function independently of its own formula):
 *   multiply / multiplyT1 / multiplyT2, bmm / bmmT1 / bmmT2 (literal + fast):
 *       pinned -- exact integer-valued inputs against int64 products (bitwise),
 *       identity / one-hot data-movement cases, transpose identities, FP64
 *       products within the forward error bound, literal == fast bitwise.
 *   SK_K_slice / slice bounds: pinned -- enumeration (lengths sum to K, last
 *       slice takes the remainder, multiple of 8) and, where the reference's
 *       micro.cuh builds, the reference's own macro.
 *   SKbuf_summary (Kahan): pinned -- against FP64 sums on adversarial data.
 *   blockNum / nstream / streamSize: pinned -- hand-derived table, brute-force
 *       tile-class decomposition, and the reference's own blockNum where
 *       micro.cuh builds.
 *   gridZ policies (Java float arithmetic): pinned by a hand-derived table of
 *       cases only; beyond that table "parity unpinned" (no JVM here).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define CLONES __attribute__((target_clones("avx2", "default")))

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------ */
/* 2-D products, literal loop order (MM/test.cuh:60-82, Java twins           */
/* alpha-Dragon-v1.2/test/test/cuda/matMul/Cuda_matMul_test.java:31-39,       */
/* Cuda_matMul_test_T1.java:34-41, Cuda_matMul_test_T2.java:31-39).           */
/* C must be zero-initialised by the caller, as in the reference's tests.    */
/* ------------------------------------------------------------------------ */

/* C[N,M] += A[N,K] * B[K,M]                      MM/test.cuh:60-66 */
void oracle_multiply(const float* A, const float* B, float* C, int N, int M, int K) {
    for (int k = 0; k < K; k++)
        for (int i = 0; i < N; i++)
            for (int j = 0; j < M; j++)
                C[(size_t)i * M + j] += A[(size_t)i * K + k] * B[(size_t)k * M + j];
}

/* C[N,M] += A[K,N]^T * B[K,M]                    MM/test.cuh:68-74 */
void oracle_multiplyT1(const float* A, const float* B, float* C, int N, int M, int K) {
    for (int k = 0; k < K; k++)
        for (int i = 0; i < N; i++)
            for (int j = 0; j < M; j++)
                C[(size_t)i * M + j] += A[(size_t)k * N + i] * B[(size_t)k * M + j];
}

/* C[N,M] += A[N,K] * B[M,K]^T                    MM/test.cuh:76-82 */
void oracle_multiplyT2(const float* A, const float* B, float* C, int N, int M, int K) {
    for (int k = 0; k < K; k++)
        for (int i = 0; i < N; i++)
            for (int j = 0; j < M; j++)
                C[(size_t)i * M + j] += A[(size_t)i * K + k] * B[(size_t)j * K + k];
}

/* ------------------------------------------------------------------------ */
/* Generic strided core used by the fast variants.                           */
/*   C[i*ldc + j] += sum_k A[i*sai + k*sak] * B[k*ldb + j]                    */
/* for k in [k0,k1) ascending, B with unit stride along j.  Blocked over      */
/* (i, j) for cache reuse; the k order seen by each element is unchanged.     */
/* ------------------------------------------------------------------------ */
#define IB 48
#define JB 256
#define KB 128

CLONES
static void core_tile(const float* A, size_t sai, size_t sak,
                      const float* B, size_t ldb,
                      float* C, size_t ldc,
                      int i0, int i1, int j0, int j1, int k0, int k1) {
    for (int kb = k0; kb < k1; kb += KB) {
        int ke = kb + KB < k1 ? kb + KB : k1;
        for (int i = i0; i < i1; i++) {
            float* __restrict__ c = C + (size_t)i * ldc;
            for (int k = kb; k < ke; k++) {
                const float a = A[(size_t)i * sai + (size_t)k * sak];
                const float* __restrict__ b = B + (size_t)k * ldb;
                for (int j = j0; j < j1; j++) c[j] += a * b[j];
            }
        }
    }
}

static void core_parallel(const float* A, size_t sai, size_t sak,
                          const float* B, size_t ldb,
                          float* C, size_t ldc,
                          int rows, int cols, int k0, int k1) {
    int nib = (rows + IB - 1) / IB, njb = (cols + JB - 1) / JB;
    long ntile = (long)nib * njb;
#pragma omp parallel for schedule(dynamic, 1)
    for (long t = 0; t < ntile; t++) {
        int ib = (int)(t / njb), jb = (int)(t % njb);
        int i0 = ib * IB, i1 = i0 + IB < rows ? i0 + IB : rows;
        int j0 = jb * JB, j1 = j0 + JB < cols ? j0 + JB : cols;
        core_tile(A, sai, sak, B, ldb, C, ldc, i0, i1, j0, j1, k0, k1);
    }
}

/* out[c*rows + r] = in[r*cols + c] */
static float* transpose_copy(const float* in, int rows, int cols) {
    float* out = (float*)malloc((size_t)rows * cols * sizeof(float));
    if (!out) return NULL;
#pragma omp parallel for schedule(static)
    for (int rb = 0; rb < rows; rb += 32)
        for (int cb = 0; cb < cols; cb += 32)
            for (int r = rb; r < rb + 32 && r < rows; r++)
                for (int c = cb; c < cb + 32 && c < cols; c++)
                    out[(size_t)c * rows + r] = in[(size_t)r * cols + c];
    return out;
}

/* variant: 0 = A*B, 1 = A^T*B, 2 = A*B^T.  Bit-identical to the literal loops
 * above (same per-element operation sequence), cache-blocked and row-parallel. */
int oracle_matMul_fast(int variant, const float* A, const float* B, float* C,
                       int N, int M, int K) {
    if (variant == 0) {
        core_parallel(A, (size_t)K, 1, B, (size_t)M, C, (size_t)M, N, M, 0, K);
    } else if (variant == 1) {
        core_parallel(A, 1, (size_t)N, B, (size_t)M, C, (size_t)M, N, M, 0, K);
    } else if (variant == 2) {
        float* Bt = transpose_copy(B, M, K); /* Bt[K,M] */
        if (!Bt) return -1;
        core_parallel(A, (size_t)K, 1, Bt, (size_t)M, C, (size_t)M, N, M, 0, K);
        free(Bt);
    } else {
        return -2;
    }
    return 0;
}

/* FP64-accumulate twin: products of two floats are exact in double, the sum is
 * carried in double.  Separates the oracle's own FP32 rounding noise from the
 * device's.  Output is double. */
int oracle_matMul_f64(int variant, const float* A, const float* B, double* C,
                      int N, int M, int K) {
    const float* Bn = B;
    float* Bt = NULL;
    if (variant == 2) { Bt = transpose_copy(B, M, K); if (!Bt) return -1; Bn = Bt; }
    size_t sai = (variant == 1) ? 1 : (size_t)K, sak = (variant == 1) ? (size_t)N : 1;
#pragma omp parallel for schedule(dynamic, 4)
    for (int i = 0; i < N; i++) {
        double* c = C + (size_t)i * M;
        for (int j = 0; j < M; j++) c[j] = 0.0;
        for (int k = 0; k < K; k++) {
            const double a = (double)A[(size_t)i * sai + (size_t)k * sak];
            const float* b = Bn + (size_t)k * M;
            for (int j = 0; j < M; j++) c[j] += a * (double)b[j];
        }
    }
    free(Bt);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Batched products, literal (BMM/test.cuh:95-138).  Strides follow the       */
/* reference exactly: padded AK/AN/CM, unpadded BK/CN/BM.                    */
/* ------------------------------------------------------------------------ */

/* C[b][N,CM] += A[b][N,AK] * B[b][BK,CM], k < BK        BMM/test.cuh:95-108 */
void oracle_bmm(const float* A, const float* B, float* C,
                int Batch, int N, int CM, int BK, int AK) {
    for (int b = 0; b < Batch; b++)
        for (int k = 0; k < BK; k++)
            for (int i = 0; i < N; i++)
                for (int j = 0; j < CM; j++)
                    C[((size_t)b * N + i) * CM + j] +=
                        A[((size_t)b * N + i) * AK + k] * B[((size_t)b * BK + k) * CM + j];
}

/* C[b][CN,CM] += A[b][K,AN]^T * B[b][K,CM], i < CN      BMM/test.cuh:110-123 */
void oracle_bmmT1(const float* A, const float* B, float* C,
                  int Batch, int CN, int AN, int CM, int K) {
    for (int b = 0; b < Batch; b++)
        for (int k = 0; k < K; k++)
            for (int i = 0; i < CN; i++)
                for (int j = 0; j < CM; j++)
                    C[((size_t)b * CN + i) * CM + j] +=
                        A[((size_t)b * K + k) * AN + i] * B[((size_t)b * K + k) * CM + j];
}

/* C[b][N,CM] += A[b][N,K] * B[b][BM,K]^T, j < BM        BMM/test.cuh:125-138 */
void oracle_bmmT2(const float* A, const float* B, float* C,
                  int Batch, int N, int CM, int BM, int K) {
    for (int b = 0; b < Batch; b++)
        for (int k = 0; k < K; k++)
            for (int i = 0; i < N; i++)
                for (int j = 0; j < BM; j++)
                    C[((size_t)b * N + i) * CM + j] +=
                        A[((size_t)b * N + i) * K + k] * B[((size_t)b * BM + j) * K + k];
}

/* Fast batched twins (bit-identical; batches in parallel on top of the tiles). */
int oracle_bmm_fast(int variant, const float* A, const float* B, float* C,
                    int Batch, int d0, int d1, int d2, int d3) {
    for (int b = 0; b < Batch; b++) {
        if (variant == 0) {          /* (N, CM, BK, AK) */
            int N = d0, CM = d1, BK = d2, AK = d3;
            core_parallel(A + (size_t)b * N * AK, (size_t)AK, 1,
                          B + (size_t)b * BK * CM, (size_t)CM,
                          C + (size_t)b * N * CM, (size_t)CM, N, CM, 0, BK);
        } else if (variant == 1) {   /* (CN, AN, CM, K) */
            int CN = d0, AN = d1, CM = d2, K = d3;
            core_parallel(A + (size_t)b * K * AN, 1, (size_t)AN,
                          B + (size_t)b * K * CM, (size_t)CM,
                          C + (size_t)b * CN * CM, (size_t)CM, CN, CM, 0, K);
        } else if (variant == 2) {   /* (N, CM, BM, K) */
            int N = d0, CM = d1, BM = d2, K = d3;
            float* Bt = transpose_copy(B + (size_t)b * BM * K, BM, K); /* [K,BM] */
            if (!Bt) return -1;
            core_parallel(A + (size_t)b * N * K, (size_t)K, 1, Bt, (size_t)BM,
                          C + (size_t)b * N * CM, (size_t)CM, N, BM, 0, K);
            free(Bt);
        } else {
            return -2;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Split-K                                                                   */
/* ------------------------------------------------------------------------ */

/* K_slice = (K / GZ) >> 3 << 3                              MM/micro.cuh:92 */
int oracle_SK_K_slice(int K, int GZ) { return ((K / GZ) >> 3) << 3; }

/* Slice z covers [z*K_slice, (z+1)*K_slice), the last slice runs to K
 * (MM/matMulSK_kernel.cuh:124-127). */
void oracle_SK_bounds(int K, int GZ, int z, int* k_start, int* k_end) {
    int ks = oracle_SK_K_slice(K, GZ);
    *k_start = ks * z;
    *k_end = (z != GZ - 1) ? (*k_start + ks) : K;
}

/* Stage 1 of the two-stage split-K product: slice 0 -> C, slice z>=1 ->
 * Cbuf[(z-1)*N*M ...] (MM/matMulSK_kernel.cuh:130-131, MM/A.cu:59-79,108-128,
 * 157-178).  Each slice is a sequential FP32 sum over its own k range. */
int oracle_matMulSK(int variant, int GZ, const float* A, const float* B,
                    float* C, float* Cbuf, int N, int M, int K) {
    const float* Bn = B;
    float* Bt = NULL;
    if (variant == 2) { Bt = transpose_copy(B, M, K); if (!Bt) return -1; Bn = Bt; }
    size_t sai = (variant == 1) ? 1 : (size_t)K, sak = (variant == 1) ? (size_t)N : 1;
    size_t sizeC = (size_t)N * M;
    for (int z = 0; z < GZ; z++) {
        int ks, ke;
        oracle_SK_bounds(K, GZ, z, &ks, &ke);
        float* dst = (z == 0) ? C : Cbuf + (size_t)(z - 1) * sizeC;
        memset(dst, 0, sizeC * sizeof(float));
        core_parallel(A, sai, sak, Bn, (size_t)M, dst, (size_t)M, N, M, ks, ke);
    }
    free(Bt);
    return 0;
}

/* Stage 2: C[i] += sum_p Cbuf[p*sizeC + i] with Kahan compensation, p ascending
 * (MM/SKbufsum.cuh:37-67).  The operation order is restated literally. */
void oracle_SKbuf_summary(const float* Cbuf, float* C, int part, int sizeC) {
    for (int i = 0; i < sizeC; i++) {
        float v = C[i];
        float c = 0.0f;
        for (int p = 0; p < part; p++) {
            float vbuf = Cbuf[(size_t)p * sizeC + i];
            vbuf -= c;
            float t = v + vbuf;
            c = (t - v) - vbuf;
            v = t;
        }
        C[i] = v;
    }
}

/* ------------------------------------------------------------------------ */
/* Host heuristics                                                           */
/* ------------------------------------------------------------------------ */

static int tile_classes(int N, int count_128_multiples) {
    /* number of tile-class rows after carving N into 128,64,32,16,8,4 */
    int bn = 0;
    for (;;) {
        if (N > 127) bn += count_128_multiples ? (N >> 7) : 1;
        N &= 127; if (N == 0) break;
        if (N > 63) bn += 1; N &= 63; if (N == 0) break;
        if (N > 31) bn += 1; N &= 31; if (N == 0) break;
        if (N > 15) bn += 1; N &= 15; if (N == 0) break;
        if (N > 7) bn += 1; N &= 7; if (N == 0) break;
        if (N > 3) bn += 1; break;
    }
    return bn;
}

/* AJ/engine/cuda/impl/math/Cuda_matMul.java:18-38 (twin: MM/micro.cuh:94-116) */
int oracle_blockNum(int N, int M) { return tile_classes(N, 1) * tile_classes(M, 1); }

/* AJ/engine/cuda/impl/math/Cuda_matMul.java:41-65 */
int oracle_nstream(int N, int M) {
    int sn = ((N & (N - 1)) == 0) ? 1 : tile_classes(N, 0);
    int sm = ((M & (M - 1)) == 0) ? 1 : tile_classes(M, 0);
    int size = sn * sm;
    return size < 10 ? size : 10;
}

/* AJ/engine/cuda/impl/math/Cuda_batchMatMul.java:18-42 */
int oracle_streamSize(int N, int M) {
    int sn = ((N & (N - 1)) == 0) ? 1 : tile_classes(N, 0);
    int sm = ((M & (M - 1)) == 0) ? 1 : tile_classes(M, 0);
    int size = sn * sm;
    if (size < 1) size = 1;
    return size < 10 ? size : 10;
}

/* AJ/engine/cuda/CudaFloat32EngineBase.java:70-74: pad to x4 (<=32) or x8,
 * clip to [16,128]. */
int oracle_smooth_maxPart(int x) {
    if (x <= 32) x = ((x + 3) >> 2) << 2; else x = ((x + 7) >> 3) << 3;
    if (x < 16) x = 16;
    if (x > 128) x = 128;
    return x;
}

/* Split-K decision of CudaFloat32EngineBase.{matMul, matMul_biased, matMulT1,
 * matMulT2} (AJ/engine/cuda/CudaFloat32EngineBase.java:1519-1562, 1594-1660,
 * 1736-1779, 1855-1896), Java float arithmetic restated in C float.
 *   kind: 0 = matMul, 1 = matMulT1, 2 = matMulT2, 3 = matMul_biased
 * Returns GridZ (1 = no split).  Defaults: threshold 512; minBlock 1.2f for
 * matMul / 1.14f for T1; maxBlock 4.0f; maxPart = smooth(SM).  matMulT2 reads
 * the matMul constants for its threshold test and clamp, as the reference does. */
int oracle_gridZ(int kind, int N, int M, int K, int SM,
                 int threshold, float minBlock, float maxBlock, int maxPart) {
    float fGridZ = 1.0f;
    int bself = 1;
    if (K >= threshold) {
        float kterm = (float)K / ((float)K + 1024.0f);
        float expect;
        if (kind == 0) expect = minBlock + 0.4f * (float)K / ((float)K + 1024.0f);
        else expect = minBlock + kterm;
        if (kind == 0 || kind == 3) {
            bself = oracle_blockNum(N, M);
            if ((float)bself < (float)SM * expect) {
                int b1 = oracle_blockNum(K, M), b2 = oracle_blockNum(N, K);
                fGridZ = (float)(b1 + b2) / ((float)bself * 2.0f);
            }
        } else if (kind == 1) {
            bself = oracle_blockNum(N, M);
            if ((float)bself < (float)SM * expect) {
                int b0 = oracle_blockNum(K, N), b2 = oracle_blockNum(K, M);
                fGridZ = (float)(b0 + b2) / ((float)bself * 2.0f);
            }
        } else {
            bself = oracle_blockNum(N, K); /* the reference tests blockNum(N,K) here */
            if ((float)bself < (float)SM * expect) {
                int b0 = oracle_blockNum(N, M), b1 = oracle_blockNum(K, M);
                fGridZ = (float)(b1 + bself) / ((float)b0 * 2.0f);
            }
        }
    }
    if (fGridZ < 1.8f) return 1;
    int GridZ = (int)fGridZ;
    int GridZ2 = K >> 8;
    if (GridZ > GridZ2) GridZ = GridZ2;
    float coef = (float)K / ((float)K + 4096.0f);
    int GridZ3 = (int)((float)SM * maxBlock * coef / (float)bself);
    if (GridZ > GridZ3) GridZ = GridZ3;
    if (GridZ < 2) GridZ = 2; else GridZ = ((GridZ + 3) >> 2) << 2;
    if (GridZ > maxPart) GridZ = maxPart;
    return GridZ;
}

/* ------------------------------------------------------------------------ */
/* Bias row                                                                  */
/* ------------------------------------------------------------------------ */

/* Y[i] = alpha*X1[i] + beta*X2[i % row_lengthv] + gamma, then the element is multiplied by
 * the 0/1 flag "column (i % stride) < width"
 * (engine-cuda-base/Cuda_function/Cuda_function/type1_linear_dual2D_row.cuh:43-66,
 * within_width: Cuda_function/micro.cuh:61-65).  Each product and sum is rounded to float
 * on its own (this file is built with contraction off); the reference's compiler may fuse a
 * product into a sum, which changes nothing for (alpha, beta, gamma) = (1, 1, 0), the bias
 * addition of matMul_biased (CudaFloat32EngineBase.java:1626-1634).  Y may alias X1. */
void oracle_linear_dual2D_row(const float* X1, const float* X2, int row_lengthv, float alpha,
                              float beta, float gamma, float* Y, int lengthv, int width,
                              int stride) {
    for (int i = 0; i < lengthv; i++) {
        float p1 = alpha * X1[i];
        float p2 = beta * X2[i % row_lengthv];
        float y = (p1 + p2) + gamma;
        y *= ((i % stride) < width) ? 1.0f : 0.0f;
        Y[i] = y;
    }
}

/* ------------------------------------------------------------------------ */
/* Scalar linear map and row softmax                                         */
/* ------------------------------------------------------------------------ */

/* Y[i] = alpha*X[i] + beta, pad columns (i % stride >= width) multiplied by zero
 * (engine-cuda-base/Cuda_function/Cuda_function/type1_linear2D.cuh, within_width: micro.cuh:61-65);
 * product and sum rounded separately. */
void oracle_linear2D(float alpha, const float* X, float beta, float* Y, int lengthv, int width, int stride) {
    for (int i = 0; i < lengthv; i++) {
        float p = alpha * X[i];
        float y = p + beta;
        y *= ((i % stride) < width) ? 1.0f : 0.0f;
        Y[i] = y;
    }
}

/* Softmax of scale*X over each field of row_lengthv floats, logical elements only
 * (column < width of every memory row), pad of Y zero: the result of the reference's sequence
 * M = row_max(X); E = exp(X - M), V = row_sum(E); Y = E / V
 * (alpha-Dragon-v1.2/src/z/dragon/engine/cuda/CudaFloat32EngineBase.java:5753-5771), every step in
 * float, the sum taken left to right.  scale = 1 is Engine.softmax; another value is the sdiv
 * (Engine.java:4002) applied first. */
void oracle_softmax2D(const float* X, float* Y, int field_length, int row_lengthv, int width, int stride,
                      float scale) {
    for (int f = 0; f < field_length; f++) {
        const float* x = X + (size_t)f * row_lengthv;
        float* y = Y + (size_t)f * row_lengthv;
        float m = -INFINITY;
        for (int i = 0; i < row_lengthv; i++)
            if ((i % stride) < width) { float t = x[i] * scale; if (t > m) m = t; }
        float sum = 0.0f;
        for (int i = 0; i < row_lengthv; i++) {
            if ((i % stride) < width) { float t = x[i] * scale; y[i] = expf(t - m); sum += y[i]; }
            else y[i] = 0.0f;
        }
        for (int i = 0; i < row_lengthv; i++) y[i] = y[i] / sum;
    }
}

/* ------------------------------------------------------------------------ */
/* Forward convolution                                                       */
/* ------------------------------------------------------------------------ */

/* Y[n][oh][ow][oc] = sum over fh, fw, ic of X[n][oh*sh-ph+fh][ow*sw-pw+fw][ic] * W[oc][fh][fw][ic],
 * pixels in the padding skipped; logical (unpadded) row-major arrays.  The loop nest and the
 * double-precision accumulator with a final cast to float of the reference's CPU check
 * (ZUTIL-STD-1.2/src/z/util/math/vector/Tense.java:141-171, used by
 * alpha-Dragon-v1.2/test/test/cuda/conv3D/Cuda_conv3D_test.java).  acc32 != 0 accumulates in float,
 * fh, fw, ic ascending, instead: the order-exact twin for integer-valued inputs. */
void oracle_conv3D(const float* X, int IH, int IW, const float* W, int FH, int FW, float* Y, int OH, int OW,
                   int N, int IC, int OC, int sh, int sw, int ph, int pw, int acc32) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++)
        for (int oc = 0; oc < OC; oc++)
            for (int oh = 0; oh < OH; oh++)
                for (int ow = 0; ow < OW; ow++) {
                    const int ih_s = oh * sh - ph, iw_s = ow * sw - pw;
                    double v = 0;
                    float vf = 0.0f;
                    for (int fh = 0; fh < FH; fh++)
                        for (int fw = 0; fw < FW; fw++)
                            for (int ic = 0; ic < IC; ic++) {
                                const int ih = ih_s + fh, iw = iw_s + fw;
                                if (ih < 0 || iw < 0 || ih >= IH || iw >= IW) continue;
                                const float x = X[(((size_t)n * IH + ih) * IW + iw) * IC + ic];
                                const float w = W[(((size_t)oc * FH + fh) * FW + fw) * IC + ic];
                                if (acc32) { float pr = x * w; vf = vf + pr; }
                                else v += (double)x * (double)w;
                            }
                    Y[(((size_t)n * OH + oh) * OW + ow) * OC + oc] = acc32 ? vf : (float)v;
                }
}

/* ------------------------------------------------------------------------ */
/* Dimension swap                                                            */
/* ------------------------------------------------------------------------ */

/* Y[x with entries i1 and i2 exchanged] = X[x] for every logical element, X taken as 4-D
 * (leading dimensions 1 for fewer), the last dimension of X stored at strideX and of Y at
 * strideY floats; Y is not touched outside its logical elements.  Index arithmetic of the
 * reference's general kernel
 * (engine-cuda-base/Cuda_expk2/Cuda_expk2/Cuda_transpose4D.cuh:91-120). */
void oracle_transpose4D(const float* X, float* Y, const int* xdim, int i1, int i2, int strideX,
                        int strideY) {
    int ydim[4] = {xdim[0], xdim[1], xdim[2], xdim[3]};
    ydim[i1] = xdim[i2]; ydim[i2] = xdim[i1];
    const long long Xdim123 = (long long)xdim[1] * xdim[2] * xdim[3], Xdim23 = (long long)xdim[2] * xdim[3];
    const long long length = Xdim123 * xdim[0];
    for (long long index = 0; index < length; index++) {
        int x[4];
        long long res = index;
        x[0] = (int)(res / Xdim123); res -= x[0] * Xdim123;
        x[1] = (int)(res / Xdim23); res -= x[1] * Xdim23;
        x[2] = (int)(res / xdim[3]);
        x[3] = (int)(res - (long long)x[2] * xdim[3]);
        int t = x[i1]; x[i1] = x[i2]; x[i2] = t;
        long long yoffset = (((long long)x[0] * ydim[1] + x[1]) * ydim[2] + x[2]) * ydim[3] + x[3];
        const long long xo = (index / xdim[3]) * strideX + (index % xdim[3]);
        const long long yo = (yoffset / ydim[3]) * strideY + (yoffset % ydim[3]);
        Y[yo] = X[xo];
    }
}

/* ------------------------------------------------------------------------ */
/* Error metrics used by the parity tests                                    */
/* ------------------------------------------------------------------------ */

/* The reference's own acceptance rule, restated literally
 * (ZUTIL-STD-1.2/src/z/util/math/vector/Vector.java:3937-3950): equal elements
 * are same; otherwise |(a-b+MIN)/(a+b+MIN)| < threshold with MIN the smallest
 * positive subnormal float; two NaNs are same.  Returned as a float ratio. */
float oracle_samePercent_relative(const float* a, const float* b, int n, float threshold) {
    const float MINV = 1.401298464324817e-45f; /* Float.MIN_VALUE */
    int same = 0;
    for (int i = 0; i < n; i++) {
        if (a[i] == b[i]) { same++; continue; }
        float dif = fabsf((a[i] - b[i] + MINV) / (a[i] + b[i] + MINV));
        if (dif < threshold) same++;
        else if (isnan(a[i]) && isnan(b[i])) same++;
    }
    return ((float)same) / (float)n;
}
