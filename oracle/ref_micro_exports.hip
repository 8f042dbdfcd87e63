// Export shim for oracle/_ref: compiles the reference's own MM/micro.cuh (found
// through -I, never copied) and exposes its host-side helpers with C linkage.
// Test infrastructure only.
#include <hip/hip_runtime.h>
#include "micro.cuh"

extern "C" {
int ref_blockNum(int N, int M) { return blockNum(N, M); }
int ref_SK_K_slice(int K, int GZ) { return SK_K_slice(K, GZ); }
int ref_matMul_gridZ(int N, int M, int K) { return matMul_gridZ(N, M, K); }
int ref_matMulT2_gridZ(int N, int M, int K) { return matMulT2_gridZ(N, M, K); }
int ref_LOG2(int n) { return LOG2(n); }
}
