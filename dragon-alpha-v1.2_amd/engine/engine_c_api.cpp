// C access to the host-side engine mirror (declared in include/dragon_hip_engine.h).
#include <string.h>

#include <string>

#include "../../include/dragon_hip_engine.h"
#include "dragon_engine.hpp"

using namespace dragon;

struct dragon_engine { Engine eg; dragon_engine(int d, int p, int64_t b = 0, int64_t m = 0) : eg(d, p, b, m) {} };
struct dragon_tensor { Tensor* ts; };

namespace {
thread_local std::string g_err;
thread_local int g_cuda_code = 0;
thread_local int g_status = DRAGON_OK;

template <typename F>
int guard(F f) {
    try {
        f();
        return g_status = DRAGON_OK;
    } catch (const NullPointerException& e) {
        g_err = e.what(); return g_status = DRAGON_E_NULL_POINTER;
    } catch (const IllegalArgumentException& e) {
        g_err = e.what(); return g_status = DRAGON_E_ILLEGAL_ARGUMENT;
    } catch (const CudaException& e) {
        g_err = e.what(); g_cuda_code = e.code; return g_status = DRAGON_E_CUDA;
    } catch (const std::exception& e) {
        g_err = e.what(); return g_status = DRAGON_E_OTHER;
    }
}
std::vector<int> dims(const int32_t* dim, int32_t ndim) {
    if (dim == nullptr) throw NullPointerException("dim for Tensor can not be null");
    return std::vector<int>(dim, dim + (ndim > 0 ? ndim : 0));
}
dragon_tensor* wrap(Tensor* t) {
    dragon_tensor* h = new dragon_tensor;
    h->ts = t;
    return h;
}
Tensor* T(dragon_tensor* h) { return h ? h->ts : nullptr; }
const SplitKKnobs kDefaultMM = {512, 0, 1.2f, 4.0f};
const SplitKKnobs kDefaultT = {512, 0, 1.14f, 4.0f};
}  // namespace

extern "C" {

const char* dragon_engine_last_error(void) { return g_err.c_str(); }
int32_t dragon_engine_last_cuda_code(void) { return g_cuda_code; }
int32_t dragon_engine_last_status(void) { return g_status; }

dragon_engine* dragon_engine_cuda_float32(int32_t device_id, int32_t stream_pool_size) {
    dragon_engine* e = nullptr;
    guard([&] { e = new dragon_engine(device_id, stream_pool_size); });
    return e;
}
dragon_engine* dragon_engine_cuda_float32_buffered(int32_t device_id, int32_t stream_pool_size,
                                                   int64_t max_trans_buf_size) {
    dragon_engine* e = nullptr;
    guard([&] { e = new dragon_engine(device_id, stream_pool_size, max_trans_buf_size); });
    return e;
}
dragon_engine* dragon_engine_cuda_float32_pooled(int32_t device_id, int32_t stream_pool_size,
                                                 int64_t max_mem_size, int64_t max_trans_buf_size) {
    dragon_engine* e = nullptr;
    guard([&] {
        if (max_mem_size <= 0) throw IllegalArgumentException("Mempool.max_mem_size must be positive");
        e = new dragon_engine(device_id, stream_pool_size, max_trans_buf_size, max_mem_size);
    });
    return e;
}
void dragon_engine_delete(dragon_engine* eg) { delete eg; }
int dragon_engine_check(dragon_engine* eg, int32_t flag) {
    return guard([&] { if (!eg) throw NullPointerException("engine"); eg->eg.check(flag != 0); });
}
int dragon_engine_sync(dragon_engine* eg, int32_t flag) {
    return guard([&] { if (!eg) throw NullPointerException("engine"); eg->eg.sync(flag != 0); });
}

int dragon_engine_set_param(dragon_engine* eg, const char* name, int32_t v) {
    return guard([&] {
        if (!eg || !name) throw NullPointerException("engine / name");
        CudaFloat32EngineBase& b = eg->eg.engineBase();
        const std::string n(name);
        if (n == "matMul_splitK_threshold") b.matMul_splitK_threshold(v);
        else if (n == "matMul_splitK_maxPart") b.matMul_splitK_maxPart(v);
        else if (n == "matMulT1_splitK_threshold") b.matMulT1_splitK_threshold(v);
        else if (n == "matMulT1_maxPart") b.matMulT1_maxPart(v);
        else if (n == "matMulT2_splitK_threshold") b.matMulT2_splitK_threshold(v);
        else if (n == "matMulT2_splitK_maxPart") b.matMulT2_splitK_maxPart(v);
        else if (n == "tf32") b.tf32(v != 0);
        else if (n == "matMul_biased_fused") b.matMul_biased_fused = (v != 0);
        else if (n == "conv3D_remode") b.conv3D_remode = (v != 0);
        else if (n == "conv3D_Gemm_useTexture") b.conv3D_Gemm_useTexture = (v != 0);
        else if (n == "conv3D_biased_fused") b.conv3D_biased_fused = (v != 0);
        else if (n == "batchMatMul_useTexture") b.batchMatMul_useTexture = (v != 0);
        else if (n == "batchMatMulT2_useTexture") b.batchMatMulT2_useTexture = (v != 0);
        else if (n == "multiProcessorCount") {
            if (v <= 0) throw IllegalArgumentException("multiProcessorCount must be positive");
            b.device().overrideMultiProcessorCount(v);
            b.recomputeMaxParts();
        } else throw IllegalArgumentException("unknown parameter: " + n);
    });
}
int32_t dragon_engine_get_param(dragon_engine* eg, const char* name) {
    int32_t out = -1;
    guard([&] {
        if (!eg || !name) throw NullPointerException("engine / name");
        CudaFloat32EngineBase& b = eg->eg.engineBase();
        const std::string n(name);
        if (n == "matMul_splitK_threshold") out = b.matMul_sk_threshold;
        else if (n == "matMul_splitK_maxPart") out = b.matMul_sk_maxPart;
        else if (n == "matMulT1_splitK_threshold") out = b.matMulT1_sk_threshold;
        else if (n == "matMulT1_maxPart") out = b.matMulT1_sk_maxPart;
        else if (n == "matMulT2_splitK_threshold") out = b.matMulT2_sk_threshold;
        else if (n == "matMulT2_splitK_maxPart") out = b.matMulT2_sk_maxPart;
        else if (n == "matMul_biased_fused") out = b.matMul_biased_fused ? 1 : 0;
        else if (n == "conv3D_remode") out = b.conv3D_remode ? 1 : 0;
        else if (n == "conv3D_biased_fused") out = b.conv3D_biased_fused ? 1 : 0;
        else if (n == "multiProcessorCount") out = b.device().multiProcessorCount();
        else if (n == "last_gridZ") out = b.last_gridZ;
        else if (n == "last_stream_count") out = b.last_stream_count;
        else if (n == "live_blocks") out = (int32_t)eg->eg.engineCore().live_blocks();
        else if (n == "stream_pool_size") out = b.streamPool().total_stream_size();
        else if (n == "pooled_events") out = b.streamPool().pooled_event_count();
        else if (n == "buf_physical_blocks") out = b.buf_mempool() ? b.buf_mempool()->physical_block_num() : -1;
        else if (n == "buf_buffered_blocks") out = b.buf_mempool() ? b.buf_mempool()->buffered_block_num() : -1;
        else if (n == "buf_used_mem_size") out = b.buf_mempool() ? (int32_t)b.buf_mempool()->used_mem_size() : -1;
        else if (n == "buf_total_mem_size_MB") out = b.buf_mempool() ? (int32_t)(b.buf_mempool()->total_mem_size() >> 20) : -1;
        else if (n == "memp_physical_blocks" || n == "memp_buffered_blocks" || n == "memp_used_mem_size_KB" ||
                 n == "memp_total_mem_size_KB") {
            Memp1* mp = eg->eg.engineCore().mempool();
            out = !mp ? -1 : n == "memp_physical_blocks" ? mp->physical_block_num()
                : n == "memp_buffered_blocks" ? mp->buffered_block_num()
                : n == "memp_used_mem_size_KB" ? (int32_t)(mp->used_mem_size() >> 10)
                : (int32_t)(mp->total_mem_size() >> 10);
        }
        else throw IllegalArgumentException("unknown parameter: " + n);
    });
    return out;
}

int32_t dragon_engine_gridZ(dragon_engine* eg, int32_t kind, int32_t N, int32_t M, int32_t K) {
    int32_t out = -1;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        CudaFloat32EngineBase& b = eg->eg.engineBase();
        out = kind == 0 ? b.matMul_gridZ(N, M, K) : kind == 1 ? b.matMulT1_gridZ(N, M, K)
            : kind == 3 ? b.matMul_biased_gridZ(N, M, K) : b.matMulT2_gridZ(N, M, K);
    });
    return out;
}
int32_t dragon_policy_smooth_maxPart(int32_t x) { return policy_smooth_maxPart(x); }
int32_t dragon_policy_gridZ(int32_t kind, int32_t N, int32_t M, int32_t K, int32_t SM) {
    SplitKKnobs mm = kDefaultMM, t = kDefaultT;
    mm.maxPart = t.maxPart = policy_smooth_maxPart(SM);
    if (kind == 0) return policy_matMul_gridZ(N, M, K, SM, mm);
    if (kind == 1) return policy_matMulT1_gridZ(N, M, K, SM, t);
    if (kind == 3) return policy_matMul_biased_gridZ(N, M, K, SM, mm);
    return policy_matMulT2_gridZ(N, M, K, SM, t, mm);
}

dragon_tensor* dragon_engine_empty(dragon_engine* eg, const int32_t* dim, int32_t ndim) {
    Tensor* t = nullptr;
    guard([&] { if (!eg) throw NullPointerException("engine"); t = eg->eg.empty(dims(dim, ndim)); });
    return t ? wrap(t) : nullptr;
}
dragon_tensor* dragon_engine_zeros(dragon_engine* eg, const int32_t* dim, int32_t ndim) {
    Tensor* t = nullptr;
    guard([&] { if (!eg) throw NullPointerException("engine"); t = eg->eg.zeros(dims(dim, ndim)); });
    return t ? wrap(t) : nullptr;
}
dragon_tensor* dragon_engine_tensor(dragon_engine* eg, const float* value, int32_t value_length,
                                    const int32_t* dim, int32_t ndim) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        t = eg->eg.tensor(value, value_length, dims(dim, ndim));
    });
    return t ? wrap(t) : nullptr;
}
int dragon_engine_set(dragon_engine* eg, dragon_tensor* X, const float* value, int32_t n) {
    return guard([&] {
        if (!eg) throw NullPointerException("engine");
        if (!value) throw NullPointerException("value is null");
        eg->eg.set(T(X), value, n);
    });
}
int dragon_engine_valueOf(dragon_engine* eg, dragon_tensor* ts, float* out, int32_t out_length) {
    return guard([&] {
        if (!eg || !out) throw NullPointerException("engine / out");
        std::vector<float> v = eg->eg.valueOf(T(ts));
        if ((int32_t)v.size() > out_length) throw IllegalArgumentException("output buffer too small");
        memcpy(out, v.data(), v.size() * sizeof(float));
    });
}
int dragon_engine_delete_tensor(dragon_engine* eg, dragon_tensor* ts) {
    return guard([&] {
        if (!eg) throw NullPointerException("engine");
        if (!ts) return;
        eg->eg.deleteTensor(ts->ts);
        delete ts;
    });
}
int dragon_tensor_c(dragon_tensor* ts) {
    return guard([&] { if (!ts) throw NullPointerException("tensor"); ts->ts->c(); });
}
int32_t dragon_tensor_ndim(const dragon_tensor* ts) { return ts ? ts->ts->ndim() : -1; }
int32_t dragon_tensor_dim(const dragon_tensor* ts, int32_t i) {
    if (!ts || i >= ts->ts->ndim() || i < -ts->ts->ndim()) return -1;
    return ts->ts->dimAt(i);
}
int32_t dragon_tensor_length(const dragon_tensor* ts) { return ts ? ts->ts->length : -1; }
int32_t dragon_tensor_lengthv(const dragon_tensor* ts) { return ts ? ts->ts->lengthv : -1; }
int32_t dragon_tensor_length_4x(const dragon_tensor* ts) { return ts ? ts->ts->length_4x : -1; }
int64_t dragon_tensor_address(const dragon_tensor* ts) { return ts ? ts->ts->address : 0; }

dragon_tensor* dragon_engine_product(dragon_engine* eg, int32_t op, int32_t likeA,
                                     dragon_tensor* A, dragon_tensor* B) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        Engine& e = eg->eg;
        switch (op) {
            case 0: t = e.matMul(T(A), T(B)); break;
            case 1: t = e.matMulT1(T(A), T(B)); break;
            case 2: t = e.matMulT2(T(A), T(B)); break;
            case 3: t = e.batchMatMul(likeA != 0, T(A), T(B)); break;
            case 4: t = e.batchMatMulT1(likeA != 0, T(A), T(B)); break;
            case 5: t = e.batchMatMulT2(likeA != 0, T(A), T(B)); break;
            default: throw IllegalArgumentException("unknown product");
        }
    });
    return t ? wrap(t) : nullptr;
}
int dragon_engine_product_into(dragon_engine* eg, int32_t op, dragon_tensor* C, dragon_tensor* A,
                               dragon_tensor* B) {
    return guard([&] {
        if (!eg) throw NullPointerException("engine");
        Engine& e = eg->eg;
        switch (op) {
            case 0: e.matMul(T(C), T(A), T(B)); break;
            case 1: e.matMulT1(T(C), T(A), T(B)); break;
            case 2: e.matMulT2(T(C), T(A), T(B)); break;
            case 3: e.batchMatMul(T(C), T(A), T(B)); break;
            case 4: e.batchMatMulT1(T(C), T(A), T(B)); break;
            case 5: e.batchMatMulT2(T(C), T(A), T(B)); break;
            default: throw IllegalArgumentException("unknown product");
        }
    });
}

dragon_tensor* dragon_engine_fullconnect(dragon_engine* eg, int32_t op, dragon_tensor* X,
                                         dragon_tensor* W, dragon_tensor* Bias) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        Engine& e = eg->eg;
        switch (op) {
            case 0: t = e.fullconnect(T(X), T(W)); break;
            case 1: t = e.fullconnect_biased(T(X), T(W), T(Bias)); break;
            case 2: t = e.fullconnect_deltaX(T(X), T(W)); break;
            case 3: t = e.fullconnect_deltaW(T(X), T(W)); break;
            case 4: t = e.matMul_biased(T(X), T(W), T(Bias)); break;
            default: throw IllegalArgumentException("unknown fullconnect operation");
        }
    });
    return t ? wrap(t) : nullptr;
}
int dragon_engine_fullconnect_into(dragon_engine* eg, int32_t op, dragon_tensor* Y, dragon_tensor* X,
                                   dragon_tensor* W, dragon_tensor* Bias) {
    return guard([&] {
        if (!eg) throw NullPointerException("engine");
        Engine& e = eg->eg;
        switch (op) {
            case 0: e.fullconnect(T(Y), T(X), T(W)); break;
            case 1: e.fullconnect_biased(T(Y), T(X), T(W), T(Bias)); break;
            case 4: e.matMul_biased(T(Y), T(X), T(W), T(Bias)); break;
            default: throw IllegalArgumentException("unknown fullconnect operation");
        }
    });
}
dragon_tensor* dragon_engine_conv3D(dragon_engine* eg, dragon_tensor* X, dragon_tensor* W, int32_t OH, int32_t OW,
                                    int32_t sh, int32_t sw, int32_t ph, int32_t pw, dragon_tensor* Bias) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        t = eg->eg.conv3D_biased(T(X), T(W), OH, OW, sh, sw, ph, pw, Bias ? T(Bias) : nullptr);
    });
    return t ? wrap(t) : nullptr;
}
int dragon_engine_conv3D_into(dragon_engine* eg, dragon_tensor* Y, dragon_tensor* X, dragon_tensor* W, int32_t sh,
                              int32_t sw, int32_t ph, int32_t pw, dragon_tensor* Bias) {
    return guard([&] {
        if (!eg) throw NullPointerException("engine");
        eg->eg.conv3D_biased(T(Y), T(X), T(W), sh, sw, ph, pw, Bias ? T(Bias) : nullptr);
    });
}
int32_t dragon_policy_conv3D_GEMM_nstream(int32_t GM, int32_t OC) { return policy_conv3D_GEMM_nstream(GM, OC); }
dragon_tensor* dragon_engine_linear(dragon_engine* eg, int32_t inplace, float alpha, dragon_tensor* X,
                                    float beta) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        t = eg->eg.linear(inplace != 0, alpha, T(X), beta);
    });
    if (!t) return nullptr;
    return inplace ? X : wrap(t);
}
dragon_tensor* dragon_engine_softmax(dragon_engine* eg, int32_t inplace, dragon_tensor* X, int32_t features,
                                     float scale) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        t = eg->eg.softmax_scaled(inplace != 0, T(X), scale, features);
    });
    if (!t) return nullptr;
    return inplace ? X : wrap(t);
}
dragon_tensor* dragon_engine_attention(dragon_engine* eg, dragon_tensor* Q, dragon_tensor* K, dragon_tensor* V,
                                       int32_t head, float scale) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        t = eg->eg.attention(T(Q), T(K), T(V), head, scale);
    });
    return t ? wrap(t) : nullptr;
}
dragon_tensor* dragon_engine_attention_masked(dragon_engine* eg, dragon_tensor* Q, dragon_tensor* K, dragon_tensor* V,
                                              dragon_tensor* Mask, int32_t head, float scale) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        if (!Mask) throw NullPointerException("Tensor mask is null");
        t = eg->eg.attention(T(Q), T(K), T(V), head, scale, T(Mask));
    });
    return t ? wrap(t) : nullptr;
}
dragon_tensor* dragon_engine_transpose(dragon_engine* eg, int32_t inplace, dragon_tensor* X,
                                       int32_t dimIdx1, int32_t dimIdx2) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        t = eg->eg.transpose(inplace != 0, T(X), dimIdx1, dimIdx2);
    });
    if (!t) return nullptr;
    return (X && t == X->ts) ? X : wrap(t);
}
dragon_tensor* dragon_engine_linear2_row(dragon_engine* eg, int32_t inplace, dragon_tensor* X1,
                                         dragon_tensor* X2, float alpha, float beta, float gamma) {
    Tensor* t = nullptr;
    guard([&] {
        if (!eg) throw NullPointerException("engine");
        t = eg->eg.linear2_row(inplace != 0, T(X1), T(X2), alpha, beta, gamma);
    });
    if (!t) return nullptr;
    return inplace ? X1 : wrap(t);
}

}  // extern "C"
