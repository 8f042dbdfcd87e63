// Host side of the matrix-multiplication path, above the C ABI: a C++ mirror of the
// Java classes that drive the reference's native libraries, with the same names,
// argument meaning and error behaviour.  It calls nothing but the C ABI of
// include/dragon_hip_gemm.h and include/dragon_hip_runtime.h -- exactly what the
// reference's Java code would call through JNI.
//
//   CudaDevice             z/dragon/engine/cuda/impl/CudaDevice.java (multiProcessorCount only)
//   CudaStreamPool         z/dragon/engine/cuda/impl/CudaStreamp1.java:34-63 (round-robin, never blocks)
//   Syncer and its kinds   z/dragon/engine/cuda/CudaFloat32EngineBase.java:649-694, 1008-1054
//   CudaFloat32EngineBase  z/dragon/engine/cuda/CudaFloat32EngineBase.java:70-92, 1148-1260, 1471-2020,
//                          4517-4530 (linear2_2D_row)
//   EngineCore             z/dragon/engine/EngineCore.java:693-811 (checks and x4 padding)
//   PinnedMempool          z/dragon/engine/cuda/impl/PinnedMempool.java:96-200
//   Tensor                 z/dragon/engine/Tensor.java:206-239 (length / lengthv / length_4x)
//   Engine                 z/dragon/engine/Engine.java:522-551, 671-676, 824-837, 908-914, 955-1470,
//                          4185-4207 (add_row / linear2_row), 1797-1831 (transpose), 4002-4013 (linear / sdiv), 6082-6100 (softmax)
// (paths relative to source/alpha-Dragon-v1.2/src of the reference tree)
#pragma once
#include <stdint.h>
#include <map>
#include <memory>
#include <set>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

namespace dragon {

// ---- exceptions: the Java types the reference throws ---------------------------------
struct NullPointerException : std::runtime_error { using std::runtime_error::runtime_error; };
struct IllegalArgumentException : std::runtime_error { using std::runtime_error::runtime_error; };
struct CudaException : std::runtime_error {
    int code;
    explicit CudaException(int c);
};

// ---- device ----------------------------------------------------------------------------
class CudaDevice {
public:
    explicit CudaDevice(int id = 0);
    int getId() const { return id_; }
    int multiProcessorCount() const { return sm_count_; }
    // lets a test drive the split-K policy as a device with another unit count would
    void overrideMultiProcessorCount(int n) { sm_count_ = n; }
private:
    int id_, sm_count_;
};

// ---- stream pool: hands out streams round-robin, returning them is a no-op ----------------
class CudaStreamPool {
public:
    CudaStreamPool(const CudaDevice& dev, int max_streamsize, int max_getsize_oneturn);
    ~CudaStreamPool();
    int64_t getStream();
    std::vector<int64_t> getStreamArray(int length);
    void returnStream(int64_t) {}
    void returnStreamArray(const std::vector<int64_t>&) {}
    int total_stream_size();
    // Events without timing, recycled: the reference creates and destroys one per call
    // (CudaFloat32EngineBase.java:649-694, 1008-1054); handing the same few out again saves the two driver
    // calls.  An event may go back as soon as its waits are enqueued: a stream's wait refers to the record
    // that preceded it, not to later ones.
    int64_t getEvent();
    void returnEvent(int64_t event);
    int pooled_event_count();
private:
    void init();
    int dev_id_, max_streamsize_, max_getsize_oneturn_;
    std::vector<int64_t> gc_;
    std::vector<int64_t> events_;     // idle events
    int gc_index_ = 0;
    bool inited_ = false;
    std::mutex mu_;
};

// ---- memory pools ------------------------------------------------------------------------------
// The recycling policy of the reference's pools (z/dragon/engine/memp/Mempool.java:150-225 with
// Memp1.java:27-80, and cuda/impl/PinnedMempool.java:96-200, which repeats it for pinned memory):
// blocks are recycled by size -- a request takes the smallest free block of [size, 1.5*size] (equal
// sizes first in, first out), else allocates; when the budget is exhausted free blocks are released
// largest-first to make room; an address can be freed once until it is handed out again.
class RecyclingPool {
public:
    explicit RecyclingPool(int64_t maxMemorySize) : max_mem_size_(maxMemorySize) {}
    virtual ~RecyclingPool() {}
    struct Block { int64_t size, address; };   // size in floats (bytes / 4), as the Java pools report it
    Block malloc(int64_t mem_size);            // mem_size in bytes
    bool free(int64_t size, int64_t address);  // size as returned by malloc
    void clear();                              // releases every block, handed out or not
    int64_t max_mem_size() const { return max_mem_size_; }
    int64_t total_mem_size() const { return total_mem_size_; }
    int64_t used_mem_size() const { return used_mem_size_; }
    int physical_block_num() const { return (int)blocks_.size(); }
    int buffered_block_num() const { return (int)pool_.size(); }
protected:
    virtual int64_t raw_malloc(int64_t bytes) = 0;   // 0 on failure
    virtual void raw_free(int64_t address) = 0;
    virtual const char* what() const = 0;
private:
    int64_t max_mem_size_, total_mem_size_ = 0, used_mem_size_ = 0;
    std::multimap<int64_t, int64_t> pool_;     // free blocks: size in bytes -> address
    std::map<int64_t, int64_t> blocks_;        // every block this pool owns: address -> size in bytes
    std::set<int64_t> grave_;                  // addresses currently free (guards a double free)
    std::mutex mu_;
};

// pinned host staging buffers for tensor transfer (z/dragon/engine/cuda/impl/PinnedMempool.java)
class PinnedMempool : public RecyclingPool {
public:
    explicit PinnedMempool(int64_t maxMemorySize) : RecyclingPool(maxMemorySize) {}
    ~PinnedMempool() override { clear(); }
protected:
    int64_t raw_malloc(int64_t bytes) override;
    void raw_free(int64_t address) override;
    const char* what() const override { return "pinned-memory"; }
};

class CudaFloat32EngineBase;
// device memory for tensors and split-K partials (z/dragon/engine/memp/Memp1.java, the pool the
// reference's tests build their engines with: alpha.engine.memp1(size)).  Without one, EngineCore
// allocates and frees every block on the device itself.
class Memp1 : public RecyclingPool {
public:
    Memp1(int64_t maxMemorySize, CudaFloat32EngineBase* base) : RecyclingPool(maxMemorySize), base_(base) {}
    ~Memp1() override { clear(); }
protected:
    int64_t raw_malloc(int64_t bytes) override;
    void raw_free(int64_t address) override;
    const char* what() const override { return "device memory"; }
private:
    CudaFloat32EngineBase* base_;
};

// ---- completion handles ----------------------------------------------------------------------
class Syncer {
public:
    virtual ~Syncer() {}
    virtual void sync() = 0;
};
typedef std::unique_ptr<Syncer> SyncerPtr;

class EngineCore;

// ---- split-K policy, usable without a device ---------------------------------------------------
struct SplitKKnobs {
    int threshold;          // K below this never splits (default 512)
    int maxPart;            // upper bound of GridZ (default smooth(SM count))
    float minBlock_perSM;   // 1.2f for matMul, 1.14f for matMulT1 / matMulT2
    float maxBlock_perSM;   // 4.0f
};
int policy_smooth_maxPart(int x);
int policy_matMul_gridZ(int N, int M, int K, int SM, const SplitKKnobs& k);
int policy_matMul_biased_gridZ(int N, int M, int K, int SM, const SplitKKnobs& k);
int policy_matMulT1_gridZ(int N, int M, int K, int SM, const SplitKKnobs& k);
int policy_matMulT2_gridZ(int N, int M, int K, int SM, const SplitKKnobs& t2, const SplitKKnobs& mm);
// stream counts and the "padding scale up" ratio of the convolution natives (Cuda_conv3D.java:18-28, 264-327)
int policy_conv3D_GEMM_nstream(int GM, int OC);
int policy_conv3D_GEMMV2_nstream(int N, int OC);
float policy_conv3D_psu(int IH, int IW, int OH, int OW, int FH, int FW, int sh, int sw);

// ---- the engine "plugin": split-K policy, stream checkout, event protocol -----------------------
class CudaFloat32EngineBase {
public:
    CudaFloat32EngineBase(int deviceId, int streamPool_maxsize);
    CudaDevice& device() { return dev_; }
    CudaStreamPool& streamPool() { return *streamPool_; }
    void engineCore(EngineCore* core) { core_ = core; }
    // staging pool for get / set; without one the transfers stage through pageable memory
    PinnedMempool* buf_mempool() { return bufPool_.get(); }
    void buf_mempool(std::unique_ptr<PinnedMempool> pool) { bufPool_ = std::move(pool); }

    // knobs (same names and defaults as the Java fields)
    int matMul_sk_threshold = 512, matMul_sk_maxPart = 16;
    float matMul_sk_minBlock_perSM = 1.2f, matMul_sk_maxBlock_perSM = 4.0f;
    int matMulT1_sk_threshold = 512, matMulT1_sk_maxPart = 16;
    float matMulT1_sk_minBlock_perSM = 1.14f, matMulT1_sk_maxBlock_perSM = 4.0f;
    int matMulT2_sk_threshold = 512, matMulT2_sk_maxPart = 16;
    float matMulT2_sk_minBlock_perSM = 1.14f, matMulT2_sk_maxBlock_perSM = 4.0f;
    bool matMul_tf32 = false, matMulT1_tf32 = false, matMulT2_tf32 = false;
    bool batchMatMul_tf32 = false, batchMatMulT1_tf32 = false, batchMatMulT2_tf32 = false;
    bool batchMatMul_useTexture = true, batchMatMulT2_useTexture = true;
    // Not a field of the Java class: when set (the default) an unsplit matMul_biased adds the bias
    // row inside the product's launch; when cleared it issues the reference's two launches.
    bool matMul_biased_fused = true;
    // Convolution knobs.  conv3D_remode is the Java field (CudaFloat32EngineBase.java:2025): re-order W to
    // CW[FH, FW, IC, OC] in a temporary block and call the GemmR natives.  The Java default is true because
    // its CUDA kernels read CW faster; the MFMA kernel reads W as stored and never touches CW, so the
    // default here is false (one launch, no temporary block).  Set it to get the reference's sequence.
    bool conv3D_remode = false;
    bool conv3D_Gemm_useTexture = true;
    float conv3D_GemmV2_Q = 1.25f;
    // Not a Java field: conv3D_biased adds the bias inside the convolution's launch (default) or issues the
    // reference's second launch linear_dual2D_row.
    bool conv3D_biased_fused = true;

    void matMul_splitK_threshold(int threshold);     // must be a positive power of two
    void matMul_splitK_maxPart(int maxPart);         // must be >= 4
    void matMulT1_splitK_threshold(int threshold);
    void matMulT1_maxPart(int maxPart);
    void matMulT2_splitK_threshold(int threshold);
    void matMulT2_splitK_maxPart(int maxPart);
    void tf32(bool flag);
    void recomputeMaxParts();                        // maxPart = smooth(SM count), as the constructor does

    // the split-K decisions on their own (1 = no split), for inspection
    int matMul_gridZ(int N, int M, int K) const;
    int matMul_biased_gridZ(int N, int M, int K) const;
    int matMulT1_gridZ(int N, int M, int K) const;
    int matMulT2_gridZ(int N, int M, int K) const;

    // memory operations
    int64_t malloc(int64_t memsize);
    void free(int64_t address);
    SyncerPtr memset(int64_t address, int value, int64_t memsize);
    void get1D(int64_t address, float* value, int length);
    void get2D(int64_t address, float* value, int height, int width, int stride);
    void set1D(int64_t address, const float* value, int length);
    void set2D(int64_t address, const float* value, int height, int width, int stride);

    // products; dims arrive already padded by EngineCore
    SyncerPtr matMul(int64_t C, int64_t A, int64_t B, int N, int M, int K);
    SyncerPtr matMul_biased(int64_t C, int64_t A, int64_t B, int N, int M, int K, int64_t Bias,
                            int lengthv, int width);
    SyncerPtr matMulT1(int64_t C, int64_t A, int64_t B, int N, int M, int K);
    SyncerPtr matMulT2(int64_t C, int64_t A, int64_t B, int N, int M, int K);
    SyncerPtr linear2_2D_row(int64_t Y, int64_t X1, int64_t X2, int row_lengthv, float alpha,
                             float beta, float gamma, int lengthv, int width, int stride);
    // forward convolution; Bias = 0 for the plain form.  N, IC, OC arrive padded by EngineCore
    SyncerPtr conv3D(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W, int FH, int FW,
                     int N, int IC, int OC, int sh, int sw, int ph, int pw);
    SyncerPtr conv3D_biased(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W, int FH, int FW,
                            int N, int IC, int OC, int sh, int sw, int ph, int pw, int64_t Bias,
                            int lengthv, int width);
    SyncerPtr transpose(int64_t Y, const std::vector<int>& Ydim, int64_t X, const std::vector<int>& Xdim,
                        int dimIndex1, int dimIndex2, int strideX, int strideY, int length);
    SyncerPtr linear2D(int64_t Y, float alpha, int64_t X, float beta, int lengthv, int width, int stride);
    // scale is not an argument of the Java method: 1 reproduces it, another value folds a preceding sdiv
    SyncerPtr softmax2D(int64_t Y, int64_t X, int field_length, int row_lengthv, int lengthv, int width,
                        int stride, float scale = 1.0f);
    SyncerPtr memcpy(int64_t dst, int64_t src, int64_t memsize);
    // softmax(scale * Q.K^T).V per (image, head) in one launch; not a Java method (the reference's block
    // issues transposes, batchMatMulT2, sdiv, softmax, batchMatMul: nn/unit/complex/block/ChannelMHA.java:66-83)
    // Mask != 0: the probabilities are multiplied by it after the softmax (the block's mask unit); rows of
    // mask_pitch floats, one [QL, mask_pitch] slice for all or one per (image, head)
    SyncerPtr attention(int64_t Y, int64_t Q, int64_t K, int64_t V, int N, int head, int QL, int VL, int dK4,
                        int dV4, bool head_inner, float scale, int64_t Mask = 0, int mask_pitch = 0,
                        bool mask_per_head = false);
    SyncerPtr batchMatMul(int64_t C, int64_t A, int64_t B, int Batch, int N, int M, int BK, int AK);
    SyncerPtr batchMatMulT1(int64_t C, int64_t A, int64_t B, int Batch, int CN, int AN, int M, int K);
    SyncerPtr batchMatMulT2(int64_t C, int64_t A, int64_t B, int Batch, int N, int CM, int BM, int K);

    // what the last product call decided (test introspection)
    int last_gridZ = 1, last_stream_count = 0;

private:
    SyncerPtr run_2d(int variant, int gridZ, int64_t C, int64_t A, int64_t B, int N, int M, int K,
                     int64_t Bias = 0, int lengthv = 0, int width = 0);
    SyncerPtr run_conv(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W, int FH, int FW,
                       int N, int IC, int OC, int sh, int sw, int ph, int pw, int64_t Bias, int lengthv,
                       int width);
    CudaDevice dev_;
    std::unique_ptr<CudaStreamPool> streamPool_;
    std::unique_ptr<PinnedMempool> bufPool_;
    EngineCore* core_ = nullptr;
};

// ---- EngineCore: argument checks, x4 padding, memory blocks ----------------------------------------
class EngineCore {
public:
    explicit EngineCore(CudaFloat32EngineBase* base, bool check = true);
    CudaFloat32EngineBase* engineBase() { return base_; }
    bool check;

    // a block is {size in bytes, address}.  With a pool (EngineCore(mempool, check) of the reference)
    // blocks are recycled through it; without one every block is its own device allocation.
    struct Block { int64_t size, address; };
    Block malloc(int mem_length);
    void free(int64_t size, int64_t address);
    int64_t live_blocks() const { return live_blocks_; }
    void mempool(std::unique_ptr<Memp1> pool) { mempool_ = std::move(pool); }
    Memp1* mempool() { return mempool_.get(); }
    SyncerPtr memset(int64_t address, int value, int length);
    void get1D(int64_t address, float* value, int length);
    void get2D(int64_t address, float* value, int height, int width);
    void set1D(int64_t address, const float* value, int length);
    void set2D(int64_t address, const float* value, int length, int width);

    SyncerPtr matMul(int64_t C, int64_t A, int64_t B, int N, int M, int K);
    SyncerPtr matMul_biased(int64_t C, int64_t A, int64_t B, int N, int M, int K, int64_t Bias,
                            int lengthv);
    SyncerPtr matMulT1(int64_t C, int64_t A, int64_t B, int N, int M, int K);
    SyncerPtr matMulT2(int64_t C, int64_t A, int64_t B, int N, int M, int K);
    SyncerPtr linear2_2D_row(int64_t Y, int64_t X1, int64_t X2, int row_lengthv, float alpha,
                             float beta, float gamma, int lengthv, int width);
    SyncerPtr conv3D(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W, int FH, int FW,
                     int N, int IC, int OC, int sh, int sw, int ph, int pw);
    SyncerPtr conv3D_biased(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W, int FH, int FW,
                            int N, int IC, int OC, int sh, int sw, int ph, int pw, int64_t Bias, int lengthv);
    SyncerPtr transpose(int64_t Y, const std::vector<int>& Ydim, int64_t X, const std::vector<int>& Xdim,
                        int dimIndex1, int dimIndex2, int widthX, int widthY, int length);
    SyncerPtr linear2D(int64_t Y, float alpha, int64_t X, float beta, int lengthv, int width);
    SyncerPtr softmax2D(int64_t Y, int64_t X, int row_length, int lengthv, int width, float scale = 1.0f);
    SyncerPtr memcpy(int64_t dst, int64_t src, int length);
    // head dimensions arrive unpadded; with more than one head they must be multiples of 4 already
    SyncerPtr attention(int64_t Y, int64_t Q, int64_t K, int64_t V, int N, int head, int QL, int VL, int dK,
                        int dV, bool head_inner, float scale, int64_t Mask = 0, int mask_width = 0,
                        bool mask_per_head = false);
    SyncerPtr batchMatMul(int64_t C, int64_t A, int64_t B, int Batch, int N, int M, int K);
    SyncerPtr batchMatMulT1(int64_t C, int64_t A, int64_t B, int Batch, int N, int M, int K);
    SyncerPtr batchMatMulT2(int64_t C, int64_t A, int64_t B, int Batch, int N, int M, int K);

private:
    void matMul_check(int64_t C, int64_t A, int64_t B, int N, int M, int K) const;
    void func_param_check_row(int lengthv, int row_lengthv, int width, int stride) const;
    void conv3D_param_check(int OH, int OW, int IH, int IW, int FH, int FW, int N, int IC, int OC, int sh,
                            int sw, int ph, int pw) const;
    CudaFloat32EngineBase* base_;
    int64_t live_blocks_ = 0;
    std::unique_ptr<Memp1> mempool_;
    std::mutex mu_;
};

// ---- Tensor: row-major, last dimension stored with a stride rounded up to 4 ---------------------------
class Tensor {
public:
    Tensor(bool check, const std::vector<int>& dim);
    std::vector<int> dim;
    int length = 0;      // logical element count
    int lengthv = 0;     // firstDim * mid * lastDim_4x
    int length_4x = 0;   // firstDim_4x * mid * lastDim_4x: what is allocated
    int64_t mem_size = 0, address = 0;
    int ndim() const { return (int)dim.size(); }
    int dimAt(int i) const { return i < 0 ? dim[dim.size() + i] : dim[i]; }
    int lastDim() const { return dim.back(); }
    void setSyncer(SyncerPtr sc) { syncer_ = std::move(sc); }
    Tensor& c();         // wait for the pending operation that produces this tensor
private:
    SyncerPtr syncer_;
};

// ---- Engine: the tensor-level API ------------------------------------------------------------------------
class Engine {
public:
    // max_trans_buf_size > 0 gives the engine a PinnedMempool of that many bytes, max_mem_size > 0 a
    // Memp1 device pool of that many (Alpha.java:770-790)
    Engine(int deviceId, int streamPool_maxsize, int64_t max_trans_buf_size = 0, int64_t max_mem_size = 0);
    ~Engine();
    EngineCore& engineCore() { return *core_; }
    CudaFloat32EngineBase& engineBase() { return *base_; }
    Engine& check(bool flag) { check_ = flag; core_->check = flag; return *this; }
    Engine& sync(bool flag) { sync_ = flag; return *this; }

    Tensor* empty(const std::vector<int>& dim);
    Tensor* zeros(const std::vector<int>& dim);
    Tensor* tensor(const float* value, int value_length, const std::vector<int>& dim);
    Tensor* set(Tensor* X, const float* value, int value_length);
    std::vector<float> valueOf(Tensor* ts);
    void deleteTensor(Tensor* ts);

    Tensor* matMul(Tensor* A, Tensor* B);
    Tensor* matMul(Tensor* C, Tensor* A, Tensor* B);
    Tensor* matMul_biased(Tensor* A, Tensor* B, Tensor* Bias);
    Tensor* matMul_biased(Tensor* C, Tensor* A, Tensor* B, Tensor* Bias);
    Tensor* matMulT1(Tensor* A, Tensor* B);
    Tensor* matMulT1(Tensor* C, Tensor* A, Tensor* B);
    Tensor* matMulT2(Tensor* A, Tensor* B);
    Tensor* matMulT2(Tensor* C, Tensor* A, Tensor* B);
    Tensor* batchMatMul(bool likeA, Tensor* A, Tensor* B);
    Tensor* batchMatMul(Tensor* C, Tensor* A, Tensor* B);
    Tensor* batchMatMulT1(bool likeA, Tensor* A, Tensor* B);
    Tensor* batchMatMulT1(Tensor* C, Tensor* A, Tensor* B);
    Tensor* batchMatMulT2(bool likeA, Tensor* A, Tensor* B);
    Tensor* batchMatMulT2(Tensor* C, Tensor* A, Tensor* B);

    // fully connected layer over the last dimension of a tensor of any rank >= 2
    Tensor* fullconnect(Tensor* X, Tensor* W);
    Tensor* fullconnect(Tensor* Y, Tensor* X, Tensor* W);
    Tensor* fullconnect_biased(Tensor* X, Tensor* W, Tensor* Bias);
    Tensor* fullconnect_biased(Tensor* Y, Tensor* X, Tensor* W, Tensor* Bias);
    Tensor* fullconnect_deltaX(Tensor* deltaY, Tensor* W);
    Tensor* fullconnect_deltaW(Tensor* X, Tensor* deltaY);

    // forward convolution over NHWC tensors: X[N, IH, IW, IC], W[OC, FH, FW, IC] -> Y[N, OH, OW, OC].
    // With Y given, ph / pw = -1 derive the padding from the shapes (rounded up); without Y, OH / OW = -1
    // derive the output size from the padding (rounded down).  Bias[OC] is added to every output pixel.
    Tensor* conv3D(Tensor* Y, Tensor* X, Tensor* W, int sh, int sw, int ph = -1, int pw = -1);
    Tensor* conv3D(Tensor* X, Tensor* W, int OH, int OW, int sh, int sw, int ph, int pw);
    Tensor* conv3D_biased(Tensor* Y, Tensor* X, Tensor* W, int sh, int sw, int ph, int pw, Tensor* Bias);
    Tensor* conv3D_biased(Tensor* X, Tensor* W, int OH, int OW, int sh, int sw, int ph, int pw, Tensor* Bias);

    // exchange of two dimensions (negative indices count from the end); inplace gives X the new
    // shape and memory and frees the old memory once the kernel is done
    Tensor* transpose(bool inplace, Tensor* X, int dimIdx1, int dimIdx2);
    Tensor* copy(Tensor* X);

    // Y = alpha*X + beta; sdiv(X, C) = X / C = linear(1/C, X, 0)
    Tensor* linear(bool inplace, float alpha, Tensor* X, float beta);
    Tensor* sdiv(bool inplace, Tensor* X, float C) { return linear(inplace, 1.0f / C, X, 0.0f); }
    // softmax over groups of `features` elements (-1: the last dimension).  softmax_scaled is
    // softmax(scale * X) in the same launch: softmax(sdiv(X, C)) without the extra pass (not in the
    // Java class).
    Tensor* softmax(bool inplace, Tensor* X, int features = -1) { return softmax_scaled(inplace, X, 1.0f, features); }
    Tensor* softmax_scaled(bool inplace, Tensor* X, float scale, int features = -1);

    // The attention block of ChannelMHA (nn/unit/complex/block/ChannelMHA.java:66-83) in one launch:
    // Q[N, QL, KC], K[N, VL, KC], V[N, VL, VC] hold `head` heads side by side in their last dimension;
    // Y[N, QL, VC] = per head softmax(scale * Q.K^T).V.  scale = 0 means the block's own 1/sqrt(KC).
    // Needs KC/head and VC/head <= 256 (and multiples of 4 when head > 1); other shapes take the operator
    // chain (transpose, batchMatMulT2, softmax_scaled, batchMatMul, transpose).  Not a Java method.
    // mask (optional): a tensor [QL, VL] (one for every image and head) or [N, head, QL, VL] that multiplies the
    // probabilities after the softmax, which is what the block does with a mask unit that multiplies element by
    // element (ChannelMHA.java:75-76).
    Tensor* attention(Tensor* Q, Tensor* K, Tensor* V, int head, float scale = 0.0f, Tensor* mask = nullptr);

    // Y = alpha*X1 + beta*X2 + gamma with the row vector X2 broadcast over the rows of X1
    Tensor* add_row(bool inplace, Tensor* X1, Tensor* X2) { return linear2_row(inplace, X1, X2, 1.0f, 1.0f, 0.0f); }
    Tensor* linear2_row(bool inplace, Tensor* X1, Tensor* X2, float alpha, float beta, float gamma);

private:
    void finish(Tensor* C, SyncerPtr sc);
    std::unique_ptr<CudaFloat32EngineBase> base_;
    std::unique_ptr<EngineCore> core_;
    bool check_ = true, sync_ = true;
};

}  // namespace dragon
