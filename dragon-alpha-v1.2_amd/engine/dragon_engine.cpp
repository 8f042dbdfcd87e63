// Implementation of the host-side mirror declared in dragon_engine.hpp.  Every device
// action goes through the C ABI (dragon_Cuda_* entry points); no HIP call is made here.
#include "dragon_engine.hpp"

#include <math.h>
#include <string.h>

#include "../../include/dragon_hip_conv.h"
#include "../../include/dragon_hip_gemm.h"
#include "../../include/dragon_hip_runtime.h"

namespace dragon {

namespace {

inline int pad4(int x) { return ((x + 3) >> 2) << 2; }

inline void cu(int code) {
    if (code != 0) throw CudaException(code);
}
inline int64_t cu_handle(int64_t h) {
    if (h == 0) {
        int code = dragon_Cuda_getLastExceptionType();
        throw CudaException(code ? code : 2);
    }
    return h;
}

std::string fmt(const char* f, long long a = 0, long long b = 0) {
    char buf[256];
    snprintf(buf, sizeof(buf), f, a, b);
    return buf;
}

// an event of the pool that goes back when the scope ends, also when an exception leaves it
struct ScopedEvent {
    CudaStreamPool* pool;
    int64_t handle;
    explicit ScopedEvent(CudaStreamPool* p) : pool(p), handle(p->getEvent()) {}
    ~ScopedEvent() { if (handle) pool->returnEvent(handle); }
    ScopedEvent(const ScopedEvent&) = delete;
    ScopedEvent& operator=(const ScopedEvent&) = delete;
};

// streams -> streams[0]  (CudaFloat32EngineBase.java:649-654).  With a single stream there is nothing to
// join: what follows on it is ordered behind what was issued.
void sync_streamArray_2_stream0(CudaStreamPool* pool, const std::vector<int64_t>& streams) {
    if (streams.size() < 2) return;
    ScopedEvent event1(pool);
    cu(dragon_Cuda_eventRecord_streams(event1.handle, streams.data(), (int)streams.size()));
    cu(dragon_Cuda_streamWaitEvent_default(streams[0], event1.handle));
}

// wait for a syncer's event and hand it back to the pool
void wait_and_recycle(CudaStreamPool* pool, int64_t event) {
    const int rc = dragon_Cuda_eventSynchronize(event);
    pool->returnEvent(event);
    cu(rc);
}

// CudaFloat32EngineBase.java:657-694
class StreamArraySyncer : public Syncer {
public:
    StreamArraySyncer(CudaStreamPool* pool, std::vector<int64_t> streams)
        : pool_(pool), streams_(std::move(streams)) {
        sync_streamArray_2_stream0(pool_, streams_);
        event_ = pool_->getEvent();
        cu(dragon_Cuda_eventRecord(event_, streams_[0]));
    }
    // The reference's finalizer drops the event without waiting; waiting is the safe
    // reading of the same protocol, and a completed syncer makes this a no-op.
    ~StreamArraySyncer() override {
        try { sync(); } catch (...) {}
    }
    void sync() override {
        {
            std::lock_guard<std::mutex> g(mu_);
            if (called_) return;
            wait_and_recycle(pool_, event_);
            called_ = true;
        }
        pool_->returnStreamArray(streams_);
    }
private:
    CudaStreamPool* pool_;
    std::vector<int64_t> streams_;
    int64_t event_ = 0;
    bool called_ = false;
    std::mutex mu_;
};

// CudaFloat32EngineBase.java:1008-1054: completion of the reduction on streams[0], then the
// partial-product buffer goes back to the core
class SplitKSyncer : public Syncer {
public:
    SplitKSyncer(EngineCore* core, EngineCore::Block block, CudaStreamPool* pool,
                 std::vector<int64_t> streams)
        : core_(core), block_(block), pool_(pool), streams_(std::move(streams)) {
        event_ = pool_->getEvent();
        cu(dragon_Cuda_eventRecord(event_, streams_[0]));
    }
    ~SplitKSyncer() override {
        try { sync(); } catch (...) {}
    }
    void sync() override {
        {
            std::lock_guard<std::mutex> g(mu_);
            if (called_) return;
            wait_and_recycle(pool_, event_);
            called_ = true;
        }
        core_->free(block_.size, block_.address);
        pool_->returnStreamArray(streams_);
    }
private:
    EngineCore* core_;
    EngineCore::Block block_;
    CudaStreamPool* pool_;
    std::vector<int64_t> streams_;
    int64_t event_ = 0;
    bool called_ = false;
    std::mutex mu_;
};

// one stream, one event (StreamSyncer of the reference, used by memset)
class StreamSyncer : public Syncer {
public:
    StreamSyncer(CudaStreamPool* pool, int64_t stream) : pool_(pool), stream_(stream) {
        event_ = pool_->getEvent();
        cu(dragon_Cuda_eventRecord(event_, stream_));
    }
    ~StreamSyncer() override {
        try { sync(); } catch (...) {}
    }
    void sync() override {
        if (called_) return;
        wait_and_recycle(pool_, event_);
        called_ = true;
        pool_->returnStream(stream_);
    }
private:
    CudaStreamPool* pool_;
    int64_t stream_, event_ = 0;
    bool called_ = false;
};

struct FreeAfter : Syncer {     // Syncer.dual(sc1, () -> core.free(old)): wait, then release the old memory
    SyncerPtr first; EngineCore* core; int64_t size, address; bool done = false;
    FreeAfter(SyncerPtr f, EngineCore* c, int64_t s, int64_t a) : first(std::move(f)), core(c), size(s), address(a) {}
    ~FreeAfter() override { try { sync(); } catch (...) {} }
    void sync() override {
        if (done) return;
        first->sync();
        core->free(size, address);
        done = true;
    }
};

std::mutex g_cuda_class_lock;  // the reference serialises setDevice+malloc/free on Cuda.class

}  // namespace

CudaException::CudaException(int c)
    : std::runtime_error(std::string(dragon_Cuda_getExceptionName(c) ? dragon_Cuda_getExceptionName(c)
                                                                      : "hipError") +
                         " (" + std::to_string(c) + ")"),
      code(c) {}

// ---- CudaDevice ----------------------------------------------------------------------------
CudaDevice::CudaDevice(int id) : id_(id), sm_count_(0) {
    sm_count_ = dragon_CudaDevice_multiProcessorCount(id);
    if (sm_count_ <= 0) throw CudaException(dragon_Cuda_getLastExceptionType());
}

// ---- CudaStreamPool ---------------------------------------------------------------------------
CudaStreamPool::CudaStreamPool(const CudaDevice& dev, int max_streamsize, int max_getsize_oneturn)
    : dev_id_(dev.getId()), max_streamsize_(max_streamsize),
      max_getsize_oneturn_(max_getsize_oneturn) {
    if (max_streamsize <= 0) throw IllegalArgumentException("max_streamsize must be positive");
    if (max_getsize_oneturn_ > max_streamsize_) max_getsize_oneturn_ = max_streamsize_;
}
CudaStreamPool::~CudaStreamPool() {
    for (int64_t e : events_) dragon_Cuda_deleteEvent(e);
    if (!gc_.empty()) dragon_Cuda_deleteStreams(gc_.data(), (int)gc_.size());
}
int64_t CudaStreamPool::getEvent() {
    {
        std::lock_guard<std::mutex> g(mu_);
        if (!events_.empty()) { const int64_t e = events_.back(); events_.pop_back(); return e; }
    }
    std::lock_guard<std::mutex> g(g_cuda_class_lock);
    cu(dragon_Cuda_setDevice(dev_id_));
    return cu_handle(dragon_Cuda_newEvent_DisableTiming());
}
void CudaStreamPool::returnEvent(int64_t event) {
    if (event == 0) return;
    std::lock_guard<std::mutex> g(mu_);
    if (events_.size() < 256) { events_.push_back(event); return; }
    dragon_Cuda_deleteEvent(event);
}
int CudaStreamPool::pooled_event_count() {
    std::lock_guard<std::mutex> g(mu_);
    return (int)events_.size();
}
void CudaStreamPool::init() {
    std::lock_guard<std::mutex> g(g_cuda_class_lock);
    cu(dragon_Cuda_setDevice(dev_id_));
    for (int i = 0; i < max_streamsize_; i++) gc_.push_back(cu_handle(dragon_Cuda_newStream_Blocking()));
}
int64_t CudaStreamPool::getStream() {
    std::lock_guard<std::mutex> g(mu_);
    if (!inited_) { init(); inited_ = true; }
    int64_t s = gc_[gc_index_];
    gc_index_ = (gc_index_ + 1) % max_streamsize_;
    return s;
}
std::vector<int64_t> CudaStreamPool::getStreamArray(int length) {
    std::lock_guard<std::mutex> g(mu_);
    if (!inited_) { init(); inited_ = true; }
    if (length > max_getsize_oneturn_) length = max_getsize_oneturn_;
    std::vector<int64_t> streams((size_t)length);
    for (int i = 0; i < length; i++) {
        streams[i] = gc_[gc_index_];
        gc_index_ = (gc_index_ + 1) % max_streamsize_;
    }
    return streams;
}
int CudaStreamPool::total_stream_size() {
    std::lock_guard<std::mutex> g(mu_);
    return (int)gc_.size();
}

// ---- CudaFloat32EngineBase ------------------------------------------------------------------------
CudaFloat32EngineBase::CudaFloat32EngineBase(int deviceId, int streamPool_maxsize)
    : dev_(deviceId) {
    streamPool_.reset(new CudaStreamPool(dev_, streamPool_maxsize, 16));
    recomputeMaxParts();
}

void CudaFloat32EngineBase::recomputeMaxParts() {     // CudaFloat32EngineBase.java:86-92
    const int SM_count = dev_.multiProcessorCount();
    matMul_sk_maxPart = policy_smooth_maxPart(SM_count);
    matMulT1_sk_maxPart = policy_smooth_maxPart(SM_count);
    matMulT2_sk_maxPart = policy_smooth_maxPart(SM_count);
}

static void check_threshold(int threshold) {
    if (threshold <= 0 || (threshold & (threshold - 1)) != 0)
        throw IllegalArgumentException(fmt("threshold { got %lld } must be a power of 2", threshold));
}
static void check_maxPart(int maxPart) {
    if (maxPart < 4) throw IllegalArgumentException(fmt("maxPartNum { got %lld } must >= 4", maxPart));
}
void CudaFloat32EngineBase::matMul_splitK_threshold(int t) { check_threshold(t); matMul_sk_threshold = t; }
void CudaFloat32EngineBase::matMul_splitK_maxPart(int p) { check_maxPart(p); matMul_sk_maxPart = p; }
void CudaFloat32EngineBase::matMulT1_splitK_threshold(int t) { check_threshold(t); matMulT1_sk_threshold = t; }
void CudaFloat32EngineBase::matMulT1_maxPart(int p) { check_maxPart(p); matMulT1_sk_maxPart = p; }
void CudaFloat32EngineBase::matMulT2_splitK_threshold(int t) { check_threshold(t); matMulT2_sk_threshold = t; }
void CudaFloat32EngineBase::matMulT2_splitK_maxPart(int p) { check_maxPart(p); matMulT2_sk_maxPart = p; }
void CudaFloat32EngineBase::tf32(bool flag) {
    matMul_tf32 = matMulT1_tf32 = matMulT2_tf32 = flag;
    batchMatMul_tf32 = batchMatMulT1_tf32 = batchMatMulT2_tf32 = flag;
}

// ---- split-K policy as pure functions of (shape, unit count, knobs) ---------------------------
// The restriction block shared by the three products (e.g. CudaFloat32EngineBase.java:1551-1562).
// All arithmetic in float, truncation where Java casts to int.
static int policy_clamp(float fGridZ, int K, int b, int SM, float maxBlock, int maxPart) {
    if (fGridZ < 1.8f) return 1;
    int GridZ = (int)fGridZ;
    int GridZ2 = K >> 8;
    if (GridZ > GridZ2) GridZ = GridZ2;
    float coef = (float)K / ((float)K + 4096.0f);
    int GridZ3 = (int)((float)SM * maxBlock * coef / (float)b);
    if (GridZ > GridZ3) GridZ = GridZ3;
    if (GridZ < 2) GridZ = 2; else GridZ = (GridZ + 3) >> 2 << 2;
    if (GridZ > maxPart) GridZ = maxPart;
    return GridZ;
}

int policy_smooth_maxPart(int x) {   // CudaFloat32EngineBase.java:70-74
    if (x <= 32) x = (x + 3) >> 2 << 2; else x = (x + 7) >> 3 << 3;
    return x < 16 ? 16 : (x > 128 ? 128 : x);
}

int policy_matMul_gridZ(int N, int M, int K, int SM, const SplitKKnobs& k) {   // :1523-1532
    float fGridZ = 1; int b0 = 1;
    if (K >= k.threshold) {
        b0 = dragon_Cuda_matMul_blockNum(N, M);
        float expect_block_perSM = k.minBlock_perSM + 0.4f * (float)K / ((float)K + 1024.0f);
        if ((float)b0 < (float)SM * expect_block_perSM) {
            int b1 = dragon_Cuda_matMul_blockNum(K, M);
            int b2 = dragon_Cuda_matMul_blockNum(N, K);
            fGridZ = (float)(b1 + b2) / ((float)b0 * 2.0f);
        }
    }
    return policy_clamp(fGridZ, K, b0, SM, k.maxBlock_perSM, k.maxPart);
}

// :1604-1613 -- the same test as matMul without the 0.4 factor on K/(K+1024)
int policy_matMul_biased_gridZ(int N, int M, int K, int SM, const SplitKKnobs& k) {
    float fGridZ = 1; int b0 = 1;
    if (K >= k.threshold) {
        b0 = dragon_Cuda_matMul_blockNum(N, M);
        float expect_block_perSM = k.minBlock_perSM + (float)K / ((float)K + 1024.0f);
        if ((float)b0 < (float)SM * expect_block_perSM) {
            int b1 = dragon_Cuda_matMul_blockNum(K, M);
            int b2 = dragon_Cuda_matMul_blockNum(N, K);
            fGridZ = (float)(b1 + b2) / ((float)b0 * 2.0f);
        }
    }
    return policy_clamp(fGridZ, K, b0, SM, k.maxBlock_perSM, k.maxPart);
}

int policy_matMulT1_gridZ(int N, int M, int K, int SM, const SplitKKnobs& k) {  // :1740-1749
    float fGridZ = 1; int b1 = 1;
    if (K >= k.threshold) {
        b1 = dragon_Cuda_matMul_blockNum(N, M);
        float expect_block_perSM = k.minBlock_perSM + (float)K / ((float)K + 1024.0f);
        if ((float)b1 < (float)SM * expect_block_perSM) {
            int b0 = dragon_Cuda_matMul_blockNum(K, N);
            int b2 = dragon_Cuda_matMul_blockNum(K, M);
            fGridZ = (float)(b0 + b2) / ((float)b1 * 2.0f);
        }
    }
    return policy_clamp(fGridZ, K, b1, SM, k.maxBlock_perSM, k.maxPart);
}

// :1859-1867 and :1894 -- the reference tests blockNum(N,K) against the matMul (not matMulT2)
// block constants here and clamps with them; threshold and maxPart are the T2 fields.
int policy_matMulT2_gridZ(int N, int M, int K, int SM, const SplitKKnobs& t2, const SplitKKnobs& mm) {
    float fGridZ = 1; int b2 = 1;
    if (K >= t2.threshold) {
        b2 = dragon_Cuda_matMul_blockNum(N, K);
        float expect_block_perSM = mm.minBlock_perSM + (float)K / ((float)K + 1024.0f);
        if ((float)b2 < (float)SM * expect_block_perSM) {
            int b0 = dragon_Cuda_matMul_blockNum(N, M);
            int b1 = dragon_Cuda_matMul_blockNum(K, M);
            fGridZ = (float)(b1 + b2) / ((float)b0 * 2.0f);
        }
    }
    return policy_clamp(fGridZ, K, b2, SM, mm.maxBlock_perSM, t2.maxPart);
}

int CudaFloat32EngineBase::matMul_gridZ(int N, int M, int K) const {
    SplitKKnobs k = {matMul_sk_threshold, matMul_sk_maxPart, matMul_sk_minBlock_perSM, matMul_sk_maxBlock_perSM};
    return policy_matMul_gridZ(N, M, K, dev_.multiProcessorCount(), k);
}
// Cuda_conv3D.java:264-327: one stream per power-of-two piece of each extent, ten at most
static int conv_pieces(int G) {
    if ((G & (G - 1)) == 0) return 1;
    int s = 0;
    for (int bit = 128; bit >= 4; bit >>= 1) {
        if (G >= bit) s++;
        G &= bit - 1;
        if (G == 0) break;
    }
    return s;
}
int policy_conv3D_GEMM_nstream(int GM, int OC) {
    const int size = conv_pieces(OC) * conv_pieces(GM);
    return size < 10 ? size : 10;
}
int policy_conv3D_GEMMV2_nstream(int N, int OC) { return policy_conv3D_GEMM_nstream(N, OC); }
float policy_conv3D_psu(int IH, int IW, int OH, int OW, int FH, int FW, int sh, int sw) {   // :18-22
    const int input_size = IH * IW;
    const int pad_size = ((OH - 1) * sh + FH) * ((OW - 1) * sw + FW);
    return 1.0f * pad_size / input_size;
}

int CudaFloat32EngineBase::matMul_biased_gridZ(int N, int M, int K) const {
    SplitKKnobs k = {matMul_sk_threshold, matMul_sk_maxPart, matMul_sk_minBlock_perSM, matMul_sk_maxBlock_perSM};
    return policy_matMul_biased_gridZ(N, M, K, dev_.multiProcessorCount(), k);
}
int CudaFloat32EngineBase::matMulT1_gridZ(int N, int M, int K) const {
    SplitKKnobs k = {matMulT1_sk_threshold, matMulT1_sk_maxPart, matMulT1_sk_minBlock_perSM, matMulT1_sk_maxBlock_perSM};
    return policy_matMulT1_gridZ(N, M, K, dev_.multiProcessorCount(), k);
}
int CudaFloat32EngineBase::matMulT2_gridZ(int N, int M, int K) const {
    SplitKKnobs t2 = {matMulT2_sk_threshold, matMulT2_sk_maxPart, matMulT2_sk_minBlock_perSM, matMulT2_sk_maxBlock_perSM};
    SplitKKnobs mm = {matMul_sk_threshold, matMul_sk_maxPart, matMul_sk_minBlock_perSM, matMul_sk_maxBlock_perSM};
    return policy_matMulT2_gridZ(N, M, K, dev_.multiProcessorCount(), t2, mm);
}

int64_t CudaFloat32EngineBase::malloc(int64_t memsize) {   // :1148-1156
    std::lock_guard<std::mutex> g(g_cuda_class_lock);
    cu(dragon_Cuda_setDevice(dev_.getId()));
    return cu_handle(dragon_Cuda_malloc(memsize));
}
void CudaFloat32EngineBase::free(int64_t address) {        // :1158-1164
    std::lock_guard<std::mutex> g(g_cuda_class_lock);
    cu(dragon_Cuda_setDevice(dev_.getId()));
    cu(dragon_Cuda_free(address));
}
SyncerPtr CudaFloat32EngineBase::memset(int64_t address, int value, int64_t memsize) {  // :1166-1171
    int64_t stream = streamPool_->getStream();
    cu(dragon_Cuda_memsetAsync(stream, address, value, memsize));
    return SyncerPtr(new StreamSyncer(streamPool_.get(), stream));
}
// Transfers (:1197-1260): with a staging pool the _v2 natives, else the plain ones.
namespace {
struct StagingBlock {   // returns the block to the pool on every path out
    PinnedMempool* pool;
    PinnedMempool::Block b;
    StagingBlock(PinnedMempool* p, int64_t bytes) : pool(p), b(p->malloc(bytes)) {}
    ~StagingBlock() { pool->free(b.size, b.address); }
};
}  // namespace
void CudaFloat32EngineBase::get1D(int64_t address, float* value, int length) {
    int64_t stream = streamPool_->getStream();
    if (!bufPool_) cu(dragon_Cuda_get1D(stream, address, value, length));
    else {
        StagingBlock sb(bufPool_.get(), (int64_t)length << 2);
        cu(dragon_Cuda_get1D_v2(stream, address, value, sb.b.address, length));
    }
    streamPool_->returnStream(stream);
}
void CudaFloat32EngineBase::get2D(int64_t address, float* value, int height, int width, int stride) {
    int64_t stream = streamPool_->getStream();
    if (!bufPool_) cu(dragon_Cuda_get2D(stream, address, value, height, width, stride));
    else {
        StagingBlock sb(bufPool_.get(), ((int64_t)height * stride) << 2);
        cu(dragon_Cuda_get2D_v2(stream, address, value, sb.b.address, height, width, stride));
    }
    streamPool_->returnStream(stream);
}
void CudaFloat32EngineBase::set1D(int64_t address, const float* value, int length) {
    int64_t stream = streamPool_->getStream();
    if (!bufPool_) cu(dragon_Cuda_set1D(stream, address, value, length));
    else {
        StagingBlock sb(bufPool_.get(), (int64_t)length << 2);
        cu(dragon_Cuda_set1D_v2(stream, address, value, sb.b.address, length));
    }
    streamPool_->returnStream(stream);
}
void CudaFloat32EngineBase::set2D(int64_t address, const float* value, int height, int width, int stride) {
    int64_t stream = streamPool_->getStream();
    if (!bufPool_) cu(dragon_Cuda_set2D(stream, address, value, height, width, stride));
    else {
        StagingBlock sb(bufPool_.get(), ((int64_t)height * stride) << 2);
        cu(dragon_Cuda_set2D_v2(stream, address, value, sb.b.address, height, width, stride));
    }
    streamPool_->returnStream(stream);
}

// ---- RecyclingPool: Mempool.java:150-225 + Memp1.java:27-80; PinnedMempool.java:96-200 -------------
RecyclingPool::Block RecyclingPool::malloc(int64_t mem_size) {
    std::lock_guard<std::mutex> g(mu_);
    if (mem_size <= 0) throw IllegalArgumentException("mem_size must be positive");
    mem_size = (mem_size + 3) >> 2 << 2;
    if (mem_size > max_mem_size_)
        throw IllegalArgumentException(fmt("mem_size { got %lld } > mempool.max_mem_size { got %lld }",
                                           (long long)mem_size, (long long)max_mem_size_));
    int64_t size = 0, address = 0;
    auto it = pool_.lower_bound(mem_size);                       // remove_section(size, 1.5 * size)
    if (it != pool_.end() && it->first <= (int64_t)((double)mem_size * 1.5)) {
        size = it->first; address = it->second;
        pool_.erase(it);
    } else {
        // the Java pools wait up to 10 s for the collector or another thread to free memory; this one
        // fails at once
        if (mem_size > max_mem_size_ - used_mem_size_)
            throw std::runtime_error("[Error] Maximum Memory { " + std::to_string(max_mem_size_ >> 20) +
                                     " MB } is insufficient. Try to alloc more");
        while (mem_size > max_mem_size_ - total_mem_size_ && !pool_.empty()) {   // alloc_free: largest first
            auto big = std::prev(pool_.end());
            raw_free(big->second);
            total_mem_size_ -= big->first;
            blocks_.erase(big->second);
            grave_.erase(big->second);
            pool_.erase(big);
        }
        address = raw_malloc(mem_size);
        if (address == 0)
            throw std::runtime_error(std::string("failed to alloc ") + what() + " for [mem_size = " +
                                     std::to_string(mem_size) + " ]");
        size = mem_size;
        total_mem_size_ += size;
        blocks_[address] = size;
    }
    used_mem_size_ += size;
    grave_.erase(address);
    return Block{size >> 2, address};
}
bool RecyclingPool::free(int64_t size, int64_t address) {
    std::lock_guard<std::mutex> g(mu_);
    if (address == 0 || grave_.count(address) || !blocks_.count(address)) return false;
    const int64_t bytes = blocks_[address];   // what the block really holds (the caller reports the same)
    (void)size;
    pool_.emplace(bytes, address);
    grave_.insert(address);
    used_mem_size_ -= bytes;
    return true;
}
void RecyclingPool::clear() {
    std::lock_guard<std::mutex> g(mu_);
    for (auto& kv : blocks_) raw_free(kv.first);
    blocks_.clear(); pool_.clear(); grave_.clear();
    total_mem_size_ = used_mem_size_ = 0;
}
int64_t PinnedMempool::raw_malloc(int64_t bytes) { return dragon_Cuda_mallocHost(bytes); }
void PinnedMempool::raw_free(int64_t address) { (void)dragon_Cuda_freeHost(address); }
int64_t Memp1::raw_malloc(int64_t bytes) { return base_->malloc(bytes); }
void Memp1::raw_free(int64_t address) {
    try { base_->free(address); } catch (const std::exception&) {}   // also runs from destructors
}

// Shared body of matMul / matMulT1 / matMulT2 (:1534-1589, :1751-1806, :1870-1925) and, with a
// Bias address, of matMul_biased (:1615-1686): the bias row is the last thing issued on streams[0].
SyncerPtr CudaFloat32EngineBase::run_2d(int variant, int GridZ, int64_t C, int64_t A, int64_t B,
                                        int N, int M, int K, int64_t Bias, int lengthv, int width) {
    const int length = dragon_Cuda_matMul_nstream(N, M);
    std::vector<int64_t> streamArray = streamPool_->getStreamArray(length);
    const int n = (int)streamArray.size();
    last_gridZ = GridZ;
    last_stream_count = n;
    const bool big = (N > 127) && (M > 127) && (K % 8 == 0);
    if (GridZ < 2) {   // no need to split
        int rc;
        if (Bias != 0) {
            const bool mma = matMul_tf32 && big;
            if (matMul_biased_fused && !mma) {
                cu(dragon_Cuda_matMul_matMul_biased(streamArray.data(), n, A, B, C, Bias, N, M, K,
                                                    lengthv, width));
            } else {
                cu(mma ? dragon_Cuda_matMul_matMul_mma(streamArray.data(), n, A, B, C, N, M, K)
                       : dragon_Cuda_matMul_matMul(streamArray.data(), n, A, B, C, N, M, K));
                sync_streamArray_2_stream0(streamPool_.get(), streamArray);
                cu(dragon_Cuda_function_linear_dual2D_row(streamArray[0], C, Bias, M, 1.0f, 1.0f, 0.0f,
                                                          C, lengthv, width, M));
            }
            // the reference's BiasedForwardSyncer (:924-956) waits on streams[0] alone, where the
            // bias row ran; the stream-array syncer joins the idle streams first, same result
            return SyncerPtr(new StreamArraySyncer(streamPool_.get(), streamArray));
        }
        if (variant == 0)
            rc = (matMul_tf32 && big)
                     ? dragon_Cuda_matMul_matMul_mma(streamArray.data(), n, A, B, C, N, M, K)
                     : dragon_Cuda_matMul_matMul(streamArray.data(), n, A, B, C, N, M, K);
        else if (variant == 1)
            rc = (matMulT1_tf32 && big)
                     ? dragon_Cuda_matMul_matMulT1_mma(streamArray.data(), n, A, B, C, N, M, K)
                     : dragon_Cuda_matMul_matMulT1(streamArray.data(), n, A, B, C, N, M, K);
        else
            rc = (matMulT2_tf32 && big)
                     ? dragon_Cuda_matMul_matMulT2_mma(streamArray.data(), n, A, B, C, N, M, K)
                     : dragon_Cuda_matMul_matMulT2(streamArray.data(), n, A, B, C, N, M, K);
        cu(rc);
        return SyncerPtr(new StreamArraySyncer(streamPool_.get(), streamArray));
    }
    // split K to improve parallelism
    const int part = GridZ - 1;
    const int sizeC = N * M;
    if (core_ == nullptr) throw NullPointerException("engine core is not bound");
    EngineCore::Block block = core_->malloc(sizeC * part);
    const int64_t Cbuf = block.address;
    try {
        // stage 1: local products
        int rc;
        if (variant == 0)
            rc = dragon_Cuda_matMul_matMulSK(streamArray.data(), n, GridZ, A, B, C, Cbuf, N, M, K);
        else if (variant == 1)
            rc = dragon_Cuda_matMul_matMulT1SK(streamArray.data(), n, GridZ, A, B, C, Cbuf, N, M, K);
        else
            rc = dragon_Cuda_matMul_matMulT2SK(streamArray.data(), n, GridZ, A, B, C, Cbuf, N, M, K);
        cu(rc);
        // stage 2: global reduction on streams[0] once every stream has finished stage 1
        const int64_t stream = streamArray[0];
        sync_streamArray_2_stream0(streamPool_.get(), streamArray);
        cu(dragon_Cuda_matMul_SKbuf_summary(stream, Cbuf, C, part, sizeC));
        // stage 3 of matMul_biased: the bias row, after the reduction
        if (Bias != 0)
            cu(dragon_Cuda_function_linear_dual2D_row(stream, C, Bias, M, 1.0f, 1.0f, 0.0f, C, lengthv,
                                                      width, M));
    } catch (...) {
        core_->free(block.size, block.address);
        throw;
    }
    return SyncerPtr(new SplitKSyncer(core_, block, streamPool_.get(), streamArray));
}

SyncerPtr CudaFloat32EngineBase::matMul(int64_t C, int64_t A, int64_t B, int N, int M, int K) {
    return run_2d(0, matMul_gridZ(N, M, K), C, A, B, N, M, K);
}
SyncerPtr CudaFloat32EngineBase::matMul_biased(int64_t C, int64_t A, int64_t B, int N, int M, int K,
                                               int64_t Bias, int lengthv, int width) {   // :1594-1688
    if (Bias == 0) throw NullPointerException("Tensor Bias is null");
    return run_2d(0, matMul_biased_gridZ(N, M, K), C, A, B, N, M, K, Bias, lengthv, width);
}
SyncerPtr CudaFloat32EngineBase::linear2_2D_row(int64_t Y, int64_t X1, int64_t X2, int row_lengthv,
                                                float alpha, float beta, float gamma, int lengthv,
                                                int width, int stride) {   // :4517-4530
    int64_t stream = streamPool_->getStream();
    cu(dragon_Cuda_function_linear_dual2D_row(stream, X1, X2, row_lengthv, alpha, beta, gamma, Y,
                                              lengthv, width, stride));
    return SyncerPtr(new StreamSyncer(streamPool_.get(), stream));
}
// CudaFloat32EngineBase.java:2258-2383 (conv3D), :2386-2545 (conv3D_biased).  The reference chooses among
// kernel families; every family is the same MFMA kernel here, so what remains of the dispatch is which
// native is called (it documents the shape class) and the stream / event protocol.
SyncerPtr CudaFloat32EngineBase::run_conv(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W,
                                          int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph,
                                          int pw, int64_t Bias, int lengthv, int width) {
    if ((long long)N * OH * OW > 0x7fffffffLL || (long long)FH * FW * IC * OC > 0x7fffffffLL)
        throw IllegalArgumentException("the convolution is too large: N*OH*OW and FH*FW*IC*OC must fit 31 bits");
    const int GM = N * OH * OW;
    const bool w1 = (FH == 1) && (FW == 1) && (sh == 1) && (sw == 1) && (ph == 0) && (pw == 0);
    if (conv3D_remode && (OC > 31) && (GM > 31)) {
        // stage 1: W -> CW on its own stream; stage 2 waits for it
        const int GK = FH * FW * IC;
        EngineCore::Block block = core_->malloc(GK * OC);
        int64_t stream = 0;
        std::vector<int64_t> s;
        try {
            stream = streamPool_->getStream();
            cu(dragon_Cuda_conv3D_kernel_remode(stream, W, block.address, FH, FW, OC, IC));
            ScopedEvent event(streamPool_.get());
            cu(dragon_Cuda_eventRecord(event.handle, stream));
            s = streamPool_->getStreamArray(policy_conv3D_GEMM_nstream(GM, OC));
            const int n = (int)s.size();
            last_gridZ = 1; last_stream_count = n;
            cu(dragon_Cuda_streamsWaitEvent_default(s.data(), n, event.handle));
            if (w1)
                cu(dragon_Cuda_conv3D_conv3D_GemmR_W1(s.data(), n, X, IH, IW, W, block.address, Y, N, IC, OC));
            else if (conv3D_Gemm_useTexture)
                cu(dragon_Cuda_conv3D_conv3D_GemmR_texture(s.data(), n, X, IH, IW, W, block.address, FH, FW, Y,
                                                           OH, OW, N, IC, OC, sh, sw, ph, pw));
            else
                cu(dragon_Cuda_conv3D_conv3D_GemmR(s.data(), n, X, IH, IW, W, block.address, FH, FW, Y, OH, OW,
                                                   N, IC, OC, sh, sw, ph, pw));
            if (Bias) {   // stage 3 on the first stream, after stage 2
                ScopedEvent event2(streamPool_.get());
                cu(dragon_Cuda_eventRecord_streams(event2.handle, s.data(), n));
                cu(dragon_Cuda_streamWaitEvent_default(stream, event2.handle));
                cu(dragon_Cuda_function_linear_dual2D_row(stream, Y, Bias, OC, 1.0f, 1.0f, 0.0f, Y, lengthv,
                                                          width, OC));
            }
        } catch (...) {
            if (stream) {   // the block may be in use by what was issued: drain before it goes back
                dragon_Cuda_streamSynchronize(stream);
                streamPool_->returnStream(stream);
            }
            if (!s.empty()) {
                for (int64_t q : s) dragon_Cuda_streamSynchronize(q);
                streamPool_->returnStreamArray(s);
            }
            core_->free(block.size, block.address);
            throw;
        }
        s.insert(s.begin(), stream);   // Vector.append(stream, streamArray): the syncer waits for all of them
        return SyncerPtr(new FreeAfter(SyncerPtr(new StreamArraySyncer(streamPool_.get(), s)), core_,
                                       block.size, block.address));
    }
    const bool V2 = (N > 127) && (OC > 127) &&
                    policy_conv3D_psu(IH, IW, OH, OW, FH, FW, sh, sw) >= conv3D_GemmV2_Q;
    std::vector<int64_t> s = streamPool_->getStreamArray(V2 ? policy_conv3D_GEMMV2_nstream(N, OC)
                                                            : policy_conv3D_GEMM_nstream(GM, OC));
    const int n = (int)s.size();
    last_gridZ = 1; last_stream_count = n;
    const bool useTexture = conv3D_Gemm_useTexture && (OC > 15);
    try {
        if (Bias && conv3D_biased_fused)
            cu(dragon_Cuda_conv3D_conv3D_biased(s.data(), n, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh,
                                                sw, ph, pw, Bias, lengthv, width));
        else {
            if (w1)
                cu(dragon_Cuda_conv3D_conv3D_W1(s.data(), n, X, IH, IW, W, Y, N, IC, OC));
            else if ((ph == 0) && (pw == 0))
                cu(dragon_Cuda_conv3D_conv3D_np(s.data(), n, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw));
            else if (V2)
                cu(dragon_Cuda_conv3D_conv3DV2(useTexture, s.data(), n, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC,
                                               OC, sh, sw, ph, pw));
            else if (useTexture)
                cu(dragon_Cuda_conv3D_conv3D_texture(s.data(), n, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC,
                                                     sh, sw, ph, pw));
            else
                cu(dragon_Cuda_conv3D_conv3D(s.data(), n, X, IH, IW, W, FH, FW, Y, OH, OW, N, IC, OC, sh, sw,
                                             ph, pw));
            if (Bias) {   // the second launch, on streams[0] after every stream of the first
                ScopedEvent event(streamPool_.get());
                cu(dragon_Cuda_eventRecord_streams(event.handle, s.data(), n));
                cu(dragon_Cuda_streamWaitEvent_default(s[0], event.handle));
                cu(dragon_Cuda_function_linear_dual2D_row(s[0], Y, Bias, OC, 1.0f, 1.0f, 0.0f, Y, lengthv,
                                                          width, OC));
                }
        }
    } catch (...) { streamPool_->returnStreamArray(s); throw; }
    return SyncerPtr(new StreamArraySyncer(streamPool_.get(), s));
}
SyncerPtr CudaFloat32EngineBase::conv3D(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W,
                                        int FH, int FW, int N, int IC, int OC, int sh, int sw, int ph,
                                        int pw) {
    return run_conv(Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, 0, 0, 0);
}
SyncerPtr CudaFloat32EngineBase::conv3D_biased(int64_t Y, int OH, int OW, int64_t X, int IH, int IW,
                                               int64_t W, int FH, int FW, int N, int IC, int OC, int sh,
                                               int sw, int ph, int pw, int64_t Bias, int lengthv, int width) {
    if (Bias == 0) throw NullPointerException("Tensor Bias is null");
    return run_conv(Y, OH, OW, X, IH, IW, W, FH, FW, N, IC, OC, sh, sw, ph, pw, Bias, lengthv, width);
}
SyncerPtr CudaFloat32EngineBase::transpose(int64_t Y, const std::vector<int>& Ydim, int64_t X,
                                           const std::vector<int>& Xdim, int dimIndex1, int dimIndex2,
                                           int strideX, int strideY, int length) {   // :1343-1375
    int64_t stream = streamPool_->getStream();
    if (Xdim.size() == 4)
        cu(dragon_Cuda_expk2_transpose4D(stream, X, Y, Xdim[1], Xdim[2], Xdim[3], Ydim[1], Ydim[2], Ydim[3],
                                         dimIndex1, dimIndex2, strideX, strideY, length));
    else if (Xdim.size() == 3)
        cu(dragon_Cuda_expk2_transpose3D(stream, X, Y, Xdim[1], Xdim[2], Ydim[1], Ydim[2], dimIndex1,
                                         dimIndex2, strideX, strideY, length));
    else
        cu(dragon_Cuda_expk2_transpose2D(stream, X, Y, Xdim[1], Ydim[1], strideX, strideY, length));
    return SyncerPtr(new StreamSyncer(streamPool_.get(), stream));
}
SyncerPtr CudaFloat32EngineBase::linear2D(int64_t Y, float alpha, int64_t X, float beta, int lengthv,
                                          int width, int stride) {
    int64_t stream = streamPool_->getStream();
    cu(dragon_Cuda_function_linear2D(stream, alpha, X, beta, Y, lengthv, width, stride));
    return SyncerPtr(new StreamSyncer(streamPool_.get(), stream));
}
// :5738-5774 issues row_max, row_softmax and div2D_field with two temporary blocks; one launch here
SyncerPtr CudaFloat32EngineBase::softmax2D(int64_t Y, int64_t X, int field_length, int row_lengthv,
                                           int lengthv, int width, int stride, float scale) {
    (void)lengthv;
    int64_t stream = streamPool_->getStream();
    cu(dragon_Cuda_reduce_softmax2D(stream, X, Y, field_length, row_lengthv, width, stride, scale));
    return SyncerPtr(new StreamSyncer(streamPool_.get(), stream));
}
SyncerPtr CudaFloat32EngineBase::attention(int64_t Y, int64_t Q, int64_t K, int64_t V, int N, int head, int QL,
                                           int VL, int dK4, int dV4, bool head_inner, float scale, int64_t Mask,
                                           int mask_pitch, bool mask_per_head) {
    std::vector<int64_t> s = streamPool_->getStreamArray(1);
    last_gridZ = 1; last_stream_count = (int)s.size();
    try {
        if (Mask != 0)
            cu(dragon_Cuda_attention_forward_masked(s.data(), (int)s.size(), Q, K, V, Mask, Y, N, head, QL, VL, dK4,
                                                    dV4, head_inner ? 1 : 0, scale, mask_pitch, mask_per_head ? 1 : 0));
        else
        cu(dragon_Cuda_attention_forward(s.data(), (int)s.size(), Q, K, V, Y, N, head, QL, VL, dK4, dV4,
                                         head_inner ? 1 : 0, scale));
    } catch (...) { streamPool_->returnStreamArray(s); throw; }
    return SyncerPtr(new StreamArraySyncer(streamPool_.get(), s));
}
SyncerPtr CudaFloat32EngineBase::memcpy(int64_t dst, int64_t src, int64_t memsize) {   // :1173-1179
    int64_t stream = streamPool_->getStream();
    cu(dragon_Cuda_memcpyAsyncDeviceToDevice(stream, dst, src, memsize));
    return SyncerPtr(new StreamSyncer(streamPool_.get(), stream));
}
SyncerPtr CudaFloat32EngineBase::matMulT1(int64_t C, int64_t A, int64_t B, int N, int M, int K) {
    return run_2d(1, matMulT1_gridZ(N, M, K), C, A, B, N, M, K);
}
SyncerPtr CudaFloat32EngineBase::matMulT2(int64_t C, int64_t A, int64_t B, int N, int M, int K) {
    return run_2d(2, matMulT2_gridZ(N, M, K), C, A, B, N, M, K);
}

SyncerPtr CudaFloat32EngineBase::batchMatMul(int64_t C, int64_t A, int64_t B, int Batch, int N,
                                             int M, int BK, int AK) {   // :1939-1959
    const int length = dragon_Cuda_batchMatMul_streamSize(N, M);
    std::vector<int64_t> s = streamPool_->getStreamArray(length);
    const int n = (int)s.size();
    last_gridZ = 1; last_stream_count = n;
    int rc;
    if (batchMatMul_tf32 && (N > 127) && (M > 127) && (BK % 2 == 0) && (BK > 7))
        rc = dragon_Cuda_batchMatMul_batchMatMul_mma(batchMatMul_useTexture, s.data(), n, A, B, C,
                                                     Batch, N, M, BK, AK);
    else if (batchMatMul_useTexture)
        rc = dragon_Cuda_batchMatMul_batchMatMul_texture(s.data(), n, A, B, C, Batch, N, M, BK, AK);
    else
        rc = dragon_Cuda_batchMatMul_batchMatMul(s.data(), n, A, B, C, Batch, N, M, BK, AK);
    cu(rc);
    return SyncerPtr(new StreamArraySyncer(streamPool_.get(), s));
}

SyncerPtr CudaFloat32EngineBase::batchMatMulT1(int64_t C, int64_t A, int64_t B, int Batch, int CN,
                                               int AN, int M, int K) {  // :1966-1981
    const int length = dragon_Cuda_batchMatMul_streamSize(CN, M);
    std::vector<int64_t> s = streamPool_->getStreamArray(length);
    const int n = (int)s.size();
    last_gridZ = 1; last_stream_count = n;
    int rc;
    if (batchMatMulT1_tf32 && (CN > 127) && (M > 127) && (K > 7))
        rc = dragon_Cuda_batchMatMul_batchMatMulT1_mma(s.data(), n, A, B, C, Batch, CN, AN, M, K);
    else
        rc = dragon_Cuda_batchMatMul_batchMatMulT1(s.data(), n, A, B, C, Batch, CN, AN, M, K);
    cu(rc);
    return SyncerPtr(new StreamArraySyncer(streamPool_.get(), s));
}

SyncerPtr CudaFloat32EngineBase::batchMatMulT2(int64_t C, int64_t A, int64_t B, int Batch, int N,
                                               int CM, int BM, int K) { // :1995-2017
    const int length = dragon_Cuda_batchMatMul_streamSize(N, CM);
    std::vector<int64_t> s = streamPool_->getStreamArray(length);
    const int n = (int)s.size();
    last_gridZ = 1; last_stream_count = n;
    const bool useTexture = batchMatMulT2_useTexture && (N > 47) && (CM > 47);
    int rc;
    if (batchMatMulT2_tf32 && (N > 127) && (CM > 127) && (K > 7))
        rc = dragon_Cuda_batchMatMul_batchMatMulT2_mma(batchMatMulT2_useTexture, s.data(), n, A, B, C,
                                                       Batch, N, CM, BM, K);
    else if (useTexture)
        rc = dragon_Cuda_batchMatMul_batchMatMulT2_texture(s.data(), n, A, B, C, Batch, N, CM, BM, K);
    else
        rc = dragon_Cuda_batchMatMul_batchMatMulT2(s.data(), n, A, B, C, Batch, N, CM, BM, K);
    cu(rc);
    return SyncerPtr(new StreamArraySyncer(streamPool_.get(), s));
}

// ---- EngineCore ---------------------------------------------------------------------------------------
EngineCore::EngineCore(CudaFloat32EngineBase* base, bool chk) : check(chk), base_(base) {
    base_->engineCore(this);
}

EngineCore::Block EngineCore::malloc(int mem_length) {
    if (check && mem_length <= 0)
        throw IllegalArgumentException(fmt("mem_length { got %lld } must be positive", mem_length));
    Block b;
    if (mempool_) {            // EngineCore.malloc -> Mempool.malloc (EngineCore.java:154-165)
        const RecyclingPool::Block pb = mempool_->malloc((int64_t)pad4(mem_length) * 4);
        b.size = pb.size * 4;
        b.address = pb.address;
    } else {
        b.size = (int64_t)mem_length * 4;
        b.address = base_->malloc(b.size);
    }
    std::lock_guard<std::mutex> g(mu_);
    live_blocks_++;
    return b;
}
void EngineCore::free(int64_t size, int64_t address) {
    if (address == 0) return;
    if (mempool_) {
        if (!mempool_->free(size >> 2, address)) return;   // not this pool's, or freed already
    } else base_->free(address);
    std::lock_guard<std::mutex> g(mu_);
    live_blocks_--;
}
SyncerPtr EngineCore::memset(int64_t address, int value, int length) {
    if (check) {
        if (address == 0) throw NullPointerException("Tensor is null");
        if (length <= 0) throw IllegalArgumentException(fmt("length { got %lld } must > 0", length));
    }
    return base_->memset(address, value, (int64_t)length * 4);
}
void EngineCore::get1D(int64_t address, float* value, int length) {
    if (check && address == 0) throw NullPointerException("Tensor is null");
    base_->get1D(address, value, length);
}
void EngineCore::get2D(int64_t address, float* value, int height, int width) {
    if (check && address == 0) throw NullPointerException("Tensor is null");
    base_->get2D(address, value, height, width, pad4(width));
}
void EngineCore::set1D(int64_t address, const float* value, int length) {
    if (check && address == 0) throw NullPointerException("Tensor is null");
    base_->set1D(address, value, length);
}
void EngineCore::set2D(int64_t address, const float* value, int length, int width) {
    if (check) {
        if (address == 0) throw NullPointerException("Tensor is null");
        if (width <= 0 || length % width != 0)
            throw IllegalArgumentException(fmt("value.length { got %lld } %% width { got %lld } != 0", length, width));
    }
    base_->set2D(address, value, length / width, width, pad4(width));
}

void EngineCore::matMul_check(int64_t C, int64_t A, int64_t B, int N, int M, int K) const {  // :695-705
    if (C == 0) throw NullPointerException("Tensor C is null");
    if (B == 0) throw NullPointerException("Tensor B is null");
    if (A == 0) throw NullPointerException("Tensor A is null");
    if (N <= 0) throw IllegalArgumentException(fmt("N { got %lld } must > 0", N));
    if (M <= 0) throw IllegalArgumentException(fmt("M { got %lld } must > 0", M));
    if (K <= 0) throw IllegalArgumentException(fmt("K { got %lld } must > 0", K));
}

SyncerPtr EngineCore::transpose(int64_t Y, const std::vector<int>& Ydim, int64_t X,
                                const std::vector<int>& Xdim, int dimIndex1, int dimIndex2, int widthX,
                                int widthY, int length) {   // :582-613
    if (check) {
        auto s = [](int v) { return std::to_string(v); };
        if (Y == 0) throw NullPointerException("Tensor Y is null");
        if (X == 0) throw NullPointerException("Tensor X is null");
        if (Ydim.size() < 2) throw IllegalArgumentException("Y.ndim { got " + s((int)Ydim.size()) + " } must >= 2");
        if (Xdim.size() < 2) throw IllegalArgumentException("X.ndim { got " + s((int)Xdim.size()) + " } must >= 2");
        if (widthX <= 0) throw IllegalArgumentException("widthX { got " + s(widthX) + " } <= 0");
        if (length < widthX) throw IllegalArgumentException("length { got " + s(length) + " } < widthX { got " + s(widthX) + " }");
        if (length % widthX != 0) throw IllegalArgumentException("lengthv { got " + s(length) + " } % widthX { got " + s(widthX) + " } != 0");
        if (widthY <= 0) throw IllegalArgumentException("widthY { got " + s(widthY) + " } <= 0");
        if (length < widthY) throw IllegalArgumentException("length { got " + s(length) + " } < widthY { got " + s(widthY) + " }");
        if (length % widthY != 0) throw IllegalArgumentException("lengthv { got " + s(length) + " } % widthY { got " + s(widthY) + " } != 0");
    }
    return base_->transpose(Y, Ydim, X, Xdim, dimIndex1, dimIndex2, pad4(widthX), pad4(widthY), length);
}
SyncerPtr EngineCore::linear2D(int64_t Y, float alpha, int64_t X, float beta, int lengthv, int width) {
    const int stride = pad4(width);
    if (check) {
        if (Y == 0) throw NullPointerException("Tensor Y is null");
        if (X == 0) throw NullPointerException("Tensor X is null");
        auto s = [](int v) { return std::to_string(v); };
        if (lengthv < width) throw IllegalArgumentException("lengthv { got " + s(lengthv) + " } < width { got " + s(width) + " }");
        if (width <= 0) throw IllegalArgumentException("width { got " + s(width) + " } <= 0");
        if (lengthv % stride != 0) throw IllegalArgumentException("lengthv { got " + s(lengthv) + " } % stride { got " + s(stride) + " } != 0");
    }
    return base_->linear2D(Y, alpha, X, beta, lengthv, width, stride);
}
SyncerPtr EngineCore::softmax2D(int64_t Y, int64_t X, int row_length, int lengthv, int width, float scale) {  // :3368-3384
    const int stride = pad4(width);
    if (check) {
        if (X == 0) throw NullPointerException("Tensor X is NULL");
        if (Y == 0) throw NullPointerException("Tensor Y is NULL");
        auto s = [](int v) { return std::to_string(v); };
        if (width <= 0) throw IllegalArgumentException("width { got " + s(width) + " } <= 0");   // :1646-1657
        if (lengthv < row_length) throw IllegalArgumentException("lengthv { got " + s(lengthv) + " } < row_length { got " + s(row_length) + " }");
        if (row_length < width) throw IllegalArgumentException("row_length { got " + s(row_length) + " } < width { got " + s(width) + " }");
        if (row_length % width != 0) throw IllegalArgumentException("row_length { got " + s(row_length) + " } % width { got " + s(width) + " } != 0");
    }
    const int row_lengthv = row_length / width * stride;
    if (check && lengthv % row_lengthv != 0)
        throw IllegalArgumentException("lengthv { got " + std::to_string(lengthv) + " } % row_lengthv { got " +
                                       std::to_string(row_lengthv) + " } != 0");
    const int field_length = lengthv / row_lengthv;
    return base_->softmax2D(Y, X, field_length, row_lengthv, lengthv, width, stride, scale);
}
SyncerPtr EngineCore::memcpy(int64_t dst, int64_t src, int length) {
    if (check) {
        if (dst == 0) throw NullPointerException("dst is null");
        if (src == 0) throw NullPointerException("src is null");
        if (length <= 0) throw IllegalArgumentException("length must be positive");
    }
    return base_->memcpy(dst, src, (int64_t)length << 2);
}
void EngineCore::func_param_check_row(int lengthv, int row_lengthv, int width, int stride) const {  // :1613-1622
    auto s = [](int v) { return std::to_string(v); };
    if (lengthv < row_lengthv)
        throw IllegalArgumentException("lengthv { got " + s(lengthv) + " } < row_lengthv { " + s(row_lengthv) + " }");
    if (width <= 0) throw IllegalArgumentException("width { got " + s(width) + " } <= 0");
    if (lengthv % row_lengthv != 0)
        throw IllegalArgumentException("lengthv { got " + s(lengthv) + " } % row_lengthv { " + s(row_lengthv) + " } != 0");
    if (row_lengthv % stride != 0)
        throw IllegalArgumentException("row_lengthv { " + s(row_lengthv) + " } % stride { " + s(stride) + " } != 0");
}
SyncerPtr EngineCore::matMul_biased(int64_t C, int64_t A, int64_t B, int N, int M, int K, int64_t Bias,
                                    int lengthv) {   // :719-740
    const int M_4x = pad4(M);
    if (check) {
        matMul_check(C, A, B, N, M, K);
        if (Bias == 0) throw NullPointerException("Tensor Bias is null");
        func_param_check_row(lengthv, M_4x, M, M_4x);
    }
    return base_->matMul_biased(C, A, B, pad4(N), M_4x, pad4(K), Bias, lengthv, M);
}
// EngineCore.java:816-845
void EngineCore::conv3D_param_check(int OH, int OW, int IH, int IW, int FH, int FW, int N, int IC, int OC,
                                    int sh, int sw, int ph, int pw) const {
    auto s = [](long long v) { return std::to_string(v); };
    if (OH <= 0) throw IllegalArgumentException("OH { got " + s(OH) + " } must > 0");
    if (OW <= 0) throw IllegalArgumentException("OW { got " + s(OW) + " } must > 0");
    if (N <= 0) throw IllegalArgumentException("N  { got " + s(N) + " } must > 0");
    if (IC <= 0) throw IllegalArgumentException("IC { got " + s(IC) + " } must > 0");
    if (OC <= 0) throw IllegalArgumentException("OC { got " + s(OC) + " } must > 0");
    if (sh <= 0) throw IllegalArgumentException("sh { got " + s(sh) + " } must > 0");
    if (sw <= 0) throw IllegalArgumentException("sw { got " + s(sw) + " } must > 0");
    if (ph < 0) throw IllegalArgumentException("ph { got " + s(ph) + " } must >= 0");
    if (pw < 0) throw IllegalArgumentException("pw { got " + s(pw) + " } must >= 0");
    if (FH <= ph) throw IllegalArgumentException("FH { got " + s(FH) + " } <= ph { got " + s(ph) + " }");
    if (FW <= pw) throw IllegalArgumentException("FW { got " + s(FW) + " } <= pw { got " + s(pw) + " }");
    if (FH < sh) throw IllegalArgumentException("FH { got " + s(FH) + " } < sh { got " + s(sh) + " }");
    if (FW < sw) throw IllegalArgumentException("FW { got " + s(FW) + " } < sw { got " + s(sw) + " }");
    if (FH > IH + (ph << 1))
        throw IllegalArgumentException("FH { got " + s(FH) + " } > IH { got " + s(IH) + " } + 2 * ph { " + s(ph) + " }");
    if (FW > IW + (pw << 1))
        throw IllegalArgumentException("FW { got " + s(FW) + " } > IW { got " + s(IW) + " } + 2 * pw { " + s(pw) + " }");
}
SyncerPtr EngineCore::conv3D(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W, int FH, int FW,
                             int N, int IC, int OC, int sh, int sw, int ph, int pw) {   // :848-869
    if (check) {
        if (Y == 0) throw NullPointerException("Tensor Y is null");
        if (X == 0) throw NullPointerException("Tensor X is null");
        if (W == 0) throw NullPointerException("Tensor W is null");
        conv3D_param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw);
    }
    return base_->conv3D(Y, OH, OW, X, IH, IW, W, FH, FW, pad4(N), pad4(IC), pad4(OC), sh, sw, ph, pw);
}
SyncerPtr EngineCore::conv3D_biased(int64_t Y, int OH, int OW, int64_t X, int IH, int IW, int64_t W, int FH,
                                    int FW, int N, int IC, int OC, int sh, int sw, int ph, int pw,
                                    int64_t Bias, int lengthv) {   // :871-898
    const int OC_4x = pad4(OC);
    if (check) {
        if (Y == 0) throw NullPointerException("Tensor Y is null");
        if (X == 0) throw NullPointerException("Tensor X is null");
        if (W == 0) throw NullPointerException("Tensor W is null");
        conv3D_param_check(OH, OW, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw);
        if (Bias == 0) throw NullPointerException("Tensor Bias is null");
        func_param_check_row(lengthv, OC_4x, OC, OC_4x);
    }
    return base_->conv3D_biased(Y, OH, OW, X, IH, IW, W, FH, FW, pad4(N), pad4(IC), OC_4x, sh, sw, ph, pw,
                                Bias, lengthv, OC);
}
SyncerPtr EngineCore::attention(int64_t Y, int64_t Q, int64_t K, int64_t V, int N, int head, int QL, int VL,
                                int dK, int dV, bool head_inner, float scale, int64_t Mask, int mask_width,
                                bool mask_per_head) {
    if (check) {
        if (Y == 0) throw NullPointerException("Tensor Y is null");
        if (Q == 0) throw NullPointerException("Tensor Q is null");
        if (K == 0) throw NullPointerException("Tensor K is null");
        if (V == 0) throw NullPointerException("Tensor V is null");
        auto s = [](long long v) { return std::to_string(v); };
        if (N <= 0) throw IllegalArgumentException("N { got " + s(N) + " } must > 0");
        if (head <= 0) throw IllegalArgumentException("head { got " + s(head) + " } must > 0");
        if (QL <= 0) throw IllegalArgumentException("Q.seq_len { got " + s(QL) + " } must > 0");
        if (VL <= 0) throw IllegalArgumentException("V.seq_len { got " + s(VL) + " } must > 0");
        if (dK <= 0 || dV <= 0) throw IllegalArgumentException("head dimensions must > 0");
        if (head > 1 && ((dK & 3) || (dV & 3)))
            throw IllegalArgumentException("with several heads the head dimensions { got " + s(dK) + ", " + s(dV) +
                                           " } must be multiples of 4");
        if (pad4(dK) > 256 || pad4(dV) > 256)
            throw IllegalArgumentException("head dimensions { got " + s(dK) + ", " + s(dV) + " } must <= 256");
    }
    if (check && Mask != 0 && mask_width != VL)
        throw IllegalArgumentException("mask.width { got " + std::to_string(mask_width) + " } != V.seq_len { got " +
                                       std::to_string(VL) + " }");
    return base_->attention(Y, Q, K, V, N, head, QL, VL, pad4(dK), pad4(dV), head_inner, scale, Mask, pad4(mask_width),
                            mask_per_head);
}
SyncerPtr EngineCore::linear2_2D_row(int64_t Y, int64_t X1, int64_t X2, int row_lengthv, float alpha,
                                     float beta, float gamma, int lengthv, int width) {   // :1965-1983
    const int stride = pad4(width);
    if (check) {
        if (Y == 0) throw NullPointerException("Tensor Y is null");
        if (X1 == 0) throw NullPointerException("Tensor X1 is null");
        if (X2 == 0) throw NullPointerException("Tensor X2 is null");
        func_param_check_row(lengthv, row_lengthv, width, stride);
    }
    return base_->linear2_2D_row(Y, X1, X2, row_lengthv, alpha, beta, gamma, lengthv, width, stride);
}
SyncerPtr EngineCore::matMul(int64_t C, int64_t A, int64_t B, int N, int M, int K) {    // :708-717
    if (check) matMul_check(C, A, B, N, M, K);
    return base_->matMul(C, A, B, pad4(N), pad4(M), pad4(K));
}
SyncerPtr EngineCore::matMulT1(int64_t C, int64_t A, int64_t B, int N, int M, int K) {  // :743-752
    if (check) matMul_check(C, A, B, N, M, K);
    return base_->matMulT1(C, A, B, pad4(N), pad4(M), pad4(K));
}
SyncerPtr EngineCore::matMulT2(int64_t C, int64_t A, int64_t B, int N, int M, int K) {  // :755-764
    if (check) matMul_check(C, A, B, N, M, K);
    return base_->matMulT2(C, A, B, pad4(N), pad4(M), pad4(K));
}
SyncerPtr EngineCore::batchMatMul(int64_t C, int64_t A, int64_t B, int Batch, int N, int M, int K) {  // :767-780
    if (check) {
        if (Batch <= 0) throw IllegalArgumentException("Batch MatMul: Batch must be positive");
        matMul_check(C, A, B, N, M, K);
    }
    // A[Batch, N, AK] * B[Batch, BK, M] = C[Batch, N, M]
    return base_->batchMatMul(C, A, B, pad4(Batch), N, pad4(M), K, pad4(K));
}
SyncerPtr EngineCore::batchMatMulT1(int64_t C, int64_t A, int64_t B, int Batch, int N, int M, int K) {  // :782-795
    if (check) {
        if (Batch <= 0) throw IllegalArgumentException("Batch MatMul: Batch must be positive");
        matMul_check(C, A, B, N, M, K);
    }
    // (A[Batch, K, AN])^T * B[Batch, K, M] = C[Batch, CN, M]
    return base_->batchMatMulT1(C, A, B, pad4(Batch), N, pad4(N), pad4(M), K);
}
SyncerPtr EngineCore::batchMatMulT2(int64_t C, int64_t A, int64_t B, int Batch, int N, int M, int K) {  // :797-810
    if (check) {
        if (Batch <= 0) throw IllegalArgumentException("Batch MatMul: Batch must be positive");
        matMul_check(C, A, B, N, M, K);
    }
    // A[Batch, N, K] * (B[Batch, BM, K])^T = C[Batch, N, CM]
    return base_->batchMatMulT2(C, A, B, pad4(Batch), N, pad4(M), M, pad4(K));
}

// ---- Tensor --------------------------------------------------------------------------------------------
Tensor::Tensor(bool check, const std::vector<int>& d) {   // Tensor.java:206-239
    if (check) {
        if (d.empty()) throw IllegalArgumentException("Tensor.ndim == 0");
        for (size_t i = 0; i < d.size(); i++)
            if (d[i] <= 0)
                throw IllegalArgumentException(fmt("dim[%lld] { got %lld } must be positive", (long long)i, d[i]));
    }
    const int firstDim = d[0], firstDim_4x = pad4(firstDim);
    long long L4, Lv, L;
    if (d.size() == 1) {
        L4 = firstDim_4x; Lv = firstDim_4x; L = firstDim;
    } else {
        const int lastDim = d.back(), lastDim_4x = pad4(lastDim);
        long long midlen = 1;
        for (size_t i = 1; i + 1 < d.size(); i++) midlen *= d[i];
        L4 = (long long)firstDim_4x * midlen * lastDim_4x;
        Lv = (long long)firstDim * midlen * lastDim_4x;
        L = (long long)firstDim * midlen * lastDim;
    }
    if (L4 <= 0 || L4 > 0x7fffffffLL)
        throw IllegalArgumentException("the length of Tensor is exceed the upper limit");
    length_4x = (int)L4; lengthv = (int)Lv; length = (int)L;
    dim = d;
}
Tensor& Tensor::c() {
    if (syncer_) { syncer_->sync(); syncer_.reset(); }
    return *this;
}

// ---- Engine ------------------------------------------------------------------------------------------------
Engine::Engine(int deviceId, int streamPool_maxsize, int64_t max_trans_buf_size, int64_t max_mem_size) {
    base_.reset(new CudaFloat32EngineBase(deviceId, streamPool_maxsize));
    if (max_trans_buf_size > 0)
        base_->buf_mempool(std::unique_ptr<PinnedMempool>(new PinnedMempool(max_trans_buf_size)));
    core_.reset(new EngineCore(base_.get(), true));
    if (max_mem_size > 0) core_->mempool(std::unique_ptr<Memp1>(new Memp1(max_mem_size, base_.get())));
}
Engine::~Engine() {
    core_.reset();   // the pool hands its blocks back through the engine base, which must still be there
    base_.reset();
}

static void equals(int a, const char* an, int b, const char* bn) {
    if (a != b)
        throw IllegalArgumentException(std::string(an) + " { got " + std::to_string(a) + " } != " + bn +
                                       " { got " + std::to_string(b) + " }");
}
static void must_greater_equal(int a, const char* an, int b) {
    if (a < b)
        throw IllegalArgumentException(std::string(an) + " { got " + std::to_string(a) + " } must >= " +
                                       std::to_string(b));
}
static void require(Tensor* t, const char* name) {
    if (t == nullptr) throw NullPointerException(std::string("Tensor ") + name + " is null");
}

void Engine::finish(Tensor* C, SyncerPtr sc) {
    if (sync_) sc->sync(); else C->setSyncer(std::move(sc));
}

Tensor* Engine::empty(const std::vector<int>& dim) {   // Engine.java:522-532
    std::unique_ptr<Tensor> ts(new Tensor(check_, dim));
    EngineCore::Block b = core_->malloc(ts->length_4x);
    ts->mem_size = b.size; ts->address = b.address;
    if (ts->length_4x > ts->length) {   // padded: the pad must read as zero
        SyncerPtr sc = core_->memset(ts->address, 0, ts->length_4x);
        if (sync_) sc->sync(); else ts->setSyncer(std::move(sc));
    }
    return ts.release();
}
Tensor* Engine::zeros(const std::vector<int>& dim) {   // Engine.java:545-551
    std::unique_ptr<Tensor> ts(new Tensor(check_, dim));
    EngineCore::Block b = core_->malloc(ts->length_4x);
    ts->mem_size = b.size; ts->address = b.address;
    SyncerPtr sc = core_->memset(ts->address, 0, ts->length_4x);
    if (sync_) sc->sync(); else ts->setSyncer(std::move(sc));
    return ts.release();
}
Tensor* Engine::tensor(const float* value, int value_length, const std::vector<int>& dim_in) {  // :671-676
    if (value == nullptr) throw NullPointerException("value is null");
    std::vector<int> dim = dim_in;
    int neg = -1; long long known = 1;
    for (size_t i = 0; i < dim.size(); i++) {
        if (dim[i] == -1 && neg < 0) neg = (int)i; else known *= dim[i];
    }
    if (neg >= 0) {
        if (known <= 0 || value_length % known != 0)
            throw IllegalArgumentException("value.length is not a multiple of the known dimensions");
        dim[neg] = (int)(value_length / known);
    }
    Tensor* ts = empty(dim);
    try {
        ts->c();
        set(ts, value, value_length);
    } catch (...) { deleteTensor(ts); throw; }
    return ts;
}
Tensor* Engine::set(Tensor* X, const float* value, int value_length) {   // Engine.java:824-837
    if (check_) {
        require(X, "X");
        equals(value_length, "value<float>.length", X->length, "X.length");
    }
    if (X->ndim() == 1) core_->set1D(X->address, value, value_length);
    else {
        const int width = X->lastDim();
        if ((width & 3) == 0) core_->set1D(X->address, value, value_length);
        else core_->set2D(X->address, value, value_length, width);
    }
    return X;
}
std::vector<float> Engine::valueOf(Tensor* ts) {   // Engine.java:908-914
    require(ts, "ts");
    std::vector<float> out((size_t)ts->length);
    ts->c();
    if (ts->ndim() == 1) { core_->get1D(ts->address, out.data(), ts->length); return out; }
    const int width = ts->lastDim();
    if ((width & 3) == 0) core_->get1D(ts->address, out.data(), ts->length);
    else core_->get2D(ts->address, out.data(), ts->length / width, width);
    return out;
}
void Engine::deleteTensor(Tensor* ts) {
    if (ts == nullptr) return;
    ts->c();
    core_->free(ts->mem_size, ts->address);
    delete ts;
}

// 2-D products (Engine.java:958-995, 1042-1077, 1080-1118)
Tensor* Engine::matMul(Tensor* A, Tensor* B) {
    require(A, "A"); require(B, "B");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2");
        equals(A->dimAt(1), "A.width", B->dimAt(0), "B.height");
    }
    const int AH = A->dim[0], AW = A->dimAt(1), BW = B->dim[1];
    Tensor* C = &empty({AH, BW})->c();
    try { finish(C, core_->matMul(C->address, A->address, B->address, AH, BW, AW)); }
    catch (...) { deleteTensor(C); throw; }
    return C;
}
Tensor* Engine::matMul(Tensor* C, Tensor* A, Tensor* B) {
    require(C, "C"); require(A, "A"); require(B, "B");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2"); equals(C->ndim(), "C.ndim", 2, "2");
        equals(C->dimAt(0), "C.height", A->dimAt(0), "A.height");
        equals(C->dimAt(1), "C.width", B->dimAt(1), "B.width");
        equals(A->dimAt(1), "A.width", B->dimAt(0), "B.height");
    }
    finish(C, core_->matMul(C->address, A->address, B->address, A->dim[0], B->dim[1], A->dimAt(1)));
    return C;
}
// C = A * B + Bias (Engine.java:998-1039)
Tensor* Engine::matMul_biased(Tensor* A, Tensor* B, Tensor* Bias) {
    require(A, "A"); require(B, "B"); require(Bias, "Bias");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2");
        equals(A->dimAt(1), "A.width", B->dimAt(0), "B.height");
        equals(Bias->lastDim(), "Bias.lastDim", B->dimAt(1), "B.width");
    }
    const int AH = A->dim[0], AW = A->dimAt(1), BW = B->dim[1];
    Tensor* C = &empty({AH, BW})->c();
    try {
        finish(C, core_->matMul_biased(C->address, A->address, B->address, AH, BW, AW, Bias->address,
                                       C->lengthv));
    } catch (...) { deleteTensor(C); throw; }
    return C;
}
Tensor* Engine::matMul_biased(Tensor* C, Tensor* A, Tensor* B, Tensor* Bias) {
    require(C, "C"); require(A, "A"); require(B, "B"); require(Bias, "Bias");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2"); equals(C->ndim(), "C.ndim", 2, "2");
        equals(C->dimAt(0), "C.height", A->dimAt(0), "A.height");
        equals(C->dimAt(1), "C.width", B->dimAt(1), "B.width");
        equals(A->dimAt(1), "A.width", B->dimAt(0), "B.height");
        equals(Bias->lastDim(), "Bias.lastDim", B->dimAt(1), "B.width");
    }
    finish(C, core_->matMul_biased(C->address, A->address, B->address, A->dim[0], B->dim[1], A->dimAt(1),
                                   Bias->address, C->lengthv));
    return C;
}
// Engine.java:2076-2204.  Y given: the padding defaults are derived from the shapes, rounded up.
Tensor* Engine::conv3D(Tensor* Y, Tensor* X, Tensor* W, int sh, int sw, int ph, int pw) {
    return conv3D_biased(Y, X, W, sh, sw, ph, pw, nullptr);
}
Tensor* Engine::conv3D_biased(Tensor* Y, Tensor* X, Tensor* W, int sh, int sw, int ph, int pw, Tensor* Bias) {
    require(Y, "Y"); require(X, "X"); require(W, "W");
    if (check_) {
        equals(Y->ndim(), "Y.ndim", 4, "4"); equals(X->ndim(), "X.ndim", 4, "4"); equals(W->ndim(), "W.ndim", 4, "4");
        equals(Y->dimAt(0), "Y.batch", X->dimAt(0), "X.batch");
        equals(W->dimAt(0), "W.OC", Y->dimAt(3), "Y.OC");
        equals(W->dimAt(3), "W.IC", X->dimAt(3), "X.IC");
        if (Bias) equals(Bias->lastDim(), "Bias.lastDim", W->dimAt(0), "W.OC");
    }
    const int OH = Y->dim[1], OW = Y->dim[2];
    const int XN = X->dim[0], IH = X->dim[1], IW = X->dim[2];
    const int WOC = W->dim[0], FH = W->dim[1], FW = W->dim[2], WIC = W->dim[3];
    if (ph == -1) ph = ((OH - 1) * sh + FH - IH + 1) >> 1;
    if (pw == -1) pw = ((OW - 1) * sw + FW - IW + 1) >> 1;
    finish(Y, Bias ? core_->conv3D_biased(Y->address, OH, OW, X->address, IH, IW, W->address, FH, FW, XN, WIC, WOC,
                                          sh, sw, ph, pw, Bias->address, Y->lengthv)
                   : core_->conv3D(Y->address, OH, OW, X->address, IH, IW, W->address, FH, FW, XN, WIC, WOC, sh,
                                   sw, ph, pw));
    return Y;
}
// Y created: the output size defaults are derived from the padding, rounded down
Tensor* Engine::conv3D(Tensor* X, Tensor* W, int OH, int OW, int sh, int sw, int ph, int pw) {
    return conv3D_biased(X, W, OH, OW, sh, sw, ph, pw, nullptr);
}
Tensor* Engine::conv3D_biased(Tensor* X, Tensor* W, int OH, int OW, int sh, int sw, int ph, int pw,
                              Tensor* Bias) {
    require(X, "X"); require(W, "W");
    if (check_) {
        equals(X->ndim(), "X.ndim", 4, "4"); equals(W->ndim(), "W.ndim", 4, "4");
        equals(W->dimAt(3), "W.IC", X->dimAt(3), "X.IC");
        if (Bias) equals(Bias->lastDim(), "Bias.lastDim", W->dimAt(0), "W.OC");
        if (sh <= 0 || sw <= 0) throw IllegalArgumentException("sh, sw must > 0");
    }
    const int XN = X->dim[0], IH = X->dim[1], IW = X->dim[2];
    const int WOC = W->dim[0], FH = W->dim[1], FW = W->dim[2], WIC = W->dim[3];
    if (OH == -1) OH = (IH - FH + (ph << 1)) / sh + 1;
    if (OW == -1) OW = (IW - FW + (pw << 1)) / sw + 1;
    if (check_ && (OH <= 0 || OW <= 0))
        throw IllegalArgumentException("OH { got " + std::to_string(OH) + " }, OW { got " + std::to_string(OW) +
                                       " } must > 0");
    Tensor* Y = &empty({XN, OH, OW, WOC})->c();
    try {
        finish(Y, Bias ? core_->conv3D_biased(Y->address, OH, OW, X->address, IH, IW, W->address, FH, FW, XN, WIC,
                                              WOC, sh, sw, ph, pw, Bias->address, Y->lengthv)
                       : core_->conv3D(Y->address, OH, OW, X->address, IH, IW, W->address, FH, FW, XN, WIC, WOC,
                                       sh, sw, ph, pw));
    } catch (...) { deleteTensor(Y); throw; }
    return Y;
}
Tensor* Engine::matMulT1(Tensor* A, Tensor* B) {
    require(A, "A"); require(B, "B");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2");
        equals(A->dimAt(0), "A.height", B->dimAt(0), "B.height");
    }
    const int AH = A->dim[0], AW = A->dim[1], BW = B->dim[1];   // A[K, N], B[K, M]
    Tensor* C = &empty({AW, BW})->c();
    try { finish(C, core_->matMulT1(C->address, A->address, B->address, AW, BW, AH)); }
    catch (...) { deleteTensor(C); throw; }
    return C;
}
Tensor* Engine::matMulT1(Tensor* C, Tensor* A, Tensor* B) {
    require(C, "C"); require(A, "A"); require(B, "B");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2"); equals(C->ndim(), "C.ndim", 2, "2");
        equals(C->dimAt(0), "C.height", A->dimAt(1), "A.width");
        equals(C->dimAt(1), "C.width", B->dimAt(1), "B.width");
        equals(A->dimAt(0), "A.height", B->dimAt(0), "B.height");
    }
    finish(C, core_->matMulT1(C->address, A->address, B->address, A->dim[1], B->dim[1], A->dim[0]));
    return C;
}
Tensor* Engine::matMulT2(Tensor* A, Tensor* B) {
    require(A, "A"); require(B, "B");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2");
        equals(A->dimAt(1), "A.width", B->dimAt(1), "B.width");
    }
    const int AH = A->dim[0], AW = A->dim[1], BH = B->dim[0];   // A[N, K], B[M, K]
    Tensor* C = &empty({AH, BH})->c();
    try { finish(C, core_->matMulT2(C->address, A->address, B->address, AH, BH, AW)); }
    catch (...) { deleteTensor(C); throw; }
    return C;
}
Tensor* Engine::matMulT2(Tensor* C, Tensor* A, Tensor* B) {
    require(C, "C"); require(A, "A"); require(B, "B");
    if (check_) {
        equals(A->ndim(), "A.ndim", 2, "2"); equals(B->ndim(), "B.ndim", 2, "2"); equals(C->ndim(), "C.ndim", 2, "2");
        equals(C->dimAt(0), "C.height", A->dimAt(0), "A.height");
        equals(C->dimAt(1), "C.width", B->dimAt(0), "B.height");
        equals(A->dimAt(1), "A.width", B->dimAt(1), "B.width");
    }
    finish(C, core_->matMulT2(C->address, A->address, B->address, A->dim[0], B->dim[0], A->dim[1]));
    return C;
}

// batched products (Engine.java:1121-1312): batch = product of the leading dimensions
static std::vector<int> batched_dimC(bool likeA, Tensor* A, Tensor* B, int rows, int cols) {
    Tensor* L = likeA ? A : B;
    std::vector<int> dimC(L->dim.begin(), L->dim.end());
    dimC[dimC.size() - 2] = rows;
    dimC[dimC.size() - 1] = cols;
    return dimC;
}
static int batch_of(Tensor* T) { return T->length / (T->dimAt(-2) * T->dimAt(-1)); }

Tensor* Engine::batchMatMul(bool likeA, Tensor* A, Tensor* B) {
    require(A, "A"); require(B, "B");
    if (A->ndim() == 2 && B->ndim() == 2) return matMul(A, B);
    if (check_) {
        must_greater_equal(A->ndim(), "A.ndim", 3); must_greater_equal(B->ndim(), "B.ndim", 3);
        equals(A->dimAt(-1), "A.width", B->dimAt(-2), "B.height");
        equals(batch_of(A), "A.batch", batch_of(B), "B.batch");
    }
    const int AH = A->dimAt(-2), AW = A->dimAt(-1), BW = B->dimAt(-1);
    Tensor* C = &empty(batched_dimC(likeA, A, B, AH, BW))->c();
    try { finish(C, core_->batchMatMul(C->address, A->address, B->address, batch_of(A), AH, BW, AW)); }
    catch (...) { deleteTensor(C); throw; }
    return C;
}
Tensor* Engine::batchMatMul(Tensor* C, Tensor* A, Tensor* B) {
    require(C, "C"); require(A, "A"); require(B, "B");
    if (A->ndim() == 2 && B->ndim() == 2 && C->ndim() == 2) return matMul(C, A, B);
    if (check_) {
        must_greater_equal(A->ndim(), "A.ndim", 3); must_greater_equal(B->ndim(), "B.ndim", 3);
        must_greater_equal(C->ndim(), "C.ndim", 3);
        equals(C->dimAt(-2), "C.height", A->dimAt(-2), "A.height");
        equals(C->dimAt(-1), "C.width", B->dimAt(-1), "B.width");
        equals(A->dimAt(-1), "A.width", B->dimAt(-2), "B.height");
        equals(batch_of(A), "A.batch", batch_of(B), "B.batch");
        equals(batch_of(A), "A.batch", batch_of(C), "C.batch");
    }
    finish(C, core_->batchMatMul(C->address, A->address, B->address, batch_of(A), A->dimAt(-2),
                                 B->dimAt(-1), A->dimAt(-1)));
    return C;
}
Tensor* Engine::batchMatMulT1(bool likeA, Tensor* A, Tensor* B) {
    require(A, "A"); require(B, "B");
    if (A->ndim() == 2 && B->ndim() == 2) return matMulT1(A, B);
    if (check_) {
        must_greater_equal(A->ndim(), "A.ndim", 3); must_greater_equal(B->ndim(), "B.ndim", 3);
        equals(A->dimAt(-2), "A.height", B->dimAt(-2), "B.height");
        equals(batch_of(A), "A.batch", batch_of(B), "B.batch");
    }
    const int AH = A->dimAt(-2), AW = A->dimAt(-1), BW = B->dimAt(-1);   // A^T[N: AW, K: AH]
    Tensor* C = &empty(batched_dimC(likeA, A, B, AW, BW))->c();
    try { finish(C, core_->batchMatMulT1(C->address, A->address, B->address, batch_of(A), AW, BW, AH)); }
    catch (...) { deleteTensor(C); throw; }
    return C;
}
Tensor* Engine::batchMatMulT1(Tensor* C, Tensor* A, Tensor* B) {
    require(C, "C"); require(A, "A"); require(B, "B");
    if (A->ndim() == 2 && B->ndim() == 2 && C->ndim() == 2) return matMulT1(C, A, B);
    if (check_) {
        must_greater_equal(A->ndim(), "A.ndim", 3); must_greater_equal(B->ndim(), "B.ndim", 3);
        must_greater_equal(C->ndim(), "C.ndim", 3);
        equals(C->dimAt(-2), "C.height", A->dimAt(-1), "A.width");
        equals(C->dimAt(-1), "C.width", B->dimAt(-1), "B.width");
        equals(A->dimAt(-2), "A.height", B->dimAt(-2), "B.height");
        equals(batch_of(A), "A.batch", batch_of(B), "B.batch");
        equals(batch_of(A), "A.batch", batch_of(C), "C.batch");
    }
    finish(C, core_->batchMatMulT1(C->address, A->address, B->address, batch_of(A), A->dimAt(-1),
                                   B->dimAt(-1), A->dimAt(-2)));
    return C;
}
Tensor* Engine::batchMatMulT2(bool likeA, Tensor* A, Tensor* B) {
    require(A, "A"); require(B, "B");
    if (A->ndim() == 2 && B->ndim() == 2) return matMulT2(A, B);
    if (check_) {
        must_greater_equal(A->ndim(), "A.ndim", 3); must_greater_equal(B->ndim(), "B.ndim", 3);
        equals(A->dimAt(-1), "A.width", B->dimAt(-1), "B.width");
        equals(batch_of(A), "A.batch", batch_of(B), "B.batch");
    }
    const int AH = A->dimAt(-2), AW = A->dimAt(-1), BH = B->dimAt(-2);   // B^T[K: BW, M: BH]
    Tensor* C = &empty(batched_dimC(likeA, A, B, AH, BH))->c();
    try { finish(C, core_->batchMatMulT2(C->address, A->address, B->address, batch_of(A), AH, BH, AW)); }
    catch (...) { deleteTensor(C); throw; }
    return C;
}
Tensor* Engine::batchMatMulT2(Tensor* C, Tensor* A, Tensor* B) {
    require(C, "C"); require(A, "A"); require(B, "B");
    if (A->ndim() == 2 && B->ndim() == 2 && C->ndim() == 2) return matMulT2(C, A, B);
    if (check_) {
        must_greater_equal(A->ndim(), "A.ndim", 3); must_greater_equal(B->ndim(), "B.ndim", 3);
        must_greater_equal(C->ndim(), "C.ndim", 3);
        equals(C->dimAt(-2), "C.height", A->dimAt(-2), "A.height");
        equals(C->dimAt(-1), "C.width", B->dimAt(-2), "B.height");
        equals(A->dimAt(-1), "A.width", B->dimAt(-1), "B.width");
        equals(batch_of(A), "A.batch", batch_of(B), "B.batch");
        equals(batch_of(A), "A.batch", batch_of(C), "C.batch");
    }
    finish(C, core_->batchMatMulT2(C->address, A->address, B->address, batch_of(A), A->dimAt(-2),
                                   B->dimAt(-2), A->dimAt(-1)));
    return C;
}

// ---- fully connected layer: the 2-D products over a tensor of any rank, rows = length / lastDim
// (Engine.java:1315-1470).  Only the last dimension carries a padded stride, so the leading
// dimensions fold into one row count without moving data.
static std::vector<int> with_last(const Tensor* X, int last) {
    std::vector<int> d = X->dim;
    d.back() = last;
    return d;
}
Tensor* Engine::fullconnect(Tensor* X, Tensor* W) {
    require(X, "X"); require(W, "W");
    if (X->ndim() == 2) return matMul(X, W);
    if (check_) {
        must_greater_equal(X->ndim(), "X.ndim", 3);
        equals(W->ndim(), "W.ndim", 2, "2");
        equals(X->dimAt(-1), "X.features", W->dimAt(0), "W.in_features");
    }
    const int WOW = W->dim[1], XIW = X->dimAt(-1), GN = X->length / XIW;
    Tensor* Y = &empty(with_last(X, WOW))->c();
    try { finish(Y, core_->matMul(Y->address, X->address, W->address, GN, WOW, XIW)); }
    catch (...) { deleteTensor(Y); throw; }
    return Y;
}
Tensor* Engine::fullconnect(Tensor* Y, Tensor* X, Tensor* W) {
    require(Y, "Y"); require(X, "X"); require(W, "W");
    if (X->ndim() == 2 && Y->ndim() == 2) return matMul(Y, X, W);
    if (check_) {
        must_greater_equal(Y->ndim(), "Y.ndim", 2); must_greater_equal(X->ndim(), "X.ndim", 2);
        equals(W->ndim(), "W.ndim", 2, "2");
        equals(X->dimAt(-1), "X.features", W->dimAt(0), "W.in_features");
        equals(Y->dimAt(-1), "Y.features", W->dimAt(1), "W.out_features");
        equals(X->length / X->dimAt(-1), "(X.batch * X.height)", Y->length / Y->dimAt(-1), "(Y.batch * Y.height)");
    }
    const int WOW = W->dim[1], XIW = X->dimAt(-1), GN = X->length / XIW;
    finish(Y, core_->matMul(Y->address, X->address, W->address, GN, WOW, XIW));
    return Y;
}
Tensor* Engine::fullconnect_biased(Tensor* X, Tensor* W, Tensor* Bias) {
    require(X, "X"); require(W, "W"); require(Bias, "Bias");
    if (X->ndim() == 2) return matMul_biased(X, W, Bias);
    if (check_) {
        must_greater_equal(X->ndim(), "X.ndim", 3);
        equals(W->ndim(), "W.ndim", 2, "2");
        equals(X->dimAt(-1), "X.features", W->dimAt(0), "W.in_features");
        equals(Bias->length, "Bias.length", W->dimAt(1), "W.out_features");
    }
    const int WOW = W->dim[1], XIW = X->dimAt(-1), GN = X->length / XIW;
    Tensor* Y = &empty(with_last(X, WOW))->c();
    try {
        finish(Y, core_->matMul_biased(Y->address, X->address, W->address, GN, WOW, XIW, Bias->address,
                                       Y->lengthv));
    } catch (...) { deleteTensor(Y); throw; }
    return Y;
}
Tensor* Engine::fullconnect_biased(Tensor* Y, Tensor* X, Tensor* W, Tensor* Bias) {
    require(Y, "Y"); require(X, "X"); require(W, "W"); require(Bias, "Bias");
    if (X->ndim() == 2 && Y->ndim() == 2) return matMul_biased(Y, X, W, Bias);
    if (check_) {
        must_greater_equal(Y->ndim(), "Y.ndim", 2); must_greater_equal(X->ndim(), "X.ndim", 2);
        equals(W->ndim(), "W.ndim", 2, "2");
        equals(X->dimAt(-1), "X.features", W->dimAt(0), "W.in_features");
        equals(Y->dimAt(-1), "Y.features", W->dimAt(1), "W.out_features");
        equals(X->length / X->dimAt(-1), "(X.batch * X.height)", Y->length / Y->dimAt(-1), "(Y.batch * Y.height)");
        equals(Bias->length, "Bias.length", W->dimAt(1), "W.out_features");
    }
    const int WOW = W->dim[1], XIW = X->dimAt(-1), GN = X->length / XIW;
    finish(Y, core_->matMul_biased(Y->address, X->address, W->address, GN, WOW, XIW, Bias->address,
                                   Y->lengthv));
    return Y;
}
Tensor* Engine::fullconnect_deltaX(Tensor* deltaY, Tensor* W) {   // deltaX = deltaY * W^T
    require(deltaY, "deltaY"); require(W, "W");
    if (deltaY->ndim() == 2) return matMulT2(deltaY, W);
    if (check_) {
        must_greater_equal(deltaY->ndim(), "deltaY.ndim", 3);
        equals(W->ndim(), "W.ndim", 2, "2");
        equals(deltaY->dimAt(-1), "deltaY.features", W->dimAt(1), "W.out_features");
    }
    const int WIW = W->dim[0], YOW = deltaY->dimAt(-1), GN = deltaY->length / YOW;
    Tensor* deltaX = &empty(with_last(deltaY, WIW))->c();
    try { finish(deltaX, core_->matMulT2(deltaX->address, deltaY->address, W->address, GN, WIW, YOW)); }
    catch (...) { deleteTensor(deltaX); throw; }
    return deltaX;
}
Tensor* Engine::fullconnect_deltaW(Tensor* X, Tensor* deltaY) {   // deltaW = X^T * deltaY
    require(X, "X"); require(deltaY, "deltaY");
    if (deltaY->ndim() == 2 && X->ndim() == 2) return matMulT1(X, deltaY);
    if (check_) {
        must_greater_equal(X->ndim(), "X.ndim", 3); must_greater_equal(deltaY->ndim(), "deltaY.ndim", 3);
        equals(X->length / X->dimAt(-1), "(X.batch * X.height)", deltaY->length / deltaY->dimAt(-1),
               "(deltaY.batch * Y.height)");
    }
    const int XIW = X->dimAt(-1), YOW = deltaY->dimAt(-1), GK = deltaY->length / YOW;
    Tensor* deltaW = &empty({XIW, YOW})->c();
    try { finish(deltaW, core_->matMulT1(deltaW->address, X->address, deltaY->address, XIW, YOW, GK)); }
    catch (...) { deleteTensor(deltaW); throw; }
    return deltaW;
}

// Engine.java:1797-1831.  The reference supports 2 to 4 dimensions (anything else falls through to
// its 2-D native with the wrong shape); here more than 4 is refused.
namespace {
}  // namespace
Tensor* Engine::copy(Tensor* X) {
    require(X, "X");
    Tensor* Y = &empty(X->dim)->c();
    try { finish(Y, core_->memcpy(Y->address, X->address, X->length_4x)); }
    catch (...) { deleteTensor(Y); throw; }
    return Y;
}
Tensor* Engine::transpose(bool inplace, Tensor* X, int dimIdx1, int dimIdx2) {
    require(X, "X");
    const int nd = X->ndim();
    if (dimIdx1 < 0) dimIdx1 += nd;
    if (dimIdx2 < 0) dimIdx2 += nd;
    if (dimIdx1 == dimIdx2) return inplace ? X : copy(X);
    if (check_) {
        must_greater_equal(nd, "X.ndim", 2);
        if (nd > 4) throw IllegalArgumentException("X.ndim { got " + std::to_string(nd) + " } must <= 4");
        if (dimIdx1 < 0 || dimIdx1 >= nd) throw IllegalArgumentException("dimIdx1 is out of range");
        if (dimIdx2 < 0 || dimIdx2 >= nd) throw IllegalArgumentException("dimIdx2 is out of range");
    }
    X->c();
    std::vector<int> Ydim = X->dim;
    std::swap(Ydim[dimIdx1], Ydim[dimIdx2]);
    Tensor* Y = &empty(Ydim)->c();
    SyncerPtr sc1;
    try {
        sc1 = core_->transpose(Y->address, Ydim, X->address, X->dim, dimIdx1, dimIdx2, X->lastDim(),
                               Y->lastDim(), X->length);
    } catch (...) { deleteTensor(Y); throw; }
    if (!inplace) { finish(Y, std::move(sc1)); return Y; }
    // X takes over Y's shape and memory; the old memory goes back once the kernel has read it
    const int64_t old_size = X->mem_size, old_addr = X->address;
    X->dim = Y->dim; X->length = Y->length; X->lengthv = Y->lengthv; X->length_4x = Y->length_4x;
    X->mem_size = Y->mem_size; X->address = Y->address;
    delete Y;
    finish(X, SyncerPtr(new FreeAfter(std::move(sc1), core_.get(), old_size, old_addr)));
    return X;
}

Tensor* Engine::attention(Tensor* Q, Tensor* K, Tensor* V, int head, float scale, Tensor* mask) {
    require(Q, "Q"); require(K, "K"); require(V, "V");
    if (check_) {    // ChannelMHA.java:45-63
        must_greater_equal(Q->ndim(), "Q.ndim", 2); must_greater_equal(K->ndim(), "K.ndim", 2);
        must_greater_equal(V->ndim(), "V.ndim", 2);
        equals(Q->dimAt(0), "Q.batch", K->dimAt(0), "K.batch");
        equals(Q->dimAt(0), "Q.batch", V->dimAt(0), "V.batch");
        equals(Q->lastDim(), "Q.seq_dim", K->lastDim(), "K.seq_dim");
        if (head <= 0) throw IllegalArgumentException("head { got " + std::to_string(head) + " } must > 0");
        if (Q->lastDim() % head != 0 || V->lastDim() % head != 0)
            throw IllegalArgumentException("seq_dim { got " + std::to_string(Q->lastDim()) + ", " +
                                           std::to_string(V->lastDim()) + " } mod head { got " +
                                           std::to_string(head) + " } != 0");
    }
    const int N = Q->dim[0], KC = Q->lastDim(), VC = V->lastDim();
    const int QL = Q->length / (N * KC), KL = K->length / (N * KC), VL = V->length / (N * VC);
    if (check_ && KL != VL)
        throw IllegalArgumentException("K.seq_len { got " + std::to_string(KL) + " } != V.seq_len { got " +
                                       std::to_string(VL) + " }");
    if (scale == 0.0f) scale = 1.0f / sqrtf((float)KC);
    bool mask_per_head = false;
    if (mask != nullptr) {   // [QL, VL] for every image and head, or [N, head, QL, VL]
        const std::vector<int>& md = mask->dim;
        const bool one = md.size() == 2 && md[0] == QL && md[1] == VL;
        mask_per_head = md.size() == 4 && md[0] == N && md[1] == head && md[2] == QL && md[3] == VL;
        if (!one && !mask_per_head)
            throw IllegalArgumentException("mask.dim must be [Q.seq_len, V.seq_len] or [batch, head, Q.seq_len, V.seq_len]");
    }
    std::vector<int> Ydim = Q->dim;
    Ydim.back() = VC;
    Tensor* Y = &empty(Ydim)->c();
    try {
        finish(Y, core_->attention(Y->address, Q->address, K->address, V->address, N, head, QL, VL, KC / head,
                                   VC / head, true, scale, mask ? mask->address : 0, mask ? mask->lastDim() : 0,
                                   mask_per_head));
    } catch (...) { deleteTensor(Y); throw; }
    return Y;
}

// Engine.java:4002-4013
Tensor* Engine::linear(bool inplace, float alpha, Tensor* X, float beta) {
    require(X, "X");
    Tensor* Y = inplace ? X : &empty(X->dim)->c();
    try { finish(Y, core_->linear2D(Y->address, alpha, X->address, beta, X->lengthv, X->lastDim())); }
    catch (...) { if (!inplace) deleteTensor(Y); throw; }
    return Y;
}
// Engine.java:6082-6100
Tensor* Engine::softmax_scaled(bool inplace, Tensor* X, float scale, int features) {
    require(X, "X");
    if (features == -1) features = X->lastDim();
    if (check_) {
        must_greater_equal(X->ndim(), "X.ndim", 2);
        if (features <= 0 || X->length % features != 0)
            throw IllegalArgumentException("X.length { got " + std::to_string(X->length) + " } % features { got " +
                                           std::to_string(features) + " } != 0");
    }
    Tensor* Y = inplace ? X : &empty(X->dim)->c();
    try { finish(Y, core_->softmax2D(Y->address, X->address, features, X->lengthv, X->lastDim(), scale)); }
    catch (...) { if (!inplace) deleteTensor(Y); throw; }
    return Y;
}

// Engine.java:4185-4207, check_row :3781-3788
Tensor* Engine::linear2_row(bool inplace, Tensor* X1, Tensor* X2, float alpha, float beta, float gamma) {
    require(X1, "X1"); require(X2, "X2");
    if (check_) {
        must_greater_equal(X1->ndim(), "X1.ndim", 2);
        equals(X1->lastDim(), "X1.lastDim", X2->lastDim(), "X2.lastDim");
    }
    Tensor* Y = inplace ? X1 : &empty(X1->dim)->c();
    try {
        finish(Y, core_->linear2_2D_row(Y->address, X1->address, X2->address, X2->lengthv, alpha, beta,
                                        gamma, X1->lengthv, X1->lastDim()));
    } catch (...) { if (!inplace) deleteTensor(Y); throw; }
    return Y;
}

}  // namespace dragon
