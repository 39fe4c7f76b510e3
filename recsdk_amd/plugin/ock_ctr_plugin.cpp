// lib_ock_ctr_common.so for MI355X: the reference's plugin interface over librecsdk_hip.so.
//
// The reference's host runtime finds its dedup and HBM-cache code through one C symbol, CTR_CreateFactory
// (training/tf_rec_v1/src/AccCTR/src/factory_impl.cpp:26-41, loaded by include/ock_ctr_common_def.h:28-57), and
// three abstract classes: ock::ctr::Factory (include/factory.h:45-58), ock::ctr::Unique (include/unique.h:85-125)
// and EmbCache::EmbCacheManager (include/embedding_cache.h:182-374).  This file implements those classes on the HIP
// library: ids and key lists arrive in host memory (the interface says so), are staged to the device, and the
// results come back in the caller's buffers.  It is compiled against the reference's own interface headers where
// they lie in a reference checkout (see build.py); nothing of them is kept here.
//
// Error codes are the reference's CTRCode values (common/util/error_code.h), returned for the same conditions as
// UniqueImpl (unique/unique_impl.cpp:22-318) and EmbCacheManagerImpl (embedding_cache/cache_manager/
// cache_manager.cpp:27-503).  Differences: distinct ids come out in order of first occurrence (inside a shard when
// sharding is on) where the reference's order is that of its hash buckets; the thread arguments are checked like
// the reference's and otherwise unused; an extEmbeddingSize that is not a multiple of 4 floats is rejected with
// H_EXT_EMBEDDING_SIZE_INVALID.
#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <thread>
#include <unordered_set>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "error_code.h"  // reference: AccCTR/src/common/util
#include "factory.h"     // reference: AccCTR/src/include (pulls in unique.h and embedding_cache.h)
#include "recsdk_hip.h"

using namespace ock::ctr;
using namespace EmbCache;

namespace {

ExternalLog g_log = nullptr;
enum { LOG_DEBUG = 0, LOG_INFO = 1, LOG_WARN = 2, LOG_ERROR = 3 };  // LogLevel of common/util/external_logger.h

void log_msg(int level, const std::string& msg)
{
    if (g_log != nullptr) {
        g_log(level, msg.c_str());
    }
}

bool valid_thread_num(uint32_t threads)
{
    return threads != 0 && threads <= std::thread::hardware_concurrency();
}

// limits of the reference (common/util/defines.h:27-28, embedding_cache/common.h:53-62)
constexpr uint32_t kMaxDesiredSize = 1431655765u;
constexpr uint32_t kMaxIdCount = 1u << 29;
constexpr size_t kTableNameMax = 1024;
constexpr float kMeanMax = 1e9f, kMeanMin = -1e9f, kStdMax = 100.0f, kStdMin = 0.0f;
constexpr float kConstMax = 1e9f, kConstMin = -1e9f, kInitKMax = 10000.0f, kInitKMin = -10000.0f;

float clampf(float v, float lo, float hi, const char* what)
{
    if (v > hi) {
        log_msg(LOG_WARN, std::string(what) + " is greater than " + std::to_string(hi) + ", and will use it.");
        return hi;
    }
    if (v < lo) {
        log_msg(LOG_WARN, std::string(what) + " is less than " + std::to_string(lo) + ", and will use it.");
        return lo;
    }
    return v;
}

// A device buffer that only grows.
struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    bool reserve(size_t want)
    {
        if (want <= bytes) {
            return true;
        }
        if (p != nullptr) {
            (void)hipFree(p);
            p = nullptr;
            bytes = 0;
        }
        if (hipMalloc(&p, want) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        bytes = want;
        return true;
    }
    void release()
    {
        if (p != nullptr) {
            (void)hipFree(p);
        }
        p = nullptr;
        bytes = 0;
    }
    template <typename T>
    T* as() const
    {
        return static_cast<T*>(p);
    }
};

// The stream of the calling thread.  The reference's host runtime drives the tables from a pool of threads
// (hybrid_mgmt.cpp:545-560); with one stream per thread their kernels and copies run side by side on the device, where
// the null stream would put them in one queue.  Every entry point of this library that uses the stream waits for it
// before it returns, so a table may be driven by a different thread on every call.  The streams live as long as the
// process (threads of a pool do not end before it does).
hipStream_t ThreadStream()
{
    thread_local hipStream_t stream = nullptr;
    if (stream == nullptr && hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        stream = nullptr;   // the null stream still works
    }
    return stream;
}

bool h2d(void* dst, const void* src, size_t bytes)
{
    hipStream_t s = ThreadStream();
    return bytes == 0 || (hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s) == hipSuccess &&
                          hipStreamSynchronize(s) == hipSuccess);
}
bool d2h(void* dst, const void* src, size_t bytes)
{
    hipStream_t s = ThreadStream();
    return bytes == 0 || (hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s) == hipSuccess &&
                          hipStreamSynchronize(s) == hipSuccess);
}

// ---- ock::ctr::Unique ----------------------------------------------------------------------------------------------
class HipUnique : public Unique {
public:
    ~HipUnique() override { UnInitialize(); }

    int Initialize(const UniqueConf& in) override
    {
        UniqueConf conf = in;
        int ret = CheckConf(conf);
        if (ret != H_OK) {
            return ret;
        }
        if (conf.outputType == OutputType::NORMAL || !conf.useSharding) {
            conf.shardingNum = 1;
        }
        UnInitialize();
        conf_ = conf;
        if (!Grow(std::max<uint32_t>(conf.desiredSize, 1))) {
            UnInitialize();
            log_msg(LOG_ERROR, "memory alloc error");
            return H_MEMORY_ALLOC_ERROR;
        }
        ready_ = true;
        return H_OK;
    }

    void UnInitialize() override
    {
        if (uq_ != nullptr) {
            recsdk_unique_destroy(uq_);
            uq_ = nullptr;
        }
        if (rg_ != nullptr) {
            recsdk_regroup_destroy(rg_);
            rg_ = nullptr;
        }
        for (DevBuf* b : {&in_, &off_, &uid_, &index_, &inBucket_, &cntInBucket_, &idCnt_, &idCntFill_}) {
            b->release();
        }
        cap_ = 0;
        ready_ = false;
    }

    int DoUnique(UniqueIn& in, UniqueOut& out) override
    {
        if (!Ready()) {
            return H_UNIQUE_UNINITIALIZED_ERROR;
        }
        if (conf_.outputType != OutputType::NORMAL) {
            log_msg(LOG_ERROR, "output type error, should be NORMAL");
            return H_OUTPUT_TYPE_ERROR;
        }
        if (IsNull(in.inputId, "inputId") || IsNull(out.uniqueId, "uniqueId") || IsNull(out.index, "index")) {
            log_msg(LOG_ERROR, "input or conf is error");
            return H_ADDRESS_NULL;
        }
        const uint32_t n = in.inputIdCnt;
        int ret = Run(in);
        if (ret != H_OK) {
            log_msg(LOG_ERROR, "do unique error");
            return ret;
        }
        int64_t total = 0;
        if (recsdk_unique_fetch(uq_, uid_.as<int64_t>(), nullptr, index_.as<int32_t>(), nullptr, ThreadStream()) != RECSDK_OK ||
            recsdk_unique_total(uq_, ThreadStream(), &total) != RECSDK_OK) {
            return Fail();
        }
        if (!CopyIds(out.uniqueId, uid_.as<int64_t>(), (size_t)total) || !d2h(out.index, index_.p, sizeof(uint32_t) * n)) {
            return H_COPY_ERROR;
        }
        out.uniqueIdCnt = (int)total;
        return H_OK;
    }

    int DoEnhancedUnique(UniqueIn& in, EnhancedUniqueOut& out) override
    {
        if (!Ready()) {
            return H_UNIQUE_UNINITIALIZED_ERROR;
        }
        if (conf_.outputType != OutputType::ENHANCED) {
            log_msg(LOG_ERROR, "output type error, should be ENHANCED");
            return H_OUTPUT_TYPE_ERROR;
        }
        int ret = CheckEnhancedInput(in, out);
        if (ret != H_OK) {
            log_msg(LOG_ERROR, "input or conf is error.");
            return ret;
        }
        const uint32_t n = in.inputIdCnt;
        ret = Run(in);
        if (ret != H_OK) {
            log_msg(LOG_ERROR, "do unique error");
            return ret;
        }
        const int shards = conf_.shardingNum;
        const int pad = conf_.usePadding ? conf_.paddingSize : 0;
        const bool wantCnt = conf_.useIdCount;
        int32_t filled = 0;
        int rc = recsdk_unique_sharded(rg_, uq_, shards, conf_.performance ? 1 : 0, pad, (int64_t)conf_.paddingVal,
                                       uid_.as<int64_t>(), index_.as<uint32_t>(), inBucket_.as<int64_t>(),
                                       cntInBucket_.as<int32_t>(), wantCnt ? idCnt_.as<int32_t>() : nullptr,
                                       (wantCnt && pad > 0) ? idCntFill_.as<int32_t>() : nullptr, ThreadStream(), &filled);
        if (rc == RECSDK_ECAPACITY) {
            log_msg(LOG_ERROR, "do unique error");
            return H_PADDING_SMALL;
        }
        if (rc != RECSDK_OK) {
            return Fail();
        }
        std::vector<int32_t> perShard((size_t)shards);
        if (!d2h(perShard.data(), cntInBucket_.p, sizeof(int32_t) * shards)) {
            return H_COPY_ERROR;
        }
        size_t distinct = 0;
        for (int32_t c : perShard) {
            distinct += (size_t)c;
        }
        bool ok = CopyIds(out.uniqueId, uid_.as<int64_t>(), (size_t)filled) &&
                  d2h(out.index, index_.p, sizeof(uint32_t) * n);
        if (conf_.useSharding) {
            ok = ok && CopyIds(out.uniqueIdInBucket, inBucket_.as<int64_t>(), distinct);
            std::memcpy(out.uniqueIdCntInBucket, perShard.data(), sizeof(int32_t) * shards);
        }
        if (wantCnt) {
            ok = ok && d2h(out.idCnt, idCnt_.p, sizeof(int32_t) * distinct);
            if (pad > 0) {
                ok = ok && d2h(out.idCntFill, idCntFill_.p, sizeof(int32_t) * (size_t)filled);
            }
        }
        if (!ok) {
            return H_COPY_ERROR;
        }
        out.uniqueIdCnt = conf_.usePadding ? conf_.paddingSize * conf_.shardingNum : (int)distinct;
        return H_OK;
    }

    int SetExternalThreadFuncInner(ExternalThread) override { return H_OK; }  // the device does the work

private:
    static bool NonPositive(int64_t v, const char* name)
    {
        if (v <= 0) {
            log_msg(LOG_ERROR, std::string(name) + "can not be zero or negative");
            return true;
        }
        return false;
    }
    static bool IsNull(const void* p, const char* name)
    {
        if (p == nullptr) {
            log_msg(LOG_ERROR, std::string(name) + "can not be nullptr");
            return true;
        }
        return false;
    }

    static int CheckConf(const UniqueConf& conf)
    {
        if (NonPositive(conf.maxIdVal, "maxIdVal") || NonPositive(conf.desiredSize, "desiredSize")) {
            return H_NUM_SMALL;
        }
        const uint32_t cores = std::thread::hardware_concurrency();
        if (conf.maxThreadNum > cores) {
            log_msg(LOG_ERROR, "maxThreadNum can not larger than " + std::to_string(cores));
            return H_ERROR;
        }
        if (conf.maxThreadNum == 0 || conf.minThreadNum == 0 || conf.minThreadNum > conf.maxThreadNum) {
            log_msg(LOG_ERROR, "please check minThreadNum and maxThreadNum");
            return H_ERROR;
        }
        if (conf.desiredSize > kMaxDesiredSize) {
            log_msg(LOG_ERROR, "desiredSize can not larger than" + std::to_string(kMaxDesiredSize));
            return H_ERROR;
        }
        if (conf.outputType == OutputType::ENHANCED) {
            if (conf.usePadding) {
                if (!conf.useSharding) {
                    log_msg(LOG_ERROR, "sharding is not enable.");
                    return H_SCENE_ERROR;
                }
                if (NonPositive(conf.paddingSize, "paddingSize")) {
                    return H_NUM_SMALL;
                }
            }
            if (conf.useSharding) {
                if (NonPositive(conf.shardingNum, "shardingNum")) {
                    return H_NUM_SMALL;
                }
                if (conf.performance && (conf.shardingNum & (conf.shardingNum - 1)) != 0) {
                    log_msg(LOG_ERROR, "if performance is true, shardingNum must be 2^N");
                    return H_ERROR;
                }
            }
        }
        return H_OK;
    }

    int CheckEnhancedInput(const UniqueIn& in, const EnhancedUniqueOut& out) const
    {
        if (IsNull(in.inputId, "inputId") || IsNull(out.uniqueId, "uniqueId") || IsNull(out.index, "index")) {
            return H_ADDRESS_NULL;
        }
        if (conf_.useSharding &&
            (IsNull(out.uniqueIdInBucket, "uniqueIdInBucket") || IsNull(out.uniqueIdCntInBucket, "uniqueIdCntInBucket"))) {
            return H_ADDRESS_NULL;
        }
        if (conf_.useIdCount) {
            if (IsNull(out.idCnt, "idCnt")) {
                return H_ADDRESS_NULL;
            }
            if (conf_.usePadding && IsNull(out.idCntFill, "idCntFill")) {
                return H_ADDRESS_NULL;
            }
        }
        if (NonPositive(in.inputIdCnt, "inputIdCnt")) {
            return H_NUM_SMALL;
        }
        if (in.inputIdCnt > kMaxIdCount) {
            log_msg(LOG_ERROR, "inputIdCnt can not larger than 2^29");
            return H_ERROR;
        }
        return H_OK;
    }

    bool Ready() const
    {
        if (!ready_) {
            log_msg(LOG_ERROR, "please call Initialize before DoUnique");
        }
        return ready_;
    }

    int Fail() const
    {
        log_msg(LOG_ERROR, std::string("device library: ") + recsdk_last_error());
        return H_ERROR;
    }

    // handles and buffers for up to n ids per call
    bool Grow(size_t n)
    {
        if (n <= cap_) {
            return true;
        }
        if (uq_ != nullptr) {
            recsdk_unique_destroy(uq_);
            uq_ = nullptr;
        }
        if (rg_ != nullptr) {
            recsdk_regroup_destroy(rg_);
            rg_ = nullptr;
        }
        if (recsdk_unique_create((int64_t)n, 1, &uq_) != RECSDK_OK || recsdk_unique_set_lists(uq_, 0) != RECSDK_OK ||
            recsdk_regroup_create((int64_t)n, &rg_) != RECSDK_OK) {
            return false;
        }
        const size_t shards = (size_t)std::max(conf_.shardingNum, 1);
        const size_t padded = conf_.usePadding ? shards * (size_t)conf_.paddingSize : 0;
        const size_t m = std::max(n, padded);
        cap_ = n;
        return in_.reserve(sizeof(int64_t) * n) && off_.reserve(sizeof(int64_t) * 2) && uid_.reserve(sizeof(int64_t) * m) &&
               index_.reserve(sizeof(uint32_t) * n) && inBucket_.reserve(sizeof(int64_t) * n) &&
               cntInBucket_.reserve(sizeof(int32_t) * shards) && idCnt_.reserve(sizeof(int32_t) * n) &&
               idCntFill_.reserve(sizeof(int32_t) * m);
    }

    // stage the ids, check them against maxIdVal, run the dedup
    int Run(const UniqueIn& in)
    {
        const size_t n = in.inputIdCnt;
        if (n == 0) {
            return H_NUM_SMALL;
        }
        if (!Grow(n)) {
            log_msg(LOG_ERROR, "memory alloc error");
            return H_MEMORY_ALLOC_ERROR;
        }
        const int64_t* ids = nullptr;
        if (conf_.dataType == DataType::INT32) {
            const int32_t* narrow = static_cast<const int32_t*>(in.inputId);
            wide_.assign(narrow, narrow + n);
            ids = wide_.data();
        } else {
            ids = static_cast<const int64_t*>(in.inputId);
        }
        for (size_t i = 0; i < n; ++i) {
            if (ids[i] > conf_.maxIdVal) {
                log_msg(LOG_ERROR, "id val is larger than maxIdVal");
                return H_ID_LARGE;
            }
        }
        const int64_t offsets[2] = {0, (int64_t)n};
        if (!h2d(in_.p, ids, sizeof(int64_t) * n) || !h2d(off_.p, offsets, sizeof(offsets))) {
            return H_COPY_ERROR;
        }
        if (recsdk_unique_run(uq_, in_.as<int64_t>(), nullptr, off_.as<int64_t>(), 1, (int64_t)n, 0, 0, ThreadStream()) !=
            RECSDK_OK) {
            return Fail();
        }
        return H_OK;
    }

    // ids go back in the caller's width
    bool CopyIds(void* dst, const int64_t* src, size_t count)
    {
        if (conf_.dataType == DataType::INT64) {
            return d2h(dst, src, sizeof(int64_t) * count);
        }
        wide_.resize(count);
        if (!d2h(wide_.data(), src, sizeof(int64_t) * count)) {
            return false;
        }
        int32_t* narrow = static_cast<int32_t*>(dst);
        for (size_t i = 0; i < count; ++i) {
            narrow[i] = (int32_t)wide_[i];
        }
        return true;
    }

    UniqueConf conf_;
    bool ready_ = false;
    size_t cap_ = 0;
    recsdk_unique_t* uq_ = nullptr;
    recsdk_regroup_t* rg_ = nullptr;
    DevBuf in_, off_, uid_, index_, inBucket_, cntInBucket_, idCnt_, idCntFill_;
    std::vector<int64_t> wide_;
};

// ---- EmbCache::EmbCacheManager ----------------------------------------------------------------------------------
struct Planner {
    recsdk_om_t* om = nullptr;
    std::unordered_set<uint64_t> paddingKeysOffset;
    void release()
    {
        if (om != nullptr) {
            recsdk_om_destroy(om);
            om = nullptr;
        }
        paddingKeysOffset.clear();
    }
};

struct CacheTable {
    EmbCacheInfo info{"", 0, 0, 0, 0};
    int64_t maxKeys = 0;  // keys per planner call the handles are sized for
    Planner live;
    Planner backup;
    bool hasBackup = false;
    recsdk_hostrows_t* rows = nullptr;
    DevBuf keys, inKeys, inPos, outKeys, outPos;
    void release()
    {
        live.release();
        backup.release();
        if (rows != nullptr) {
            recsdk_hostrows_destroy(rows);
            rows = nullptr;
        }
        for (DevBuf* b : {&keys, &inKeys, &inPos, &outKeys, &outPos}) {
            b->release();
        }
    }
};

class HipEmbCacheManager : public EmbCacheManager {
public:
    ~HipEmbCacheManager() override { Destroy(); }

    int CreateCacheForTable(const EmbCacheInfo& info, const std::vector<InitializerInfo>& initializerInfos,
                            int64_t invalidKey, uint64_t prefillBufferSize, uint32_t refillThreadNum) override
    {
        if (info.tableName.empty()) {
            log_msg(LOG_ERROR, "tableName can not be empty");
            return H_TABLE_NAME_EMPTY;
        }
        if (info.tableName.size() > kTableNameMax) {
            log_msg(LOG_ERROR, "tableName size can not larger than " + std::to_string(kTableNameMax));
            return H_TABLE_NAME_TOO_LONG;
        }
        if (info.extEmbeddingSize == 0 || info.embeddingSize == 0 || info.vocabSize == 0 || info.maxCacheSize == 0) {
            log_msg(LOG_ERROR, "size must be positive");
            return H_SIZE_ZERO;
        }
        if (info.vocabSize < info.maxCacheSize) {
            log_msg(LOG_ERROR, "host vocabSize too small:" + std::to_string(info.vocabSize) + " < " +
                                   std::to_string(info.maxCacheSize) +
                                   ", need increase host vocabSize in create_table interface");
            return H_HOST_VOCAB_SIZE_TOO_SMALL;
        }
        if (tables_.count(info.tableName) != 0) {
            log_msg(LOG_ERROR, "This table has already been created");
            return H_TABLE_CREATE_DUPLICATE;
        }
        if (info.extEmbeddingSize % info.embeddingSize != 0) {
            log_msg(LOG_ERROR, "extEmbeddingSize = embeddingSize + optimizerSize, which is divisible by embeddingSize");
            return H_EXT_EMBEDDING_SIZE_INVALID;
        }
        if (info.extEmbeddingSize % 4 != 0) {
            log_msg(LOG_ERROR, "extEmbeddingSize must be a multiple of 4 floats on this device");
            return H_EXT_EMBEDDING_SIZE_INVALID;
        }
        std::vector<recsdk_initializer_desc_t> descs;
        if (!CheckInitializers(info.extEmbeddingSize, initializerInfos, &descs)) {
            return H_INITIALIZER_INVALID;
        }
        if (prefillBufferSize < 1 || prefillBufferSize > info.vocabSize) {
            log_msg(LOG_ERROR, "PrefillBufferSize: " + std::to_string(prefillBufferSize) +
                                   " has to be between [1, hostVocabSize].");
            return H_PREFILL_BUFFER_SIZE_INVALID;
        }
        if (!valid_thread_num(refillThreadNum)) {
            log_msg(LOG_ERROR, "ThreadNum must be between 1 and the cpu core num");
            return H_THREAD_NUM_ERROR;
        }
        CacheTable t;
        t.info = info;
        t.maxKeys = (int64_t)std::min<uint64_t>(std::max<uint64_t>(info.maxCacheSize, 1024), uint64_t(1) << 28);
        if (recsdk_om_create((int64_t)info.maxCacheSize, t.maxKeys, &t.live.om) != RECSDK_OK ||
            recsdk_hostrows_create((int64_t)info.vocabSize, (int32_t)info.extEmbeddingSize, descs.data(),
                                   (int32_t)descs.size(), &t.rows) != RECSDK_OK) {
            log_msg(LOG_ERROR, std::string("device library: ") + recsdk_last_error());
            t.release();
            return H_MEMORY_ALLOC_ERROR;
        }
        tables_.emplace(info.tableName, std::move(t));
        invalidKey_ = invalidKey;
        return H_OK;
    }

    int GetSwapPairsAndKey2Offset(const EmbBaseInfo& info, std::vector<uint64_t>& keys, KeyOffsetPair& swapIn,
                                  KeyOffsetPair& swapOut) override
    {
        if (!swapIn.first.empty() || !swapIn.second.empty() || !swapOut.first.empty() || !swapOut.second.empty()) {
            log_msg(LOG_ERROR, "koPair should be empty");
            return H_ARG_NOT_EMPTY;
        }
        CacheTable* t = nullptr;
        int ret = Find(info.name, &t);
        if (ret != H_OK) {
            return ret;
        }
        const size_t n = keys.size();
        if (!Reserve(t, n)) {
            return H_MEMORY_ALLOC_ERROR;
        }
        if (!h2d(t->keys.p, keys.data(), sizeof(uint64_t) * n)) {
            return H_COPY_ERROR;
        }
        if (recsdk_om_compute(t->live.om, t->keys.as<int64_t>(), (int64_t)n, t->inKeys.as<int64_t>(),
                              t->inPos.as<int64_t>(), t->outKeys.as<int64_t>(), t->outPos.as<int64_t>(), ThreadStream()) !=
            RECSDK_OK) {
            return DeviceError();
        }
        int64_t nIn = 0;
        int64_t nOut = 0;
        const int rc = recsdk_om_counts(t->live.om, ThreadStream(), &nIn, &nOut, nullptr, nullptr);
        if (rc == RECSDK_EOVERFLOW) {
            log_msg(LOG_ERROR, "Device cache overflow! Max cache size is too small. Please set a grater value for "
                               "`device_vocabulary_size` parameter when invoke `create_table` function. Current table:" +
                                   info.name + ", device_vocabulary_size:" + std::to_string(t->info.maxCacheSize));
            return H_MAX_CACHESIZE_TOO_SMALL;
        }
        if (rc != RECSDK_OK) {
            return DeviceError();
        }
        swapIn.first.resize((size_t)nIn);
        swapIn.second.resize((size_t)nIn);
        swapOut.first.resize((size_t)nOut);
        swapOut.second.resize((size_t)nOut);
        if (!d2h(keys.data(), t->keys.p, sizeof(uint64_t) * n) ||
            !d2h(swapIn.first.data(), t->inKeys.p, sizeof(uint64_t) * nIn) ||
            !d2h(swapIn.second.data(), t->inPos.p, sizeof(uint64_t) * nIn) ||
            !d2h(swapOut.first.data(), t->outKeys.p, sizeof(uint64_t) * nOut) ||
            !d2h(swapOut.second.data(), t->outPos.p, sizeof(uint64_t) * nOut)) {
            return H_COPY_ERROR;
        }
        // OffsetMapper::RecordPaddingKeysOffset (offset_mapper.h:296-307): slots handed to padding keys, train only
        if (info.channelId == 0 && info.paddingKeysMask) {
            for (size_t i = 0; i < (size_t)nIn; ++i) {
                if (std::find(info.paddingKeys.begin(), info.paddingKeys.end(), (int64_t)swapIn.first[i]) !=
                    info.paddingKeys.end()) {
                    t->live.paddingKeysOffset.insert(swapIn.second[i]);
                }
            }
        }
        return H_OK;
    }

    int EmbeddingLookup(const std::string& tableName, const std::vector<uint64_t>& keys, float* embAddr,
                        uint32_t threadNum) override
    {
        CacheTable* t = nullptr;
        int ret = CheckRowCall(tableName, threadNum, &t);
        if (ret != H_OK || keys.empty()) {
            return ret;
        }
        if (embAddr == nullptr) {
            log_msg(LOG_ERROR, "embAddr is nullptr");
            return H_ADDRESS_NULL;
        }
        return RowCode(recsdk_hostrows_gather(t->rows, AsKeys(keys), (int64_t)keys.size(), embAddr, (int32_t)threadNum));
    }

    int EmbeddingLookupAddrs(const std::string& tableName, const std::vector<uint64_t>& keys, std::vector<float*>& addrs,
                             uint32_t threadNum) override
    {
        CacheTable* t = nullptr;
        int ret = CheckRowCall(tableName, threadNum, &t);
        if (ret != H_OK || keys.empty()) {
            return ret;
        }
        std::vector<int64_t> rows(keys.size());
        float* base = nullptr;
        ret = RowCode(recsdk_hostrows_find_rows(t->rows, AsKeys(keys), (int64_t)keys.size(), 1, rows.data()));
        if (ret != H_OK) {
            return ret;
        }
        if (recsdk_hostrows_arena(t->rows, &base) != RECSDK_OK) {
            return DeviceError();
        }
        addrs.resize(keys.size());
        for (size_t i = 0; i < keys.size(); ++i) {
            addrs[i] = base + rows[i] * (int64_t)t->info.extEmbeddingSize;
        }
        return H_OK;
    }

    int EmbeddingLookupAndRemove(const std::string& tableName, const std::vector<uint64_t>& keys, float* embAddr,
                                 uint32_t threadNum) override
    {
        CacheTable* t = nullptr;
        int ret = CheckRowCall(tableName, threadNum, &t);
        if (ret != H_OK || keys.empty()) {
            return ret;
        }
        if (embAddr == nullptr) {
            log_msg(LOG_ERROR, "embAddr is nullptr");
            return H_ADDRESS_NULL;
        }
        return RowCode(recsdk_hostrows_gather_and_remove(t->rows, AsKeys(keys), (int64_t)keys.size(), embAddr));
    }

    int EmbeddingUpdate(const std::string& tableName, const std::vector<uint64_t>& keys, float* embAddr,
                        uint32_t threadNum) override
    {
        CacheTable* t = nullptr;
        int ret = CheckRowCall(tableName, threadNum, &t);
        if (ret != H_OK || keys.empty()) {
            return ret;
        }
        if (embAddr == nullptr) {
            log_msg(LOG_ERROR, "embAddr is nullptr");
            return H_ADDRESS_NULL;
        }
        return RowCode(recsdk_hostrows_scatter(t->rows, AsKeys(keys), (int64_t)keys.size(), embAddr, (int32_t)threadNum));
    }

    int EmbeddingRemove(const std::string& tableName, const std::vector<uint64_t>& keys, uint32_t threadNum) override
    {
        CacheTable* t = nullptr;
        int ret = CheckRowCall(tableName, threadNum, &t);
        if (ret != H_OK || keys.empty()) {
            return ret;
        }
        return RowCode(recsdk_hostrows_remove(t->rows, AsKeys(keys), (int64_t)keys.size()));
    }

    int RemoveEmbsByKeys(const std::string& tableName, const std::vector<uint64_t>& keys) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        std::vector<int64_t> valid;
        valid.reserve(keys.size());
        for (uint64_t k : keys) {
            if ((int64_t)k == invalidKey_) {
                log_msg(LOG_WARN, "Try to evict invalid key");
                continue;
            }
            valid.push_back((int64_t)k);
        }
        if (valid.empty()) {
            return H_OK;
        }
        if (!Reserve(t, valid.size())) {
            return H_MEMORY_ALLOC_ERROR;
        }
        if (!h2d(t->keys.p, valid.data(), sizeof(int64_t) * valid.size())) {
            return H_COPY_ERROR;
        }
        if (recsdk_om_remove(t->live.om, t->keys.as<int64_t>(), (int64_t)valid.size(), ThreadStream()) != RECSDK_OK ||
            hipStreamSynchronize(ThreadStream()) != hipSuccess) {
            return DeviceError();
        }
        return RowCode(recsdk_hostrows_remove(t->rows, valid.data(), (int64_t)valid.size()));
    }

    int GetEmbTableNames(std::vector<std::string>& allTableNames) override
    {
        if (!allTableNames.empty()) {
            log_msg(LOG_ERROR, "allTableNames should be empty");
            return H_ARG_NOT_EMPTY;
        }
        for (auto& kv : tables_) {
            allTableNames.emplace_back(kv.first);
        }
        return H_OK;
    }

    int ExportDeviceKeyOffsetPairs(const std::string& tableName,
                                   std::vector<std::pair<uint64_t, uint64_t>>& koVec) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        const size_t slots = (size_t)t->info.maxCacheSize;
        DevBuf tmp;
        std::vector<int64_t> pos2key(slots);
        if (!tmp.reserve(sizeof(int64_t) * slots)) {
            return H_MEMORY_ALLOC_ERROR;
        }
        const bool ok = recsdk_om_export(t->live.om, tmp.as<int64_t>(), ThreadStream()) == RECSDK_OK &&
                        d2h(pos2key.data(), tmp.p, sizeof(int64_t) * slots);
        tmp.release();
        if (!ok) {
            return DeviceError();
        }
        koVec.clear();
        for (size_t pos = 0; pos < slots; ++pos) {  // ascending slot = ExportSortedKVPairs' order
            if (pos2key[pos] != -1) {
                koVec.emplace_back((uint64_t)pos2key[pos], (uint64_t)pos);
            }
        }
        return H_OK;
    }

    int Serialize(const std::string& tableName, std::vector<char>& buffer) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        int64_t bytes = 0;
        if (recsdk_hostrows_serialize(t->rows, nullptr, 0, &bytes) != RECSDK_OK) {
            return DeviceError();
        }
        buffer.resize((size_t)bytes);
        if (recsdk_hostrows_serialize(t->rows, buffer.data(), bytes, &bytes) != RECSDK_OK) {
            return DeviceError();
        }
        return H_OK;
    }

    int Deserialize(const std::string& tableName, const std::vector<char>& buffer) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        if (recsdk_hostrows_deserialize(t->rows, buffer.data(), (int64_t)buffer.size()) != RECSDK_OK) {
            log_msg(LOG_ERROR, recsdk_last_error());
            return H_LOAD_ERROR;
        }
        return H_OK;
    }

    void Destroy() override
    {
        for (auto& kv : tables_) {
            kv.second.release();
        }
        tables_.clear();
    }

    uint32_t GetUsage(const std::string& tableName) override
    {
        auto it = tables_.find(tableName);
        int64_t live = 0;
        if (it == tables_.end() || recsdk_hostrows_size(it->second.rows, &live) != RECSDK_OK) {
            return 0;
        }
        return (uint32_t)live;
    }

    int GetEmbTableInfos(std::string tableName, std::vector<uint64_t>& keys, std::vector<std::vector<float>>& embeddings,
                         std::vector<std::vector<float>>& optimizerSlots) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        if (!keys.empty() || !embeddings.empty() || !optimizerSlots.empty()) {
            log_msg(LOG_ERROR, "keys, embeddings and optimizerSlots should be empty");
            return H_ARG_NOT_EMPTY;
        }
        int64_t live = 0;
        if (recsdk_hostrows_size(t->rows, &live) != RECSDK_OK) {
            return DeviceError();
        }
        const size_t ext = t->info.extEmbeddingSize;
        const size_t emb = t->info.embeddingSize;
        std::vector<int64_t> k((size_t)live);
        std::vector<float> rows((size_t)live * ext);
        int64_t count = 0;
        if (recsdk_hostrows_export(t->rows, k.data(), rows.data(), live, &count) != RECSDK_OK) {
            return DeviceError();
        }
        for (int64_t i = 0; i < count; ++i) {
            const float* row = rows.data() + (size_t)i * ext;
            keys.emplace_back((uint64_t)k[(size_t)i]);
            embeddings.emplace_back(row, row + emb);
            if (ext > emb) {
                optimizerSlots.emplace_back(row + emb, row + ext);
            }
        }
        return H_OK;
    }

    int LoadEmbTableInfos(std::string tableName, const std::vector<uint64_t>& keys,
                          const std::vector<std::vector<float>>& embeddings,
                          const std::vector<std::vector<float>>& optimizerSlots) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        const size_t ext = t->info.extEmbeddingSize;
        const size_t emb = t->info.embeddingSize;
        if (keys.size() != embeddings.size()) {
            log_msg(LOG_ERROR, "the size of keys and embeddings should be same!");
            return H_LOAD_ERROR;
        }
        if (ext > emb && keys.size() != optimizerSlots.size()) {
            log_msg(LOG_ERROR, "the size of keys and optimizerSlots should be same!");
            return H_LOAD_ERROR;
        }
        std::vector<float> rows(keys.size() * ext);
        for (size_t i = 0; i < keys.size(); ++i) {
            if (embeddings[i].size() != emb) {
                log_msg(LOG_ERROR, "The size of entering Embedding does not equals to embeddingSize");
                return H_LOAD_ERROR;
            }
            std::copy(embeddings[i].begin(), embeddings[i].end(), rows.begin() + i * ext);
            if (ext > emb) {
                if (optimizerSlots[i].size() != ext - emb) {
                    log_msg(LOG_ERROR,
                            "The size of entering optimizerSlot does not equals to extEmbeddingSize - embeddingSize");
                    return H_LOAD_ERROR;
                }
                std::copy(optimizerSlots[i].begin(), optimizerSlots[i].end(), rows.begin() + i * ext + emb);
            }
        }
        if (keys.empty()) {
            return H_OK;
        }
        if (recsdk_hostrows_scatter(t->rows, AsKeys(keys), (int64_t)keys.size(), rows.data(), 1) != RECSDK_OK) {
            log_msg(LOG_ERROR, recsdk_last_error());
            return H_LOAD_ERROR;
        }
        return H_OK;
    }

    // The evaluation phase plans on an empty mapper; the training mapper waits in the backup.
    int BackUpTrainStatus(const std::string& tableName) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        t->backup.release();
        t->backup = std::move(t->live);
        t->live = Planner();
        t->hasBackup = true;
        if (recsdk_om_create((int64_t)t->info.maxCacheSize, t->maxKeys, &t->live.om) != RECSDK_OK) {
            return H_MEMORY_ALLOC_ERROR;
        }
        return H_OK;
    }

    int RecoverTrainStatus(const std::string& tableName) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            return ret;
        }
        if (!t->hasBackup) {  // the reference assigns its empty backup mapper
            return ResetPlanner(t);
        }
        // the backup stays valid for a later recovery, as the reference's copy assignment leaves it
        Planner fresh;
        if (recsdk_om_create((int64_t)t->info.maxCacheSize, t->maxKeys, &fresh.om) != RECSDK_OK) {
            return H_MEMORY_ALLOC_ERROR;
        }
        if (recsdk_om_copy_state(fresh.om, t->backup.om, ThreadStream()) != RECSDK_OK ||
            hipStreamSynchronize(ThreadStream()) != hipSuccess) {
            fresh.release();
            return DeviceError();
        }
        fresh.paddingKeysOffset = t->backup.paddingKeysOffset;
        t->live.release();
        t->live = std::move(fresh);
        return H_OK;
    }

    int ResetOffsetMappers() override
    {
        for (auto& kv : tables_) {
            int ret = ResetPlanner(&kv.second);
            if (ret != H_OK) {
                return ret;
            }
        }
        return H_OK;
    }

    std::unordered_set<uint64_t> GetPaddingKeysOffset(const std::string& tableName) override
    {
        CacheTable* t = nullptr;
        int ret = Find(tableName, &t);
        if (ret != H_OK) {
            throw std::invalid_argument("Table: " + tableName + " is invalid, please check error log, and error code is " +
                                        std::to_string(ret) + ".");
        }
        return t->live.paddingKeysOffset;
    }

private:
    static const int64_t* AsKeys(const std::vector<uint64_t>& keys)
    {
        return reinterpret_cast<const int64_t*>(keys.data());
    }

    int Find(const std::string& tableName, CacheTable** out)
    {
        if (tableName.size() > kTableNameMax) {
            log_msg(LOG_ERROR, "tableName size can not larger than " + std::to_string(kTableNameMax));
            return H_TABLE_NAME_TOO_LONG;
        }
        auto it = tables_.find(tableName);
        if (it == tables_.end()) {
            log_msg(LOG_ERROR, "can not find table");
            return H_TABLE_NOT_EXIST;
        }
        *out = &it->second;
        return H_OK;
    }

    int CheckRowCall(const std::string& tableName, uint32_t threadNum, CacheTable** out)
    {
        int ret = Find(tableName, out);
        if (ret != H_OK) {
            return ret;
        }
        if (!valid_thread_num(threadNum)) {
            log_msg(LOG_ERROR, "ThreadNum must be between 1 and the cpu core num");
            return H_THREAD_NUM_ERROR;
        }
        return H_OK;
    }

    int DeviceError()
    {
        log_msg(LOG_ERROR, std::string("device library: ") + recsdk_last_error());
        return H_ERROR;
    }

    int RowCode(int rc)
    {
        if (rc == RECSDK_OK) {
            return H_OK;
        }
        log_msg(LOG_ERROR, recsdk_last_error());
        return rc == RECSDK_ECAPACITY ? H_HOST_VOCAB_SIZE_TOO_SMALL : H_ERROR;
    }

    static int ResetPlanner(CacheTable* t)
    {
        t->live.release();
        if (recsdk_om_create((int64_t)t->info.maxCacheSize, t->maxKeys, &t->live.om) != RECSDK_OK) {
            return H_MEMORY_ALLOC_ERROR;
        }
        return H_OK;
    }

    // device lists for n keys; a planner sized for fewer keys is replaced by a larger one with the same state
    bool Reserve(CacheTable* t, size_t n)
    {
        if ((int64_t)n > t->maxKeys) {
            int64_t want = t->maxKeys;
            while (want < (int64_t)n) {
                want *= 2;
            }
            for (Planner* p : {&t->live, &t->backup}) {
                if (p->om == nullptr) {
                    continue;
                }
                recsdk_om_t* bigger = nullptr;
                if (recsdk_om_create((int64_t)t->info.maxCacheSize, want, &bigger) != RECSDK_OK) {
                    return false;
                }
                if (recsdk_om_copy_state(bigger, p->om, ThreadStream()) != RECSDK_OK ||
                    hipStreamSynchronize(ThreadStream()) != hipSuccess) {
                    recsdk_om_destroy(bigger);
                    return false;
                }
                recsdk_om_destroy(p->om);
                p->om = bigger;
            }
            t->maxKeys = want;
        }
        const size_t bytes = sizeof(int64_t) * std::max<size_t>(n, 1);
        return t->keys.reserve(bytes) && t->inKeys.reserve(bytes) && t->inPos.reserve(bytes) &&
               t->outKeys.reserve(bytes) && t->outPos.reserve(bytes);
    }

    // CheckInitializer (cache_manager.cpp:402-424): the initializers must tile [0, extEmbeddingSize) without gaps
    static bool CheckInitializers(uint32_t ext, std::vector<InitializerInfo> infos,
                                  std::vector<recsdk_initializer_desc_t>* descs)
    {
        std::sort(infos.begin(), infos.end(), [](const auto& u, const auto& v) { return u.start < v.start; });
        uint32_t at = 0;
        for (const InitializerInfo& info : infos) {
            if (info.initializer == nullptr) {
                log_msg(LOG_ERROR, "initializer is nullptr");
                return false;
            }
            if (info.start != at) {
                log_msg(LOG_ERROR, "Initializers got coverage problems");
                return false;
            }
            at += info.len;
            recsdk_initializer_desc_t d{};
            d.start = info.start;
            d.len = info.len;
            if (info.initializerType == InitializerType::CONSTANT) {
                d.kind = RECSDK_INIT_CONSTANT;
                d.value_or_mean = info.constantInitializerInfo.constantValue;
                d.init_k = info.constantInitializerInfo.initK;
            } else {
                d.kind = info.initializerType == InitializerType::RANDOM_NORMAL ? RECSDK_INIT_RANDOM_NORMAL
                                                                                 : RECSDK_INIT_TRUNCATED_NORMAL;
                d.value_or_mean = info.normalInitializerInfo.mean;
                d.stddev = info.normalInitializerInfo.stddev;
                d.seed = info.normalInitializerInfo.seed;
                d.init_k = info.normalInitializerInfo.initK;
            }
            descs->push_back(d);
        }
        if (at != ext) {
            log_msg(LOG_ERROR, "Initializers got coverage problems");
            return false;
        }
        return true;
    }

    std::map<std::string, CacheTable> tables_;
    int64_t invalidKey_ = -1;
};

// ---- ock::ctr::Factory ---------------------------------------------------------------------------------------------
class HipFactory : public Factory {
public:
    int CreateUnique(UniquePtr& out) override
    {
        auto* u = new (std::nothrow) HipUnique();
        if (u == nullptr) {
            return H_NEW_OBJECT_FAILED;
        }
        out.reset(u);
        return H_OK;
    }
    int CreateEmbCacheManager(EmbCacheManagerPtr& out) override
    {
        auto* m = new (std::nothrow) HipEmbCacheManager();
        if (m == nullptr) {
            return H_NEW_OBJECT_FAILED;
        }
        out.reset(m);
        return H_OK;
    }
    int SetExternalLogFuncInner(ExternalLog logFunc) override
    {
        g_log = logFunc;
        return H_OK;
    }
};

std::mutex g_factoryLock;
HipFactory* g_factory = nullptr;

}  // namespace

// ---- the parts of include/embedding_cache.h that the reference's library defines and its callers link ------------
// (embedding_cache/initializer/initializer.cpp:22-58 and the three initializer sources)
namespace EmbCache {

ConstantInitializerInfo::ConstantInitializerInfo(float constantValue, float initK)
    : constantValue(constantValue), initK(initK)
{
}

NormalInitializerInfo::NormalInitializerInfo(float mean, float stddev, uint32_t seed, float initK)
    : mean(mean), stddev(stddev), seed(seed), initK(initK)
{
}

InitializerInfo::InitializerInfo(std::string& name, uint32_t start, uint32_t len, ConstantInitializerInfo constantInfo)
    : name(name), start(start), len(len), constantInitializerInfo(constantInfo)
{
    if (name == "constant_initializer") {
        initializerType = InitializerType::CONSTANT;
        initializer = std::make_shared<ConstantInitializer>(start, len, constantInfo.constantValue, constantInfo.initK);
    } else {
        log_msg(LOG_ERROR, "Invalid Initializer Type.");
    }
}

InitializerInfo::InitializerInfo(std::string& name, uint32_t start, uint32_t len, NormalInitializerInfo normalInfo)
    : name(name), start(start), len(len), normalInitializerInfo(normalInfo)
{
    if (name == "truncated_normal_initializer") {
        initializerType = InitializerType::TRUNCATED_NORMAL;
        initializer = std::make_shared<TruncatedNormalInitializer>(start, len, normalInfo);
    } else if (name == "random_normal_initializer") {
        initializerType = InitializerType::RANDOM_NORMAL;
        initializer = std::make_shared<RandomNormalInitializer>(start, len, normalInfo);
    } else {
        log_msg(LOG_ERROR, "Invalid Initializer Type.");
    }
}

static bool range_fits(uint32_t start, uint32_t len, int embSize)
{
    if (len == 0) {
        return false;
    }
    if (embSize != -1 && embSize < static_cast<int>(start + len)) {
        log_msg(LOG_WARN, "InitializeInfo start " + std::to_string(start) + " + len " + std::to_string(len) +
                              " is larger than embedding size " + std::to_string(embSize));
        return false;
    }
    return true;
}

ConstantInitializer::ConstantInitializer(uint32_t start, uint32_t len, float value, float initK) : start(start), len(len)
{
    constantValue = clampf(value, kConstMin, kConstMax, "constant value");
    initParam = clampf(initK, kInitKMin, kInitKMax, "constant initK");
}

void ConstantInitializer::GenerateData(float* emb, int embSize)
{
    if (range_fits(start, len, embSize)) {
        std::fill_n(emb + start, len, initParam * constantValue);
    }
}

RandomNormalInitializer::RandomNormalInitializer(uint32_t start, uint32_t len, NormalInitializerInfo& info)
    : start(start), len(len), seed(info.seed)
{
    mean = clampf(info.mean, kMeanMin, kMeanMax, "random normal mean");
    stddev = clampf(info.stddev, kStdMin, kStdMax, "random normal stddev");
    initParam = clampf(info.initK, kInitKMin, kInitKMax, "random normal initK");
    generator = std::default_random_engine(seed);
    distribution = std::normal_distribution<float>(mean, stddev);
}

void RandomNormalInitializer::GenerateData(float* emb, int embSize)
{
    if (range_fits(start, len, embSize)) {
        for (uint32_t j = 0; j < len; ++j) {
            emb[start + j] = initParam * distribution(generator);
        }
    }
}

TruncatedNormalInitializer::TruncatedNormalInitializer(uint32_t start, uint32_t len, NormalInitializerInfo& info)
    : start(start), len(len), seed(info.seed)
{
    mean = clampf(info.mean, kMeanMin, kMeanMax, "truncated normal mean");
    stddev = clampf(info.stddev, kStdMin, kStdMax, "truncated normal stddev");
    initParam = clampf(info.initK, kInitKMin, kInitKMax, "truncated normal initK");
    generator = std::default_random_engine(seed);
    distribution = std::normal_distribution<float>(mean, stddev);
    minBound = initParam * (mean - (float)boundNum * stddev);
    maxBound = initParam * (mean + (float)boundNum * stddev);
}

void TruncatedNormalInitializer::GenerateData(float* emb, int embSize)
{
    if (range_fits(start, len, embSize)) {
        for (uint32_t j = 0; j < len; ++j) {
            float v = initParam * distribution(generator);
            while (v < minBound || v > maxBound) {
                v = initParam * distribution(generator);
            }
            emb[start + j] = v;
        }
    }
}

}  // namespace EmbCache

extern "C" __attribute__((visibility("default"))) int CTR_CreateFactory(uintptr_t* outFactory)
{
    if (outFactory == nullptr) {
        return H_ADDRESS_NULL;
    }
    std::lock_guard<std::mutex> lock(g_factoryLock);
    if (g_factory == nullptr) {
        g_factory = new (std::nothrow) HipFactory();
        if (g_factory == nullptr) {
            return H_NEW_OBJECT_FAILED;
        }
    }
    *outFactory = reinterpret_cast<uintptr_t>(g_factory);
    return H_OK;
}
