// Embcache::FeatureFilter over the HIP library: a drop-in for the reference's
// training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/feature_filter/feature_filter.cpp.
//
// It compiles against the reference's own header (feature_filter/feature_filter.h:26-66, in place in the reference
// checkout) and defines the class's member functions; the counts and timestamps live in a device-resident history
// (recsdk_faae_*), one handle per filter, kept in a registry keyed by the object's address: the class has no spare
// member and no destructor, EmbcacheManager holds its filters by unique_ptr (embcache_manager.h:211), so the address
// is stable, and the constructor drops whatever an earlier object at the same address left behind.  The two maps the class exposes for checkpoints are rebuilt from the device records when
// they are asked for.  The pointer arguments are host memory, as in the reference: a slice goes up, the filtered keys
// come back.
#include "feature_filter/feature_filter.h"

#include <algorithm>
#include <cstdlib>
#include <limits>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "recsdk_hip.h"
#include "thread_stream.h"

namespace {

using recsdk_embcache::CopyDown;
using recsdk_embcache::CopyUp;
using recsdk_embcache::ThreadStream;
constexpr const char* kWho = "FeatureFilter";

struct DeviceState {
    recsdk_faae_t* h = nullptr;
    int64_t capacity = 0;
    int64_t maxKeys = 0;
    int64_t* keys = nullptr;      // [maxKeys]
    int64_t* times = nullptr;     // [maxKeys]
    uint32_t* counts = nullptr;   // [maxKeys]
    int64_t* offsets = nullptr;   // [2]
    int64_t* evicted = nullptr;   // [capacity]
};

std::mutex g_lock;
std::unordered_map<const void*, DeviceState> g_states;

void Release(DeviceState& s)
{
    if (s.h != nullptr) {
        recsdk_faae_destroy(s.h);
    }
    for (void* p : {static_cast<void*>(s.keys), static_cast<void*>(s.times), static_cast<void*>(s.counts),
                    static_cast<void*>(s.offsets), static_cast<void*>(s.evicted)}) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    s = DeviceState();
}

void Check(hipError_t e, const char* what)
{
    if (e != hipSuccess) {
        throw std::runtime_error(std::string("FeatureFilter (HIP): ") + what + ": " + hipGetErrorString(e));
    }
}

void Check(int rc, const char* what)
{
    if (rc != RECSDK_OK) {
        throw std::runtime_error(std::string("FeatureFilter (HIP): ") + what + ": " + recsdk_last_error());
    }
}

int64_t EnvOr(const char* name, int64_t fallback)
{
    const char* env = std::getenv(name);
    const long long v = env != nullptr ? std::atoll(env) : 0;
    return v > 0 ? v : fallback;
}

// RECSDK_EMBCACHE_FILTER_CAPACITY: live records a filter can hold (default 2^22); RECSDK_EMBCACHE_MAX_KEYS: keys per
// call (default 2^20; longer slices go up in pieces).
// The state is built aside and entered into the registry only when every allocation has succeeded: a failure half
// way leaves no entry whose buffers are missing.
DeviceState& StateOf(const void* self, int64_t admitThreshold, uint64_t evictThreshold)
{
    std::lock_guard<std::mutex> lock(g_lock);
    auto it = g_states.find(self);
    if (it != g_states.end()) {
        return it->second;
    }
    DeviceState s;
    try {
        s.capacity = EnvOr("RECSDK_EMBCACHE_FILTER_CAPACITY", 1LL << 22);
        s.maxKeys = EnvOr("RECSDK_EMBCACHE_MAX_KEYS", 1LL << 20);
        const int32_t countThreshold = admitThreshold == Embcache::INVALID_KEY ? -1 : static_cast<int32_t>(admitThreshold);
        const int32_t timeThreshold = evictThreshold == 0 ? -1 : static_cast<int32_t>(evictThreshold);
        const int32_t one = 1;
        Check(recsdk_faae_create(1, &s.capacity, &countThreshold, &timeThreshold, &one, &one, s.maxKeys, &s.h),
              "recsdk_faae_create");
        Check(hipMalloc(reinterpret_cast<void**>(&s.keys), sizeof(int64_t) * s.maxKeys), "hipMalloc");
        Check(hipMalloc(reinterpret_cast<void**>(&s.times), sizeof(int64_t) * s.maxKeys), "hipMalloc");
        Check(hipMalloc(reinterpret_cast<void**>(&s.counts), sizeof(uint32_t) * s.maxKeys), "hipMalloc");
        Check(hipMalloc(reinterpret_cast<void**>(&s.offsets), sizeof(int64_t) * 2), "hipMalloc");
        Check(hipMalloc(reinterpret_cast<void**>(&s.evicted), sizeof(int64_t) * s.capacity), "hipMalloc");
    } catch (...) {
        (void)hipGetLastError();
        Release(s);
        throw;
    }
    return g_states.emplace(self, s).first->second;
}

void SetSlice(DeviceState& s, const int64_t* keys, int64_t n)
{
    const int64_t off[2] = {0, n};
    CopyUp(s.offsets, off, sizeof(off), kWho);
    CopyUp(s.keys, keys, sizeof(int64_t) * n, kWho);
}

}  // namespace

namespace Embcache {

FeatureFilter::FeatureFilter(const std::string& tableName, int64_t admitThreshold, uint64_t evictThreshold,
                             uint64_t evictStepInterval)
    : tableName_(tableName), admitThreshold_(admitThreshold), evictThreshold_(evictThreshold),
      evictStepInterval_(evictStepInterval)
{
    std::lock_guard<std::mutex> lock(g_lock);
    auto it = g_states.find(this);
    if (it != g_states.end()) {
        Release(it->second);
        g_states.erase(it);
    }
}

bool FeatureFilter::IsAdmitEnabled() const
{
    return admitThreshold_ != INVALID_KEY;
}

void FeatureFilter::StatisticsKeyCount(const int64_t* featureDataPtr, const int64_t* countDataPtr, int64_t startIndex,
                                       int64_t endIndex, bool isCountDataEmpty)
{
    if (featureDataPtr == nullptr) {
        throw std::invalid_argument("featureDataPtr should not be nullptr");
    }
    if (!isCountDataEmpty && countDataPtr == nullptr) {
        throw std::invalid_argument("countDataPtr should not be nullptr when counts data is not empty");
    }
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    std::vector<uint32_t> counts;
    for (int64_t first = startIndex; first < endIndex; first += s.maxKeys) {
        const int64_t n = std::min(s.maxKeys, endIndex - first);
        SetSlice(s, featureDataPtr + first, n);
        if (!isCountDataEmpty) {
            counts.resize(static_cast<size_t>(n));
            for (int64_t i = 0; i < n; ++i) {
                const int64_t raw = countDataPtr[first + i];   // negative counts count as 0 (feature_filter.cpp:124-127)
                counts[i] = raw < 0 ? 0u : static_cast<uint32_t>(std::min<int64_t>(raw, 0xFFFFFFFELL));
            }
            CopyUp(s.counts, counts.data(), sizeof(uint32_t) * n, kWho);
        }
        Check(recsdk_faae_count_add(s.h, s.keys, isCountDataEmpty ? nullptr : s.counts, s.offsets, 1, n, ThreadStream()),
              "recsdk_faae_count_add");
    }
    Check(hipStreamSynchronize(ThreadStream()), "hipStreamSynchronize");
}

void FeatureFilter::CountFilter(int64_t* featureDataPtr, int64_t startIndex, int64_t endIndex)
{
    if (featureDataPtr == nullptr) {
        throw std::invalid_argument("featureDataPtr should not be nullptr");
    }
    if (!IsAdmitEnabled()) {
        return;
    }
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    for (int64_t first = startIndex; first < endIndex; first += s.maxKeys) {
        const int64_t n = std::min(s.maxKeys, endIndex - first);
        SetSlice(s, featureDataPtr + first, n);
        Check(recsdk_faae_count_filter(s.h, s.keys, s.offsets, 1, n, ThreadStream()), "recsdk_faae_count_filter");
        CopyDown(featureDataPtr + first, s.keys, sizeof(int64_t) * n, kWho);
    }
}

void FeatureFilter::RecordTimestamp(const int64_t* featureDataPtr, int64_t startIndex, int64_t endIndex,
                                    const int64_t* timestampDataPtr)
{
    if (featureDataPtr == nullptr || timestampDataPtr == nullptr) {
        throw std::invalid_argument("featureDataPtr and timestampDataPtr should not be nullptr");
    }
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    for (int64_t first = startIndex; first < endIndex; first += s.maxKeys) {
        const int64_t n = std::min(s.maxKeys, endIndex - first);
        SetSlice(s, featureDataPtr + first, n);
        CopyUp(s.times, timestampDataPtr + first, sizeof(int64_t) * n, kWho);
        Check(recsdk_faae_record_timestamp(s.h, s.keys, s.times, s.offsets, 1, n, ThreadStream()),
              "recsdk_faae_record_timestamp");
        for (int64_t i = 0; i < n; ++i) {
            latestTimestamp_ = std::max(latestTimestamp_, static_cast<std::time_t>(timestampDataPtr[first + i]));
        }
    }
    Check(hipStreamSynchronize(ThreadStream()), "hipStreamSynchronize");
    // the reference's cadence (feature_filter.cpp:48-52)
    if (evictStepInterval_ != 0 && recordTsBatchId_ > 0 && (recordTsBatchId_ + 1) % evictStepInterval_ == 0) {
        FeatureEvict();
    }
    recordTsBatchId_++;
}

void FeatureFilter::FeatureEvict()
{
    if (evictThreshold_ == 0) {
        return;
    }
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    int64_t offs[2] = {0, 0};
    Check(recsdk_faae_evict(s.h, /*strict=*/1, s.evicted, s.capacity, offs, ThreadStream()), "recsdk_faae_evict");
    std::vector<int64_t>& evictKeys = evictFeatureRecord_.GetEvictKeys();
    const size_t before = evictKeys.size();
    evictKeys.resize(before + static_cast<size_t>(offs[1]));
    if (offs[1] > 0) {
        CopyDown(evictKeys.data() + before, s.evicted, sizeof(int64_t) * offs[1], kWho);
    }
}

// The two maps are views for the checkpoint writer (embcache_manager.cpp:824-950): rebuilt from the device records.
static void Snapshot(DeviceState& s, std::vector<int64_t>& keys, std::vector<uint32_t>& counts,
                     std::vector<int64_t>& times)
{
    int64_t n = 0;
    int64_t* dTimes = nullptr;
    uint32_t* dCounts = nullptr;
    Check(hipMalloc(reinterpret_cast<void**>(&dTimes), sizeof(int64_t) * s.capacity), "hipMalloc");
    Check(hipMalloc(reinterpret_cast<void**>(&dCounts), sizeof(uint32_t) * s.capacity), "hipMalloc");
    Check(recsdk_faae_dump(s.h, 0, s.evicted, dCounts, dTimes, s.capacity, &n, ThreadStream()), "recsdk_faae_dump");
    keys.resize(static_cast<size_t>(n));
    counts.resize(static_cast<size_t>(n));
    times.resize(static_cast<size_t>(n));
    if (n > 0) {
        CopyDown(keys.data(), s.evicted, sizeof(int64_t) * n, kWho);
        CopyDown(counts.data(), dCounts, sizeof(uint32_t) * n, kWho);
        CopyDown(times.data(), dTimes, sizeof(int64_t) * n, kWho);
    }
    Check(hipFree(dTimes), "hipFree");
    Check(hipFree(dCounts), "hipFree");
}

const std::unordered_map<int64_t, FeatureRecord>& FeatureFilter::GetFeatureCountMap()
{
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    std::vector<int64_t> keys;
    std::vector<uint32_t> counts;
    std::vector<int64_t> times;
    Snapshot(s, keys, counts, times);
    featureRecordMap_.clear();
    for (size_t i = 0; i < keys.size(); ++i) {
        if (counts[i] != 0xFFFFFFFFu) {   // a record without a count only carries a timestamp
            featureRecordMap_[keys[i]] = FeatureRecord{counts[i]};
        }
    }
    return featureRecordMap_;
}

const std::unordered_map<int64_t, std::time_t>& FeatureFilter::GetFeatureTimestampMap()
{
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    std::vector<int64_t> keys;
    std::vector<uint32_t> counts;
    std::vector<int64_t> times;
    Snapshot(s, keys, counts, times);
    timestampRecordMap_.clear();
    for (size_t i = 0; i < keys.size(); ++i) {
        if (times[i] != std::numeric_limits<int64_t>::min()) {
            timestampRecordMap_[keys[i]] = static_cast<std::time_t>(times[i]);
        }
    }
    return timestampRecordMap_;
}

void FeatureFilter::LoadFeatureRecords(const std::vector<int64_t>& keys, std::vector<uint64_t>& counts)
{
    if (keys.size() != counts.size()) {
        throw std::runtime_error("Failed to load key count info, vector size is not same between keys and counts.");
    }
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    std::vector<uint32_t> c32;
    for (size_t first = 0; first < keys.size(); first += static_cast<size_t>(s.maxKeys)) {
        const int64_t n = static_cast<int64_t>(std::min<size_t>(static_cast<size_t>(s.maxKeys), keys.size() - first));
        c32.resize(static_cast<size_t>(n));
        for (int64_t i = 0; i < n; ++i) {
            c32[i] = static_cast<uint32_t>(std::min<uint64_t>(counts[first + i], 0xFFFFFFFEULL));
        }
        CopyUp(s.keys, keys.data() + first, sizeof(int64_t) * n, kWho);
        CopyUp(s.counts, c32.data(), sizeof(uint32_t) * n, kWho);
        Check(recsdk_faae_load(s.h, 0, s.keys, s.counts, nullptr, n, 0, std::numeric_limits<int64_t>::min(), ThreadStream()),
              "recsdk_faae_load");
    }
    Check(hipStreamSynchronize(ThreadStream()), "hipStreamSynchronize");
}

void FeatureFilter::LoadTimestampRecords(const std::vector<int64_t>& keys, std::vector<int64_t>& timestamps)
{
    if (keys.size() != timestamps.size()) {
        throw std::runtime_error("Failed to load timestamp info, vector size is not same between keys and timestamps.");
    }
    DeviceState& s = StateOf(this, admitThreshold_, evictThreshold_);
    for (size_t first = 0; first < keys.size(); first += static_cast<size_t>(s.maxKeys)) {
        const int64_t n = static_cast<int64_t>(std::min<size_t>(static_cast<size_t>(s.maxKeys), keys.size() - first));
        CopyUp(s.keys, keys.data() + first, sizeof(int64_t) * n, kWho);
        CopyUp(s.times, timestamps.data() + first, sizeof(int64_t) * n, kWho);
        Check(recsdk_faae_load(s.h, 0, s.keys, nullptr, s.times, n, 0, std::numeric_limits<int64_t>::min(), ThreadStream()),
              "recsdk_faae_load");
    }
    Check(hipStreamSynchronize(ThreadStream()), "hipStreamSynchronize");
}

}  // namespace Embcache

// Frees the device state of every FeatureFilter made so far (they must not be used afterwards).
extern "C" __attribute__((visibility("default"))) void recsdk_embcache_release_feature_filters()
{
    std::lock_guard<std::mutex> lock(g_lock);
    for (auto& kv : g_states) {
        Release(kv.second);
    }
    g_states.clear();
}
