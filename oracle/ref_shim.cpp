// C entry points around the REFERENCE's own torch-side sources (SwapManager, FeatureFilter, IdsMapper), which
// oracle/ref.mk compiles in place from the reference checkout into oracle/_ref/libref_torch.so.
// TEST INFRASTRUCTURE ONLY: used to validate the CPU oracle's restatement; never linked into the product.
// This file contains no reference code: it only calls the reference's public methods.
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <tuple>
#include <vector>

#include "embedding_cache/swap_manager.h"
#include "feature_filter/feature_filter.h"
#include "ids_mapper.h"
#include "unique.h"

#include <torch/custom_class.h>
#include <torch/library.h>

#define REF_API extern "C" __attribute__((visibility("default")))

namespace {
struct SwapBox {
    Embcache::SwapManager mgr;
    std::vector<int64_t> out[5];
    SwapBox(int64_t c, int64_t m) : mgr(c, m) {}
};

void CopyOut(const std::vector<int64_t>& v, int64_t* dst, int64_t cap)
{
    for (size_t i = 0; i < v.size() && static_cast<int64_t>(i) < cap; ++i) {
        dst[i] = v[i];
    }
}
}  // namespace

REF_API void* ref_swap_create(int64_t cacheSize, int64_t memStart) { return new SwapBox(cacheSize, memStart); }
REF_API void ref_swap_destroy(void* h) { delete static_cast<SwapBox*>(h); }

// returns 0, or -1 when the reference throws ("cacheSize_ too small")
REF_API int32_t ref_swap_compute(void* h, const int64_t* keys, int64_t n)
{
    auto* b = static_cast<SwapBox*>(h);
    std::vector<int64_t> k(keys, keys + n);
    try {
        auto r = b->mgr.ComputeSwapInfo(k);
        b->out[0] = std::get<0>(r);
        b->out[1] = std::get<1>(r);
        b->out[2] = std::get<2>(r);
        b->out[3] = std::get<3>(r);
        b->out[4] = std::get<4>(r);
    } catch (const std::runtime_error&) {
        return -1;
    }
    return 0;
}

REF_API int64_t ref_swap_result(void* h, int32_t which, int64_t* out, int64_t cap)
{
    auto* b = static_cast<SwapBox*>(h);
    CopyOut(b->out[which], out, cap);
    return static_cast<int64_t>(b->out[which].size());
}

REF_API void ref_swap_remove(void* h, const int64_t* keys, int64_t n)
{
    static_cast<SwapBox*>(h)->mgr.RemoveKeys(std::vector<int64_t>(keys, keys + n));
}

REF_API void* ref_filter_create(int64_t admitThreshold, uint64_t evictThreshold, uint64_t evictStepInterval)
{
    return new Embcache::FeatureFilter("t", admitThreshold, evictThreshold, evictStepInterval);
}
REF_API void ref_filter_destroy(void* h) { delete static_cast<Embcache::FeatureFilter*>(h); }

REF_API void ref_filter_statistics(void* h, const int64_t* keys, const int64_t* counts, int64_t n)
{
    static_cast<Embcache::FeatureFilter*>(h)->StatisticsKeyCount(keys, counts, 0, n, counts == nullptr);
}

REF_API void ref_filter_count_filter(void* h, int64_t* keys, int64_t n)
{
    static_cast<Embcache::FeatureFilter*>(h)->CountFilter(keys, 0, n);
}

// returns the number of keys the call evicted (the reference appends them to evictFeatureRecord_), copied to out
REF_API int64_t ref_filter_record_timestamp(void* h, const int64_t* keys, const int64_t* ts, int64_t n, int64_t* out,
                                            int64_t cap)
{
    auto* f = static_cast<Embcache::FeatureFilter*>(h);
    f->evictFeatureRecord_.GetEvictKeys().clear();
    f->RecordTimestamp(keys, 0, n, ts);
    const auto& ev = f->evictFeatureRecord_.GetEvictKeys();
    CopyOut(ev, out, cap);
    return static_cast<int64_t>(ev.size());
}

REF_API int64_t ref_filter_counts(void* h, int64_t* keys, uint64_t* counts, int64_t cap)
{
    const auto& m = static_cast<Embcache::FeatureFilter*>(h)->GetFeatureCountMap();
    int64_t i = 0;
    for (const auto& kv : m) {
        if (i < cap) {
            keys[i] = kv.first;
            counts[i] = kv.second.count;
        }
        ++i;
    }
    return i;
}

// c10::List of a custom class needs the class registered with the dispatcher (checker-local namespace)
TORCH_LIBRARY(recsdk_ref_shim, m)
{
    m.class_<hybrid::IdsMapper>("IdsMapper").def(torch::init<int64_t, bool>());
}

// IdsMapper::ParallelUniqueHashOut over T mappers; outputs are caller-allocated (n or T+1 entries)
REF_API void* ref_ids_create(int64_t T, const int64_t* initMaxIndex)
{
    auto* v = new c10::List<c10::intrusive_ptr<hybrid::IdsMapper>>();
    for (int64_t t = 0; t < T; ++t) {
        v->push_back(c10::make_intrusive<hybrid::IdsMapper>(initMaxIndex[t], true));
    }
    return v;
}
REF_API void ref_ids_destroy(void* h) { delete static_cast<c10::List<c10::intrusive_ptr<hybrid::IdsMapper>>*>(h); }

REF_API int32_t ref_ids_parallel_unique_hash_out(void* h, const int64_t* ids, int64_t n, const int64_t* offsets,
                                                 int64_t T, int64_t* hashIndices, int64_t* unique, int64_t* uniqueIds,
                                                 int64_t* uniqueInverse, int64_t* uniqueOffset)
{
    auto* mappers = static_cast<c10::List<c10::intrusive_ptr<hybrid::IdsMapper>>*>(h);
    auto opt = torch::TensorOptions().dtype(torch::kInt64);
    auto tIds = torch::from_blob(const_cast<int64_t*>(ids), {n}, opt);
    auto tOff = torch::from_blob(const_cast<int64_t*>(offsets), {T + 1}, opt);
    auto tHash = torch::from_blob(hashIndices, {n}, opt);
    auto tUniq = torch::from_blob(unique, {n}, opt);
    auto tUids = torch::from_blob(uniqueIds, {n}, opt);
    auto tInv = torch::from_blob(uniqueInverse, {n}, opt);
    auto tUoff = torch::from_blob(uniqueOffset, {T + 1}, opt);
    try {
        hybrid::IdsMapper::ParallelUniqueHashOut(*mappers, tIds, tHash, tOff, tUniq, tUids, tInv, tUoff);
    } catch (const std::exception&) {
        return -1;
    }
    return 0;
}

// hybrid::UniqueParallel: sorted distinct ids and the int64 inverse; returns the number of distinct ids
REF_API int64_t ref_unique_parallel(const int64_t* ids, int64_t n, int64_t* sorted, int64_t* inverse)
{
    auto opt = torch::TensorOptions().dtype(torch::kInt64);
    auto tIds = torch::from_blob(const_cast<int64_t*>(ids), {n}, opt);
    auto res = hybrid::UniqueParallel(tIds);
    const at::Tensor& u = std::get<0>(res);
    const at::Tensor& inv = std::get<1>(res);
    std::memcpy(sorted, u.data_ptr<int64_t>(), sizeof(int64_t) * u.numel());
    std::memcpy(inverse, inv.data_ptr<int64_t>(), sizeof(int64_t) * inv.numel());
    return u.numel();
}
