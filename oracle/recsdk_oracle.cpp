// CPU oracle for the sparse-embedding hot path.  TEST INFRASTRUCTURE ONLY.
//
// This file restates, on the CPU and from scratch, the algorithms of the
// reference's host key pipeline and device operators so that the HIP kernels
// can be checked against them.  Nothing in the shipped library links, loads or
// calls it: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
// may use it, and only as the checker or as the timed CPU baseline.
//
// Every function cites the reference file:line it follows (paths relative to
// the reference checkout).  Integer results follow the reference's sequential
// order (first occurrence, LIFO slot reuse); floating-point results are computed
// in fp32 in the reference's operation order with contraction disabled
// (compile with -ffp-contract=off).
//
// Pinning status (what checks the restatement itself, see tests/test_oracle_*.py):
//   orc_hash_split / orc_build_restore_vec : KATs key_process_test.cpp:744-787,855-885 + numpy brute force
//   orc_global_unique                      : numpy brute force (np.unique + first index)
//   orc_read_emb_key / orc_padding_keys_mask : numpy slicing / np.isin (brute force)
//   orc_hot_*                              : numpy/dict model written from the text of HotHashSplit + invariants (no KAT in the reference)
//   orc_static_*                           : KAT key_process_test.cpp:925-954, embedding_static_test.cpp:78-160
//   orc_faae_*                             : KATs feature_admit_and_evict_test.cpp:283-325, :405-421 (explicit timestamps)
//   orc_swap_*                             : the reference-built checker under oracle/_ref when it builds, invariants otherwise
//   orc_filter_*                           : python dict model written from the feature_filter.cpp text + invariants (no KAT in the reference)
//   orc_lookup/update_by_addr              : closed form gen_lookup_data.py:22-38, gen_update_data.py:22-38
//   orc_lazy_adam / orc_sgd                : closed form aclnn_lazy_adam_test gen_data.py:90-127; textbook SGD(+L2)
//   orc_byaddr_* algebra                   : numpy restatement + torch.optim cross-check
//   orc_tbe_forward                        : torch.nn.EmbeddingBag(sum/mean) (third-party)
//   orc_tbe_backward                       : torch.optim.{SGD,Adagrad,SparseAdam} on loss = sum(out*g)
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <queue>
#include <unordered_map>
#include <utility>
#include <random>
#include <vector>

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

// Open-addressing int64 -> V map (linear probing, tombstones).  Same class of data
// structure as the reference's absl::flat_hash_map; iteration order is never relied on.
template <typename V>
class FlatMap {
public:
    explicit FlatMap(size_t expected = 16) { Rehash(Pow2(expected * 2 + 16)); }

    V* Find(int64_t key)
    {
        size_t pos = Hash(key) & mask_;
        while (state_[pos] != kEmpty) {
            if (state_[pos] == kFull && keys_[pos] == key) {
                return &vals_[pos];
            }
            pos = (pos + 1) & mask_;
        }
        return nullptr;
    }

    // returns {pointer, inserted}
    std::pair<V*, bool> TryEmplace(int64_t key, const V& v)
    {
        if ((used_ + 1) * 10 > (mask_ + 1) * 7) {
            Rehash((size_ * 10 > (mask_ + 1) * 3) ? (mask_ + 1) * 2 : (mask_ + 1));
        }
        size_t pos = Hash(key) & mask_;
        size_t firstTomb = SIZE_MAX;
        while (state_[pos] != kEmpty) {
            if (state_[pos] == kFull && keys_[pos] == key) {
                return {&vals_[pos], false};
            }
            if (state_[pos] == kTomb && firstTomb == SIZE_MAX) {
                firstTomb = pos;
            }
            pos = (pos + 1) & mask_;
        }
        if (firstTomb != SIZE_MAX) {
            pos = firstTomb;
        } else {
            used_++;
        }
        state_[pos] = kFull;
        keys_[pos] = key;
        vals_[pos] = v;
        size_++;
        return {&vals_[pos], true};
    }

    bool Erase(int64_t key)
    {
        size_t pos = Hash(key) & mask_;
        while (state_[pos] != kEmpty) {
            if (state_[pos] == kFull && keys_[pos] == key) {
                state_[pos] = kTomb;
                size_--;
                return true;
            }
            pos = (pos + 1) & mask_;
        }
        return false;
    }

    size_t Size() const { return size_; }

    template <typename F>
    void ForEach(F&& f) const
    {
        for (size_t i = 0; i <= mask_; ++i) {
            if (state_[i] == kFull) {
                f(keys_[i], vals_[i]);
            }
        }
    }

    void Clear()
    {
        std::fill(state_.begin(), state_.end(), kEmpty);
        size_ = 0;
        used_ = 0;
    }

private:
    static constexpr uint8_t kEmpty = 0, kFull = 1, kTomb = 2;

    static size_t Pow2(size_t n)
    {
        size_t p = 16;
        while (p < n) {
            p <<= 1;
        }
        return p;
    }

    static size_t Hash(int64_t key)
    {
        uint64_t x = static_cast<uint64_t>(key);
        x ^= x >> 33;
        x *= 0xff51afd7ed558ccdULL;
        x ^= x >> 33;
        return static_cast<size_t>(x);
    }

    void Rehash(size_t newCap)
    {
        std::vector<uint8_t> os;
        std::vector<int64_t> ok;
        std::vector<V> ov;
        os.swap(state_);
        ok.swap(keys_);
        ov.swap(vals_);
        state_.assign(newCap, kEmpty);
        keys_.assign(newCap, 0);
        vals_.assign(newCap, V());
        mask_ = newCap - 1;
        size_ = 0;
        used_ = 0;
        for (size_t i = 0; i < os.size(); ++i) {
            if (os[i] == kFull) {
                size_t pos = Hash(ok[i]) & mask_;
                while (state_[pos] != kEmpty) {
                    pos = (pos + 1) & mask_;
                }
                state_[pos] = kFull;
                keys_[pos] = ok[i];
                vals_[pos] = ov[i];
                size_++;
                used_++;
            }
        }
    }

    std::vector<uint8_t> state_;
    std::vector<int64_t> keys_;
    std::vector<V> vals_;
    size_t mask_ = 0;
    size_t size_ = 0;
    size_t used_ = 0;  // full + tombstones
};

inline int64_t AbsMod(int64_t key, int64_t m)
{
    int64_t r = key % m;
    return r < 0 ? -r : r;
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// A1  KeyProcess::HashSplit / HashSplitWithFAAE
//     training/tf_rec_v1/src/core/key_process/key_process.cpp:1134-1156, 1170-1216
// Dedup in first-occurrence order, bucket by abs(key % rankSize); restore[i] = index of
// key[i] inside its bucket; counts[j] = multiplicity of the j-th emitted key.
// Output: splitKeys = buckets concatenated in rank order, splitOffsets[rankSize+1].
// Returns the number of distinct keys.
ORC_API int64_t orc_hash_split(const int64_t* keys, int64_t n, int32_t rankSize, int64_t* splitKeys,
                               int64_t* splitOffsets, int32_t* restore, uint32_t* counts)
{
    struct Rec {
        int32_t pos;   // index inside its bucket
        int32_t dev;   // bucket
        uint32_t cnt;  // multiplicity
    };
    FlatMap<Rec> seen(static_cast<size_t>(n));
    std::vector<std::vector<int64_t>> buckets(rankSize);
    for (int64_t i = 0; i < n; ++i) {
        int64_t key = keys[i];
        Rec* r = seen.Find(key);
        if (r == nullptr) {
            int32_t dev = static_cast<int32_t>(AbsMod(key, rankSize));
            Rec rec{static_cast<int32_t>(buckets[dev].size()), dev, 1};
            buckets[dev].push_back(key);
            seen.TryEmplace(key, rec);
            restore[i] = rec.pos;
        } else {
            restore[i] = r->pos;
            r->cnt++;
        }
    }
    int64_t total = 0;
    for (int32_t d = 0; d < rankSize; ++d) {
        splitOffsets[d] = total;
        for (int64_t key : buckets[d]) {
            splitKeys[total] = key;
            if (counts != nullptr) {
                counts[total] = seen.Find(key)->cnt;
            }
            total++;
        }
    }
    splitOffsets[rankSize] = total;
    return total;
}

// KeyProcess::BuildRestoreVec, key_process.cpp:1416-1431: restore entries that are not hot
// (>= hotPosSize) are shifted by the start offset of their bucket in the received block.
ORC_API void orc_build_restore_vec(const int64_t* keys, int64_t n, int32_t rankSize, const int32_t* blockOffset,
                                   int32_t* restore, int32_t hotPosSize)
{
    for (int64_t i = 0; i < n; ++i) {
        int64_t dev = AbsMod(keys[i], rankSize);
        if (restore[i] >= hotPosSize) {
            restore[i] += blockOffset[dev];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Batch ingestion  ReadEmbKeyV2::EnqueueBatchData + ParseTimestampAndCheck, hybrid_dataset_ops.cpp:467-531.
// data: the batch tensor (dataSize elements, int32 when isInt32 else int64).  Returns the number of keys written to
// sample (the per-table batches back to back, bounds in offsets[used+1]); -1 "Timestamp field not found",
// -2 "Timestamp should greater than 0".
ORC_API int64_t orc_read_emb_key(const void* data, int32_t isInt32, int64_t dataSize, const int64_t* splits,
                                 const uint8_t* tableUsed, int32_t nTables, int32_t isTimestamp, int64_t fieldNum,
                                 int64_t* sample, int64_t* offsets, int64_t* timestamp)
{
    *timestamp = -1;
    if (isTimestamp) {
        if (dataSize - fieldNum != 1) {
            return -1;
        }
        std::memcpy(timestamp, data, sizeof(int64_t));  // time_t: the first 8 bytes
        if (*timestamp <= 0) {
            return -2;
        }
    }
    size_t offset = isTimestamp ? 1 : 0;
    int64_t total = 0;
    int32_t used = 0;
    offsets[0] = 0;
    for (int32_t i = 0; i < nTables; ++i) {
        const size_t len = static_cast<size_t>(splits[i]);
        if (tableUsed != nullptr && !tableUsed[i]) {
            offset += len;
            continue;
        }
        if (isInt32) {
            const int32_t* src = static_cast<const int32_t*>(data);
            std::copy(src + offset, src + offset + len, sample + total);
        } else {
            const int64_t* src = static_cast<const int64_t*>(data);
            std::copy(src + offset, src + offset + len, sample + total);
        }
        offset += len;
        total += static_cast<int64_t>(len);
        offsets[++used] = total;
    }
    return total;
}

// KeyProcess::PushPaddingKeysTensors, key_process.cpp:1808-1827: mask 1, 0 where the value is in the padding set.
ORC_API void orc_padding_keys_mask(const int64_t* values, int64_t n, const int64_t* padding, int32_t nPadding,
                                   int32_t* mask)
{
    std::unordered_map<int64_t, int> pad;
    for (int32_t j = 0; j < nPadding; ++j) {
        pad[padding[j]] = 1;
    }
    for (int64_t i = 0; i < n; ++i) {
        mask[i] = pad.find(values[i]) != pad.end() ? 0 : 1;
    }
}

// ---------------------------------------------------------------------------------------------
// A1 (hot keys)  KeyProcess::HotHashSplit, key_process.cpp:1218-1293, for rankSize 1 (every key goes to bucket 0,
// AddCountStartToHotPos adds bucket start 0), with KeyProcess::UpdateHotMap, key_process.cpp:1335-1356.
// One object per embedding table: hotKey[name] (key -> -1) and hotEmbTotCount[name].
struct OrcHot {
    std::unordered_map<int64_t, int> hotMap;
    int32_t hotTot = 0;
};

ORC_API void* orc_hot_create(int32_t hotEmbTotCount)
{
    auto* h = new OrcHot();
    h->hotTot = hotEmbTotCount;
    return h;
}

ORC_API void orc_hot_destroy(void* p) { delete static_cast<OrcHot*>(p); }

// restore[n], hotPos[hotEmbTotCount], splitKeys[n], keyCount[n]; returns the number of distinct keys.
ORC_API int64_t orc_hot_hash_split(void* p, const int64_t* batchData, int64_t miniBs, int32_t refresh,
                                   int64_t* splitKeys, int32_t* restore, int32_t* hotPos, uint32_t* keyCount)
{
    auto* h = static_cast<OrcHot*>(p);
    std::unordered_map<int64_t, std::pair<int32_t, uint32_t>> uKey;
    std::unordered_map<int64_t, int> keyCountMap;
    std::unordered_map<int64_t, int> hotMap = h->hotMap;  // per-batch copy: marks are not kept
    for (int32_t j = 0; j < h->hotTot; ++j) {
        hotPos[j] = 0;
    }
    int32_t hotCount = 0;
    const int32_t hotOffset = h->hotTot;
    int64_t splitSize = 0;
    for (int64_t i = 0; i < miniBs; ++i) {
        const int64_t key = batchData[i];
        if (refresh) {
            keyCountMap[key]++;
        }
        auto seen = uKey.find(key);
        if (seen != uKey.end()) {
            restore[i] = seen->second.first;
            seen->second.second++;
            continue;
        }
        splitKeys[splitSize++] = key;
        auto hot = hotMap.find(key);
        if (hot != hotMap.end()) {
            if (hot->second == -1) {
                hotPos[hotCount] = static_cast<int32_t>(splitSize) - 1;
                hot->second = hotCount;
                restore[i] = hotCount++;
            } else {
                restore[i] = hot->second;
            }
        } else {
            restore[i] = static_cast<int32_t>(splitSize + (hotOffset - 1));
        }
        uKey[key] = {restore[i], 1u};
    }
    for (int64_t k = 0; k < splitSize; ++k) {
        keyCount[k] = uKey[splitKeys[k]].second;
    }
    if (refresh) {
        // max-heap of (-count, key) cut to hotTot entries: what stays are the largest counts, ties to the smaller key
        std::priority_queue<std::pair<int, int64_t>> pq;
        for (auto& kv : keyCountMap) {
            pq.push({-kv.second, kv.first});
            if (pq.size() > static_cast<size_t>(h->hotTot)) {
                pq.pop();
            }
        }
        h->hotMap.clear();
        while (!pq.empty()) {
            h->hotMap.insert({pq.top().second, -1});
            pq.pop();
        }
    }
    return splitSize;
}

// The current hot set, ascending; returns its size.
ORC_API int64_t orc_hot_keys(void* p, int64_t* out, int64_t cap)
{
    auto* h = static_cast<OrcHot*>(p);
    std::vector<int64_t> k;
    for (auto& kv : h->hotMap) {
        k.push_back(kv.first);
    }
    std::sort(k.begin(), k.end());
    for (size_t j = 0; j < k.size() && static_cast<int64_t>(j) < cap; ++j) {
        out[j] = k[j];
    }
    return static_cast<int64_t>(k.size());
}

// ---------------------------------------------------------------------------------------------
// A2  KeyProcess::GlobalUnique, key_process.h:114-145
// Second dedup over lookup keys/offsets.  With useStatic the padding value (-1, or 0 under dynamic
// expansion) is skipped (restoreVecSec = -1) and uniqueKeys is padded to m with the padding value.
// Returns the number of distinct keys (before padding).
ORC_API int64_t orc_global_unique(const int64_t* lookupKeys, int64_t m, int32_t useStatic, int32_t useDynamicExpansion,
                                  int64_t* uniqueKeys, int32_t* restoreVecSec)
{
    FlatMap<int32_t> umap(static_cast<size_t>(m));
    int32_t length = 0;
    const int64_t pad = useDynamicExpansion ? 0 : -1;
    for (int64_t i = 0; i < m; ++i) {
        restoreVecSec[i] = -1;
        int64_t key = lookupKeys[i];
        if (useStatic && key == pad) {
            continue;
        }
        int32_t* r = umap.Find(key);
        if (r == nullptr) {
            uniqueKeys[length] = key;
            umap.TryEmplace(key, length);
            restoreVecSec[i] = length;
            length++;
        } else {
            restoreVecSec[i] = *r;
        }
    }
    if (useStatic) {
        for (int64_t i = length; i < m; ++i) {
            uniqueKeys[i] = pad;
        }
    }
    return length;
}

// ---------------------------------------------------------------------------------------------
// A4/A5/A8  key -> slot tables
//   EmbeddingStatic::Key2Offset   emb_table/embedding_static.cpp:38-99
//   EmbeddingDynamic::Key2Offset  emb_table/embedding_dynamic.cpp:59-85 (+118-144 address minting)
//   EmbeddingTable::EvictKeys     emb_table/embedding_table.cpp:66-85
struct OrcTable {
    FlatMap<int64_t> keyOffset;
    std::vector<int64_t> evictPos;
    int64_t maxOffset = 0;
    int64_t devVocabSize = 0;
    // dynamic mode: address = arenaBase + seq * rowBytes (the reference mints addresses row by row from
    // 100000-row blocks, embedding_dynamic.h:54; one contiguous arena gives the same sequence shape)
    int32_t dynamic = 0;
    int64_t arenaBase = 0;
    int64_t rowBytes = 0;
    explicit OrcTable(size_t expected) : keyOffset(expected) {}
};

ORC_API void* orc_table_create(int64_t devVocabSize, int32_t dynamic, int64_t arenaBase, int64_t rowBytes)
{
    auto* t = new OrcTable(static_cast<size_t>(std::min<int64_t>(devVocabSize, 1 << 20)));
    t->devVocabSize = devVocabSize;
    t->dynamic = dynamic;
    t->arenaBase = arenaBase;
    t->rowBytes = rowBytes;
    return t;
}

ORC_API void orc_table_destroy(void* h) { delete static_cast<OrcTable*>(h); }

ORC_API int64_t orc_table_size(void* h) { return static_cast<OrcTable*>(h)->maxOffset; }

ORC_API int64_t orc_table_live(void* h) { return static_cast<int64_t>(static_cast<OrcTable*>(h)->keyOffset.Size()); }

ORC_API int64_t orc_table_evict_count(void* h) { return static_cast<int64_t>(static_cast<OrcTable*>(h)->evictPos.size()); }

ORC_API void orc_table_evict_pos(void* h, int64_t* out)
{
    auto* t = static_cast<OrcTable*>(h);
    std::copy(t->evictPos.begin(), t->evictPos.end(), out);
}

// In place: keys[i] -> offset (static) or address (dynamic).  channel 0 = train, 1 = eval.
// Returns 0, or -1 when the static table overflowed (the reference throws after mutating state,
// embedding_static.cpp:90-98).
ORC_API int32_t orc_table_key2offset(void* h, int64_t* keys, int64_t n, int32_t channel)
{
    auto* t = static_cast<OrcTable*>(h);
    if (t->dynamic) {
        for (int64_t i = 0; i < n; ++i) {
            int64_t key = keys[i];
            if (key == -1) {
                keys[i] = 0;
                continue;
            }
            int64_t* found = t->keyOffset.Find(key);
            if (found != nullptr) {
                keys[i] = *found;
                continue;
            }
            if (channel == 0) {
                int64_t addr = t->arenaBase + t->maxOffset * t->rowBytes;
                t->keyOffset.TryEmplace(key, addr);
                keys[i] = addr;
                t->maxOffset++;
                continue;
            }
            keys[i] = 0;
        }
        return (t->maxOffset > t->devVocabSize) ? -1 : 0;
    }
    // static: FindKeyOffset pass then EmplaceKeyOffset pass over the indices that missed
    std::vector<int64_t> newIdx;
    for (int64_t i = 0; i < n; ++i) {
        int64_t key = keys[i];
        if (key == -1) {
            continue;
        }
        int64_t* found = t->keyOffset.Find(key);
        if (found != nullptr) {
            keys[i] = *found;
            continue;
        }
        newIdx.push_back(i);
    }
    for (int64_t i : newIdx) {
        int64_t key = keys[i];
        if (!t->evictPos.empty() && channel == 0) {
            int64_t offset = t->evictPos.back();
            auto ret = t->keyOffset.TryEmplace(key, offset);
            if (ret.second) {
                t->evictPos.pop_back();
            }
            keys[i] = *ret.first;
            continue;
        } else if (channel != 0) {
            keys[i] = -1;
            continue;
        }
        auto ret = t->keyOffset.TryEmplace(key, t->maxOffset);
        if (ret.second) {
            t->maxOffset++;
        }
        keys[i] = *ret.first;
    }
    return (t->maxOffset > t->devVocabSize) ? -1 : 0;
}

// EvictKeys: erase key -> slot, append slot to evictPos in call order.  Returns #erased.
ORC_API int64_t orc_table_evict(void* h, const int64_t* keys, int64_t n)
{
    auto* t = static_cast<OrcTable*>(h);
    int64_t erased = 0;
    for (int64_t i = 0; i < n; ++i) {
        int64_t key = keys[i];
        if (key == -1) {
            continue;
        }
        int64_t* found = t->keyOffset.Find(key);
        if (found == nullptr) {
            continue;
        }
        int64_t slot = *found;
        t->keyOffset.Erase(key);
        t->evictPos.push_back(slot);
        erased++;
    }
    return erased;
}

// ---------------------------------------------------------------------------------------------
// A6/A7  FeatureAdmitAndEvict  key_process/feature_admit_and_evict.cpp:46-145 (admit), 148-200 (evict)
struct OrcFaaeRec {
    uint32_t count = 0;
    int64_t lastTime = 0;
};

struct OrcFaae {
    FlatMap<OrcFaaeRec> history;
    int64_t timestamp = 0;
    int32_t countThreshold = -1;
    int32_t timeThreshold = -1;
    int32_t coef = 1;
    int32_t isEnableSum = 1;
    OrcFaae() : history(1024) {}
};

ORC_API void* orc_faae_create(int32_t countThreshold, int32_t timeThreshold, int32_t coef, int32_t isEnableSum)
{
    auto* f = new OrcFaae();
    f->countThreshold = countThreshold;
    f->timeThreshold = timeThreshold;
    f->coef = coef;
    f->isEnableSum = isEnableSum;
    return f;
}

ORC_API void orc_faae_destroy(void* h) { delete static_cast<OrcFaae*>(h); }

ORC_API int64_t orc_faae_size(void* h) { return static_cast<int64_t>(static_cast<OrcFaae*>(h)->history.Size()); }

// Dump history sorted by key: keys[], counts[], lastTimes[]; returns size.
ORC_API int64_t orc_faae_dump(void* h, int64_t* keys, uint32_t* counts, int64_t* lastTimes)
{
    auto* f = static_cast<OrcFaae*>(h);
    std::vector<std::pair<int64_t, OrcFaaeRec>> all;
    f->history.ForEach([&](int64_t k, const OrcFaaeRec& r) { all.emplace_back(k, r); });
    std::sort(all.begin(), all.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    for (size_t i = 0; i < all.size(); ++i) {
        keys[i] = all[i].first;
        counts[i] = all[i].second.count;
        lastTimes[i] = all[i].second.lastTime;
    }
    return static_cast<int64_t>(all.size());
}

// FeatureAdmit (feature_admit_and_evict.cpp:46-104) + FeatureAdmitHelper (:106-145).
// keys may repeat; counts[i] is the multiplicity carried by occurrence i (PreProcessKeys :218-233 merges them).
// In place: every occurrence of a key that fails admission becomes -1.
ORC_API int32_t orc_faae_admit(void* h, int32_t channel, int64_t* keys, const uint32_t* counts, int64_t n,
                               int64_t batchTimestamp)
{
    auto* f = static_cast<OrcFaae*>(h);
    FlatMap<uint32_t> merge(static_cast<size_t>(n));
    for (int64_t i = 0; i < n; ++i) {
        if (keys[i] == -1) {
            continue;
        }
        auto ret = merge.TryEmplace(keys[i], counts[i]);
        if (!ret.second) {
            *ret.first += counts[i];
        }
    }
    if (batchTimestamp > f->timestamp) {
        f->timestamp = batchTimestamp;
    }
    FlatMap<uint8_t> visited(static_cast<size_t>(n));
    for (int64_t i = 0; i < n; ++i) {
        int64_t key = keys[i];
        if (key == -1) {
            continue;
        }
        uint8_t* seen = visited.Find(key);
        if (seen != nullptr) {
            if (!*seen) {
                keys[i] = -1;
            }
            continue;
        }
        uint32_t featureCnt = *merge.Find(key);
        uint32_t curr = 0;
        OrcFaaeRec* rec = f->history.Find(key);
        if (channel == 1 || !f->isEnableSum) {
            if (rec != nullptr) {
                curr = rec->count;
            }
        } else if (channel == 0) {
            if (rec == nullptr) {
                OrcFaaeRec info;
                info.count = featureCnt;
                info.lastTime = f->timestamp;
                info.count *= static_cast<uint32_t>(f->coef);
                f->history.TryEmplace(key, info);
                curr = info.count;
            } else {
                rec->count += static_cast<uint32_t>(f->coef) * featureCnt;
                rec->lastTime = f->timestamp;
                curr = rec->count;
            }
        }
        bool ok = curr >= static_cast<uint32_t>(f->countThreshold);
        visited.TryEmplace(key, ok ? 1 : 0);
        if (!ok) {
            keys[i] = -1;
        }
    }
    return 0;
}

// FeatureEvictHelper (:163-200): evict every record with currTime - lastTime >= timeThreshold and erase it.
// The reference pops a priority queue ordered by lastTime (ties in hash-map order, unspecified); the set is
// what is specified.  Emitted here in ascending (lastTime, key) order.  Returns the number of evicted keys.
ORC_API int64_t orc_faae_evict(void* h, int64_t* outKeys, int64_t cap)
{
    auto* f = static_cast<OrcFaae*>(h);
    std::vector<std::pair<int64_t, int64_t>> ev;  // (lastTime, key)
    f->history.ForEach([&](int64_t k, const OrcFaaeRec& r) {
        if (f->timestamp - r.lastTime >= f->timeThreshold) {
            ev.emplace_back(r.lastTime, k);
        }
    });
    std::sort(ev.begin(), ev.end());
    int64_t cnt = 0;
    for (auto& e : ev) {
        f->history.Erase(e.second);
        if (cnt < cap) {
            outKeys[cnt] = e.second;
        }
        cnt++;
    }
    return cnt;
}

// ---------------------------------------------------------------------------------------------
// A11  torch FeatureFilter
//      training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/feature_filter/feature_filter.cpp:27-80,112-160
// Separate count and timestamp maps; eviction every evictStepInterval RecordTimestamp calls.
struct OrcFilter {
    FlatMap<uint64_t> counts;
    FlatMap<int64_t> times;
    int64_t admitThreshold = -1;  // -1 = admission off (INVALID_KEY)
    uint64_t evictThreshold = 0;
    uint64_t evictStepInterval = 1;
    int64_t latest = 0;
    uint64_t recordTsBatchId = 0;
    std::vector<int64_t> evicted;  // keys of the last eviction, ascending (timestamp, key)
    OrcFilter() : counts(1024), times(1024) {}
};

ORC_API void* orc_filter_create(int64_t admitThreshold, uint64_t evictThreshold, uint64_t evictStepInterval)
{
    auto* f = new OrcFilter();
    f->admitThreshold = admitThreshold;
    f->evictThreshold = evictThreshold;
    f->evictStepInterval = evictStepInterval;
    return f;
}

ORC_API void orc_filter_destroy(void* h) { delete static_cast<OrcFilter*>(h); }

// StatisticsKeyCount :112-138 (negative counts clamp to 0; counts == NULL means 1 each)
ORC_API void orc_filter_statistics(void* h, const int64_t* keys, const int64_t* counts, int64_t n)
{
    auto* f = static_cast<OrcFilter*>(h);
    for (int64_t i = 0; i < n; ++i) {
        int64_t raw = counts ? counts[i] : 1;
        uint64_t c = raw < 0 ? 0 : static_cast<uint64_t>(raw);
        auto ret = f->counts.TryEmplace(keys[i], c);
        if (!ret.second) {
            *ret.first += c;
        }
    }
}

// CountFilter :140-160
ORC_API void orc_filter_count_filter(void* h, int64_t* keys, int64_t n)
{
    auto* f = static_cast<OrcFilter*>(h);
    if (f->admitThreshold == -1) {
        return;
    }
    for (int64_t i = 0; i < n; ++i) {
        uint64_t* c = f->counts.Find(keys[i]);
        if (c != nullptr && *c < static_cast<uint64_t>(f->admitThreshold)) {
            keys[i] = -1;
        }
    }
}

static void OrcFilterEvict(OrcFilter* f)
{
    f->evicted.clear();
    if (f->evictThreshold == 0) {
        return;
    }
    std::vector<std::pair<int64_t, int64_t>> ev;
    f->times.ForEach([&](int64_t k, const int64_t& ts) {
        if (k == -1) {
            return;
        }
        if (f->latest - ts > static_cast<int64_t>(f->evictThreshold)) {
            ev.emplace_back(ts, k);
        }
    });
    std::sort(ev.begin(), ev.end());
    for (auto& e : ev) {
        f->times.Erase(e.second);
        if (f->admitThreshold != -1) {
            f->counts.Erase(e.second);
        }
        f->evicted.push_back(e.second);
    }
}

// RecordTimestamp :27-50; returns 1 when this call ran an eviction
ORC_API int32_t orc_filter_record_timestamp(void* h, const int64_t* keys, const int64_t* timestamps, int64_t n)
{
    auto* f = static_cast<OrcFilter*>(h);
    for (int64_t i = 0; i < n; ++i) {
        auto ret = f->times.TryEmplace(keys[i], timestamps[i]);
        if (!ret.second) {
            *ret.first = timestamps[i];
        }
        f->latest = std::max(f->latest, timestamps[i]);
    }
    int32_t ran = 0;
    if (f->recordTsBatchId > 0 && (f->recordTsBatchId + 1) % f->evictStepInterval == 0) {
        OrcFilterEvict(f);
        ran = 1;
    }
    f->recordTsBatchId++;
    return ran;
}

ORC_API int64_t orc_filter_evicted(void* h, int64_t* out, int64_t cap)
{
    auto* f = static_cast<OrcFilter*>(h);
    int64_t n = static_cast<int64_t>(f->evicted.size());
    for (int64_t i = 0; i < n && i < cap; ++i) {
        out[i] = f->evicted[i];
    }
    return n;
}

// ---------------------------------------------------------------------------------------------
// A10  torch SwapManager
//      training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/embedding_cache/swap_manager.cpp:32-159
struct OrcSwap {
    int64_t memStart = 0;
    int64_t cacheSize = 0;
    int64_t occupied = 0;
    int64_t now = 0;
    int64_t swapIdx = 0;
    FlatMap<int64_t> key2off;
    std::vector<int64_t> key;
    std::vector<int64_t> version;
    std::vector<int64_t> out[4];  // swapoutKeys, swapoutOffs, swapinKeys, swapinOffs of the last call
    explicit OrcSwap(int64_t n) : key2off(static_cast<size_t>(std::min<int64_t>(n, 1 << 20))) {}
};

ORC_API void* orc_swap_create(int64_t cacheSize, int64_t memStartOffset)
{
    auto* s = new OrcSwap(cacheSize);
    s->cacheSize = cacheSize;
    s->memStart = memStartOffset;
    s->occupied = memStartOffset;
    s->swapIdx = memStartOffset;
    s->key.assign(cacheSize, 0);
    s->version.assign(cacheSize, 0);
    return s;
}

ORC_API void orc_swap_destroy(void* h) { delete static_cast<OrcSwap*>(h); }

// Returns 0, or -1 for "cacheSize_ too small" (the reference throws there).
ORC_API int32_t orc_swap_compute(void* h, const int64_t* keys, int64_t n, int64_t* batchOffs)
{
    auto* s = static_cast<OrcSwap*>(h);
    for (auto& v : s->out) {
        v.clear();
    }
    std::vector<int64_t> missed;
    for (int64_t i = 0; i < n; ++i) {
        int64_t key = keys[i];
        if (key == -1) {
            batchOffs[i] = 0;
            continue;
        }
        int64_t* off = s->key2off.Find(key);
        if (off != nullptr) {
            batchOffs[i] = *off;
            s->version[*off] = s->now;
        } else {
            missed.push_back(i);
        }
    }
    for (int64_t i : missed) {
        int64_t key = keys[i];
        int64_t* known = s->key2off.Find(key);
        if (known != nullptr) {
            batchOffs[i] = *known;
            continue;
        }
        int64_t off;
        if (s->occupied < s->cacheSize) {
            off = s->occupied++;
            s->out[2].push_back(key);
            s->out[3].push_back(off);
            s->key[off] = key;
            s->version[off] = s->now;
            s->key2off.TryEmplace(key, off);
            batchOffs[i] = off;
            continue;
        }
        while (s->swapIdx < s->cacheSize && s->version[s->swapIdx] >= s->now - 1) {
            s->swapIdx++;
        }
        if (s->swapIdx == s->cacheSize) {
            s->swapIdx = s->memStart;
            while (s->swapIdx < s->cacheSize && s->version[s->swapIdx] >= s->now - 1) {
                s->swapIdx++;
            }
            if (s->swapIdx == s->cacheSize) {
                return -1;
            }
        }
        bool evictedPos = s->version[s->swapIdx] == -2;
        off = s->swapIdx++;
        s->out[2].push_back(key);
        s->out[3].push_back(off);
        int64_t oldKey = s->key[off];
        if (oldKey != -1) {
            s->key2off.Erase(oldKey);
        }
        if (!evictedPos) {
            s->out[0].push_back(oldKey);
            s->out[1].push_back(off);
        }
        s->key[off] = key;
        s->version[off] = s->now;
        s->key2off.TryEmplace(key, off);
        batchOffs[i] = off;
    }
    s->now++;
    return 0;
}

ORC_API int64_t orc_swap_result(void* h, int32_t which, int64_t* out, int64_t cap)
{
    auto* s = static_cast<OrcSwap*>(h);
    const auto& v = s->out[which];
    for (size_t i = 0; i < v.size() && static_cast<int64_t>(i) < cap; ++i) {
        out[i] = v[i];
    }
    return static_cast<int64_t>(v.size());
}

ORC_API void orc_swap_remove(void* h, const int64_t* keys, int64_t n)
{
    auto* s = static_cast<OrcSwap*>(h);
    for (int64_t i = 0; i < n; ++i) {
        int64_t* off = s->key2off.Find(keys[i]);
        if (off == nullptr) {
            continue;
        }
        s->version[*off] = -2;
        s->key[*off] = -1;
        s->key2off.Erase(keys[i]);
    }
}

// ---------------------------------------------------------------------------------------------
// A13  embedding_lookup_by_address
//      cust_op/ascendc_op/ai_core_op/cust_op_by_addr/v220/op_kernel/embedding_lookup_by_address.cpp:117-132
// y[i,:] = *(T*)address[i]; address 0 -> zero row.  elemBytes = sizeof(T).
ORC_API void orc_lookup_by_addr(const int64_t* address, int64_t n, int32_t dim, int32_t elemBytes, void* y)
{
    size_t rowBytes = static_cast<size_t>(dim) * elemBytes;
    char* out = static_cast<char*>(y);
    for (int64_t i = 0; i < n; ++i) {
        if (address[i] != 0) {
            std::memcpy(out + i * rowBytes, reinterpret_cast<const void*>(address[i]), rowBytes);
        } else {
            std::memset(out + i * rowBytes, 0, rowBytes);
        }
    }
}

// A14  embedding_update_by_address  .../op_kernel/embedding_update_by_address.cpp:107-144,158-188
// updateType 0: *(float*)address[i] += emb[i,:] (duplicates accumulate, applied in index order here);
// updateType 1: overwrite.  address 0 skipped.  fp32 only in the oracle.
ORC_API void orc_update_by_addr_f32(const int64_t* address, int64_t n, int32_t dim, const float* emb, int32_t updateType)
{
    for (int64_t i = 0; i < n; ++i) {
        if (address[i] == 0) {
            continue;
        }
        float* dst = reinterpret_cast<float*>(address[i]);
        const float* src = emb + i * dim;
        if (updateType == 0) {
            for (int32_t d = 0; d < dim; ++d) {
                dst[d] += src[d];
            }
        } else {
            for (int32_t d = 0; d < dim; ++d) {
                dst[d] = src[d];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// A16  lazy_adam   cust_op/ascendc_op/ai_core_op/fused_lazy_adam/v220/op_kernel/lazy_adam.cpp:138-205
// rows with index >= 0: m = b1*m + (1-b1)*g; v = b2*v + (1-b2)*g*g; var += (-lr*m) / (sqrt(|v|) + eps).
// (golden generator: cust_op/test/aclnn_lazy_adam_test/tf/scripts/gen_data.py:90-127)
ORC_API void orc_lazy_adam(const float* grad, const int32_t* indices, int64_t n, int32_t dim, float* m, float* v,
                           float* var, float lr, float beta1, float beta2, float eps)
{
    const float omb1 = 1.0f - beta1;
    const float omb2 = 1.0f - beta2;
    for (int64_t i = 0; i < n; ++i) {
        int64_t idx = indices[i];
        if (idx < 0) {
            continue;
        }
        const float* g = grad + i * dim;
        float* mr = m + idx * dim;
        float* vr = v + idx * dim;
        float* wr = var + idx * dim;
        for (int32_t d = 0; d < dim; ++d) {
            float mn = mr[d] * beta1 + g[d] * omb1;
            float vn = vr[d] * beta2 + (g[d] * g[d]) * omb2;
            float den = std::sqrt(std::fabs(vn)) + eps;
            float upd = (mn * -lr) / den;
            mr[d] = mn;
            vr[d] = vn;
            wr[d] = upd + wr[d];
        }
    }
}

// A17  sgd   cust_op/ascendc_op/ai_core_op/fused_sgd/v220/op_kernel/sgd_kernel.h:83-95,169-184
// var[idx] += -lr * (g + wd * var[idx]); duplicates accumulate; applied in index order, each
// occurrence reading the row as it was at the start of the call is NOT what the kernel does:
// the device op reads var when it computes the term, so with duplicate indices the result is
// order dependent.  The oracle applies occurrences in index order against the current row.
ORC_API void orc_sgd(const float* grad, const int32_t* indices, int64_t n, int32_t dim, float* var, float lr,
                     float weightDecay)
{
    for (int64_t i = 0; i < n; ++i) {
        int64_t idx = indices[i];
        if (idx < 0) {
            continue;
        }
        const float* g = grad + i * dim;
        float* wr = var + idx * dim;
        for (int32_t d = 0; d < dim; ++d) {
            float t = g[d];
            if (weightDecay != 0.0f) {
                t = t + weightDecay * wr[d];
            }
            wr[d] = wr[d] + (-lr) * t;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Segment sum of per-lookup gradients (TF unsorted_segment_sum as used by optimizers/base.py:87-115 and
// core/emb/base_sparse_embedding.py:546-573).  seg[i] < 0 is skipped.  The reference fixes no order of the additions
// (unsorted_segment_sum and the Ascend kernels add atomically); this restatement fixes one, and the device code
// follows it bit for bit:
//   a segment with at most kTwoLevelMin members: its rows are added in ascending lookup order, starting from 0;
//   a longer segment: its members, in ascending lookup order, are cut into chunks of kChunkRows; each chunk is summed
//   in order starting from 0, then the chunk sums are added in chunk order starting from 0.
// (One chain of a hundred thousand dependent additions is what a single hot key would otherwise cost.)
namespace {
constexpr int64_t kTwoLevelMin = 1024;
constexpr int64_t kChunkRows = 256;

// Accumulator of one segment that follows the order above; count = members of the segment (known beforehand).
struct OrderedSum {
    bool twoLevel = false;
    int64_t inChunk = 0;
    std::vector<float> chunk;  // two-level only: the running chunk sum

    void Begin(int64_t count, int64_t dim)
    {
        twoLevel = count > kTwoLevelMin;
        inChunk = 0;
        if (twoLevel) {
            chunk.assign(static_cast<size_t>(dim), 0.0f);
        }
    }
    // total[0:dim] is the segment's result, zero-initialised by the caller
    void Add(float* total, const float* row, int64_t dim, float scale, bool scaled)
    {
        float* dst = twoLevel ? chunk.data() : total;
        for (int64_t d = 0; d < dim; ++d) {
            float x = row[d];
            if (scaled) {
                x = x * scale;
            }
            dst[d] += x;
        }
        if (twoLevel && ++inChunk == kChunkRows) {
            Flush(total, dim);
        }
    }
    void Flush(float* total, int64_t dim)
    {
        if (twoLevel && inChunk > 0) {
            for (int64_t d = 0; d < dim; ++d) {
                total[d] += chunk[d];
                chunk[d] = 0.0f;
            }
            inChunk = 0;
        }
    }
};
}  // namespace

ORC_API void orc_segment_sum(const float* grad, const int32_t* seg, int64_t n, int32_t dim, int64_t numSeg, float* out)
{
    std::memset(out, 0, sizeof(float) * numSeg * dim);
    std::vector<int64_t> count(static_cast<size_t>(numSeg), 0);
    for (int64_t i = 0; i < n; ++i) {
        if (seg[i] >= 0) {
            count[seg[i]]++;
        }
    }
    // the long segments (few) carry a chunk accumulator each
    std::vector<int32_t> accOf(static_cast<size_t>(numSeg), -1);
    std::vector<OrderedSum> accs;
    for (int64_t s = 0; s < numSeg; ++s) {
        if (count[s] > kTwoLevelMin) {
            accOf[s] = static_cast<int32_t>(accs.size());
            accs.emplace_back();
            accs.back().Begin(count[s], dim);
        }
    }
    for (int64_t i = 0; i < n; ++i) {
        int64_t s = seg[i];
        if (s < 0) {
            continue;
        }
        const float* g = grad + i * dim;
        float* o = out + s * dim;
        if (accOf[s] >= 0) {
            accs[accOf[s]].Add(o, g, dim, 1.0f, false);
        } else {
            for (int32_t d = 0; d < dim; ++d) {
                o[d] += g[d];
            }
        }
    }
    for (int64_t s = 0; s < numSeg; ++s) {
        if (accOf[s] >= 0) {
            accs[accOf[s]].Flush(out + s * dim, dim);
        }
    }
}

// A15  by-address optimizer algebra on rows [w | s1 | s2] addressed by rowPtr(u) = base + slot[u]*stride.
//   Adam    training/tf_rec_v1/python/optimizers/lazy_adam_by_addr.py:126-157
//           lr_t = lr*sqrt(1-b2^t)/(1-b1^t) is computed by the caller and passed as lrT.
//   Adagrad training/tf_rec_v1/python/optimizers/adagrad_by_addr.py:101-125   (eps 1e-7 inside the sqrt)
//   SGD     training/tf_rec_v1/python/optimizers/gradient_descent_by_addr.py:86-109
// The reference writes deltas with an atomic add (update_by_address, update_type 0); with deltaForm != 0 adding
// the delta to the old value is restated literally: new = old + (x' - old).  deltaForm == 0 stores x' itself,
// which is what a fused row update (lazy_adam.cpp:189-201) does; the two differ by at most one rounding of the state.
// optim: 0 sgd, 1 adagrad, 2 adam.  slot < 0 rows are skipped.  w, s1, s2 are separate base pointers so that
// both the extended-row layout (s1 = w + dim, stride 3*dim) and split tables (stride dim) are covered.
ORC_API void orc_byaddr_apply(int32_t optim, const float* g, const int64_t* slots, int64_t u, int32_t dim, float* w,
                              float* s1, float* s2, int64_t stride, float lrT, float beta1, float beta2, float eps,
                              float weightDecay, int32_t deltaForm)
{
    const float omb1 = 1.0f - beta1;
    const float omb2 = 1.0f - beta2;
    for (int64_t r = 0; r < u; ++r) {
        int64_t slot = slots[r];
        if (slot < 0) {
            continue;
        }
        const float* gr = g + r * dim;
        float* wr = w + slot * stride;
        if (optim == 2) {
            float* mr = s1 + slot * stride;
            float* vr = s2 + slot * stride;
            for (int32_t d = 0; d < dim; ++d) {
                float mt = beta1 * mr[d] + omb1 * gr[d];
                float vt = beta2 * vr[d] + omb2 * (gr[d] * gr[d]);
                float den = std::sqrt(std::fabs(vt)) + eps;
                float nd = (-lrT * mt) / den;
                wr[d] = wr[d] + nd;
                mr[d] = deltaForm ? mr[d] + (mt - mr[d]) : mt;
                vr[d] = deltaForm ? vr[d] + (vt - vr[d]) : vt;
            }
        } else if (optim == 1) {
            float* sr = s1 + slot * stride;
            for (int32_t d = 0; d < dim; ++d) {
                float st = sr[d] + gr[d] * gr[d];
                float den = std::sqrt(st + eps);
                float nd = (-lrT * gr[d]) / den;
                wr[d] = wr[d] + nd;
                sr[d] = deltaForm ? sr[d] + (st - sr[d]) : st;
            }
        } else {
            for (int32_t d = 0; d < dim; ++d) {
                float t = gr[d];
                if (weightDecay != 0.0f) {
                    t = t + weightDecay * wr[d];
                }
                wr[d] = wr[d] + (-(t * lrT));
            }
        }
    }
}

// Row gather by slot: out[i,:] = w[slot[i]*stride : +dim]; slot < 0 -> zeros (tf.gather on the static path,
// core/emb/sparse_embedding.py:49-50; zero rows for inadmissible keys follow the by-address op's address-0 rule).
ORC_API void orc_gather_rows(const float* w, int64_t stride, const int64_t* slots, int64_t n, int32_t dim, float* out)
{
    for (int64_t i = 0; i < n; ++i) {
        if (slots[i] < 0) {
            std::memset(out + i * dim, 0, sizeof(float) * dim);
        } else {
            std::memcpy(out + i * dim, w + slots[i] * stride, sizeof(float) * dim);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// A18  split_embedding_codegen_forward_unweighted
//      cust_op/ascendc_op/ai_core_op/split_embedding_codegen_forward_unweighted/v220/README.md:81-127
// poolingMode 0 sum, 1 mean, 2 none.  offsets are feature-major: bag (t,b) at t*B+b.
// Mean multiplies each row by the float reciprocal of the bag length (op_kernel ..._kernel.h:246).
// weights are fp32 (wBf16 = 0) or bf16 (wBf16 = 1, widened to fp32 before accumulation).
static inline float Bf16ToF32(uint16_t b)
{
    uint32_t u = static_cast<uint32_t>(b) << 16;
    float f;
    std::memcpy(&f, &u, sizeof(f));
    return f;
}

static inline uint16_t F32ToBf16(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, sizeof(u));
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x40);
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return static_cast<uint16_t>(u >> 16);
}

ORC_API void orc_tbe_forward(const void* devWeights, int32_t wBf16, const int64_t* weightsOffsets,
                             const int32_t* dOffsets, int64_t totalD, const int64_t* indices, const int64_t* offsets,
                             int32_t T, int64_t B, int32_t poolingMode, float* out)
{
    const float* wf = static_cast<const float*>(devWeights);
    const uint16_t* wb = static_cast<const uint16_t*>(devWeights);
    if (poolingMode == 2) {
        int64_t D = totalD / T;
        int64_t row = 0;
        for (int64_t bag = 0; bag < T * B; ++bag) {
            int64_t t = bag / B;
            for (int64_t k = offsets[bag]; k < offsets[bag + 1]; ++k) {
                int64_t base = weightsOffsets[t] + indices[k] * D;
                for (int64_t d = 0; d < D; ++d) {
                    out[row * D + d] = wBf16 ? Bf16ToF32(wb[base + d]) : wf[base + d];
                }
                row++;
            }
        }
        return;
    }
    std::memset(out, 0, sizeof(float) * B * totalD);
    for (int32_t t = 0; t < T; ++t) {
        int64_t D = dOffsets[t + 1] - dOffsets[t];
        for (int64_t b = 0; b < B; ++b) {
            int64_t s = offsets[t * B + b];
            int64_t e = offsets[t * B + b + 1];
            float scale = 1.0f;
            if (poolingMode == 1 && e > s) {
                scale = 1.0f / static_cast<float>(e - s);
            }
            float* o = out + b * totalD + dOffsets[t];
            for (int64_t k = s; k < e; ++k) {
                int64_t base = weightsOffsets[t] + indices[k] * D;
                for (int64_t d = 0; d < D; ++d) {
                    float x = wBf16 ? Bf16ToF32(wb[base + d]) : wf[base + d];
                    if (poolingMode == 1) {
                        x = x * scale;
                    }
                    o[d] += x;
                }
            }
        }
    }
}

// A19  backward_codegen_{adagrad,adam,sgd}_unweighted_exact
//      cust_op/ascendc_op/ai_core_op/backward_codegen_adagrad_unweighted_exact/v220/README.md:101-160,233-303,358-416
//      arithmetic as the kernels do it: ..._adam_unweighted_exact_kernel.h:128-166 with
//      stepSize = -lr*sqrt(1-b2^iter)/(1-b1^iter) (op_host/...cpp:98-108, eps not rescaled);
//      ..._adagrad_unweighted_exact_kernel.h:108-139: m1 += G*G; w += -lr*G/(sqrt(m1)+eps); sgd: w += -lr*G.
// Position k of `indices` belongs to bag (t, b), t = feature.  Its gradient row is grad_out[b, D-slice of t] (mean:
// times the float reciprocal of the bag length) or, without pooling (poolingMode 2), grad_out[k, :].  The gradient
// of a table row is the sum of the gradient rows of all positions that name it, whichever feature they belong to:
// features that share a table carry the same hashSizeCumsum entry, and the kernel accumulates at
// hashSizeCumsum[t] + row (op_kernel/backward_codegen_unweighted_exact_kernel.h:314-316,373-378).  The sum is formed
// in ascending position (the order a sequential scatter-add visits them; the reference's atomic adds have no order).
// Then one optimizer step per touched row.  optim: 0 sgd, 1 adagrad, 2 adam.
// weights fp32 or bf16 (bf16: widened, updated in fp32, rounded to nearest even on store); momenta fp32.
namespace {
struct TbeOpt {
    int32_t optim;
    float lr, eps, beta1, beta2, stepSize;
};

TbeOpt MakeTbeOpt(int32_t optim, float lr, float eps, float beta1, float beta2, int64_t iter)
{
    TbeOpt o{optim, lr, eps, beta1, beta2, -lr};
    if (optim == 2) {
        // op_host/backward_codegen_adagrad_unweighted_exact.cpp:98-108: pow in double, narrowed to float
        float b1c = static_cast<float>(1 - std::pow(static_cast<double>(beta1), static_cast<double>(iter)));
        float b2c = static_cast<float>(1 - std::pow(static_cast<double>(beta2), static_cast<double>(iter)));
        float beta2sqrt = std::sqrt(b2c) / b1c;
        o.stepSize = -lr * beta2sqrt;
    }
    return o;
}

void TbeUpdateRow(const TbeOpt& o, const float* g, int64_t base, int64_t D, void* devWeights, int32_t wBf16,
                  float* momentum1, float* momentum2)
{
    float* wf = static_cast<float*>(devWeights);
    uint16_t* wb = static_cast<uint16_t*>(devWeights);
    const float omb1 = 1.0f - o.beta1;
    const float omb2 = 1.0f - o.beta2;
    for (int64_t d = 0; d < D; ++d) {
        float w = wBf16 ? Bf16ToF32(wb[base + d]) : wf[base + d];
        float delta;
        if (o.optim == 2) {
            float m1 = momentum1[base + d] * o.beta1 + g[d] * omb1;
            float m2 = momentum2[base + d] * o.beta2 + (g[d] * g[d]) * omb2;
            momentum1[base + d] = m1;
            momentum2[base + d] = m2;
            delta = (m1 / (std::sqrt(m2) + o.eps)) * o.stepSize;
        } else if (o.optim == 1) {
            float m1 = momentum1[base + d] + g[d] * g[d];
            momentum1[base + d] = m1;
            delta = -((o.lr / (std::sqrt(m1) + o.eps)) * g[d]);
        } else {
            delta = g[d] * o.stepSize;
        }
        w = w + delta;
        if (wBf16) {
            wb[base + d] = F32ToBf16(w);
        } else {
            wf[base + d] = w;
        }
    }
}

// acc[0:D] += gradient row of position k of bag (t, b)
void TbeAddGradRow(float* acc, const float* gradOutput, int64_t totalD, const int32_t* dOffsets, int32_t t, int64_t b,
                   int64_t k, int64_t D, int32_t poolingMode, float scale)
{
    const float* go = poolingMode == 2 ? gradOutput + k * D : gradOutput + b * totalD + dOffsets[t];
    for (int64_t d = 0; d < D; ++d) {
        float x = go[d];
        if (poolingMode == 1) {
            x = x * scale;
        }
        acc[d] += x;
    }
}
}  // namespace

ORC_API void orc_tbe_backward(int32_t optim, const float* gradOutput, void* devWeights, int32_t wBf16,
                              const int64_t* weightsOffsets, const int32_t* dOffsets, int64_t totalD,
                              const int64_t* hashSizeCumsum, const int64_t* indices, const int64_t* offsets, int32_t T,
                              int64_t B, int32_t poolingMode, float* momentum1, float* momentum2, float lr, float eps,
                              float beta1, float beta2, int64_t iter)
{
    const TbeOpt opt = MakeTbeOpt(optim, lr, eps, beta1, beta2, iter);
    // table-global row (hashSizeCumsum[t] + row) -> place in `rows`, rows in first-touch order
    FlatMap<int64_t> rowPos(static_cast<size_t>(offsets[static_cast<int64_t>(T) * B]));
    struct Touched {
        int64_t base;  // first element of the row in the weight buffer
        int64_t D;
        size_t g;      // start of its sum in G
        int64_t count; // positions that name the row
        int32_t acc;   // its chunk accumulator when the sum takes the two-level order of orc_segment_sum, else -1
    };
    std::vector<Touched> rows;
    size_t gSize = 0;
    // first pass: the touched rows and how often each is named (the order of a row's sum depends on it)
    for (int32_t t = 0; t < T; ++t) {
        const int64_t D = poolingMode == 2 ? totalD / T : dOffsets[t + 1] - dOffsets[t];
        for (int64_t k = offsets[static_cast<int64_t>(t) * B]; k < offsets[static_cast<int64_t>(t + 1) * B]; ++k) {
            auto ret = rowPos.TryEmplace(hashSizeCumsum[t] + indices[k], static_cast<int64_t>(rows.size()));
            if (ret.second) {
                rows.push_back(Touched{weightsOffsets[t] + indices[k] * D, D, gSize, 0, -1});
                gSize += static_cast<size_t>(D);
            }
            rows[*ret.first].count++;
        }
    }
    std::vector<float> G(gSize, 0.0f);
    std::vector<OrderedSum> accs;
    for (Touched& r : rows) {
        if (r.count > kTwoLevelMin) {
            r.acc = static_cast<int32_t>(accs.size());
            accs.emplace_back();
            accs.back().Begin(r.count, r.D);
        }
    }
    for (int32_t t = 0; t < T; ++t) {
        const int64_t D = poolingMode == 2 ? totalD / T : dOffsets[t + 1] - dOffsets[t];
        for (int64_t b = 0; b < B; ++b) {
            int64_t s = offsets[t * B + b];
            int64_t e = offsets[t * B + b + 1];
            float scale = 1.0f;
            if (poolingMode == 1 && e > s) {
                scale = 1.0f / static_cast<float>(e - s);
            }
            for (int64_t k = s; k < e; ++k) {
                Touched& r = rows[*rowPos.Find(hashSizeCumsum[t] + indices[k])];
                if (r.acc >= 0) {
                    const float* go = poolingMode == 2 ? gradOutput + k * D : gradOutput + b * totalD + dOffsets[t];
                    accs[r.acc].Add(G.data() + r.g, go, D, scale, poolingMode == 1);
                } else {
                    TbeAddGradRow(G.data() + r.g, gradOutput, totalD, dOffsets, t, b, k, D, poolingMode, scale);
                }
            }
        }
    }
    for (Touched& r : rows) {
        if (r.acc >= 0) {
            accs[r.acc].Flush(G.data() + r.g, r.D);
        }
    }
    for (const Touched& r : rows) {
        TbeUpdateRow(opt, G.data() + r.g, r.base, r.D, devWeights, wBf16, momentum1, momentum2);
    }
}

// The unique variant of the same operator (op_kernel/backward_codegen_unweighted_exact_kernel_unique.h:47-95,115-270,
// ..._adam_unweighted_exact_kernel_unique.h:52-66,110-160): the caller brings the distinct rows of every table
// (uniqueIds, table after table; uniqueOffsets[t] = start of feature t's table in it, one entry per feature plus the
// total, features of one table carrying the same start) and uniqueInverse[k] = place of position k's row inside its
// table's slice.  The gradient of distinct row j is accumulated at j = uniqueOffsets[t] + uniqueInverse[k]
// (ComputeGradBag / ComputeGradNoBag), then every distinct row uniqueIds[j] of every table gets one optimizer step
// (AdamScheduler: the feature whose start differs from the one before owns the slice).  `indices` is not read.
ORC_API void orc_tbe_backward_unique(int32_t optim, const float* gradOutput, void* devWeights, int32_t wBf16,
                                     const int64_t* weightsOffsets, const int32_t* dOffsets, int64_t totalD,
                                     const int64_t* offsets, int32_t T, int64_t B, int32_t poolingMode,
                                     const int64_t* uniqueIds, const int64_t* uniqueOffsets,
                                     const int64_t* uniqueInverse, float* momentum1, float* momentum2, float lr,
                                     float eps, float beta1, float beta2, int64_t iter)
{
    const TbeOpt opt = MakeTbeOpt(optim, lr, eps, beta1, beta2, iter);
    const int64_t U = uniqueOffsets[T];
    int64_t maxD = 0;
    for (int32_t t = 0; t < T; ++t) {
        maxD = std::max<int64_t>(maxD, poolingMode == 2 ? totalD / T : dOffsets[t + 1] - dOffsets[t]);
    }
    std::vector<float> G(static_cast<size_t>(U * maxD), 0.0f);
    // how often each distinct row is named decides the order of its sum (see orc_segment_sum)
    std::vector<int64_t> count(static_cast<size_t>(U), 0);
    for (int32_t t = 0; t < T; ++t) {
        for (int64_t k = offsets[static_cast<int64_t>(t) * B]; k < offsets[static_cast<int64_t>(t + 1) * B]; ++k) {
            count[uniqueOffsets[t] + uniqueInverse[k]]++;
        }
    }
    std::vector<int32_t> accOf(static_cast<size_t>(U), -1);
    std::vector<OrderedSum> accs;
    for (int32_t t = 0; t < T; ++t) {
        const int64_t D = poolingMode == 2 ? totalD / T : dOffsets[t + 1] - dOffsets[t];
        for (int64_t j = uniqueOffsets[t]; j < uniqueOffsets[t + 1]; ++j) {
            if (count[j] > kTwoLevelMin && accOf[j] < 0) {
                accOf[j] = static_cast<int32_t>(accs.size());
                accs.emplace_back();
                accs.back().Begin(count[j], D);
            }
        }
    }
    for (int32_t t = 0; t < T; ++t) {
        const int64_t D = poolingMode == 2 ? totalD / T : dOffsets[t + 1] - dOffsets[t];
        for (int64_t b = 0; b < B; ++b) {
            int64_t s = offsets[t * B + b];
            int64_t e = offsets[t * B + b + 1];
            float scale = 1.0f;
            if (poolingMode == 1 && e > s) {
                scale = 1.0f / static_cast<float>(e - s);
            }
            for (int64_t k = s; k < e; ++k) {
                const int64_t j = uniqueOffsets[t] + uniqueInverse[k];
                if (accOf[j] >= 0) {
                    const float* go = poolingMode == 2 ? gradOutput + k * D : gradOutput + b * totalD + dOffsets[t];
                    accs[accOf[j]].Add(G.data() + j * maxD, go, D, scale, poolingMode == 1);
                } else {
                    TbeAddGradRow(G.data() + j * maxD, gradOutput, totalD, dOffsets, t, b, k, D, poolingMode, scale);
                }
            }
        }
    }
    for (int32_t t = 0; t < T; ++t) {
        const int64_t D = poolingMode == 2 ? totalD / T : dOffsets[t + 1] - dOffsets[t];
        for (int64_t j = uniqueOffsets[t]; j < uniqueOffsets[t + 1]; ++j) {
            if (accOf[j] >= 0) {
                accs[accOf[j]].Flush(G.data() + j * maxD, D);
            }
        }
    }
    int64_t last = 0;
    for (int32_t i = 1; i <= T; ++i) {
        if (uniqueOffsets[i] != last) {
            const int32_t t = i - 1;
            const int64_t D = poolingMode == 2 ? totalD / T : dOffsets[t + 1] - dOffsets[t];
            for (int64_t j = last; j < uniqueOffsets[i]; ++j) {
                TbeUpdateRow(opt, G.data() + j * maxD, weightsOffsets[t] + uniqueIds[j] * D, D, devWeights, wBf16,
                             momentum1, momentum2);
            }
            last = uniqueOffsets[i];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// A3  ock::ctr::Unique::DoEnhancedUnique with sharding / padding / id counts
//     training/tf_rec_v1/src/AccCTR/src/unique/unique_func.h:271-329 (Compute), :400-453 (TileAndFill),
//     :455-468 (HandleFill), unique_func.cpp:173-180 (GetFillOffset), unique_impl.cpp:131-140 (uniqueIdCnt)
// The reference emits the keys of a shard in hash-bucket order (and its overflow keys in unordered_map order);
// its tests assert order-free properties only (unique_test.cpp:614-641, 762-792).  This restatement fixes the
// order inside a shard to first occurrence.  shard = (uint64)key % shards, or key & (shards-1) in mask form.
// Returns uniqueIdCnt, or -1 when a shard needs more than paddingSize places (H_PADDING_SMALL).
ORC_API int64_t orc_unique_sharded(const int64_t* ids, int64_t n, int32_t shards, int32_t useMask, int32_t paddingSize,
                                   int64_t paddingVal, int64_t* uniqueId, uint32_t* index, int64_t* uniqueIdInBucket,
                                   int32_t* cntInBucket, int32_t* idCnt, int32_t* idCntFill)
{
    FlatMap<int64_t> seen(static_cast<size_t>(n));  // key -> rank inside its shard
    std::vector<std::vector<int64_t>> perShard(shards);
    std::vector<std::vector<int32_t>> perShardCnt(shards);
    std::vector<int32_t> shardOf(n);
    std::vector<int64_t> rankOf(n);
    for (int64_t i = 0; i < n; ++i) {
        const uint64_t v = static_cast<uint64_t>(ids[i]);
        const int32_t s = useMask ? static_cast<int32_t>(v & static_cast<uint64_t>(shards - 1))
                                  : static_cast<int32_t>(v % static_cast<uint64_t>(shards));
        auto res = seen.TryEmplace(ids[i], static_cast<int64_t>(perShard[s].size()));
        if (res.second) {
            perShard[s].push_back(ids[i]);
            perShardCnt[s].push_back(0);
        }
        perShardCnt[s][*res.first]++;
        shardOf[i] = s;
        rankOf[i] = *res.first;
    }
    std::vector<int64_t> base(shards + 1, 0);
    for (int32_t s = 0; s < shards; ++s) {
        cntInBucket[s] = static_cast<int32_t>(perShard[s].size());
        base[s + 1] = base[s] + cntInBucket[s];
        if (paddingSize > 0 && cntInBucket[s] > paddingSize) {
            return -1;
        }
    }
    if (paddingSize > 0) {
        for (int64_t j = 0; j < static_cast<int64_t>(paddingSize) * shards; ++j) {
            uniqueId[j] = paddingVal;
            if (idCntFill != nullptr) {
                idCntFill[j] = 0;
            }
        }
    }
    for (int32_t s = 0; s < shards; ++s) {
        for (size_t r = 0; r < perShard[s].size(); ++r) {
            const int64_t compact = base[s] + static_cast<int64_t>(r);
            const int64_t dest = paddingSize > 0 ? static_cast<int64_t>(s) * paddingSize + static_cast<int64_t>(r) : compact;
            uniqueId[dest] = perShard[s][r];
            if (uniqueIdInBucket != nullptr) {
                uniqueIdInBucket[compact] = perShard[s][r];
            }
            if (idCnt != nullptr) {
                idCnt[compact] = perShardCnt[s][r];
            }
            if (idCntFill != nullptr) {
                idCntFill[dest] = perShardCnt[s][r];
            }
        }
    }
    for (int64_t i = 0; i < n; ++i) {
        const int32_t s = shardOf[i];
        index[i] = static_cast<uint32_t>(paddingSize > 0 ? static_cast<int64_t>(s) * paddingSize + rankOf[i]
                                                         : base[s] + rankOf[i]);
    }
    return paddingSize > 0 ? static_cast<int64_t>(paddingSize) * shards : base[shards];
}

// ---------------------------------------------------------------------------------------------
// A12 hybrid::UniqueParallel  training/torch_rec_v1/hybrid_torchrec/src/ids_process/unique.cpp:55-118
// Sorted distinct ids and, per input position, the place of its id among them.  Returns the number of distinct ids.
ORC_API int64_t orc_unique_sorted(const int64_t* ids, int64_t n, int64_t* sorted, int64_t* inverse)
{
    std::vector<int64_t> perm(n);
    for (int64_t i = 0; i < n; ++i) {
        perm[i] = i;
    }
    std::stable_sort(perm.begin(), perm.end(), [&](int64_t a, int64_t b) { return ids[a] < ids[b]; });
    int64_t u = 0;
    for (int64_t j = 0; j < n; ++j) {
        if (j == 0 || ids[perm[j]] != ids[perm[j - 1]]) {
            sorted[u++] = ids[perm[j]];
        }
        inverse[perm[j]] = u - 1;
    }
    return u;
}

// ---------------------------------------------------------------------------------------------
// A9  EmbCache::OffsetMapper  training/tf_rec_v1/src/AccCTR/src/embedding_cache/offset_mapper/offset_mapper.h
//     GetSwapPairsAndKey2Offset :135-171, FindInUsedPos :178-244, FindInOffsetMapper :246-271, FilterKeys :273-295,
//     Remove :107-119; LimitedSet (slot set with most-recently-inserted-first iteration) limited_set.h:25-140.
// HBM-cache planner: keys found in the cache are replaced by their slot; the others ("swap in") take, in input
// order, (1) slots freed by Remove, most recently freed first, (2) when the cache cannot hold them all, slots of
// keys that neither this batch nor the previous one used, most recently released first (their keys are "swapped
// out"), (3) never-used slots.  The slot sets are intrusive lists here as in the reference: insertion at the head,
// iteration from the head.
namespace {

struct OrcSlotList {  // the reference's LimitedSet over slots [0, n)
    std::vector<int64_t> prev, next;
    std::vector<uint8_t> in;
    int64_t head;  // index n = head sentinel, n+1 = tail sentinel
    int64_t tail;
    explicit OrcSlotList(int64_t n) : prev(n + 2, -1), next(n + 2, -1), in(n, 0), head(n), tail(n + 1)
    {
        next[head] = tail;
        prev[tail] = head;
    }
    void Insert(int64_t v)
    {
        if (in[v]) {
            return;
        }
        in[v] = 1;
        const int64_t nx = next[head];
        next[v] = nx;
        prev[v] = head;
        next[head] = v;
        prev[nx] = v;
    }
    void Remove(int64_t v)
    {
        if (!in[v]) {
            return;
        }
        in[v] = 0;
        next[prev[v]] = next[v];
        prev[next[v]] = prev[v];
    }
};

struct OrcOffsetMapper {
    int64_t maxCacheSize;
    int64_t useLength = 0;
    int64_t evictSize = 0;
    OrcSlotList validPos;
    OrcSlotList evictPos;
    std::vector<int64_t> pos2Key;
    std::vector<int64_t> lastBatchPos;
    FlatMap<int64_t> map;
    std::vector<int64_t> swapInKeys, swapInPos, swapOutKeys, swapOutPos;
    explicit OrcOffsetMapper(int64_t m)
        : maxCacheSize(m), validPos(m), evictPos(m), pos2Key(m, -1), map(static_cast<size_t>(m))
    {
    }
};

}  // namespace

ORC_API void* orc_om_create(int64_t maxCacheSize) { return new OrcOffsetMapper(maxCacheSize); }
ORC_API void orc_om_destroy(void* h) { delete static_cast<OrcOffsetMapper*>(h); }

// keys[n] in place -> slots (entries equal to -1 are left alone).  Returns 0, or -1 for the reference's
// H_MAX_CACHESIZE_TOO_SMALL (the state is then left as the reference leaves it: partly updated).
ORC_API int32_t orc_om_compute(void* h, int64_t* keys, int64_t n)
{
    auto* om = static_cast<OrcOffsetMapper*>(h);
    om->swapInKeys.clear();
    om->swapInPos.clear();
    om->swapOutKeys.clear();
    om->swapOutPos.clear();
    std::vector<int64_t> swapInId;
    // FilterKeys :273-295
    for (int64_t i = 0; i < n; ++i) {
        if (keys[i] == -1) {
            continue;
        }
        int64_t* pos = om->map.Find(keys[i]);
        if (pos != nullptr) {
            keys[i] = *pos;
            om->validPos.Remove(keys[i]);
        } else {
            om->swapInKeys.push_back(keys[i]);
            swapInId.push_back(i);
        }
    }
    const int64_t swapIn = static_cast<int64_t>(om->swapInKeys.size());
    om->swapInPos.assign(swapIn, 0);
    // FindInUsedPos :178-244
    const int64_t freeLen = om->maxCacheSize - om->useLength + om->evictSize;
    const int64_t swapOutNum = swapIn <= freeLen ? 0 : swapIn - freeLen;
    om->swapOutKeys.assign(swapOutNum, 0);
    om->swapOutPos.assign(swapOutNum, 0);
    int64_t inCnt = 0;
    for (int64_t p = om->evictPos.next[om->evictPos.head]; p != om->evictPos.tail; p = om->evictPos.next[p]) {
        if (inCnt == swapIn) {
            break;
        }
        om->swapInPos[inCnt] = p;
        keys[swapInId[inCnt]] = p;
        om->map.TryEmplace(om->swapInKeys[inCnt], p);
        om->pos2Key[p] = om->swapInKeys[inCnt];
        inCnt++;
        om->evictSize--;
    }
    int64_t outCnt = 0;
    for (int64_t p = om->validPos.next[om->validPos.head]; p != om->validPos.tail; p = om->validPos.next[p]) {
        if (outCnt == swapOutNum) {
            break;
        }
        om->swapInPos[inCnt] = p;
        keys[swapInId[inCnt]] = p;
        const int64_t old = om->pos2Key[p];
        om->map.Erase(old);
        om->map.TryEmplace(om->swapInKeys[inCnt], p);
        om->swapOutKeys[outCnt] = old;
        om->swapOutPos[outCnt] = p;
        om->pos2Key[p] = om->swapInKeys[inCnt];
        inCnt++;
        outCnt++;
    }
    if (outCnt < swapOutNum) {
        return -1;
    }
    // FindInOffsetMapper :246-271
    for (int64_t i = inCnt; i < swapIn; ++i) {
        om->swapInPos[i] = om->useLength++;
        if (om->swapInPos[i] >= om->maxCacheSize) {
            return -1;
        }
        om->map.TryEmplace(om->swapInKeys[i], om->swapInPos[i]);
        om->pos2Key[om->swapInPos[i]] = om->swapInKeys[i];
        keys[swapInId[i]] = om->swapInPos[i];
    }
    // :153-168
    for (int64_t p : om->lastBatchPos) {
        if (p != -1) {
            om->validPos.Insert(p);
        }
    }
    for (int64_t i = 0; i < n; ++i) {
        if (keys[i] != -1) {
            om->validPos.Remove(keys[i]);
            om->evictPos.Remove(keys[i]);
        }
    }
    om->lastBatchPos.assign(keys, keys + n);
    return 0;
}

// which: 0 swapInKeys, 1 swapInPos, 2 swapOutKeys, 3 swapOutPos.  Returns the length (copies when cap suffices).
ORC_API int64_t orc_om_result(void* h, int32_t which, int64_t* out, int64_t cap)
{
    auto* om = static_cast<OrcOffsetMapper*>(h);
    const std::vector<int64_t>* v[4] = {&om->swapInKeys, &om->swapInPos, &om->swapOutKeys, &om->swapOutPos};
    const auto& src = *v[which];
    if (out != nullptr && cap >= static_cast<int64_t>(src.size())) {
        std::copy(src.begin(), src.end(), out);
    }
    return static_cast<int64_t>(src.size());
}

// OffsetMapper::Remove :107-119 for each key (keys not in the cache are ignored)
ORC_API void orc_om_remove(void* h, const int64_t* keys, int64_t n)
{
    auto* om = static_cast<OrcOffsetMapper*>(h);
    for (int64_t i = 0; i < n; ++i) {
        int64_t* pos = om->map.Find(keys[i]);
        if (pos == nullptr) {
            continue;
        }
        const int64_t p = *pos;
        om->validPos.Remove(p);
        auto it = std::find(om->lastBatchPos.begin(), om->lastBatchPos.end(), p);
        if (it != om->lastBatchPos.end()) {
            om->lastBatchPos.erase(it);
        }
        om->evictPos.Insert(p);
        om->evictSize++;
        om->map.Erase(keys[i]);
    }
}

// state[0] = useLength, [1] = evictSize, [2] = live keys; pairs (optional, capacity = live keys): key, slot
// sorted by slot (ExportSortedKVPairs :121-126)
ORC_API void orc_om_state(void* h, int64_t* state, int64_t* pairKeys, int64_t* pairSlots)
{
    auto* om = static_cast<OrcOffsetMapper*>(h);
    state[0] = om->useLength;
    state[1] = om->evictSize;
    state[2] = static_cast<int64_t>(om->map.Size());
    if (pairKeys != nullptr && pairSlots != nullptr) {
        std::vector<std::pair<int64_t, int64_t>> kv;
        om->map.ForEach([&](int64_t k, int64_t v) { kv.emplace_back(v, k); });
        std::sort(kv.begin(), kv.end());
        for (size_t i = 0; i < kv.size(); ++i) {
            pairKeys[i] = kv[i].second;
            pairSlots[i] = kv[i].first;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// A21 row initializers  training/tf_rec_v1/src/AccCTR/src/embedding_cache/initializer/
//     constant_initializer/constant_initializer.cpp:25-63, random_normal_initializer/random_normal_initializer.cpp:24-79,
//     truncated_normal_initializer/truncated_normal_initializer.cpp:23-95 (limits embedding_cache/common.h:55-62)
// The reference draws from std::default_random_engine + std::normal_distribution<float>; those are third-party
// (libstdc++: minstd_rand0 = x*16807 mod 2^31-1; generate_canonical<float,24> = one draw, (x-1)/2147483648f;
// Marsaglia polar method in float, second value saved for the next call).  The algorithm is restated here by hand,
// not by calling the std classes, so that the product (which calls them) can be checked against it.
namespace {

struct OrcNormal {
    uint64_t state;
    float mean, stddev;
    bool saved = false;
    float savedVal = 0.0f;
    OrcNormal(uint32_t seed, float m, float s) : mean(m), stddev(s)
    {
        state = seed % 2147483647u;
        if (state == 0) {
            state = 1;
        }
    }
    uint32_t Next()
    {
        state = state * 16807u % 2147483647u;
        return static_cast<uint32_t>(state);
    }
    float Canonical()
    {
        const float r = static_cast<float>(Next() - 1u) / 2147483648.0f;
        return r >= 1.0f ? std::nextafterf(1.0f, 0.0f) : r;
    }
    float Draw()
    {
        float ret;
        if (saved) {
            saved = false;
            ret = savedVal;
        } else {
            float x, y, r2;
            do {
                x = 2.0f * Canonical() - 1.0f;
                y = 2.0f * Canonical() - 1.0f;
                r2 = x * x + y * y;
            } while (r2 > 1.0f || r2 == 0.0f);
            const float mult = std::sqrt(-2.0f * std::log(r2) / r2);
            savedVal = x * mult;
            saved = true;
            ret = y * mult;
        }
        return ret * stddev + mean;
    }
};

inline float OrcClamp(float v, float lo, float hi) { return v > hi ? hi : (v < lo ? lo : v); }

struct OrcInit {
    int32_t kind;
    uint32_t start, len;
    float value, initK, minBound, maxBound;
    OrcNormal gen;
    OrcInit(int32_t k, uint32_t s, uint32_t l, float a, float b, uint32_t seed, float ik)
        : kind(k), start(s), len(l), value(0), initK(OrcClamp(ik, -10000.0f, 10000.0f)), minBound(0), maxBound(0),
          gen(seed, OrcClamp(a, -1e9f, 1e9f), OrcClamp(b, 0.0f, 100.0f))
    {
        if (kind == 0) {
            value = initK * OrcClamp(a, -1e9f, 1e9f);
        } else {
            minBound = initK * (gen.mean - 2.0f * gen.stddev);
            maxBound = initK * (gen.mean + 2.0f * gen.stddev);
        }
    }
    void Generate(float* row)
    {
        for (uint32_t j = 0; j < len; ++j) {
            if (kind == 0) {
                row[start + j] = value;
            } else if (kind == 1) {
                row[start + j] = initK * gen.Draw();
            } else {
                float t = initK * gen.Draw();
                while (t < minBound || t > maxBound) {
                    t = initK * gen.Draw();
                }
                row[start + j] = t;
            }
        }
    }
};

}  // namespace

// descs: n records of {kind, start, len, seed} in `ints` (4 per record) and {value_or_mean, stddev, init_k} in `floats`
ORC_API void* orc_init_create(const int64_t* ints, const float* floats, int32_t n)
{
    auto* v = new std::vector<OrcInit>();
    for (int32_t k = 0; k < n; ++k) {
        v->emplace_back(static_cast<int32_t>(ints[4 * k]), static_cast<uint32_t>(ints[4 * k + 1]),
                        static_cast<uint32_t>(ints[4 * k + 2]), floats[3 * k], floats[3 * k + 1],
                        static_cast<uint32_t>(ints[4 * k + 3]), floats[3 * k + 2]);
    }
    return v;
}
ORC_API void orc_init_destroy(void* h) { delete static_cast<std::vector<OrcInit>*>(h); }
ORC_API void orc_init_generate(void* h, float* rows, int64_t n, int32_t extDim)
{
    auto* v = static_cast<std::vector<OrcInit>*>(h);
    for (int64_t r = 0; r < n; ++r) {
        for (OrcInit& it : *v) {
            it.Generate(rows + r * extDim);
        }
    }
}
// The same stream drawn from the std classes themselves (what the reference's initializers call): pins the hand
// restatement above, now that the library generates the stream on its own as well.
ORC_API void orc_std_normal(uint32_t seed, float mean, float stddev, int64_t n, float* out)
{
    std::default_random_engine gen(seed);
    std::normal_distribution<float> dist(mean, stddev);
    for (int64_t i = 0; i < n; ++i) {
        out[i] = dist(gen);
    }
}
// the raw engine: out[i] = i-th output of minstd_rand0 seeded with `seed`
ORC_API void orc_minstd_rand0(uint32_t seed, int64_t n, uint32_t* out)
{
    OrcNormal g(seed, 0.0f, 1.0f);
    for (int64_t i = 0; i < n; ++i) {
        out[i] = g.Next();
    }
}
