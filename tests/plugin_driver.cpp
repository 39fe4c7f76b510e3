// Test driver of the AccCTR plugin replacement (recsdk_amd/plugin): loads lib_ock_ctr_common.so the way the
// reference's host runtime does - ock::ctr::Factory::Create, i.e. dlopen + CTR_CreateFactory through the reference's
// own include/ock_ctr_common_def.h - and drives ock::ctr::Unique and EmbCache::EmbCacheManager through cases
// modelled on the reference's unit tests (AccCTR/tests/ut/src/unique_test.cpp, emb_cache_test.cpp): the same
// configurations, return codes and order-free assertions.  Compiled against the reference's interface headers where
// they lie; run by tests/test_gpu_plugin.py with the plugin's directory on LD_LIBRARY_PATH.
// Prints one line per failed check and a final "plugin_driver: <checks> checks, <failures> failures".
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <numeric>
#include <random>
#include <set>
#include <stdexcept>
#include <string>
#include <thread>
#include <unordered_set>
#include <vector>

#include "factory.h"

using namespace ock::ctr;
using namespace EmbCache;

static int g_checks = 0;
static int g_failures = 0;

#define CHECK(cond)                                                        \
    do {                                                                   \
        ++g_checks;                                                        \
        if (!(cond)) {                                                     \
            ++g_failures;                                                  \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
        }                                                                  \
    } while (0)

#define CHECK_EQ(a, b)                                                                                       \
    do {                                                                                                     \
        ++g_checks;                                                                                          \
        const long long _a = (long long)(a);                                                                 \
        const long long _b = (long long)(b);                                                                 \
        if (_a != _b) {                                                                                      \
            ++g_failures;                                                                                    \
            std::printf("FAILED %s:%d: %s == %s (%lld vs %lld)\n", __FILE__, __LINE__, #a, #b, _a, _b);     \
        }                                                                                                    \
    } while (0)

static std::vector<std::string> g_logs;
static std::mutex g_logLock;
static void CollectLog(int level, const char* msg)
{
    std::lock_guard<std::mutex> lock(g_logLock);
    if (level >= 2) {
        g_logs.emplace_back(msg);
    }
}

static FactoryPtr g_factory;

// ---- Unique -----------------------------------------------------------------------------------------------------
static UniqueConf EnhancedConf(uint32_t desired, int shards, bool padding, int paddingSize, bool idCount)
{
    UniqueConf conf;
    conf.desiredSize = desired;
    conf.dataType = DataType::INT64;
    conf.minThreadNum = 1;
    conf.maxThreadNum = 1;
    conf.maxIdVal = 1LL << 40;
    conf.outputType = OutputType::ENHANCED;
    conf.useSharding = shards > 0;
    conf.shardingNum = shards > 0 ? shards : -1;
    conf.usePadding = padding;
    conf.paddingSize = paddingSize;
    conf.useIdCount = idCount;
    return conf;
}

static void UniqueConfCodes()
{
    UniquePtr unique;
    CHECK_EQ(g_factory->CreateUnique(unique), 0);
    FactoryPtr again;
    CHECK_EQ(Factory::Create(again), -1);  // the library is loaded once per process
    UniqueConf conf = EnhancedConf(6, 2, true, 1, true);
    conf.maxIdVal = 0;
    CHECK_EQ(unique->Initialize(conf), 4);  // maxIdVal must be positive
    conf.maxIdVal = 9;
    conf.shardingNum = 0;
    CHECK_EQ(unique->Initialize(conf), 4);
    conf.shardingNum = 4;
    conf.maxThreadNum = 0;
    CHECK_EQ(unique->Initialize(conf), 1);
    conf.maxThreadNum = 1;
    conf.paddingSize = 0;
    CHECK_EQ(unique->Initialize(conf), 4);
    conf.desiredSize = 0;
    CHECK_EQ(unique->Initialize(conf), 4);
    conf.desiredSize = 1431655766u;
    CHECK_EQ(unique->Initialize(conf), 1);
    conf.desiredSize = 6;
    conf.minThreadNum = 100000;
    conf.maxThreadNum = 100000;
    CHECK_EQ(unique->Initialize(conf), 1);
    conf.minThreadNum = 1;
    conf.maxThreadNum = 1;
    conf.paddingSize = 1;
    CHECK_EQ(unique->Initialize(conf), 0);

    std::vector<int64_t> ids = {5, 5, 3, 1, 5, 2};
    std::vector<int64_t> uniqueId(8), inBucket(8);
    std::vector<uint32_t> index(6);
    std::vector<int> idCnt(8), idCntFill(8), cntInBucket(4);
    UniqueIn in;
    in.inputIdCnt = 6;
    in.inputId = ids.data();
    EnhancedUniqueOut out;
    out.uniqueId = nullptr;
    out.index = index.data();
    out.idCnt = idCnt.data();
    out.idCntFill = idCntFill.data();
    out.uniqueIdCntInBucket = cntInBucket.data();
    out.uniqueIdInBucket = inBucket.data();
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 3);
    out.uniqueId = uniqueId.data();
    out.uniqueIdCntInBucket = nullptr;
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 3);
    out.uniqueIdCntInBucket = cntInBucket.data();
    out.idCntFill = nullptr;
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 3);
    out.idCntFill = idCntFill.data();
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 7);  // 4 shards of 1 cannot hold {5, 1} in shard 1
    in.inputIdCnt = 0;
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 4);
    unique->UnInitialize();
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 11);

    conf = EnhancedConf(6, 0, true, 1, false);  // padding without sharding
    CHECK_EQ(unique->Initialize(conf), 9);
    conf = UniqueConf();
    conf.desiredSize = (uint32_t)-1;
    conf.maxIdVal = 9;
    CHECK_EQ(unique->Initialize(conf), 1);
    conf = EnhancedConf(16, 3, false, 0, false);
    conf.performance = true;  // the mask variant needs a power of two
    CHECK_EQ(unique->Initialize(conf), 1);
}

static std::vector<int64_t> ZipfLikeIds(size_t n, uint64_t seed, int64_t range)
{
    std::mt19937_64 rng(seed);
    std::vector<int64_t> ids(n);
    for (auto& v : ids) {
        const double u = std::generate_canonical<double, 53>(rng);
        v = (int64_t)((double)range * u * u * u);
    }
    return ids;
}

static void UniqueNormal(DataType type)
{
    UniquePtr unique;
    CHECK_EQ(g_factory->CreateUnique(unique), 0);
    UniqueConf conf;
    conf.desiredSize = 1000;  // an estimate: the call below brings more ids
    conf.dataType = type;
    conf.maxIdVal = 10000000000LL;
    conf.outputType = OutputType::NORMAL;
    CHECK_EQ(unique->Initialize(conf), 0);
    const size_t n = 30000;
    std::vector<int64_t> ids = ZipfLikeIds(n, 30, 200000);
    std::vector<int32_t> ids32(ids.begin(), ids.end());
    std::vector<int64_t> uniqueId(n);
    std::vector<int32_t> uniqueId32(n);
    std::vector<uint32_t> index(n);
    UniqueIn in;
    in.inputIdCnt = (uint32_t)n;
    in.inputId = nullptr;
    UniqueOut out;
    out.uniqueId = type == DataType::INT64 ? (void*)uniqueId.data() : (void*)uniqueId32.data();
    out.index = index.data();
    CHECK_EQ(unique->DoUnique(in, out), 3);
    in.inputId = type == DataType::INT64 ? (void*)ids.data() : (void*)ids32.data();
    EnhancedUniqueOut wrong;
    wrong.uniqueId = out.uniqueId;
    wrong.index = out.index;
    CHECK_EQ(unique->DoEnhancedUnique(in, wrong), 8);
    for (int round = 0; round < 2; ++round) {  // a handle serves many batches
        CHECK_EQ(unique->DoUnique(in, out), 0);
        std::set<int64_t> distinct(ids.begin(), ids.end());
        CHECK_EQ(out.uniqueIdCnt, distinct.size());
        bool restored = true;
        std::set<int64_t> emitted;
        for (size_t i = 0; i < n; ++i) {
            const int64_t v = type == DataType::INT64 ? uniqueId[index[i]] : (int64_t)uniqueId32[index[i]];
            restored = restored && index[i] < (uint32_t)out.uniqueIdCnt && v == ids[i];
        }
        for (int i = 0; i < out.uniqueIdCnt; ++i) {
            emitted.insert(type == DataType::INT64 ? uniqueId[i] : (int64_t)uniqueId32[i]);
        }
        CHECK(restored);
        CHECK(emitted == distinct);
        std::rotate(ids.begin(), ids.begin() + 7, ids.end());
        std::rotate(ids32.begin(), ids32.begin() + 7, ids32.end());
    }
    unique->UnInitialize();
}

static void UniqueSharded(bool padding, bool performance)
{
    UniquePtr unique;
    CHECK_EQ(g_factory->CreateUnique(unique), 0);
    const int shards = 8;
    const size_t n = 20000;
    std::vector<int64_t> ids = ZipfLikeIds(n, 7, 50000);
    std::map<int64_t, int> want;
    for (int64_t v : ids) {
        want[v] += 1;
    }
    std::vector<int> perShard(shards, 0);
    for (auto& kv : want) {
        perShard[kv.first % shards] += 1;
    }
    const int pad = padding ? *std::max_element(perShard.begin(), perShard.end()) + 3 : 0;
    UniqueConf conf = EnhancedConf((uint32_t)n, shards, padding, pad, true);
    conf.performance = performance;
    conf.paddingVal = -1;
    CHECK_EQ(unique->Initialize(conf), 0);
    UniqueOut normalOut;
    std::vector<int64_t> uniqueId(std::max<size_t>(n, (size_t)pad * shards)), inBucket(n);
    std::vector<uint32_t> index(n);
    std::vector<int> idCnt(n), idCntFill(uniqueId.size()), cntInBucket(shards);
    UniqueIn in;
    in.inputIdCnt = (uint32_t)n;
    in.inputId = ids.data();
    normalOut.uniqueId = uniqueId.data();
    normalOut.index = index.data();
    CHECK_EQ(unique->DoUnique(in, normalOut), 8);
    EnhancedUniqueOut out;
    out.uniqueId = uniqueId.data();
    out.index = index.data();
    out.uniqueIdInBucket = inBucket.data();
    out.uniqueIdCntInBucket = cntInBucket.data();
    out.idCnt = idCnt.data();
    out.idCntFill = idCntFill.data();
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 0);
    CHECK_EQ(out.uniqueIdCnt, padding ? pad * shards : (int)want.size());
    for (int s = 0; s < shards; ++s) {
        CHECK_EQ(cntInBucket[s], perShard[s]);
    }
    bool restored = true;
    for (size_t i = 0; i < n; ++i) {
        restored = restored && uniqueId[index[i]] == ids[i];
    }
    CHECK(restored);
    bool inShard = true;
    bool counts = true;
    bool layout = true;
    size_t at = 0;
    for (int s = 0; s < shards; ++s) {
        for (int r = 0; r < cntInBucket[s]; ++r, ++at) {
            const int64_t id = inBucket[at];
            inShard = inShard && (id % shards) == s;
            counts = counts && want.count(id) != 0 && idCnt[at] == want[id];
            const size_t place = padding ? (size_t)s * pad + r : at;
            layout = layout && uniqueId[place] == id;
            if (padding) {
                counts = counts && idCntFill[place] == want[id];
            }
        }
        if (padding) {
            for (int r = cntInBucket[s]; r < pad; ++r) {
                layout = layout && uniqueId[(size_t)s * pad + r] == -1 && idCntFill[(size_t)s * pad + r] == 0;
            }
        }
    }
    CHECK_EQ(at, want.size());
    CHECK(inShard);
    CHECK(counts);
    CHECK(layout);
    unique->UnInitialize();
}

static void UniqueIdLarge()
{
    UniquePtr unique;
    CHECK_EQ(g_factory->CreateUnique(unique), 0);
    UniqueConf conf;
    conf.desiredSize = 6;
    conf.useIdCount = true;
    conf.maxIdVal = 1;
    conf.outputType = OutputType::ENHANCED;
    CHECK_EQ(unique->Initialize(conf), 0);
    std::vector<int64_t> ids = {5, 5, 3, 1, 5, 2}, uniqueId(6);
    std::vector<uint32_t> index(6);
    std::vector<int> idCnt(6);
    UniqueIn in;
    in.inputIdCnt = 6;
    in.inputId = ids.data();
    EnhancedUniqueOut out;
    out.uniqueId = uniqueId.data();
    out.index = index.data();
    out.idCnt = idCnt.data();
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 6);
    // without sharding the bucket outputs may stay NULL
    conf.maxIdVal = 9;
    CHECK_EQ(unique->Initialize(conf), 0);
    CHECK_EQ(unique->DoEnhancedUnique(in, out), 0);
    CHECK_EQ(out.uniqueIdCnt, 4);
    std::map<int64_t, int> got;
    for (int i = 0; i < 4; ++i) {
        got[uniqueId[i]] = idCnt[i];
    }
    CHECK((got == std::map<int64_t, int>{{5, 3}, {3, 1}, {1, 1}, {2, 1}}));
    unique->UnInitialize();
}

// ---- EmbCacheManager --------------------------------------------------------------------------------------------
static std::vector<InitializerInfo> ConstantInit(uint32_t emb, uint32_t ext, float w, float slot)
{
    std::string name = "constant_initializer";
    std::vector<InitializerInfo> infos;
    infos.emplace_back(name, 0, emb, ConstantInitializerInfo(w, 1.0f));
    if (ext > emb) {
        infos.emplace_back(name, emb, ext - emb, ConstantInitializerInfo(slot, 2.0f));
    }
    return infos;
}

static void CacheCreateCodes(EmbCacheManagerPtr& mgr)
{
    auto init = ConstantInit(8, 16, 0.5f, 0.25f);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("", 100, 8, 16, 10), init), 22);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo(std::string(1025, 'x'), 100, 8, 16, 10), init), 24);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 0, 8, 16, 10), init), 21);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 0), init), 21);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 5, 8, 16, 10), init), 17);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 20, 10), init), 15);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 24, 10), init), 14);   // columns 16..24 uncovered
    auto gap = init;
    gap[1].start = 9;
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), gap), 14);
    std::string bad = "no_such_initializer";
    std::vector<InitializerInfo> invalid;
    invalid.emplace_back(bad, 0, 16, ConstantInitializerInfo(1.0f, 1.0f));
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), invalid), 14);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), init, -1, 0), 23);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), init, -1, 101), 23);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), init), 23);  // the default 500000 > 100 rows
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), init, -1, 50, 0), 18);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), init, -1, 50, 1000000), 18);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), init, -1, 50, 1), 0);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("t", 100, 8, 16, 10), init, -1, 50, 1), 19);
    std::vector<std::string> names;
    CHECK_EQ(mgr->GetEmbTableNames(names), 0);
    CHECK(names == std::vector<std::string>{"t"});
    CHECK_EQ(mgr->GetEmbTableNames(names), 20);
}

static void CacheRows(EmbCacheManagerPtr& mgr)
{
    const uint32_t ext = 16;
    std::vector<uint64_t> keys = {11, 7, 1ULL << 40, 3};
    std::vector<float> rows(keys.size() * ext, -1.0f);
    CHECK_EQ(mgr->EmbeddingLookup("missing", keys, rows.data()), 12);
    CHECK_EQ(mgr->EmbeddingLookup("t", keys, rows.data(), 0), 18);
    CHECK_EQ(mgr->EmbeddingLookup("t", keys, nullptr), 3);
    CHECK_EQ(mgr->EmbeddingLookup("t", {}, nullptr), 0);
    CHECK_EQ(mgr->EmbeddingLookup("t", keys, rows.data()), 0);
    bool initial = true;
    for (size_t i = 0; i < keys.size(); ++i) {
        for (uint32_t c = 0; c < ext; ++c) {
            initial = initial && rows[i * ext + c] == (c < 8 ? 0.5f : 0.5f);  // 0.5 * 1 and 0.25 * initK 2
        }
    }
    CHECK(initial);
    CHECK_EQ(mgr->GetUsage("t"), 4);
    for (size_t i = 0; i < rows.size(); ++i) {
        rows[i] = (float)i;
    }
    CHECK_EQ(mgr->EmbeddingUpdate("t", keys, rows.data()), 0);
    std::vector<uint64_t> some = {3, 11, 99};
    std::vector<float> got(some.size() * ext);
    CHECK_EQ(mgr->EmbeddingLookup("t", some, got.data()), 0);
    CHECK(std::equal(got.begin(), got.begin() + ext, rows.begin() + 3 * ext));
    CHECK(std::equal(got.begin() + ext, got.begin() + 2 * ext, rows.begin()));
    CHECK(got[2 * ext] == 0.5f);  // key 99 is new
    CHECK_EQ(mgr->GetUsage("t"), 5);
    std::vector<float*> addrs;
    CHECK_EQ(mgr->EmbeddingLookupAddrs("t", keys, addrs), 0);
    CHECK_EQ(addrs.size(), keys.size());
    if (addrs.size() != keys.size() || addrs[1] == nullptr) {
        return;
    }
    CHECK(std::equal(addrs[1], addrs[1] + ext, rows.begin() + ext));
    addrs[1][2] = 1234.0f;  // the addresses are the rows themselves
    std::vector<uint64_t> one = {7};
    CHECK_EQ(mgr->EmbeddingLookupAndRemove("t", one, got.data()), 0);
    CHECK(got[2] == 1234.0f && got[3] == rows[ext + 3]);
    CHECK_EQ(mgr->GetUsage("t"), 4);
    CHECK_EQ(mgr->EmbeddingLookupAndRemove("t", one, got.data()), 0);  // gone: initial values, nothing stored
    CHECK(got[2] == 0.5f);
    CHECK_EQ(mgr->GetUsage("t"), 4);
    CHECK_EQ(mgr->EmbeddingRemove("t", {11, 424242}), 0);
    CHECK_EQ(mgr->GetUsage("t"), 3);
    // the host table holds vocabSize rows and no more
    std::vector<uint64_t> many(200);
    std::iota(many.begin(), many.end(), 1000);
    std::vector<float> big(many.size() * ext);
    CHECK_EQ(mgr->EmbeddingLookup("t", many, big.data()), 17);
}

static void CachePlanner(EmbCacheManagerPtr& mgr)
{
    auto init = ConstantInit(4, 8, 1.0f, 0.0f);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("plan", 64, 4, 8, 5), init, -1, 16, 1), 0);
    EmbBaseInfo info(0, 0, "plan", false, true, {9});
    std::vector<uint64_t> keys = {6, 9, (uint64_t)-1, 4, 2};
    KeyOffsetPair in, out;
    in.first.push_back(1);
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(info, keys, in, out), 20);
    in.first.clear();
    EmbBaseInfo unknown(0, 0, "nope", false, false, {});
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(unknown, keys, in, out), 12);
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(info, keys, in, out), 0);
    CHECK((keys == std::vector<uint64_t>{0, 1, (uint64_t)-1, 2, 3}));
    CHECK((in.first == std::vector<uint64_t>{6, 9, 4, 2}) && (in.second == std::vector<uint64_t>{0, 1, 2, 3}));
    CHECK(out.first.empty() && out.second.empty());
    CHECK((mgr->GetPaddingKeysOffset("plan") == std::unordered_set<uint64_t>{1}));
    // slots used by the previous call cannot be taken: three new keys, one free slot, no victim allowed yet
    keys = {9, 20, 21, 22};
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(info, keys, in, out), 16);
    keys = {9};
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(info, keys, in, out), 0);
    CHECK(in.first.empty() && out.first.empty());
    // now the slots of 6, 4 and 2 may go: 9 stays, three new keys take the free slot and two victims' slots
    keys = {9, 20, 21, 22};
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(info, keys, in, out), 0);
    CHECK_EQ(keys[0], 1);
    CHECK_EQ(in.first.size(), 3);
    CHECK_EQ(out.first.size(), 2);
    std::set<uint64_t> used(keys.begin(), keys.end());
    CHECK_EQ(used.size(), 4);
    for (size_t i = 0; i < out.first.size(); ++i) {
        CHECK(out.first[i] == 6 || out.first[i] == 4 || out.first[i] == 2);
        CHECK(std::find(in.second.begin(), in.second.end(), out.second[i]) != in.second.end());
    }
    // a batch that cannot fit: six keys in five slots
    keys = {30, 31, 32, 33, 34, 35};
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(info, keys, in, out), 16);
    std::vector<std::pair<uint64_t, uint64_t>> ko;
    CHECK_EQ(mgr->ExportDeviceKeyOffsetPairs("plan", ko), 0);
    CHECK_EQ(ko.size(), 5);
    bool sorted = true;
    std::map<uint64_t, uint64_t> byKey;
    for (size_t i = 0; i < ko.size(); ++i) {
        sorted = sorted && ko[i].second == i;
        byKey[ko[i].first] = ko[i].second;
    }
    CHECK(sorted);
    CHECK(byKey.count(9) && byKey[9] == 1 && byKey.count(20) && byKey.count(21) && byKey.count(22));
    // evaluation phase: an empty planner, then the training state again
    CHECK_EQ(mgr->BackUpTrainStatus("plan"), 0);
    CHECK_EQ(mgr->ExportDeviceKeyOffsetPairs("plan", ko), 0);
    CHECK(ko.empty());
    CHECK(mgr->GetPaddingKeysOffset("plan").empty());
    keys = {77, 9};
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    EmbBaseInfo eval(1, 1, "plan", false, true, {9});
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(eval, keys, in, out), 0);
    CHECK((keys == std::vector<uint64_t>{0, 1}));
    CHECK(mgr->GetPaddingKeysOffset("plan").empty());  // recorded on the train channel only
    CHECK_EQ(mgr->RecoverTrainStatus("plan"), 0);
    CHECK_EQ(mgr->ExportDeviceKeyOffsetPairs("plan", ko), 0);
    CHECK_EQ(ko.size(), 5);
    std::map<uint64_t, uint64_t> after;
    for (auto& p : ko) {
        after[p.first] = p.second;
    }
    CHECK(after == byKey);
    CHECK((mgr->GetPaddingKeysOffset("plan") == std::unordered_set<uint64_t>{1}));
    // RemoveEmbsByKeys frees the slot and the host row; the invalid key is skipped
    std::vector<uint64_t> h = {20};
    std::vector<float> row(8);
    CHECK_EQ(mgr->EmbeddingLookup("plan", h, row.data()), 0);
    CHECK_EQ(mgr->GetUsage("plan"), 1);
    CHECK_EQ(mgr->RemoveEmbsByKeys("plan", {20, (uint64_t)-1, 555}), 0);
    CHECK_EQ(mgr->GetUsage("plan"), 0);
    CHECK_EQ(mgr->ExportDeviceKeyOffsetPairs("plan", ko), 0);
    CHECK_EQ(ko.size(), 4);
    keys = {40};
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(info, keys, in, out), 0);
    CHECK_EQ(keys[0], byKey[20]);  // the freed slot is the first to be reused
    CHECK(out.first.empty());
    CHECK_EQ(mgr->ResetOffsetMappers(), 0);
    CHECK_EQ(mgr->ExportDeviceKeyOffsetPairs("plan", ko), 0);
    CHECK(ko.empty());
    bool thrown = false;
    try {
        (void)mgr->GetPaddingKeysOffset("nope");
    } catch (const std::invalid_argument&) {
        thrown = true;
    }
    CHECK(thrown);
    // a batch larger than the planner was sized for grows its workspace and keeps its state
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("wide", 4000, 4, 8, 3000), init, -1, 100, 1), 0);
    EmbBaseInfo wide(0, 0, "wide", false, false, {});
    keys = {1, 2, 3};
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(wide, keys, in, out), 0);
    std::vector<uint64_t> lots(3500, (uint64_t)-1);  // mostly invalid keys: more entries than slots
    lots[10] = 2;
    lots[3400] = 50;
    in = KeyOffsetPair();
    out = KeyOffsetPair();
    CHECK_EQ(mgr->GetSwapPairsAndKey2Offset(wide, lots, in, out), 0);
    CHECK_EQ(lots[10], 1);
    CHECK_EQ(lots[3400], 3);
    CHECK_EQ(lots[0], (uint64_t)-1);
}

// One step of the DDR pipeline on one table, as HybridMgmt::ProcessEmbInfoDDR drives it (hybrid_mgmt.cpp:660-716):
// plan the batch, fetch the rows that move in, store rows that moved out.  Everything the calls return goes to `log`.
static int PipelineSteps(EmbCacheManagerPtr& mgr, const std::string& table, uint64_t seed, int steps,
                         std::vector<uint64_t>& log)
{
    const uint32_t ext = 8;
    for (int s = 0; s < steps; ++s) {
        std::vector<uint64_t> keys;   // distinct, first occurrence first, as KeyProcess hands them over
        std::set<int64_t> seen;
        for (int64_t id : ZipfLikeIds(600, seed + (uint64_t)s, 5000)) {
            if (seen.insert(id).second) {
                keys.push_back((uint64_t)id);
            }
        }
        EmbBaseInfo info(s, 0, table, false, false, {});
        KeyOffsetPair in, out;
        int ret = mgr->GetSwapPairsAndKey2Offset(info, keys, in, out);
        if (ret != 0) {
            return ret;
        }
        log.insert(log.end(), keys.begin(), keys.end());
        log.push_back(in.first.size());
        log.insert(log.end(), in.first.begin(), in.first.end());
        log.insert(log.end(), in.second.begin(), in.second.end());
        log.push_back(out.first.size());
        std::vector<std::pair<uint64_t, uint64_t>> gone;   // victims come in no fixed order in the reference either
        for (size_t i = 0; i < out.first.size(); ++i) {
            gone.emplace_back(out.first[i], out.second[i]);
        }
        std::sort(gone.begin(), gone.end());
        for (auto& g : gone) {
            log.push_back(g.first);
            log.push_back(g.second);
        }
        std::vector<float> rows(in.first.size() * ext);
        ret = mgr->EmbeddingLookup(table, in.first, rows.data());
        if (ret != 0) {
            return ret;
        }
        for (size_t i = 0; i < rows.size(); ++i) {
            uint32_t bits;
            std::memcpy(&bits, &rows[i], sizeof(bits));
            log.push_back(bits);
            rows[i] += (float)(s + 1);
        }
        ret = mgr->EmbeddingUpdate(table, in.first, rows.data());
        if (ret != 0) {
            return ret;
        }
    }
    return 0;
}

// HybridMgmt hands every table's batch to a thread pool (hybrid_mgmt.cpp:545-560): two tables driven from two threads
// at once give what the same calls give one after the other.
static void CacheTwoThreads(EmbCacheManagerPtr& mgr)
{
    auto init = ConstantInit(4, 8, 1.0f, 0.5f);
    const char* names[4] = {"pairA", "pairB", "soloA", "soloB"};
    for (const char* name : names) {
        CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo(name, 20000, 4, 8, 1500), init, -1, 100, 1), 0);
    }
    const int steps = 12;
    std::vector<uint64_t> logs[4];
    int rets[4] = {-1, -1, -1, -1};
    std::thread first([&]() { rets[0] = PipelineSteps(mgr, names[0], 100, steps, logs[0]); });
    std::thread second([&]() { rets[1] = PipelineSteps(mgr, names[1], 900, steps, logs[1]); });
    first.join();
    second.join();
    rets[2] = PipelineSteps(mgr, names[2], 100, steps, logs[2]);
    rets[3] = PipelineSteps(mgr, names[3], 900, steps, logs[3]);
    for (int r : rets) {
        CHECK_EQ(r, 0);
    }
    CHECK(logs[0].size() > (size_t)steps * 300);
    CHECK(logs[0] == logs[2]);
    CHECK(logs[1] == logs[3]);
    CHECK(logs[0] != logs[1]);
    CHECK_EQ(mgr->GetUsage(names[0]), mgr->GetUsage(names[2]));
    CHECK_EQ(mgr->GetUsage(names[1]), mgr->GetUsage(names[3]));
    std::vector<std::pair<uint64_t, uint64_t>> a, b;
    CHECK_EQ(mgr->ExportDeviceKeyOffsetPairs(names[1], a), 0);
    CHECK_EQ(mgr->ExportDeviceKeyOffsetPairs(names[3], b), 0);
    CHECK(a == b && !a.empty());
}

static void CachePersistence(EmbCacheManagerPtr& mgr)
{
    auto init = ConstantInit(4, 8, 1.0f, 0.0f);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("a", 100, 4, 8, 10), init, -1, 20, 1), 0);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("b", 100, 4, 8, 10), init, -1, 20, 1), 0);
    std::vector<uint64_t> keys = {42, 5, 1ULL << 50};
    std::vector<float> rows(keys.size() * 8);
    for (size_t i = 0; i < rows.size(); ++i) {
        rows[i] = 0.5f * (float)i;
    }
    CHECK_EQ(mgr->EmbeddingUpdate("a", keys, rows.data()), 0);
    std::vector<char> buffer;
    CHECK_EQ(mgr->Serialize("nope", buffer), 12);
    CHECK_EQ(mgr->Serialize("a", buffer), 0);
    CHECK_EQ(buffer.size(), keys.size() * (8 + 8 * 4));
    CHECK_EQ(mgr->Deserialize("b", buffer), 0);
    std::vector<float> got(rows.size());
    CHECK_EQ(mgr->EmbeddingLookup("b", keys, got.data()), 0);
    CHECK(got == rows);
    CHECK_EQ(mgr->GetUsage("b"), 3);
    std::vector<char> cut(buffer.begin(), buffer.begin() + 50);
    CHECK_EQ(mgr->Deserialize("b", cut), 13);
    std::vector<uint64_t> k;
    std::vector<std::vector<float>> emb, slots;
    CHECK_EQ(mgr->GetEmbTableInfos("a", k, emb, slots), 0);
    CHECK_EQ(k.size(), 3);
    CHECK_EQ(emb.size(), 3);
    CHECK_EQ(slots.size(), 3);
    for (size_t i = 0; i < k.size(); ++i) {
        const size_t src = std::find(keys.begin(), keys.end(), k[i]) - keys.begin();
        CHECK(src < keys.size() && emb[i].size() == 4 && slots[i].size() == 4 &&
              std::equal(emb[i].begin(), emb[i].end(), rows.begin() + src * 8) &&
              std::equal(slots[i].begin(), slots[i].end(), rows.begin() + src * 8 + 4));
    }
    CHECK_EQ(mgr->GetEmbTableInfos("a", k, emb, slots), 20);
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("c", 100, 4, 8, 10), init, -1, 20, 1), 0);
    CHECK_EQ(mgr->LoadEmbTableInfos("c", k, emb, slots), 0);
    CHECK_EQ(mgr->EmbeddingLookup("c", keys, got.data()), 0);
    CHECK(got == rows);
    auto shortSlots = slots;
    shortSlots.pop_back();
    CHECK_EQ(mgr->LoadEmbTableInfos("c", k, emb, shortSlots), 13);
    auto wrongEmb = emb;
    wrongEmb[0].push_back(1.0f);
    CHECK_EQ(mgr->LoadEmbTableInfos("c", k, wrongEmb, slots), 13);
}

// The rows a table hands out are the stream the interface's own initializer classes produce.
static void CacheRandomInit(EmbCacheManagerPtr& mgr)
{
    std::string normal = "random_normal_initializer";
    std::string truncated = "truncated_normal_initializer";
    std::vector<InitializerInfo> infos;
    infos.emplace_back(normal, 0, 8, NormalInitializerInfo(0.0f, 0.05f, 17, 1.0f));
    infos.emplace_back(truncated, 8, 8, NormalInitializerInfo(1.0f, 0.5f, 99, 0.5f));
    CHECK_EQ(mgr->CreateCacheForTable(EmbCacheInfo("rnd", 1000, 8, 16, 100), infos, -1, 200, 1), 0);
    std::vector<uint64_t> keys(20);
    std::iota(keys.begin(), keys.end(), 500);
    std::vector<float> got(keys.size() * 16);
    CHECK_EQ(mgr->EmbeddingLookup("rnd", keys, got.data()), 0);
    NormalInitializerInfo a(0.0f, 0.05f, 17, 1.0f);
    NormalInitializerInfo b(1.0f, 0.5f, 99, 0.5f);
    RandomNormalInitializer first(0, 8, a);
    TruncatedNormalInitializer second(8, 8, b);
    std::vector<float> want(got.size(), 0.0f);
    for (size_t i = 0; i < keys.size(); ++i) {
        first.GenerateData(want.data() + i * 16, 16);
        second.GenerateData(want.data() + i * 16, 16);
    }
    CHECK(got == want);
    bool bounded = true;
    for (size_t i = 0; i < keys.size(); ++i) {
        for (int c = 8; c < 16; ++c) {
            bounded = bounded && got[i * 16 + c] >= 0.5f * (1.0f - 1.0f) && got[i * 16 + c] <= 0.5f * (1.0f + 1.0f);
        }
    }
    CHECK(bounded);
    ConstantInitializer big(0, 2, 5e9f, 1.0f);  // clamped to 1e9
    float two[2] = {0, 0};
    big.GenerateData(two, 2);
    CHECK(two[0] == 1e9f && two[1] == 1e9f);
}

#define SECTION(call)                          \
    do {                                       \
        std::printf("section %s\n", #call);    \
        call;                                  \
    } while (0)

// ---- timing of the boundary, host vectors in and out (plugin_driver --bench <file>) ---------------------------------
// File: int64 header {T, B, K}, then T * B int64 ids (table after table), then K batches of distinct keys, each an
// int64 count followed by that many uint64 keys.  Prints one line per measurement:
//   bench <name> <calls> <median microseconds per round> <ids or keys per round>
#include <chrono>
#include <fstream>

static double MedianUs(std::vector<double> v)
{
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
}

static int BenchBoundaries(const char* path)
{
    std::ifstream f(path, std::ios::binary);
    int64_t head[3] = {0, 0, 0};
    f.read(reinterpret_cast<char*>(head), sizeof(head));
    const int64_t T = head[0], B = head[1], K = head[2];
    if (!f || T <= 0 || B <= 0 || K < 0) {
        std::printf("plugin_driver: bad bench file %s\n", path);
        return 2;
    }
    std::vector<int64_t> ids((size_t)(T * B));
    f.read(reinterpret_cast<char*>(ids.data()), sizeof(int64_t) * ids.size());
    std::vector<std::vector<uint64_t>> batches((size_t)K);
    for (auto& b : batches) {
        int64_t m = 0;
        f.read(reinterpret_cast<char*>(&m), sizeof(m));
        b.resize((size_t)m);
        f.read(reinterpret_cast<char*>(b.data()), sizeof(uint64_t) * b.size());
    }
    if (!f) {
        std::printf("plugin_driver: short bench file %s\n", path);
        return 2;
    }
    using Clock = std::chrono::steady_clock;
    {
        // DoEnhancedUnique as KeyProcess calls it (key_process.cpp:205-251): enhanced output, 8 shards, id counts,
        // one call per table and batch; a round is the T tables of one batch
        UniquePtr unique;
        if (g_factory->CreateUnique(unique) != 0) {
            return 2;
        }
        UniqueConf conf = EnhancedConf((uint32_t)B, 8, false, 0, true);
        conf.maxIdVal = INT64_MAX;
        if (unique->Initialize(conf) != 0) {
            return 2;
        }
        std::vector<int64_t> uniqueId((size_t)B), inBucket((size_t)B);
        std::vector<uint32_t> index((size_t)B);
        std::vector<int> idCnt((size_t)B), idCntFill((size_t)B), cntInBucket(8);
        std::vector<double> rounds;
        int64_t distinct = 0;
        for (int round = 0; round < 8; ++round) {
            const auto t0 = Clock::now();
            distinct = 0;
            for (int64_t t = 0; t < T; ++t) {
                UniqueIn in;
                in.inputIdCnt = (uint32_t)B;
                in.inputId = ids.data() + t * B;
                EnhancedUniqueOut out;
                out.uniqueId = uniqueId.data();
                out.index = index.data();
                out.uniqueIdInBucket = inBucket.data();
                out.uniqueIdCntInBucket = cntInBucket.data();
                out.idCnt = idCnt.data();
                out.idCntFill = idCntFill.data();
                if (unique->DoEnhancedUnique(in, out) != 0) {
                    return 2;
                }
                distinct += out.uniqueIdCnt;
            }
            const double us = std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
            if (round >= 3) {
                rounds.push_back(us);
            }
        }
        std::printf("bench DoEnhancedUnique %lld %.1f %lld %lld\n", (long long)T, MedianUs(rounds), (long long)(T * B),
                    (long long)distinct);
        unique->UnInitialize();
    }
    if (K > 0) {
        // GetSwapPairsAndKey2Offset as HybridMgmt calls it (hybrid_mgmt.cpp:545-560): the distinct keys of a batch in,
        // offsets and the two swap lists out; the cache (4 M slots) is full after the first batches
        EmbCacheManagerPtr mgr;
        if (g_factory->CreateEmbCacheManager(mgr) != 0) {
            return 2;
        }
        auto init = ConstantInit(4, 8, 1.0f, 0.0f);
        if (mgr->CreateCacheForTable(EmbCacheInfo("c5", 8000000, 4, 8, 4000000), init, -1, 16, 1) != 0) {
            return 2;
        }
        EmbBaseInfo info(0, 0, "c5", false, false, {});
        std::vector<double> calls;
        size_t keysPerCall = 0, swapIn = 0, swapOut = 0;
        for (int64_t k = 0; k < K; ++k) {
            std::vector<uint64_t> keys = batches[(size_t)k];   // the call rewrites its argument
            KeyOffsetPair in, out;
            const auto t0 = Clock::now();
            const int rc = mgr->GetSwapPairsAndKey2Offset(info, keys, in, out);
            const double us = std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
            if (rc != 0) {
                std::printf("plugin_driver: GetSwapPairsAndKey2Offset returned %d on bench batch %lld\n", rc, (long long)k);
                return 2;
            }
            if (k >= K - 8) {
                calls.push_back(us);
                keysPerCall = keys.size();
                swapIn = in.first.size();
                swapOut = out.first.size();
            }
        }
        std::printf("bench GetSwapPairsAndKey2Offset 1 %.1f %zu %zu %zu\n", MedianUs(calls), keysPerCall, swapIn, swapOut);
        mgr->Destroy();
    }
    std::fflush(stdout);
    return 0;
}

int main(int argc, char** argv)
{
    std::setvbuf(stdout, nullptr, _IONBF, 0);
    if (Factory::Create(g_factory) != 0 || g_factory == nullptr) {
        std::printf("plugin_driver: lib_ock_ctr_common.so could not be loaded\n");
        return 2;
    }
    if (argc >= 3 && std::strcmp(argv[1], "--bench") == 0) {
        return BenchBoundaries(argv[2]);
    }
    CHECK_EQ(g_factory->SetExternalLogFuncInner(CollectLog), 0);
    SECTION(UniqueConfCodes());
    SECTION(UniqueNormal(DataType::INT64));
    SECTION(UniqueNormal(DataType::INT32));
    SECTION(UniqueSharded(false, false));
    SECTION(UniqueSharded(true, false));
    SECTION(UniqueSharded(true, true));
    SECTION(UniqueIdLarge());
    EmbCacheManagerPtr mgr;
    CHECK_EQ(g_factory->CreateEmbCacheManager(mgr), 0);
    SECTION(CacheCreateCodes(mgr));
    SECTION(CacheRows(mgr));
    SECTION(CachePlanner(mgr));
    SECTION(CacheTwoThreads(mgr));
    SECTION(CachePersistence(mgr));
    SECTION(CacheRandomInit(mgr));
    CHECK(!g_logs.empty());  // the errors above went to the external log function
    mgr->Destroy();
    std::vector<std::string> names;
    CHECK_EQ(mgr->GetEmbTableNames(names), 0);
    CHECK(names.empty());
    std::printf("plugin_driver: %d checks, %d failures\n", g_checks, g_failures);
    std::fflush(stdout);
    return g_failures == 0 ? 0 : 1;
}
