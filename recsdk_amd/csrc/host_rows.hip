// Host-DRAM row store behind the HBM cache, its row initializers, and the device kernels that move rows between
// the two.
//
// Reference: EmbLocalTable (AccCTR embedding_cache/embedding_local_table/emb_local_table.cpp:106-335) keeps one
// malloc'd row of extEmbeddingSize floats per key behind a hash map; new rows come from a pool that background
// threads pre-fill by running every initializer over the row (address_mapper.h:72-231); initializers are
// constant / random normal / truncated normal over a column range of the row, one std::default_random_engine per
// initializer object seeded once (initializer/*/*.cpp).
// Here the rows live in ONE pinned, device-mapped arena (row index instead of address) so that swap-in and
// swap-out are two device kernels that read / write host memory over the host link, with no staging copy and no
// host memcpy threads.  The key -> row map stays on the host, like the reference's; the j-th row ever created
// receives the j-th row of the initializer stream, which is what a single refill thread produces.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <random>
#include <thread>
#include <unordered_map>
#include <vector>

#include "common.h"
#include "fileio.h"

namespace recsdk {

// limits the reference clamps to (embedding_cache/common.h:55-62)
constexpr float kMeanMax = 1e9f, kMeanMin = -1e9f, kStdMax = 100.0f, kStdMin = 0.0f;
constexpr float kConstMax = 1e9f, kConstMin = -1e9f, kInitKMax = 10000.0f, kInitKMin = -10000.0f;

inline float clampf(float v, float lo, float hi) { return v > hi ? hi : (v < lo ? lo : v); }

// One initializer over columns [start, start+len) of a row.
struct RowInit {
    int32_t kind;
    uint32_t start;
    uint32_t len;
    float value;  // constant: initK * value
    float initK;
    float minBound, maxBound;
    std::default_random_engine gen;
    std::normal_distribution<float> dist;

    explicit RowInit(const recsdk_initializer_desc_t& d) : kind(d.kind), start(d.start), len(d.len)
    {
        initK = clampf(d.init_k, kInitKMin, kInitKMax);
        if (kind == RECSDK_INIT_CONSTANT) {
            value = initK * clampf(d.value_or_mean, kConstMin, kConstMax);
        } else {
            const float mean = clampf(d.value_or_mean, kMeanMin, kMeanMax);
            const float stddev = clampf(d.stddev, kStdMin, kStdMax);
            gen = std::default_random_engine(d.seed);
            dist = std::normal_distribution<float>(mean, stddev);
            // truncated_normal_initializer.cpp:69-70, boundNum = 2 (include/embedding_cache.h:133)
            minBound = initK * (mean - 2.0f * stddev);
            maxBound = initK * (mean + 2.0f * stddev);
            value = 0.0f;
        }
    }

    void Generate(float* row)
    {
        float* p = row + start;
        if (kind == RECSDK_INIT_CONSTANT) {
            std::fill_n(p, len, value);
        } else if (kind == RECSDK_INIT_RANDOM_NORMAL) {
            for (uint32_t j = 0; j < len; ++j) {
                p[j] = initK * dist(gen);
            }
        } else {
            for (uint32_t j = 0; j < len; ++j) {
                float t = initK * dist(gen);
                while (t < minBound || t > maxBound) {
                    t = initK * dist(gen);
                }
                p[j] = t;
            }
        }
    }
};

// device row <-> host row, one 16-byte chunk per thread; hostRow / devSlot index the two row arrays
__global__ __launch_bounds__(kBlock) void k_rows_host_to_dev(const float* __restrict__ arena, int64_t hostStride,
                                                             const int64_t* __restrict__ hostRow,
                                                             float* __restrict__ cache, int64_t cacheStride,
                                                             const int64_t* __restrict__ devSlot, int64_t n,
                                                             int32_t chunksPerRow)
{
    const int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t i = q / chunksPerRow;
    const int c = (int)(q - i * chunksPerRow);
    if (i >= n) {
        return;
    }
    const float4 v = *reinterpret_cast<const float4*>(arena + hostRow[i] * hostStride + c * 4);
    *reinterpret_cast<float4*>(cache + devSlot[i] * cacheStride + c * 4) = v;
}

__global__ __launch_bounds__(kBlock) void k_rows_dev_to_host(float* __restrict__ arena, int64_t hostStride,
                                                             const int64_t* __restrict__ hostRow,
                                                             const float* __restrict__ cache, int64_t cacheStride,
                                                             const int64_t* __restrict__ devSlot, int64_t n,
                                                             int32_t chunksPerRow)
{
    const int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t i = q / chunksPerRow;
    const int c = (int)(q - i * chunksPerRow);
    if (i >= n) {
        return;
    }
    const float4 v = *reinterpret_cast<const float4*>(cache + devSlot[i] * cacheStride + c * 4);
    *reinterpret_cast<float4*>(arena + hostRow[i] * hostStride + c * 4) = v;
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_initializer {
    std::vector<RowInit> inits;
};

static int check_descs(const recsdk_initializer_desc_t* descs, int32_t n, int32_t extDim, const char* who)
{
    RECSDK_REQUIRE(n >= 0 && (n == 0 || descs != nullptr), RECSDK_ENULL, "initializer descriptors missing");
    for (int32_t k = 0; k < n; ++k) {
        RECSDK_REQUIRE(descs[k].kind >= RECSDK_INIT_CONSTANT && descs[k].kind <= RECSDK_INIT_TRUNCATED_NORMAL,
                       RECSDK_EINVAL, "Invalid Initializer Type.");
        RECSDK_REQUIRE(extDim <= 0 || (uint64_t)descs[k].start + descs[k].len <= (uint64_t)extDim, RECSDK_EINVAL,
                       "an initializer's start + len is larger than the row");
    }
    (void)who;
    return RECSDK_OK;
}

extern "C" int recsdk_initializer_create(const recsdk_initializer_desc_t* descs, int32_t n_descs,
                                         recsdk_initializer_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_initializer_create: out is NULL");
    int rc = check_descs(descs, n_descs, 0, "recsdk_initializer_create");
    if (rc != RECSDK_OK) {
        return rc;
    }
    auto* h = new recsdk_initializer();
    for (int32_t k = 0; k < n_descs; ++k) {
        h->inits.emplace_back(descs[k]);
    }
    *out = h;
    return RECSDK_OK;
}

extern "C" int recsdk_initializer_destroy(recsdk_initializer_t* h)
{
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_initializer_generate(recsdk_initializer_t* h, float* h_rows, int64_t rows, int32_t ext_dim)
{
    RECSDK_REQUIRE(h != nullptr && (rows == 0 || h_rows != nullptr), RECSDK_ENULL,
                   "recsdk_initializer_generate: NULL argument");
    for (const RowInit& ri : h->inits) {
        RECSDK_REQUIRE((uint64_t)ri.start + ri.len <= (uint64_t)ext_dim, RECSDK_EINVAL,
                       "recsdk_initializer_generate: an initializer's start + len is larger than ext_dim");
    }
    for (int64_t r = 0; r < rows; ++r) {
        for (RowInit& ri : h->inits) {
            ri.Generate(h_rows + r * ext_dim);
        }
    }
    return RECSDK_OK;
}

// ---- host row store ----------------------------------------------------------------------------------------
struct recsdk_hostrows {
    int64_t vocab = 0;
    int32_t ext = 0;
    float* arena = nullptr;      // pinned host memory, vocab * ext floats
    float* arenaDev = nullptr;   // the same memory as the device sees it
    std::unordered_map<int64_t, int64_t> map;  // key -> row
    std::vector<int64_t> freeRows;             // rows of removed keys (reused last-in first-out)
    int64_t used = 0;                          // rows handed out so far from the arena's front
    std::vector<RowInit> inits;
    // staging for row-index lists the kernels read: a small ring of pinned buffers, each guarded by an event
    static constexpr int kRing = 4;
    int64_t* stage[kRing] = {nullptr, nullptr, nullptr, nullptr};
    int64_t* stageDev[kRing] = {nullptr, nullptr, nullptr, nullptr};
    int64_t stageCap[kRing] = {0, 0, 0, 0};
    hipEvent_t stageDone[kRing] = {nullptr, nullptr, nullptr, nullptr};
    bool stageBusy[kRing] = {false, false, false, false};
    int next = 0;

    // row of `key`, created (and initialised) when absent and create is set; -1 when absent; -2 when full
    int64_t RowOf(int64_t key, bool create, bool* created)
    {
        auto it = map.find(key);
        if (it != map.end()) {
            return it->second;
        }
        if (!create) {
            return -1;
        }
        int64_t row;
        if (!freeRows.empty()) {
            row = freeRows.back();
            freeRows.pop_back();
        } else if (used < vocab) {
            row = used++;
        } else {
            return -2;
        }
        for (RowInit& ri : inits) {
            ri.Generate(arena + row * ext);
        }
        map.emplace(key, row);
        if (created != nullptr) {
            *created = true;
        }
        return row;
    }
};

extern "C" int recsdk_hostrows_destroy(recsdk_hostrows_t* h)
{
    if (h == nullptr) {
        return RECSDK_OK;
    }
    for (int k = 0; k < recsdk_hostrows::kRing; ++k) {
        if (h->stageBusy[k]) {
            (void)hipEventSynchronize(h->stageDone[k]);
        }
        if (h->stageDone[k] != nullptr) {
            (void)hipEventDestroy(h->stageDone[k]);
        }
        if (h->stage[k] != nullptr) {
            (void)hipHostFree(h->stage[k]);
        }
    }
    if (h->arena != nullptr) {
        (void)hipHostFree(h->arena);
    }
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_create(int64_t vocab_size, int32_t ext_dim, const recsdk_initializer_desc_t* descs,
                                      int32_t n_descs, recsdk_hostrows_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_hostrows_create: out is NULL");
    RECSDK_REQUIRE(vocab_size > 0 && ext_dim > 0 && ext_dim % 4 == 0, RECSDK_EINVAL,
                   "recsdk_hostrows_create: vocab_size must be positive and ext_dim a positive multiple of 4");
    int rc = check_descs(descs, n_descs, ext_dim, "recsdk_hostrows_create");
    if (rc != RECSDK_OK) {
        return rc;
    }
    auto* h = new recsdk_hostrows();
    h->vocab = vocab_size;
    h->ext = ext_dim;
    for (int32_t k = 0; k < n_descs; ++k) {
        h->inits.emplace_back(descs[k]);
    }
    const size_t bytes = sizeof(float) * (size_t)vocab_size * (size_t)ext_dim;
    bool ok = hipHostMalloc(reinterpret_cast<void**>(&h->arena), bytes, hipHostMallocMapped) == hipSuccess &&
              hipHostGetDevicePointer(reinterpret_cast<void**>(&h->arenaDev), h->arena, 0) == hipSuccess;
    for (int k = 0; ok && k < recsdk_hostrows::kRing; ++k) {
        ok = hipEventCreateWithFlags(&h->stageDone[k], hipEventDisableTiming) == hipSuccess;
    }
    if (!ok) {
        (void)hipGetLastError();
        recsdk_hostrows_destroy(h);
        set_error("recsdk_hostrows_create: pinned host allocation failed");
        return RECSDK_ENOMEM;
    }
    *out = h;
    return RECSDK_OK;
}

// parallel row copies over `threads` host threads (contiguous index ranges, like the reference's split)
template <typename F>
static void for_rows(int64_t n, int32_t threads, F&& body)
{
    if (threads <= 1 || n < 4096) {
        for (int64_t i = 0; i < n; ++i) {
            body(i);
        }
        return;
    }
    std::vector<std::thread> pool;
    const int64_t per = (n + threads - 1) / threads;
    for (int32_t t = 0; t < threads; ++t) {
        const int64_t b = std::min<int64_t>(n, per * t);
        const int64_t e = std::min<int64_t>(n, b + per);
        pool.emplace_back([=, &body]() {
            for (int64_t i = b; i < e; ++i) {
                body(i);
            }
        });
    }
    for (auto& t : pool) {
        t.join();
    }
}

static int resolve_rows(recsdk_hostrows* h, const int64_t* keys, int64_t n, bool create, int64_t* rows,
                        const char* who)
{
    for (int64_t i = 0; i < n; ++i) {
        rows[i] = h->RowOf(keys[i], create, nullptr);
        if (rows[i] == -2) {
            set_error("%s: host vocabulary size is too small", who);
            return RECSDK_ECAPACITY;
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_find_rows(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, int32_t create,
                                         int64_t* h_rows)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_rows != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_find_rows: NULL argument");
    return resolve_rows(h, h_keys, n, create != 0, h_rows, "recsdk_hostrows_find_rows");
}

extern "C" int recsdk_hostrows_gather(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, float* h_dst,
                                      int32_t threads)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_dst != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_gather: NULL argument");
    std::vector<int64_t> rows(n);
    int rc = resolve_rows(h, h_keys, n, true, rows.data(), "recsdk_hostrows_gather");
    if (rc != RECSDK_OK) {
        return rc;
    }
    const size_t rb = sizeof(float) * h->ext;
    for_rows(n, threads, [&](int64_t i) { std::memcpy(h_dst + i * h->ext, h->arena + rows[i] * h->ext, rb); });
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_scatter(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const float* h_src,
                                       int32_t threads)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_src != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_scatter: NULL argument");
    std::vector<int64_t> rows(n);
    int rc = resolve_rows(h, h_keys, n, true, rows.data(), "recsdk_hostrows_scatter");
    if (rc != RECSDK_OK) {
        return rc;
    }
    const size_t rb = sizeof(float) * h->ext;
    // rows of one key written twice keep the later copy, as a sequential loop would
    for_rows(n, 1, [&](int64_t i) { std::memcpy(h->arena + rows[i] * h->ext, h_src + i * h->ext, rb); });
    (void)threads;
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_gather_and_remove(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, float* h_dst)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_dst != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_gather_and_remove: NULL argument");
    const size_t rb = sizeof(float) * h->ext;
    for (int64_t i = 0; i < n; ++i) {
        auto it = h->map.find(h_keys[i]);
        if (it != h->map.end()) {
            std::memcpy(h_dst + i * h->ext, h->arena + it->second * h->ext, rb);
            h->freeRows.push_back(it->second);
            h->map.erase(it);
        } else {
            // a key that has no row gets fresh initial values and is not stored (emb_local_table.cpp:247-253)
            for (RowInit& ri : h->inits) {
                ri.Generate(h_dst + i * h->ext);
            }
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_remove(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || h_keys != nullptr), RECSDK_ENULL, "recsdk_hostrows_remove: NULL argument");
    for (int64_t i = 0; i < n; ++i) {
        auto it = h->map.find(h_keys[i]);
        if (it != h->map.end()) {
            h->freeRows.push_back(it->second);
            h->map.erase(it);
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_size(recsdk_hostrows_t* h, int64_t* h_live)
{
    RECSDK_REQUIRE(h != nullptr && h_live != nullptr, RECSDK_ENULL, "recsdk_hostrows_size: NULL argument");
    *h_live = (int64_t)h->map.size();
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_export(recsdk_hostrows_t* h, int64_t* h_keys, float* h_rows, int64_t cap,
                                      int64_t* h_count)
{
    RECSDK_REQUIRE(h != nullptr && h_count != nullptr, RECSDK_ENULL, "recsdk_hostrows_export: NULL argument");
    *h_count = (int64_t)h->map.size();
    if (h_keys == nullptr || h_rows == nullptr || cap < *h_count) {
        return RECSDK_OK;
    }
    std::vector<int64_t> keys;
    keys.reserve(h->map.size());
    for (const auto& kv : h->map) {
        keys.push_back(kv.first);
    }
    std::sort(keys.begin(), keys.end());
    for (size_t i = 0; i < keys.size(); ++i) {
        h_keys[i] = keys[i];
        std::memcpy(h_rows + i * h->ext, h->arena + h->map[keys[i]] * h->ext, sizeof(float) * h->ext);
    }
    return RECSDK_OK;
}

// ---- serialized forms -----------------------------------------------------------------------------------

static std::vector<int64_t> sorted_keys(recsdk_hostrows* h)
{
    std::vector<int64_t> keys;
    keys.reserve(h->map.size());
    for (const auto& kv : h->map) {
        keys.push_back(kv.first);
    }
    std::sort(keys.begin(), keys.end());
    return keys;
}

extern "C" int recsdk_hostrows_serialize(recsdk_hostrows_t* h, char* h_buf, int64_t cap, int64_t* h_bytes)
{
    RECSDK_REQUIRE(h != nullptr && h_bytes != nullptr, RECSDK_ENULL, "recsdk_hostrows_serialize: NULL argument");
    const size_t rec = sizeof(uint64_t) + sizeof(float) * h->ext;
    *h_bytes = (int64_t)(rec * h->map.size());
    if (h_buf == nullptr || cap < *h_bytes) {
        return RECSDK_OK;
    }
    char* p = h_buf;
    for (int64_t key : sorted_keys(h)) {
        const uint64_t k = (uint64_t)key;
        std::memcpy(p, &k, sizeof(k));
        std::memcpy(p + sizeof(k), h->arena + h->map[key] * h->ext, sizeof(float) * h->ext);
        p += rec;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_deserialize(recsdk_hostrows_t* h, const char* h_buf, int64_t bytes)
{
    RECSDK_REQUIRE(h != nullptr && (bytes == 0 || h_buf != nullptr), RECSDK_ENULL,
                   "recsdk_hostrows_deserialize: NULL argument");
    const int64_t rec = (int64_t)(sizeof(uint64_t) + sizeof(float) * h->ext);
    int64_t i = 0;
    while (i < bytes) {
        if (i + (int64_t)sizeof(uint64_t) > bytes) {
            set_error("get data failed!");
            return RECSDK_EINVAL;
        }
        uint64_t k;
        std::memcpy(&k, h_buf + i, sizeof(k));
        // the row is found or created (a created row takes its initial values first, as FindAndPutIfNotFound does)
        const int64_t row = h->RowOf((int64_t)k, true, nullptr);
        if (row == -2) {
            set_error("recsdk_hostrows_deserialize: host vocabulary size is too small");
            return RECSDK_ECAPACITY;
        }
        if (i + rec > bytes) {
            // a cut record: the floats that are there are taken, then the reference reports failure
            const int64_t have = (bytes - i - (int64_t)sizeof(uint64_t)) / (int64_t)sizeof(float);
            std::memcpy(h->arena + row * h->ext, h_buf + i + sizeof(uint64_t), sizeof(float) * have);
            set_error("get data failed!");
            return RECSDK_EINVAL;
        }
        std::memcpy(h->arena + row * h->ext, h_buf + i + sizeof(uint64_t), sizeof(float) * h->ext);
        i += rec;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_save(recsdk_hostrows_t* h, const char* prefix, int32_t emb_dim, int32_t optim_num)
{
    RECSDK_REQUIRE(h != nullptr && prefix != nullptr, RECSDK_ENULL, "recsdk_hostrows_save: NULL argument");
    RECSDK_REQUIRE(emb_dim > 0 && optim_num >= 0 && optim_num <= 2 && (int64_t)emb_dim * (1 + optim_num) <= h->ext,
                   RECSDK_EINVAL, "recsdk_hostrows_save: emb_dim * (1 + optim_num) exceeds the row width");
    const std::vector<int64_t> keys = sorted_keys(h);
    const int64_t count = (int64_t)keys.size();
    const std::string base(prefix);
    int rc = write_file(base + "/key/slice.data", keys.data(), sizeof(int64_t) * keys.size());
    const int64_t keyAttr[2] = {(int64_t)sizeof(int64_t), count};
    if (rc == RECSDK_OK) {
        rc = write_file(base + "/key/slice.attribute", keyAttr, sizeof(keyAttr));
    }
    const int64_t rowAttr[3] = {(int64_t)sizeof(float), count, emb_dim};
    // embedding at float 0 of the row, momentum1 at embDim, momentum2 at optimNum * embDim
    const char* dirs[3] = {"/embedding", "/momentum1", "/momentum2"};
    const int64_t at[3] = {0, emb_dim, (int64_t)optim_num * emb_dim};
    std::vector<float> packed((size_t)count * emb_dim);
    for (int part = 0; part <= optim_num && rc == RECSDK_OK; ++part) {
        for (int64_t i = 0; i < count; ++i) {
            std::memcpy(packed.data() + i * emb_dim, h->arena + h->map[keys[i]] * h->ext + at[part],
                        sizeof(float) * emb_dim);
        }
        rc = write_file(base + dirs[part] + "/slice.data", packed.data(), sizeof(float) * packed.size());
        if (rc == RECSDK_OK) {
            rc = write_file(base + dirs[part] + "/slice.attribute", rowAttr, sizeof(rowAttr));
        }
    }
    return rc;
}

static int read_attribute(const std::string& path, int count, std::vector<int64_t>* out)
{
    std::vector<char> raw;
    const int rc = read_file(path, 1, &raw);
    if (rc != RECSDK_OK) {
        return rc;
    }
    if (raw.size() < sizeof(int64_t) * (size_t)count) {
        set_error("Read key attribute file error, expect read bytes:%zu, actual read bytes:%zu, file:%s",
                  sizeof(int64_t) * (size_t)count, raw.size(), path.c_str());
        return RECSDK_EIO;
    }
    out->resize((size_t)count);
    std::memcpy(out->data(), raw.data(), sizeof(int64_t) * (size_t)count);
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_load(recsdk_hostrows_t* h, const char* prefix, int32_t emb_dim, int32_t optim_num)
{
    RECSDK_REQUIRE(h != nullptr && prefix != nullptr, RECSDK_ENULL, "recsdk_hostrows_load: NULL argument");
    RECSDK_REQUIRE(emb_dim > 0 && optim_num >= 0 && optim_num <= 2 && (int64_t)emb_dim * (1 + optim_num) <= h->ext,
                   RECSDK_EINVAL, "recsdk_hostrows_load: emb_dim * (1 + optim_num) exceeds the row width");
    const std::string base(prefix);
    std::vector<int64_t> attr;
    int rc = read_attribute(base + "/key/slice.attribute", 2, &attr);
    if (rc != RECSDK_OK) {
        return rc;
    }
    if (attr[1] < 0 || attr[1] > 1000000000LL) {
        set_error("Read key attribute file error, keys count is invalid:%ld, file:%s.", (long)attr[1],
                  (base + "/key/slice.attribute").c_str());
        return RECSDK_EINVAL;
    }
    std::vector<char> rawKeys;
    rc = read_file(base + "/key/slice.data", 1, &rawKeys);
    if (rc != RECSDK_OK) {
        return rc;
    }
    if (rawKeys.size() % sizeof(int64_t) != 0 || (int64_t)(rawKeys.size() / sizeof(int64_t)) != attr[1]) {
        set_error("Key file bytes is not an integer multiple of type int64_t, key file:%s",
                  (base + "/key/slice.data").c_str());
        return RECSDK_EINVAL;
    }
    const int64_t count = attr[1];
    const int64_t* keys = reinterpret_cast<const int64_t*>(rawKeys.data());
    const char* dirs[3] = {"/embedding", "/momentum1", "/momentum2"};
    const int64_t at[3] = {0, emb_dim, (int64_t)optim_num * emb_dim};
    std::vector<std::vector<char>> parts((size_t)optim_num + 1);
    for (int part = 0; part <= optim_num; ++part) {
        const std::string dataFile = base + dirs[part] + "/slice.data";
        rc = read_attribute(base + dirs[part] + "/slice.attribute", 3, &attr);
        if (rc != RECSDK_OK) {
            return rc;
        }
        if (attr[2] != emb_dim) {
            set_error("Embedding or momentum dim error, load data dim from attribute:%ld, current table dim:%d, file:%s.",
                      (long)attr[2], emb_dim, (base + dirs[part] + "/slice.attribute").c_str());
            return RECSDK_EINVAL;
        }
        rc = read_file(dataFile, 1, &parts[part]);
        if (rc != RECSDK_OK) {
            return rc;
        }
        if ((int64_t)parts[part].size() != count * emb_dim * (int64_t)sizeof(float)) {
            set_error("Read data to file error, expect read bytes:%ld, actual read bytes:%zu, file:%s",
                      (long)(count * emb_dim * (int64_t)sizeof(float)), parts[part].size(), dataFile.c_str());
            return RECSDK_EIO;
        }
    }
    // InsertOrAssign: the row of each key becomes [embedding | momentum1 | momentum2]
    for (int64_t i = 0; i < count; ++i) {
        const int64_t row = h->RowOf(keys[i], true, nullptr);
        if (row == -2) {
            set_error("recsdk_hostrows_load: host vocabulary size is too small");
            return RECSDK_ECAPACITY;
        }
        for (int part = 0; part <= optim_num; ++part) {
            std::memcpy(h->arena + row * h->ext + at[part], parts[part].data() + i * emb_dim * sizeof(float),
                        sizeof(float) * emb_dim);
        }
    }
    return RECSDK_OK;
}

// pinned staging for 2n row indices (host rows, then nothing else); waits for the slot's previous user
static int stage_acquire(recsdk_hostrows* h, int64_t n, int* slot)
{
    const int k = h->next;
    h->next = (h->next + 1) % recsdk_hostrows::kRing;
    if (h->stageBusy[k]) {
        RECSDK_HIP_TRY(hipEventSynchronize(h->stageDone[k]));
        h->stageBusy[k] = false;
    }
    if (h->stageCap[k] < n) {
        if (h->stage[k] != nullptr) {
            RECSDK_HIP_TRY(hipHostFree(h->stage[k]));
            h->stage[k] = nullptr;
            h->stageCap[k] = 0;
        }
        const int64_t cap = std::max<int64_t>(n, 4096);
        RECSDK_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&h->stage[k]), sizeof(int64_t) * cap, hipHostMallocMapped));
        RECSDK_HIP_TRY(hipHostGetDevicePointer(reinterpret_cast<void**>(&h->stageDev[k]), h->stage[k], 0));
        h->stageCap[k] = cap;
    }
    *slot = k;
    return RECSDK_OK;
}

static int swap_common(recsdk_hostrows* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots, float* d_cache,
                       int64_t cache_stride, bool toHost, hipStream_t s, const char* who)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "host row store handle is NULL");
    if (n <= 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(h_keys != nullptr && d_slots != nullptr && d_cache != nullptr, RECSDK_ENULL, "NULL argument");
    RECSDK_REQUIRE(cache_stride >= h->ext && cache_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(d_cache) % 16) == 0,
                   RECSDK_EINVAL, "cache rows must be 16-byte aligned, their stride a multiple of 4 and >= ext_dim");
    int k = 0;
    int rc = stage_acquire(h, n, &k);
    if (rc != RECSDK_OK) {
        return rc;
    }
    rc = resolve_rows(h, h_keys, n, true, h->stage[k], who);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const int32_t cpr = h->ext / 4;
    const unsigned grid = (unsigned)cdiv(n * cpr, kBlock);
    if (toHost) {
        RECSDK_LAUNCH(k_rows_dev_to_host, dim3(grid), dim3(kBlock), s, h->arenaDev, (int64_t)h->ext, h->stageDev[k],
                      d_cache, cache_stride, d_slots, n, cpr);
    } else {
        RECSDK_LAUNCH(k_rows_host_to_dev, dim3(grid), dim3(kBlock), s, h->arenaDev, (int64_t)h->ext, h->stageDev[k],
                      d_cache, cache_stride, d_slots, n, cpr);
    }
    RECSDK_HIP_TRY(hipEventRecord(h->stageDone[k], s));
    h->stageBusy[k] = true;
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_swap_out(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots,
                                        const float* d_cache, int64_t cache_stride, void* stream)
{
    return swap_common(h, h_keys, n, d_slots, const_cast<float*>(d_cache), cache_stride, true,
                       static_cast<hipStream_t>(stream), "recsdk_hostrows_swap_out");
}

extern "C" int recsdk_hostrows_swap_in(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots,
                                       float* d_cache, int64_t cache_stride, void* stream)
{
    return swap_common(h, h_keys, n, d_slots, d_cache, cache_stride, false, static_cast<hipStream_t>(stream),
                       "recsdk_hostrows_swap_in");
}
