// Re-ordered views of a unique run: the distinct keys grouped by shard (with optional fixed-size padding per shard)
// and the distinct keys in ascending order, each with the matching inverse index.
//
// Both are a stable sort of the first-occurrence-ordered distinct keys by a small sort key, followed by a scatter:
//   sharded : sort key = shard of the key              (ock::ctr::Unique::DoEnhancedUnique, unique_func.h:271-329,
//             TileAndFill unique_func.h:400-453, GetFillOffset unique_func.cpp:173-180)
//   sorted  : sort key = the key itself (sign flipped) (hybrid::UniqueParallel, unique.cpp:55-118)
// The number of distinct keys lives on the device, so the sort runs over the n input positions with the surplus
// entries keyed past every real one.
#include <string.h>

#include <hip/hip_runtime.h>

#include "common.h"
#include "dedup.h"
#include "radix_sort.h"

namespace recsdk {

__device__ __forceinline__ uint32_t shard_of(int64_t key, int32_t shards, int32_t useMask)
{
    // the reference groups by the unsigned value: `val % groupCount` on uint64_t, or `val & (shards-1)`
    const uint64_t v = (uint64_t)key;
    return useMask ? (uint32_t)(v & (uint64_t)(shards - 1)) : (uint32_t)(v % (uint64_t)shards);
}

__global__ __launch_bounds__(kBlock) void k_regroup_shard_keys(const int64_t* __restrict__ uniq,
                                                               const int64_t* __restrict__ total, int64_t n,
                                                               int32_t shards, int32_t useMask,
                                                               uint32_t* __restrict__ sid, int32_t* __restrict__ rank)
{
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= n) {
        return;
    }
    sid[r] = (r < total[0]) ? shard_of(uniq[r], shards, useMask) : (uint32_t)shards;
    rank[r] = (int32_t)r;
}

// Sort keys of the distinct keys (sign bit flipped: unsigned order = signed order) and, per block, the smallest and
// the largest of them, so that the host can leave the bits all keys share out of the sort.
__global__ __launch_bounds__(kBlock) void k_regroup_sort_keys(const int64_t* __restrict__ uniq,
                                                              const int64_t* __restrict__ total, int64_t n,
                                                              uint64_t* __restrict__ skey, int32_t* __restrict__ rank,
                                                              uint64_t* __restrict__ blockMin,
                                                              uint64_t* __restrict__ blockMax)
{
    __shared__ uint64_t sMin[kBlock / kWave];
    __shared__ uint64_t sMax[kBlock / kWave];
    const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    uint64_t lo = ~0ull;
    uint64_t hi = 0;
    if (r < n) {
        const bool live = r < total[0];
        const uint64_t k = live ? ((uint64_t)uniq[r] ^ 0x8000000000000000ull) : ~0ull;
        skey[r] = k;
        rank[r] = (int32_t)r;
        if (live) {
            lo = k;
            hi = k;
        }
    }
    for (int d = kWave / 2; d > 0; d >>= 1) {
        const uint64_t olo = __shfl_xor(lo, d, kWave);
        const uint64_t ohi = __shfl_xor(hi, d, kWave);
        lo = olo < lo ? olo : lo;
        hi = ohi > hi ? ohi : hi;
    }
    if (lane_id() == 0) {
        sMin[threadIdx.x >> 6] = lo;
        sMax[threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kBlock / kWave; ++w) {
            lo = sMin[w] < lo ? sMin[w] : lo;
            hi = sMax[w] > hi ? sMax[w] : hi;
        }
        blockMin[blockIdx.x] = lo;
        blockMax[blockIdx.x] = hi;
    }
}

// single block: out = {smallest sort key, largest sort key, number of distinct keys}
__global__ __launch_bounds__(kBlock) void k_regroup_key_range(const uint64_t* __restrict__ blockMin,
                                                              const uint64_t* __restrict__ blockMax, int64_t blocks,
                                                              const int64_t* __restrict__ total,
                                                              uint64_t* __restrict__ out)
{
    __shared__ uint64_t sMin[kBlock / kWave];
    __shared__ uint64_t sMax[kBlock / kWave];
    uint64_t lo = ~0ull;
    uint64_t hi = 0;
    for (int64_t b = threadIdx.x; b < blocks; b += kBlock) {
        lo = blockMin[b] < lo ? blockMin[b] : lo;
        hi = blockMax[b] > hi ? blockMax[b] : hi;
    }
    for (int d = kWave / 2; d > 0; d >>= 1) {
        const uint64_t olo = __shfl_xor(lo, d, kWave);
        const uint64_t ohi = __shfl_xor(hi, d, kWave);
        lo = olo < lo ? olo : lo;
        hi = ohi > hi ? ohi : hi;
    }
    if (lane_id() == 0) {
        sMin[threadIdx.x >> 6] = lo;
        sMax[threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kBlock / kWave; ++w) {
            lo = sMin[w] < lo ? sMin[w] : lo;
            hi = sMax[w] > hi ? sMax[w] : hi;
        }
        out[0] = lo;
        out[1] = hi;
        out[2] = (uint64_t)total[0];
    }
}

// start[s] = first sorted position whose shard is >= s, for s in [0, shards]; cnt[s] = start[s+1] - start[s].
// `flag` is raised when a shard holds more than paddingSize keys (paddingSize > 0).
__global__ __launch_bounds__(kBlock) void k_regroup_shard_bounds(const uint32_t* __restrict__ sidSorted,
                                                                 const int64_t* __restrict__ total, int32_t shards,
                                                                 int32_t paddingSize, int32_t* __restrict__ start,
                                                                 int32_t* __restrict__ cnt, int32_t* __restrict__ flag)
{
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s > shards) {
        return;
    }
    const int64_t U = total[0];
    auto lower = [&](uint32_t want) {
        int64_t lo = 0;
        int64_t hi = U;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (sidSorted[mid] < want) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        return lo;
    };
    const int64_t b = lower((uint32_t)s);
    start[s] = (int32_t)b;
    if (s < shards) {
        const int64_t e = lower((uint32_t)s + 1);
        cnt[s] = (int32_t)(e - b);
        if (paddingSize > 0 && e - b > paddingSize) {
            flag[0] = 1;
        }
    }
}

__global__ __launch_bounds__(kBlock) void k_regroup_fill(int64_t* __restrict__ ids, int32_t* __restrict__ cntFill,
                                                         int64_t m, int64_t paddingVal)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= m) {
        return;
    }
    ids[j] = paddingVal;
    if (cntFill != nullptr) {
        cntFill[j] = 0;
    }
}

// sorted position j -> output places; newPos[rank] = where the key's inverse index now points
__global__ __launch_bounds__(kBlock) void k_regroup_shard_scatter(
    const int64_t* __restrict__ uniq, const uint32_t* __restrict__ ucount, const int64_t* __restrict__ total,
    const uint32_t* __restrict__ sidSorted, const int32_t* __restrict__ order, const int32_t* __restrict__ start,
    const int32_t* __restrict__ flag, int32_t paddingSize, int64_t* __restrict__ uniqueId,
    int64_t* __restrict__ inBucket, int32_t* __restrict__ idCnt, int32_t* __restrict__ idCntFill,
    int32_t* __restrict__ newPos)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= total[0] || flag[0] != 0) {
        return;
    }
    const int32_t r = order[j];
    const uint32_t s = sidSorted[j];
    const int64_t key = uniq[r];
    const int64_t dest = paddingSize > 0 ? (int64_t)s * paddingSize + (j - start[s]) : j;
    uniqueId[dest] = key;
    newPos[r] = (int32_t)dest;
    if (inBucket != nullptr) {
        inBucket[j] = key;
    }
    if (idCnt != nullptr) {
        idCnt[j] = (int32_t)ucount[r];
    }
    if (idCntFill != nullptr) {
        idCntFill[dest] = (int32_t)ucount[r];
    }
}

__global__ __launch_bounds__(kBlock) void k_regroup_sorted_scatter(const uint64_t* __restrict__ skeySorted,
                                                                   const int32_t* __restrict__ order,
                                                                   const int64_t* __restrict__ total,
                                                                   int64_t* __restrict__ sorted,
                                                                   int32_t* __restrict__ newPos)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= total[0]) {
        return;
    }
    sorted[j] = (int64_t)(skeySorted[j] ^ 0x8000000000000000ull);
    newPos[order[j]] = (int32_t)j;
}

template <typename OUT>
__global__ __launch_bounds__(kBlock) void k_regroup_index(const int32_t* __restrict__ grank,
                                                          const int32_t* __restrict__ newPos,
                                                          const int32_t* __restrict__ flag, int64_t n,
                                                          OUT* __restrict__ index)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n || (flag != nullptr && flag[0] != 0)) {
        return;
    }
    const int32_t r = grank[i];
    index[i] = r >= 0 ? (OUT)newPos[r] : (OUT)-1;
}

}  // namespace recsdk

using namespace recsdk;

// The sorts here (shard ids of up to 17 bits over every position; the distinct 64-bit keys over the bits in which
// they differ) are the library's own one-sweep radix sort (radix_sort.h).
struct recsdk_regroup {
    int64_t maxKeys = 0;
    uint64_t* keyA = nullptr;  // sort keys (uint32 shard ids use the low half of the allocation)
    uint64_t* keyB = nullptr;
    int32_t* valA = nullptr;
    int32_t* valB = nullptr;
    int32_t* newPos = nullptr;
    int32_t* start = nullptr;  // [kMaxShards + 1]
    int32_t* flag = nullptr;
    uint64_t* range = nullptr;  // per block of distinct keys: smallest, largest sort key; then {min, max, distinct}
    void* tmp = nullptr;       // the radix sort's workspace, cut up in sortWs
    rsort::Workspace sortWs;
};

static constexpr int32_t kMaxShards = 65536;

extern "C" int recsdk_regroup_destroy(recsdk_regroup_t* g)
{
    if (g == nullptr) {
        return RECSDK_OK;
    }
    void* ptrs[] = {g->keyA, g->keyB, g->valA, g->valB, g->newPos, g->start, g->flag, g->range, g->tmp};
    for (void* p : ptrs) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    delete g;
    return RECSDK_OK;
}

extern "C" int recsdk_regroup_create(int64_t max_keys, recsdk_regroup_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_regroup_create: out is NULL");
    RECSDK_REQUIRE(max_keys > 0 && max_keys <= (int64_t(1) << 28), RECSDK_EINVAL,
                   "recsdk_regroup_create: max_keys must be in (0, 2^28]");
    auto* g = new recsdk_regroup();
    g->maxKeys = max_keys;
    bool ok = true;
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes) != hipSuccess) {
            ok = false;
        }
    };
    alloc(&g->keyA, sizeof(uint64_t) * max_keys);
    alloc(&g->keyB, sizeof(uint64_t) * max_keys);
    alloc(&g->valA, sizeof(int32_t) * max_keys);
    alloc(&g->valB, sizeof(int32_t) * max_keys);
    alloc(&g->newPos, sizeof(int32_t) * max_keys);
    alloc(&g->start, sizeof(int32_t) * (kMaxShards + 2));
    alloc(&g->flag, sizeof(int32_t) * 4);
    alloc(&g->range, sizeof(uint64_t) * (2 * (size_t)cdiv(max_keys, kBlock) + 4));
    alloc(&g->tmp, rsort::workspace_bytes(max_keys, sizeof(uint64_t)));
    if (!ok) {
        (void)hipGetLastError();
        recsdk_regroup_destroy(g);
        recsdk::set_error("recsdk_regroup_create: out of device memory");
        return RECSDK_ENOMEM;
    }
    g->sortWs = rsort::workspace_carve(g->tmp, max_keys, sizeof(uint64_t));
    *out = g;
    return RECSDK_OK;
}

static int regroup_check(const recsdk_regroup* g, const UniqueView* v, const char* who)
{
    RECSDK_REQUIRE(v->T == 1, RECSDK_EINVAL, "the unique run must cover one table (offsets of length 2)");
    RECSDK_REQUIRE(v->n <= g->maxKeys, RECSDK_ECAPACITY, "the unique run is larger than the regroup workspace");
    (void)who;
    return RECSDK_OK;
}

extern "C" int recsdk_unique_sharded(recsdk_regroup_t* g, recsdk_unique_t* u, int32_t shards, int32_t use_mask,
                                     int32_t padding_size, int64_t padding_val, int64_t* d_unique_id,
                                     uint32_t* d_index, int64_t* d_unique_in_bucket, int32_t* d_cnt_in_bucket,
                                     int32_t* d_id_cnt, int32_t* d_id_cnt_fill, void* stream,
                                     int32_t* h_unique_id_cnt)
{
    RECSDK_REQUIRE(g != nullptr && u != nullptr && d_unique_id != nullptr && d_index != nullptr &&
                       d_cnt_in_bucket != nullptr && h_unique_id_cnt != nullptr,
                   RECSDK_ENULL, "recsdk_unique_sharded: NULL argument");
    RECSDK_REQUIRE(shards > 0 && shards <= kMaxShards, RECSDK_EINVAL,
                   "recsdk_unique_sharded: shards must be in [1, 65536]");
    RECSDK_REQUIRE(!use_mask || (shards & (shards - 1)) == 0, RECSDK_EINVAL,
                   "recsdk_unique_sharded: the mask form needs a power-of-two shard count");
    RECSDK_REQUIRE(padding_size >= 0 && (int64_t)padding_size * shards <= (int64_t(1) << 30), RECSDK_EINVAL,
                   "recsdk_unique_sharded: padding_size * shards out of range");
    const UniqueView* v = recsdk_unique_view(u);
    int rc = regroup_check(g, v, "recsdk_unique_sharded");
    if (rc != RECSDK_OK) {
        return rc;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t n = v->n;
    const int64_t padded = (int64_t)padding_size * shards;
    uint32_t* sidA = reinterpret_cast<uint32_t*>(g->keyA);
    uint32_t* sidB = reinterpret_cast<uint32_t*>(g->keyB);
    RECSDK_HIP_TRY(hipMemsetAsync(g->flag, 0, sizeof(int32_t) * 4, s));
    if (padded > 0) {
        RECSDK_LAUNCH(k_regroup_fill, dim3((unsigned)cdiv(padded, kBlock)), dim3(kBlock), s, d_unique_id,
                      d_id_cnt_fill, padded, padding_val);
    }
    if (n > 0) {
        const unsigned grid = (unsigned)cdiv(n, kBlock);
        RECSDK_LAUNCH(k_regroup_shard_keys, dim3(grid), dim3(kBlock), s, v->uniq, v->total, n, shards, use_mask, sidA,
                      g->valA);
        int bits = 1;
        while ((1u << bits) <= (uint32_t)shards) {
            ++bits;
        }
        rc = rsort::sort_pairs<uint32_t>(g->sortWs, "sort_positions_by_shard", sidA, sidB,
                                         reinterpret_cast<const uint32_t*>(g->valA), reinterpret_cast<uint32_t*>(g->valB),
                                         n, bits, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    // with no keys the bounds kernel still writes zero counts (total[0] is 0 after an empty run)
    RECSDK_LAUNCH(k_regroup_shard_bounds, dim3((unsigned)cdiv(shards + 1, kBlock)), dim3(kBlock), s, sidB, v->total,
                  shards, padding_size, g->start, d_cnt_in_bucket, g->flag);
    if (n > 0) {
        const unsigned grid = (unsigned)cdiv(n, kBlock);
        RECSDK_HIP_TRY(recsdk_unique_wait_counts(v, s));
        RECSDK_LAUNCH(k_regroup_shard_scatter, dim3(grid), dim3(kBlock), s, v->uniq, v->ucount, v->total, sidB,
                      g->valB, g->start, g->flag, padding_size, d_unique_id, d_unique_in_bucket, d_id_cnt,
                      d_id_cnt_fill, g->newPos);
        RECSDK_LAUNCH(k_regroup_index<uint32_t>, dim3(grid), dim3(kBlock), s, v->grank, g->newPos, g->flag, n,
                      d_index);
    }
    int32_t hflag = 0;
    int64_t htotal = 0;
    RECSDK_HIP_TRY(hipMemcpyAsync(&hflag, g->flag, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(&htotal, v->total, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    RECSDK_REQUIRE(hflag == 0, RECSDK_ECAPACITY,
                   "recsdk_unique_sharded: a shard holds more distinct keys than padding_size");
    *h_unique_id_cnt = padding_size > 0 ? (int32_t)padded : (int32_t)htotal;
    return RECSDK_OK;
}

extern "C" int recsdk_unique_sorted(recsdk_regroup_t* g, recsdk_unique_t* u, int64_t* d_sorted, int64_t* d_inverse,
                                    void* stream)
{
    RECSDK_REQUIRE(g != nullptr && u != nullptr && d_sorted != nullptr && d_inverse != nullptr, RECSDK_ENULL,
                   "recsdk_unique_sorted: NULL argument");
    const UniqueView* v = recsdk_unique_view(u);
    int rc = regroup_check(g, v, "recsdk_unique_sorted");
    if (rc != RECSDK_OK) {
        return rc;
    }
    const int64_t n = v->n;
    if (n == 0) {
        return RECSDK_OK;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned grid = (unsigned)cdiv(n, kBlock);
    uint64_t* blockMin = g->range;
    uint64_t* blockMax = g->range + grid;
    uint64_t* range = g->range + 2 * (size_t)grid;
    RECSDK_LAUNCH(k_regroup_sort_keys, dim3(grid), dim3(kBlock), s, v->uniq, v->total, n, g->keyA, g->valA, blockMin,
                  blockMax);
    RECSDK_LAUNCH(k_regroup_key_range, dim3(1), dim3(kBlock), s, blockMin, blockMax, (int64_t)grid, v->total, range);
    // The sort covers the distinct keys only, over the bits in which they differ (ids below 2^32 need half of the
    // passes of a 64-bit sort), so the host has to know both: one small copy and a wait.  The caller needs the number
    // of distinct keys to size its result anyway.
    uint64_t h[3] = {0, 0, 0};
    RECSDK_HIP_TRY(hipMemcpyAsync(h, range, sizeof(h), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    const size_t distinct = (size_t)h[2];
    if (distinct > 0) {
        const uint64_t diff = h[0] ^ h[1];
        const int endBit = diff == 0 ? 1 : 64 - __builtin_clzll(diff);
        rc = rsort::sort_pairs<uint64_t>(g->sortWs, "sort_distinct_keys", g->keyA, g->keyB,
                                         reinterpret_cast<const uint32_t*>(g->valA), reinterpret_cast<uint32_t*>(g->valB),
                                         (int64_t)distinct, endBit, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    RECSDK_LAUNCH(k_regroup_sorted_scatter, dim3(grid), dim3(kBlock), s, g->keyB, g->valB, v->total, d_sorted,
                  g->newPos);
    RECSDK_LAUNCH(k_regroup_index<int64_t>, dim3(grid), dim3(kBlock), s, v->grank, g->newPos,
                  (const int32_t*)nullptr, n, d_inverse);
    return RECSDK_OK;
}
