// HBM-cache planner with most-recently-released-first reuse (the TF path's device cache in front of host rows).
//
// Sequential definition (AccCTR embedding_cache/offset_mapper/offset_mapper.h:135-295, limited_set.h:25-140):
// keys found in the cache turn into their slot; the others ("swap in"), in input order, take
//   (1) slots freed by Remove, most recently freed first,
//   (2) when the cache cannot hold them all: slots whose key neither this call nor the previous one used, most
//       recently released first (the reference walks an intrusive list that gets the previous call's slots pushed
//       at its head, in input order, at the end of every call); their keys are reported as "swap out",
//   (3) never-used slots, ascending.
// Parallel form used here: every slot carries a stamp = call * 2^28 + index of the key inside that call, written
// when the slot is used (hit or assigned).  The reference's list, read from its head, is exactly the set of slots
// with stamp.call <= now - 2 in descending stamp order, so "the first K slots of the list" is a top-K selection:
// a 4-pass radix select (14 bits per pass) finds the K-th largest stamp, the K slots at or above it are gathered
// and sorted descending.  Freed slots carry no stamp and sit on a stack.
#include <string.h>

#include <algorithm>

#include <hip/hip_runtime.h>
#include <rocprim/rocprim.hpp>

#include "common.h"
#include "hashmap.h"

namespace recsdk {

constexpr int kOmIdxBits = 28;          // index of a key inside its call
constexpr int kOmDigitBits = 14;
constexpr int kOmBins = 1 << kOmDigitBits;
constexpr int kOmPasses = 4;            // 56 stamp bits
constexpr int64_t kOmNoStamp = -1;
constexpr int64_t kOmMergeSortMax = int64_t(1) << 20;   // candidate lists up to this length take the merge sort
using OmSortConfig = rocprim::merge_sort_config<512, 512, 4, 128, 128, 4, (1u << 30)>;  // never the merge-path kernels

struct OmState {
    int64_t useLength;
    int64_t evictSize;
    int64_t call;         // number of the current call (first call = 0)
    int64_t misses;       // keys of the current call that are not in the cache
    int64_t evictTake;    // of those, how many take freed slots
    int64_t swapOutNum;   // how many take a slot whose key is swapped out
    int64_t fresh;        // the rest: never-used slots
    int64_t prefix;       // radix select: the high digits of the K-th largest eligible stamp found so far
    int64_t remaining;    // radix select: victims still to find among the stamps that share `prefix`
    int64_t gathered;     // victims appended so far
    int64_t removed;      // keys erased by the current remove call
    int32_t error;        // cache too small for the current call
    int32_t pad;
};

__device__ __forceinline__ bool om_eligible(int64_t stamp, int64_t call)
{
    return stamp >= 0 && (stamp >> kOmIdxBits) <= call - 2;
}

// ---- hits --------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kTile) void k_om_hit(MapRef map, const OmState* __restrict__ st, int64_t* __restrict__ keys,
                                                  int64_t n, int64_t* __restrict__ stamp, uint8_t* __restrict__ miss,
                                                  uint32_t* __restrict__ tileM)
{
    __shared__ uint32_t red[kTile / kWave];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    const int64_t call = st->call;
    // one key per thread, a tile per block: a probe is a chain of dependent trips to memory
    const int64_t i = tile0 + (int64_t)threadIdx.x;
    uint32_t f = 0;
    if (i < n) {
        const long long key = keys[i];
        if (key != kEmptyKey) {
            const int64_t pos = map_find(map, key);
            if (pos >= 0) {
                const int64_t slot = map.entries[pos].slot;
                keys[i] = slot;
                stamp[slot] = (call << kOmIdxBits) | i;
            } else {
                f = 1;
            }
        }
    }
    miss[i] = (uint8_t)f;  // whole tiles of flags
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
        f += __shfl_down(f, d, kWave);
    }
    if (lane_id() == 0) {
        red[threadIdx.x >> 6] = f;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t s = 0;
        for (int k = 0; k < kTile / kWave; ++k) {
            s += red[k];
        }
        tileM[blockIdx.x] = s;
    }
}

// single block: exclusive scan of the tile counts in place, total through *carry
__device__ __forceinline__ void om_scan_tiles(uint32_t* tiles, int64_t ntiles, uint32_t* smem, uint32_t* carry)
{
    if (threadIdx.x == 0) {
        *carry = 0;
    }
    __syncthreads();
    for (int64_t b = 0; b < ntiles; b += kBlock) {
        const int64_t j = b + threadIdx.x;
        const uint32_t v = (j < ntiles) ? tiles[j] : 0;
        uint32_t tot;
        const uint32_t e = block_exclusive_scan(v, smem, &tot);
        if (j < ntiles) {
            tiles[j] = *carry + e;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            *carry += tot;
        }
        __syncthreads();
    }
}

// split of the misses over the three slot sources (offset_mapper.h:187-190); clears the select histograms
__global__ __launch_bounds__(kBlock) void k_om_plan(OmState* st, uint32_t* tileM, int64_t ntiles, int64_t maxCacheSize,
                                                    uint32_t* __restrict__ hist, uint64_t* __restrict__ candKey,
                                                    int64_t n)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carry;
    if (blockIdx.x == 0) {
        om_scan_tiles(tileM, ntiles, smem, &carry);
        if (threadIdx.x == 0) {
            const int64_t m = carry;
            const int64_t freeLen = maxCacheSize - st->useLength + st->evictSize;
            const int64_t out = m <= freeLen ? 0 : m - freeLen;
            const int64_t take = st->evictSize < m ? st->evictSize : m;
            st->misses = m;
            st->swapOutNum = out;
            st->evictTake = take;
            st->fresh = m - take - out;
            st->prefix = 0;
            st->remaining = out;
            st->gathered = 0;
            st->error = 0;
        }
    }
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < (int64_t)kOmPasses * kOmBins; j += stride) {
        hist[j] = 0;
    }
    for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < n; j += stride) {
        candKey[j] = 0;
    }
}

// ---- radix select of the swapOutNum-th largest eligible stamp -----------------------------------------------
__global__ __launch_bounds__(kBlock) void k_om_select_hist(const OmState* __restrict__ st,
                                                           const int64_t* __restrict__ stamp, int pass,
                                                           uint32_t* __restrict__ hist)
{
    extern __shared__ uint32_t bins[];
    if (st->swapOutNum == 0 || st->error) {
        return;
    }
    for (int j = threadIdx.x; j < kOmBins; j += kBlock) {
        bins[j] = 0;
    }
    __syncthreads();
    const int64_t use = st->useLength;
    const int64_t call = st->call;
    const int shift = kOmDigitBits * (kOmPasses - 1 - pass);
    const int64_t prefix = st->prefix;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x; p < use; p += stride) {
        const int64_t s = stamp[p];
        if (om_eligible(s, call) && (pass == 0 || (s >> (shift + kOmDigitBits)) == prefix)) {
            atomicAdd(&bins[(s >> shift) & (kOmBins - 1)], 1u);
        }
    }
    __syncthreads();
    uint32_t* out = hist + (int64_t)pass * kOmBins;
    for (int j = threadIdx.x; j < kOmBins; j += kBlock) {
        if (bins[j] != 0) {
            atomicAdd(&out[j], bins[j]);
        }
    }
}

// single block: the digit of this pass = the highest bin b with count(bins > b) < remaining <= count(bins >= b)
__global__ __launch_bounds__(kBlock) void k_om_select_pick(OmState* st, int pass, const uint32_t* __restrict__ hist)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    if (st->swapOutNum == 0 || st->error) {
        return;
    }
    constexpr int kPer = kOmBins / kBlock;
    const uint32_t* h = hist + (int64_t)pass * kOmBins;
    // thread t owns bins [top - kPer + 1, top], top = kOmBins - 1 - t * kPer (descending order over threads)
    const int top = kOmBins - 1 - (int)threadIdx.x * kPer;
    uint32_t mine = 0;
    for (int k = 0; k < kPer; ++k) {
        mine += h[top - k];
    }
    uint32_t total;
    const uint32_t above = block_exclusive_scan(mine, smem, &total);
    const int64_t remaining = st->remaining;
    __syncthreads();
    if (threadIdx.x == 0 && (int64_t)total < remaining) {
        st->error = 1;  // fewer reusable slots than the call needs (offset_mapper.h:234-241)
    }
    if ((int64_t)total >= remaining && (int64_t)above < remaining && (int64_t)(above + mine) >= remaining) {
        uint32_t cum = above;
        for (int k = 0; k < kPer; ++k) {
            const uint32_t c = h[top - k];
            if ((int64_t)(cum + c) >= remaining) {
                st->prefix = (st->prefix << kOmDigitBits) | (int64_t)(top - k);
                st->remaining = remaining - cum;
                break;
            }
            cum += c;
        }
    }
}

// victims = eligible slots whose stamp is at least the selected one (unordered append)
__global__ __launch_bounds__(kBlock) void k_om_select_gather(OmState* st, const int64_t* __restrict__ stamp,
                                                             uint64_t* __restrict__ candKey,
                                                             uint32_t* __restrict__ candSlot)
{
    if (st->swapOutNum == 0 || st->error) {
        return;
    }
    __shared__ BlockAppend<1024> found;
    const int64_t use = st->useLength;
    const int64_t call = st->call;
    const int64_t threshold = st->prefix;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    unsigned long long* counter = reinterpret_cast<unsigned long long*>(&st->gathered);
    found.init();
    for (int64_t base = (int64_t)blockIdx.x * kBlock; base < use; base += stride) {
        const int64_t p = base + threadIdx.x;
        const int64_t s = p < use ? stamp[p] : 0;
        const bool take = p < use && om_eligible(s, call) && s >= threshold;
        // key + 1: 0 marks an unused entry of the sort buffer
        found.push(take, (unsigned long long)s + 1, (uint32_t)p);
        found.maybe_flush(counter, reinterpret_cast<unsigned long long*>(candKey), candSlot, INT64_MAX);
    }
    found.flush(counter, reinterpret_cast<unsigned long long*>(candKey), candSlot, INT64_MAX);
}

// victims in list order: erase their keys, report them as swapped out
__global__ __launch_bounds__(kBlock) void k_om_victims(MapRef map, const OmState* __restrict__ st,
                                                       const uint32_t* __restrict__ victimSlot,
                                                       const int64_t* __restrict__ pos2Key,
                                                       int64_t* __restrict__ swapOutKeys,
                                                       int64_t* __restrict__ swapOutPos)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (st->error || j >= st->swapOutNum) {
        return;
    }
    const int64_t slot = victimSlot[j];
    const long long old = pos2Key[slot];
    long long unused;
    (void)map_erase(map, old, &unused);
    swapOutKeys[j] = old;
    swapOutPos[j] = slot;
}

// misses in input order take their slots
__global__ __launch_bounds__(kTile) void k_om_assign(MapRef map, const OmState* __restrict__ st,
                                                     int64_t* __restrict__ keys, int64_t n,
                                                     const uint8_t* __restrict__ miss,
                                                     const uint32_t* __restrict__ tileM,
                                                     const int64_t* __restrict__ evictStack,
                                                     const uint32_t* __restrict__ victimSlot,
                                                     int64_t* __restrict__ pos2Key, int64_t* __restrict__ stamp,
                                                     int64_t* __restrict__ swapInKeys, int64_t* __restrict__ swapInPos)
{
    __shared__ uint32_t smem[kTile / kWave];
    if (st->error) {
        return;
    }
    // one key per thread, a tile per block: an insert is a chain of dependent trips to memory
    const int64_t i = (int64_t)blockIdx.x * kTile + (int64_t)threadIdx.x;
    const uint32_t f = miss[i];  // whole tiles of flags
    uint32_t tot;
    const int64_t r = (int64_t)block_exclusive_scan_n<kTile>(f, smem, &tot) + tileM[blockIdx.x];
    if (f == 0 || i >= n) {
        return;
    }
    const int64_t take = st->evictTake;
    const int64_t out = st->swapOutNum;
    const int64_t evictSize = st->evictSize;
    const int64_t use = st->useLength;
    const int64_t call = st->call;
    const long long key = keys[i];
    int64_t slot;
    if (r < take) {
        slot = evictStack[evictSize - 1 - r];
    } else if (r < take + out) {
        slot = victimSlot[r - take];
    } else {
        slot = use + (r - take - out);
    }
    map_insert(map, key, slot);
    pos2Key[slot] = key;
    stamp[slot] = (call << kOmIdxBits) | i;
    keys[i] = slot;
    swapInKeys[r] = key;
    swapInPos[r] = slot;
}

__global__ void k_om_finish(OmState* st, int64_t* counts)
{
    if (threadIdx.x == 0) {
        counts[0] = st->error ? 0 : st->misses;
        counts[1] = st->error ? 0 : st->swapOutNum;
        counts[2] = st->error;
        if (!st->error) {
            st->useLength += st->fresh;
            st->evictSize -= st->evictTake;
        }
        st->call += 1;
    }
}

// ---- Remove (offset_mapper.h:107-119): freed slots go on the stack in input order -----------------------------
__global__ __launch_bounds__(kBlock) void k_om_remove_mark(MapRef map, const int64_t* __restrict__ keys, int64_t n,
                                                           int64_t* __restrict__ pos2Key, int64_t* __restrict__ stamp,
                                                           int64_t* __restrict__ freed, uint32_t* __restrict__ tileM)
{
    __shared__ uint32_t red[kBlock / kWave];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    uint32_t f = 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t i = tile0 + (int64_t)threadIdx.x * kItems + k;
        int64_t slot = -1;
        if (i < n) {
            const long long key = keys[i];
            long long v;
            if (key != kEmptyKey && map_erase(map, key, &v)) {
                slot = v;
                pos2Key[slot] = kEmptyKey;
                stamp[slot] = kOmNoStamp;
                f += 1;
            }
        }
        freed[tile0 + (int64_t)threadIdx.x * kItems + k] = slot;
    }
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
        f += __shfl_down(f, d, kWave);
    }
    if (lane_id() == 0) {
        red[threadIdx.x >> 6] = f;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t s = 0;
        for (int k = 0; k < kBlock / kWave; ++k) {
            s += red[k];
        }
        tileM[blockIdx.x] = s;
    }
}

__global__ __launch_bounds__(kBlock) void k_om_remove_scan(OmState* st, uint32_t* tileM, int64_t ntiles)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carry;
    om_scan_tiles(tileM, ntiles, smem, &carry);
    if (threadIdx.x == 0) {
        st->removed = carry;
    }
}

__global__ __launch_bounds__(kBlock) void k_om_remove_push(const OmState* __restrict__ st,
                                                           const int64_t* __restrict__ freed,
                                                           const uint32_t* __restrict__ tileM,
                                                           int64_t* __restrict__ evictStack)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    const int64_t i0 = (int64_t)blockIdx.x * kTile + (int64_t)threadIdx.x * kItems;
    int64_t sl[kItems];
    uint32_t f = 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        sl[k] = freed[i0 + k];
        f += sl[k] >= 0 ? 1 : 0;
    }
    uint32_t tot;
    int64_t r = (int64_t)block_exclusive_scan(f, smem, &tot) + tileM[blockIdx.x] + st->evictSize;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (sl[k] >= 0) {
            evictStack[r] = sl[k];
            r += 1;
        }
    }
}

__global__ void k_om_remove_finish(OmState* st)
{
    if (threadIdx.x == 0) {
        st->evictSize += st->removed;
    }
}

// ---- map rebuild (erased map slots lengthen probe chains) --------------------------------------------------------
__global__ __launch_bounds__(kBlock) void k_om_map_clear(MapRef map)
{
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    TableEntry e;
    e.key = kEmptyKey;
    e.slot = -1;
    for (; i <= map.mask + 1; i += stride) {
        map.entries[i] = e;
    }
}

__global__ __launch_bounds__(kBlock) void k_om_map_refill(MapRef map, const OmState* __restrict__ st,
                                                          const int64_t* __restrict__ pos2Key)
{
    const int64_t use = st->useLength;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x; p < use; p += stride) {
        if (pos2Key[p] != kEmptyKey) {
            map_insert(map, pos2Key[p], p);
        }
    }
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_om {
    int64_t maxCacheSize = 0;
    int64_t maxKeys = 0;
    int64_t insertBound = 0;
    int64_t calls = 0;
    MapRef map{};
    int64_t* pos2Key = nullptr;
    int64_t* stamp = nullptr;
    int64_t* evictStack = nullptr;
    OmState* st = nullptr;
    uint8_t* miss = nullptr;
    uint32_t* tileM = nullptr;
    uint32_t* hist = nullptr;
    uint64_t* candKeyA = nullptr;
    uint64_t* candKeyB = nullptr;
    uint32_t* candSlotA = nullptr;
    uint32_t* candSlotB = nullptr;
    int64_t* freed = nullptr;
    int64_t* counts = nullptr;
    void* tmp = nullptr;
    size_t tmpBytes = 0;
};

extern "C" int recsdk_om_destroy(recsdk_om_t* h)
{
    if (h == nullptr) {
        return RECSDK_OK;
    }
    void* ptrs[] = {h->map.entries, h->pos2Key,  h->stamp,     h->evictStack, h->st,    h->miss,   h->tileM, h->hist,
                    h->candKeyA,    h->candKeyB, h->candSlotA, h->candSlotB,  h->freed, h->counts, h->tmp};
    for (void* p : ptrs) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_om_create(int64_t max_cache_size, int64_t max_keys, recsdk_om_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_om_create: out is NULL");
    RECSDK_REQUIRE(max_cache_size > 0 && max_cache_size < (int64_t(1) << 31), RECSDK_EINVAL,
                   "recsdk_om_create: max_cache_size must be in (0, 2^31)");
    RECSDK_REQUIRE(max_keys > 0 && max_keys <= (int64_t(1) << kOmIdxBits), RECSDK_EINVAL,
                   "recsdk_om_create: max_keys must be in (0, 2^28]");
    auto* h = new recsdk_om();
    h->maxCacheSize = max_cache_size;
    h->maxKeys = max_keys;
    uint64_t cap = 64;
    while (cap < 2 * (uint64_t)max_cache_size) {
        cap <<= 1;
    }
    h->map.mask = cap - 1;
    size_t sortBytes = 0;
    (void)rocprim::radix_sort_pairs_desc(nullptr, sortBytes, (uint64_t*)nullptr, (uint64_t*)nullptr, (uint32_t*)nullptr,
                                         (uint32_t*)nullptr, (size_t)max_keys, 0, 64, (hipStream_t) nullptr);
    {
        size_t mergeBytes = 0;
        (void)rocprim::merge_sort<OmSortConfig>(nullptr, mergeBytes, (uint64_t*)nullptr, (uint64_t*)nullptr,
                                                (uint32_t*)nullptr, (uint32_t*)nullptr,
                                                (size_t)std::min<int64_t>(max_keys, kOmMergeSortMax),
                                                rocprim::greater<uint64_t>(), (hipStream_t) nullptr);
        sortBytes = std::max(sortBytes, mergeBytes);
    }
    h->tmpBytes = sortBytes + 256;
    bool ok = true;
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes) != hipSuccess) {
            ok = false;
        }
    };
    const int64_t padded = cdiv(max_keys, kTile) * kTile;
    alloc(&h->map.entries, sizeof(TableEntry) * (cap + 1));
    alloc(&h->pos2Key, sizeof(int64_t) * max_cache_size);
    alloc(&h->stamp, sizeof(int64_t) * max_cache_size);
    alloc(&h->evictStack, sizeof(int64_t) * max_cache_size);
    alloc(&h->st, sizeof(OmState));
    alloc(&h->miss, padded);
    alloc(&h->tileM, sizeof(uint32_t) * (padded / kTile + 1));
    alloc(&h->hist, sizeof(uint32_t) * kOmPasses * kOmBins);
    alloc(&h->candKeyA, sizeof(uint64_t) * padded);
    alloc(&h->candKeyB, sizeof(uint64_t) * padded);
    alloc(&h->candSlotA, sizeof(uint32_t) * padded);
    alloc(&h->candSlotB, sizeof(uint32_t) * padded);
    alloc(&h->freed, sizeof(int64_t) * padded);
    alloc(&h->counts, sizeof(int64_t) * 4);
    alloc(&h->tmp, h->tmpBytes);
    if (ok) {
        // all-ones bytes: empty map entries, no key in any slot, no stamp
        ok = hipMemset(h->map.entries, 0xFF, sizeof(TableEntry) * (cap + 1)) == hipSuccess &&
             hipMemset(h->pos2Key, 0xFF, sizeof(int64_t) * max_cache_size) == hipSuccess &&
             hipMemset(h->stamp, 0xFF, sizeof(int64_t) * max_cache_size) == hipSuccess &&
             hipMemset(h->st, 0, sizeof(OmState)) == hipSuccess;
    }
    if (!ok) {
        (void)hipGetLastError();
        recsdk_om_destroy(h);
        set_error("recsdk_om_create: allocation failed");
        return RECSDK_ENOMEM;
    }
    *out = h;
    return RECSDK_OK;
}

static int om_maybe_rebuild(recsdk_om* h, int64_t inserts, hipStream_t s)
{
    h->insertBound += inserts;
    if ((uint64_t)h->insertBound > (h->map.mask + 1) / 4) {
        const unsigned g1 = (unsigned)std::min<uint64_t>((h->map.mask + 2 + kBlock - 1) / kBlock, 256 * 16);
        const unsigned g2 = (unsigned)std::min<int64_t>(cdiv(h->maxCacheSize, kBlock), 256 * 16);
        RECSDK_LAUNCH(k_om_map_clear, dim3(g1), dim3(kBlock), s, h->map);
        RECSDK_LAUNCH(k_om_map_refill, dim3(g2), dim3(kBlock), s, h->map, h->st, h->pos2Key);
        h->insertBound = inserts;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_om_compute(recsdk_om_t* h, int64_t* d_keys, int64_t n, int64_t* d_swapin_keys,
                                 int64_t* d_swapin_pos, int64_t* d_swapout_keys, int64_t* d_swapout_pos, void* stream)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_om_compute: NULL handle");
    RECSDK_REQUIRE(n >= 0 && n <= h->maxKeys, RECSDK_ECAPACITY, "recsdk_om_compute: n exceeds max_keys");
    RECSDK_REQUIRE(n == 0 || (d_keys && d_swapin_keys && d_swapin_pos && d_swapout_keys && d_swapout_pos), RECSDK_ENULL,
                   "recsdk_om_compute: NULL argument");
    RECSDK_REQUIRE(h->calls < (int64_t(1) << 27), RECSDK_EOVERFLOW, "recsdk_om_compute: call counter exhausted");
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc = om_maybe_rebuild(h, n, s);
    if (rc != RECSDK_OK) {
        return rc;
    }
    h->calls += 1;
    const int64_t ntiles = cdiv(n, kTile);
    const unsigned gridK = (unsigned)std::max<int64_t>(ntiles, 1);
    const unsigned gridS = (unsigned)std::min<int64_t>(cdiv(h->maxCacheSize, kTile), 512);
    const unsigned gridV = (unsigned)std::max<int64_t>(cdiv(n, kBlock), 1);
    if (n > 0) {
        RECSDK_LAUNCH(k_om_hit, dim3(gridK), dim3(kTile), s, h->map, h->st, d_keys, n, h->stamp, h->miss, h->tileM);
    }
    RECSDK_LAUNCH(k_om_plan, dim3(64), dim3(kBlock), s, h->st, h->tileM, ntiles, h->maxCacheSize, h->hist, h->candKeyA,
                  n);
    if (n > 0) {
        // Stamps are call * 2^28 + index: the digits above the current call number are zero in every eligible stamp,
        // so the select starts at the first digit that can differ (three passes instead of four for the first 16383
        // calls; every pass reads the stamps of the whole cache).
        int stampBits = kOmIdxBits;
        while ((h->calls >> (stampBits - kOmIdxBits)) != 0) {
            ++stampBits;
        }
        const int firstPass = std::max(0, kOmPasses - (stampBits + kOmDigitBits - 1) / kOmDigitBits);
        for (int pass = firstPass; pass < kOmPasses; ++pass) {
            {
                recsdk::KernelScope scope("k_om_select_hist", s);
                hipLaunchKernelGGL(k_om_select_hist, dim3(gridS), dim3(kBlock), sizeof(uint32_t) * kOmBins, s, h->st,
                                   h->stamp, pass, h->hist);
            }
            RECSDK_HIP_TRY(hipGetLastError());
            RECSDK_LAUNCH(k_om_select_pick, dim3(1), dim3(kBlock), s, h->st, pass, h->hist);
        }
        RECSDK_LAUNCH(k_om_select_gather, dim3(gridS), dim3(kBlock), s, h->st, h->stamp, h->candKeyA, h->candSlotA);
        size_t bytes = h->tmpBytes;
        if (n <= kOmMergeSortMax) {
            // a few hundred thousand candidates: the work is small and the launches count (this sort is among the last
            // kernels before the host learns the lists' lengths).  Merge sort with 2048-pair blocks and one kernel per
            // merge pass: 9 launches for 432 k candidates where the radix-sort entry point takes 21.
            RECSDK_HIP_TRY(rocprim::merge_sort<OmSortConfig>(h->tmp, bytes, h->candKeyA, h->candKeyB, h->candSlotA,
                                                             h->candSlotB, (size_t)n, rocprim::greater<uint64_t>(), s));
        } else {
            RECSDK_HIP_TRY(rocprim::radix_sort_pairs_desc(h->tmp, bytes, h->candKeyA, h->candKeyB, h->candSlotA,
                                                          h->candSlotB, (size_t)n, 0, 2 * kOmIdxBits + 1, s));
        }
        RECSDK_LAUNCH(k_om_victims, dim3(gridV), dim3(kBlock), s, h->map, h->st, h->candSlotB, h->pos2Key,
                      d_swapout_keys, d_swapout_pos);
        RECSDK_LAUNCH(k_om_assign, dim3(gridK), dim3(kTile), s, h->map, h->st, d_keys, n, h->miss, h->tileM,
                      h->evictStack, h->candSlotB, h->pos2Key, h->stamp, d_swapin_keys, d_swapin_pos);
    }
    RECSDK_LAUNCH(k_om_finish, dim3(1), dim3(64), s, h->st, h->counts);
    return RECSDK_OK;
}

extern "C" int recsdk_om_counts(recsdk_om_t* h, void* stream, int64_t* h_swapins, int64_t* h_swapouts,
                                int64_t* h_use_length, int64_t* h_evict_size)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_om_counts: NULL handle");
    hipStream_t s = static_cast<hipStream_t>(stream);
    OmState st;
    int64_t counts[4];
    RECSDK_HIP_TRY(hipMemcpyAsync(&st, h->st, sizeof(st), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(counts, h->counts, sizeof(counts), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    if (h_swapins) {
        *h_swapins = counts[0];
    }
    if (h_swapouts) {
        *h_swapouts = counts[1];
    }
    if (h_use_length) {
        *h_use_length = st.useLength;
    }
    if (h_evict_size) {
        *h_evict_size = st.evictSize;
    }
    if (counts[2] != 0) {
        set_error("device cache overflow: max cache size is too small for this batch");
        return RECSDK_EOVERFLOW;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_om_remove(recsdk_om_t* h, const int64_t* d_keys, int64_t n, void* stream)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_om_remove: NULL handle");
    if (n <= 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_keys != nullptr, RECSDK_ENULL, "recsdk_om_remove: d_keys is NULL");
    RECSDK_REQUIRE(n <= h->maxKeys, RECSDK_ECAPACITY, "recsdk_om_remove: n exceeds max_keys");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t ntiles = cdiv(n, kTile);
    RECSDK_LAUNCH(k_om_remove_mark, dim3((unsigned)ntiles), dim3(kBlock), s, h->map, d_keys, n, h->pos2Key, h->stamp,
                  h->freed, h->tileM);
    RECSDK_LAUNCH(k_om_remove_scan, dim3(1), dim3(kBlock), s, h->st, h->tileM, ntiles);
    RECSDK_LAUNCH(k_om_remove_push, dim3((unsigned)ntiles), dim3(kBlock), s, h->st, h->freed, h->tileM, h->evictStack);
    RECSDK_LAUNCH(k_om_remove_finish, dim3(1), dim3(64), s, h->st);
    return RECSDK_OK;
}

extern "C" int recsdk_om_export(recsdk_om_t* h, int64_t* d_pos2key, void* stream)
{
    RECSDK_REQUIRE(h != nullptr && d_pos2key != nullptr, RECSDK_ENULL, "recsdk_om_export: NULL argument");
    RECSDK_HIP_TRY(hipMemcpyAsync(d_pos2key, h->pos2Key, sizeof(int64_t) * h->maxCacheSize, hipMemcpyDeviceToDevice,
                                  static_cast<hipStream_t>(stream)));
    return RECSDK_OK;
}

extern "C" int recsdk_om_copy_state(recsdk_om_t* dst, const recsdk_om_t* src, void* stream)
{
    RECSDK_REQUIRE(dst != nullptr && src != nullptr, RECSDK_ENULL, "recsdk_om_copy_state: NULL handle");
    RECSDK_REQUIRE(dst->maxCacheSize == src->maxCacheSize, RECSDK_EINVAL,
                   "recsdk_om_copy_state: the two planners have different cache sizes");
    if (dst == src) {
        return RECSDK_OK;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t slots = (size_t)src->maxCacheSize;
    // the persistent state: key -> slot map, slot -> key, hit stamps, freed-slot stack, counters
    RECSDK_HIP_TRY(hipMemcpyAsync(dst->map.entries, src->map.entries, sizeof(TableEntry) * (src->map.mask + 2),
                                  hipMemcpyDeviceToDevice, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(dst->pos2Key, src->pos2Key, sizeof(int64_t) * slots, hipMemcpyDeviceToDevice, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(dst->stamp, src->stamp, sizeof(int64_t) * slots, hipMemcpyDeviceToDevice, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(dst->evictStack, src->evictStack, sizeof(int64_t) * slots, hipMemcpyDeviceToDevice, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(dst->st, src->st, sizeof(OmState), hipMemcpyDeviceToDevice, s));
    dst->insertBound = src->insertBound;
    dst->calls = src->calls;
    return RECSDK_OK;
}
