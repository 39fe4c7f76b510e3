// HBM-cache planner with a version clock (hit / miss resolve, swap-in / swap-out lists, batch offsets).
//
// Sequential definition (torchrec_embcache/csrc/embedding_cache/swap_manager.cpp:32-139): hits are stamped with
// the current version; misses, in batch order, take fresh slots while the cache is not full, then the next slot
// of a clock sweep whose version is older than the previous batch; a swept slot that was not removed before is
// swapped out.
// Parallel form used here: the distinct keys of the batch come in first-occurrence order from the dedup kernels,
// so "misses in batch order" is a scan over their miss flags; "next eligible slot of the sweep" is a scan over the
// slots' eligibility flags in cyclic order from the sweep position.  The k-th miss that needs a victim takes the
// k-th eligible slot, exactly the slot the sequential sweep would have reached.
#include <algorithm>

#include "common.h"
#include "dedup.h"
#include "hashmap.h"

namespace recsdk {

constexpr long long kReuseVersion = -2;  // CAN_REUSE_KEY_VERSION, swap_manager.h:21

struct SwapState {
    int64_t occupied;
    int64_t nowVersion;
    int64_t swapIdx;
    int64_t misses;        // distinct missed keys of the current call
    int64_t fresh;         // of those, how many take never-used slots
    int64_t needVictims;   // the rest
    int64_t eligible;      // sweepable slots
    int64_t swapouts;      // victims that are swapped out
    int64_t lastVictim;    // slot of the last victim taken
    int32_t error;         // cache too small for this batch (state left as it was)
    int32_t pad;
};

// distinct keys: hit -> offset + version stamp, miss -> flag
__global__ __launch_bounds__(kBlock) void k_swap_hit(MapRef map, const SwapState* __restrict__ st,
                                                     const int64_t* __restrict__ ukeys,
                                                     const int64_t* __restrict__ total, int64_t* __restrict__ offOf,
                                                     int64_t* __restrict__ cacheVer, uint8_t* __restrict__ miss,
                                                     uint32_t* __restrict__ tileM, int64_t nMax)
{
    __shared__ uint32_t red[kBlock / kWave];
    const int64_t U = total[0];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= U || tile0 >= nMax) {
        return;
    }
    const int64_t now = st->nowVersion;
    uint32_t f = 0;
    uint8_t fl[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t R = tile0 + (int64_t)threadIdx.x * kItems + k;
        fl[k] = 0;
        if (R < U) {
            const long long key = ukeys[R];
            const int64_t pos = map_find(map, key);
            if (pos >= 0) {
                const int64_t off = map.entries[pos].slot;
                offOf[R] = off;
                cacheVer[off] = now;
            } else {
                fl[k] = 1;
                f += 1;
            }
        }
    }
    *reinterpret_cast<uchar4*>(miss + tile0 + (int64_t)threadIdx.x * kItems) = make_uchar4(fl[0], fl[1], fl[2], fl[3]);
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

// single block: exclusive scan of tile counts in place; returns the total through *out
__device__ __forceinline__ void scan_tiles(uint32_t* tiles, int64_t ntiles, uint32_t* smem, uint32_t* carry,
                                           uint32_t* tiles2, uint32_t* carry2)
{
    if (threadIdx.x == 0) {
        *carry = 0;
        if (carry2) {
            *carry2 = 0;
        }
    }
    __syncthreads();
    for (int64_t b = 0; b < ntiles; b += kBlock) {
        const int64_t j = b + threadIdx.x;
        uint32_t v = (j < ntiles) ? tiles[j] : 0;
        uint32_t tot;
        uint32_t e = block_exclusive_scan(v, smem, &tot);
        uint32_t tot2 = 0;
        uint32_t e2 = 0;
        if (tiles2) {
            uint32_t v2 = (j < ntiles) ? tiles2[j] : 0;
            e2 = block_exclusive_scan(v2, smem, &tot2);
        }
        if (j < ntiles) {
            tiles[j] = *carry + e;
            if (tiles2) {
                tiles2[j] = *carry2 + e2;
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            *carry += tot;
            if (carry2) {
                *carry2 += tot2;
            }
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(kBlock) void k_swap_miss_scan(SwapState* st, uint32_t* tileM,
                                                           const int64_t* __restrict__ total, int64_t cacheSize,
                                                           int64_t nMax)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carry;
    const int64_t U = total[0] < nMax ? total[0] : nMax;
    scan_tiles(tileM, (U + kTile - 1) / kTile, smem, &carry, nullptr, nullptr);
    if (threadIdx.x == 0) {
        const int64_t m = carry;
        const int64_t room = cacheSize - st->occupied;
        st->misses = m;
        st->fresh = m < room ? m : room;
        st->needVictims = m - st->fresh;
        st->eligible = 0;
        st->swapouts = 0;
        st->lastVictim = -1;
        st->error = 0;
    }
}

// cyclic position c in [0, span) -> slot
__device__ __forceinline__ int64_t sweep_slot(int64_t c, int64_t memStart, int64_t span, int64_t swapIdx)
{
    int64_t rel = swapIdx - memStart + c;
    if (rel >= span) {
        rel -= span;
    }
    return memStart + rel;
}

// eligibility of every slot in sweep order (only when victims are needed)
__global__ __launch_bounds__(kBlock) void k_swap_eligible(const SwapState* __restrict__ st,
                                                          const int64_t* __restrict__ cacheVer, int64_t memStart,
                                                          int64_t cacheSize, uint32_t* __restrict__ tileE,
                                                          uint32_t* __restrict__ tileO)
{
    __shared__ uint32_t red[2 * kBlock / kWave];
    if (st->needVictims == 0) {
        return;
    }
    const int64_t span = cacheSize - memStart;
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= span) {
        return;
    }
    const int64_t now = st->nowVersion;
    const int64_t occupied = st->occupied;
    int64_t swapIdx = st->swapIdx;
    if (swapIdx >= cacheSize) {
        swapIdx = memStart;
    }
    uint32_t e = 0;
    uint32_t o = 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t c = tile0 + (int64_t)threadIdx.x * kItems + k;
        if (c < span) {
            const int64_t sl = sweep_slot(c, memStart, span, swapIdx);
            const int64_t ver = cacheVer[sl];
            // slots at or past `occupied` are the ones this call's first misses fill: they carry the current
            // version by the time the sequential sweep starts, so they are never victims
            if (sl < occupied && ver < now - 1) {
                e += 1;
                o += (ver != kReuseVersion) ? 1 : 0;
            }
        }
    }
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
        e += __shfl_down(e, d, kWave);
        o += __shfl_down(o, d, kWave);
    }
    if (lane_id() == 0) {
        red[threadIdx.x >> 6] = e;
        red[kBlock / kWave + (threadIdx.x >> 6)] = o;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t se = 0;
        uint32_t so = 0;
        for (int k = 0; k < kBlock / kWave; ++k) {
            se += red[k];
            so += red[kBlock / kWave + k];
        }
        tileE[blockIdx.x] = se;
        tileO[blockIdx.x] = so;
    }
}

__global__ __launch_bounds__(kBlock) void k_swap_eligible_scan(SwapState* st, uint32_t* tileE, uint32_t* tileO,
                                                               int64_t memStart, int64_t cacheSize)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carryE;
    __shared__ uint32_t carryO;
    if (st->needVictims == 0) {
        return;
    }
    const int64_t span = cacheSize - memStart;
    scan_tiles(tileE, (span + kTile - 1) / kTile, smem, &carryE, tileO, &carryO);
    if (threadIdx.x == 0) {
        st->eligible = carryE;
        if (st->needVictims > (int64_t)carryE) {
            st->error = 1;  // "cacheSize_ too small" (swap_manager.cpp:103-105)
        }
    }
}

// the first needVictims eligible slots of the sweep become victims
__global__ __launch_bounds__(kBlock) void k_swap_victims(MapRef map, SwapState* st, int64_t* __restrict__ cacheKey,
                                                         const int64_t* __restrict__ cacheVer, int64_t memStart,
                                                         int64_t cacheSize, const uint32_t* __restrict__ tileE,
                                                         const uint32_t* __restrict__ tileO,
                                                         int64_t* __restrict__ victimSlot,
                                                         int64_t* __restrict__ swapoutKeys,
                                                         int64_t* __restrict__ swapoutOffs)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    const int64_t need = st->needVictims;
    if (need == 0 || st->error) {
        return;
    }
    const int64_t span = cacheSize - memStart;
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= span || (int64_t)tileE[blockIdx.x] >= need) {
        return;  // the whole tile lies behind the last victim
    }
    const int64_t now = st->nowVersion;
    const int64_t occupied = st->occupied;
    int64_t swapIdx = st->swapIdx;
    if (swapIdx >= cacheSize) {
        swapIdx = memStart;
    }
    int64_t slot[kItems];
    bool el[kItems];
    bool out[kItems];
    uint32_t e = 0;
    uint32_t o = 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t c = tile0 + (int64_t)threadIdx.x * kItems + k;
        el[k] = false;
        out[k] = false;
        slot[k] = 0;
        if (c < span) {
            slot[k] = sweep_slot(c, memStart, span, swapIdx);
            const int64_t ver = cacheVer[slot[k]];
            el[k] = slot[k] < occupied && ver < now - 1;
            out[k] = el[k] && ver != kReuseVersion;
            e += el[k] ? 1 : 0;
            o += out[k] ? 1 : 0;
        }
    }
    uint32_t te;
    uint32_t to;
    int64_t re = (int64_t)block_exclusive_scan(e, smem, &te) + tileE[blockIdx.x];
    int64_t ro = (int64_t)block_exclusive_scan(o, smem, &to) + tileO[blockIdx.x];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (el[k]) {
            if (re < need) {
                victimSlot[re] = slot[k];
                const long long oldKey = cacheKey[slot[k]];
                if (oldKey != kEmptyKey) {
                    long long unused;
                    (void)map_erase(map, oldKey, &unused);
                }
                if (out[k]) {
                    swapoutKeys[ro] = oldKey;
                    swapoutOffs[ro] = slot[k];
                }
                if (re == need - 1) {
                    st->swapouts = ro + (out[k] ? 1 : 0);
                    st->lastVictim = slot[k];
                }
            }
            re += 1;
            ro += out[k] ? 1 : 0;
        }
    }
}

// misses in batch order take their slots
__global__ __launch_bounds__(kBlock) void k_swap_assign(MapRef map, const SwapState* __restrict__ st,
                                                        const int64_t* __restrict__ ukeys,
                                                        const int64_t* __restrict__ total,
                                                        const uint8_t* __restrict__ miss,
                                                        const uint32_t* __restrict__ tileM,
                                                        const int64_t* __restrict__ victimSlot,
                                                        int64_t* __restrict__ offOf, int64_t* __restrict__ cacheKey,
                                                        int64_t* __restrict__ cacheVer,
                                                        int64_t* __restrict__ swapinKeys,
                                                        int64_t* __restrict__ swapinOffs, int64_t nMax)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    const int64_t U = total[0];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= U || tile0 >= nMax || st->error) {
        return;
    }
    const int64_t i0 = tile0 + (int64_t)threadIdx.x * kItems;
    uchar4 f4 = *reinterpret_cast<const uchar4*>(miss + i0);
    uint8_t fl[kItems] = {f4.x, f4.y, f4.z, f4.w};
    uint32_t f = fl[0] + fl[1] + fl[2] + fl[3];
    uint32_t tot;
    int64_t r = (int64_t)block_exclusive_scan(f, smem, &tot) + tileM[blockIdx.x];
    if (f == 0) {
        return;
    }
    const int64_t fresh = st->fresh;
    const int64_t occupied = st->occupied;
    const int64_t now = st->nowVersion;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (!fl[k] || i0 + k >= U) {
            continue;
        }
        const long long key = ukeys[i0 + k];
        const int64_t off = (r < fresh) ? occupied + r : victimSlot[r - fresh];
        swapinKeys[r] = key;
        swapinOffs[r] = off;
        cacheKey[off] = key;
        cacheVer[off] = now;
        map_insert(map, key, off);
        offOf[i0 + k] = off;
        r += 1;
    }
}

__global__ void k_swap_finish(SwapState* st, int64_t* counts)
{
    if (threadIdx.x == 0) {
        counts[0] = st->error ? 0 : st->swapouts;
        counts[1] = st->error ? 0 : st->misses;
        if (!st->error) {
            st->occupied += st->fresh;
            if (st->lastVictim >= 0) {
                st->swapIdx = st->lastVictim + 1;
            }
        }
        st->nowVersion += 1;
    }
}

// RemoveKeys (swap_manager.cpp:141-159)
__global__ __launch_bounds__(kBlock) void k_swap_remove(MapRef map, const int64_t* __restrict__ keys, int64_t n,
                                                        int64_t* __restrict__ cacheKey, int64_t* __restrict__ cacheVer)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) {
        return;
    }
    const long long key = keys[i];
    if (key == kEmptyKey) {
        return;
    }
    long long off;
    if (map_erase(map, key, &off)) {
        cacheVer[off] = kReuseVersion;
        cacheKey[off] = kEmptyKey;
    }
}

// Rebuild of the key -> offset map from the slot arrays (erased map slots lengthen probe chains)
__global__ __launch_bounds__(kBlock) void k_swap_map_clear(MapRef map)
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

__global__ __launch_bounds__(kBlock) void k_swap_map_refill(MapRef map, const SwapState* __restrict__ st,
                                                            const int64_t* __restrict__ cacheKey,
                                                            const int64_t* __restrict__ cacheVer, int64_t memStart)
{
    int64_t off = memStart + (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    const int64_t occupied = st->occupied;
    for (; off < occupied; off += stride) {
        if (cacheVer[off] != kReuseVersion && cacheKey[off] != kEmptyKey) {
            map_insert(map, cacheKey[off], off);
        }
    }
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_swap {
    int64_t insertBound = 0;  // upper bound of map insertions since the last rebuild
    int64_t cacheSize = 0;
    int64_t memStart = 0;
    int64_t maxKeys = 0;
    MapRef map{};
    int64_t* cacheKey = nullptr;
    int64_t* cacheVer = nullptr;
    SwapState* st = nullptr;
    recsdk_unique_t* uq = nullptr;
    int64_t* offOf = nullptr;
    uint8_t* miss = nullptr;
    uint32_t* tileM = nullptr;
    uint32_t* tileE = nullptr;
    uint32_t* tileO = nullptr;
    int64_t* victimSlot = nullptr;
    int64_t* counts = nullptr;  // device: {swapouts, swapins}
    int64_t* oneOffset = nullptr;
};

extern "C" int recsdk_swap_destroy(recsdk_swap_t* h)
{
    if (h == nullptr) {
        return RECSDK_OK;
    }
    recsdk_unique_destroy(h->uq);
    void* ptrs[] = {h->map.entries, h->cacheKey, h->cacheVer, h->st,   h->offOf,  h->miss,
                    h->tileM,       h->tileE,    h->tileO,    h->victimSlot, h->counts, h->oneOffset};
    for (void* p : ptrs) {
        if (p) {
            (void)hipFree(p);
        }
    }
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_swap_create(int64_t cache_size, int64_t mem_start_offset, int64_t max_keys, recsdk_swap_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_swap_create: out is NULL");
    RECSDK_REQUIRE(cache_size > 0 && mem_start_offset >= 0 && mem_start_offset < cache_size && max_keys > 0, RECSDK_EINVAL,
                   "recsdk_swap_create: need 0 <= mem_start_offset < cache_size and max_keys > 0");
    auto* h = new recsdk_swap();
    h->cacheSize = cache_size;
    h->memStart = mem_start_offset;
    h->maxKeys = max_keys;
    uint64_t cap = 64;
    while (cap < 2 * (uint64_t)cache_size) {
        cap <<= 1;
    }
    h->map.mask = cap - 1;
    bool ok = recsdk_unique_create(max_keys, 1, &h->uq) == RECSDK_OK && recsdk_unique_set_lists(h->uq, 0) == RECSDK_OK;
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes) != hipSuccess) {
            ok = false;
        }
    };
    const int64_t padded = cdiv(max_keys, kTile) * kTile;
    const int64_t slotTiles = cdiv(cache_size, kTile) + 1;
    alloc(&h->map.entries, sizeof(TableEntry) * (cap + 1));
    alloc(&h->cacheKey, sizeof(int64_t) * cache_size);
    alloc(&h->cacheVer, sizeof(int64_t) * cache_size);
    alloc(&h->st, sizeof(SwapState));
    alloc(&h->offOf, sizeof(int64_t) * padded);
    alloc(&h->miss, padded);
    alloc(&h->tileM, sizeof(uint32_t) * (padded / kTile + 1));
    alloc(&h->tileE, sizeof(uint32_t) * slotTiles);
    alloc(&h->tileO, sizeof(uint32_t) * slotTiles);
    alloc(&h->victimSlot, sizeof(int64_t) * padded);
    alloc(&h->counts, sizeof(int64_t) * 2);
    alloc(&h->oneOffset, sizeof(int64_t) * 2);
    if (ok) {
        SwapState init{};
        init.occupied = mem_start_offset;
        init.swapIdx = mem_start_offset;
        init.lastVictim = -1;
        // slots start as {key 0, version 0} like the reference's value-initialised vector (swap_manager.cpp:29)
        ok = hipMemset(h->map.entries, 0xFF, sizeof(TableEntry) * (cap + 1)) == hipSuccess &&
             hipMemset(h->cacheKey, 0, sizeof(int64_t) * cache_size) == hipSuccess &&
             hipMemset(h->cacheVer, 0, sizeof(int64_t) * cache_size) == hipSuccess &&
             hipMemcpy(h->st, &init, sizeof(init), hipMemcpyHostToDevice) == hipSuccess;
    }
    if (!ok) {
        (void)hipGetLastError();
        recsdk_swap_destroy(h);
        set_error("recsdk_swap_create: allocation failed");
        return RECSDK_ENOMEM;
    }
    *out = h;
    return RECSDK_OK;
}

extern "C" int recsdk_swap_compute(recsdk_swap_t* h, const int64_t* d_keys, int64_t n, int64_t* d_swapout_keys,
                                   int64_t* d_swapout_offs, int64_t* d_swapin_keys, int64_t* d_swapin_offs,
                                   int64_t* d_batch_offs, void* stream)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_swap_compute: NULL handle");
    RECSDK_REQUIRE(n >= 0 && n <= h->maxKeys, RECSDK_ECAPACITY, "recsdk_swap_compute: n exceeds max_keys");
    RECSDK_REQUIRE(n == 0 || (d_keys && d_swapout_keys && d_swapout_offs && d_swapin_keys && d_swapin_offs && d_batch_offs),
                   RECSDK_ENULL, "recsdk_swap_compute: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    // every insertion may consume an empty map slot; rebuild before erased slots fill a quarter of the map
    h->insertBound += n;
    if ((uint64_t)h->insertBound > (h->map.mask + 1) / 4) {
        const unsigned g1 = (unsigned)std::min<uint64_t>((h->map.mask + 2 + kBlock - 1) / kBlock, 256 * 16);
        const unsigned g2 = (unsigned)std::min<int64_t>(cdiv(h->cacheSize, kBlock), 256 * 16);
        RECSDK_LAUNCH(k_swap_map_clear, dim3(g1), dim3(kBlock), s, h->map);
        RECSDK_LAUNCH(k_swap_map_refill, dim3(g2), dim3(kBlock), s, h->map, h->st, h->cacheKey, h->cacheVer, h->memStart);
        h->insertBound = n;
    }
    const int64_t offs[2] = {0, n};
    RECSDK_HIP_TRY(hipMemcpyAsync(h->oneOffset, offs, sizeof(offs), hipMemcpyHostToDevice, s));
    // INVALID_KEY (-1) is not looked up; its batch offset is 0 (OFFSET_OF_INVALID_KEY)
    int rc = recsdk_unique_run(h->uq, d_keys, nullptr, h->oneOffset, 1, n, 1, -1, stream);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const UniqueView* v = recsdk_unique_view(h->uq);
    const unsigned gridK = (unsigned)std::max<int64_t>(cdiv(n, kTile), 1);
    const unsigned gridS = (unsigned)cdiv(h->cacheSize - h->memStart, kTile);
    if (n > 0) {
        RECSDK_LAUNCH(k_swap_hit, dim3(gridK), dim3(kBlock), s, h->map, h->st, v->uniq, v->total, h->offOf, h->cacheVer,
                      h->miss, h->tileM, n);
    }
    RECSDK_LAUNCH(k_swap_miss_scan, dim3(1), dim3(kBlock), s, h->st, h->tileM, v->total, h->cacheSize, n);
    RECSDK_LAUNCH(k_swap_eligible, dim3(gridS), dim3(kBlock), s, h->st, h->cacheVer, h->memStart, h->cacheSize, h->tileE,
                  h->tileO);
    RECSDK_LAUNCH(k_swap_eligible_scan, dim3(1), dim3(kBlock), s, h->st, h->tileE, h->tileO, h->memStart, h->cacheSize);
    RECSDK_LAUNCH(k_swap_victims, dim3(gridS), dim3(kBlock), s, h->map, h->st, h->cacheKey, h->cacheVer, h->memStart,
                  h->cacheSize, h->tileE, h->tileO, h->victimSlot, d_swapout_keys, d_swapout_offs);
    if (n > 0) {
        RECSDK_LAUNCH(k_swap_assign, dim3(gridK), dim3(kBlock), s, h->map, h->st, v->uniq, v->total, h->miss, h->tileM,
                      h->victimSlot, h->offOf, h->cacheKey, h->cacheVer, d_swapin_keys, d_swapin_offs, n);
    }
    RECSDK_LAUNCH(k_swap_finish, dim3(1), dim3(64), s, h->st, h->counts);
    if (n > 0) {
        rc = recsdk_unique_expand(h->uq, h->offOf, 0, d_batch_offs, stream);
    }
    return rc;
}

extern "C" int recsdk_swap_counts(recsdk_swap_t* h, void* stream, int64_t* h_swapouts, int64_t* h_swapins,
                                  int64_t* h_occupied)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_swap_counts: NULL handle");
    hipStream_t s = static_cast<hipStream_t>(stream);
    SwapState st;
    int64_t counts[2];
    RECSDK_HIP_TRY(hipMemcpyAsync(&st, h->st, sizeof(st), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(counts, h->counts, sizeof(counts), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    if (h_swapouts) {
        *h_swapouts = counts[0];
    }
    if (h_swapins) {
        *h_swapins = counts[1];
    }
    if (h_occupied) {
        *h_occupied = st.occupied;
    }
    if (st.error) {
        set_error("cacheSize_ too small: the batch needs more slots than the sweep can free");
        return RECSDK_EOVERFLOW;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_swap_export(recsdk_swap_t* h, int64_t* d_cache_keys, void* stream)
{
    RECSDK_REQUIRE(h != nullptr && d_cache_keys != nullptr, RECSDK_ENULL, "recsdk_swap_export: NULL argument");
    RECSDK_HIP_TRY(hipMemcpyAsync(d_cache_keys, h->cacheKey, sizeof(int64_t) * h->cacheSize, hipMemcpyDeviceToDevice,
                                  static_cast<hipStream_t>(stream)));
    return RECSDK_OK;
}

extern "C" int recsdk_swap_remove(recsdk_swap_t* h, const int64_t* d_keys, int64_t n, void* stream)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_swap_remove: NULL handle");
    if (n <= 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_keys != nullptr, RECSDK_ENULL, "recsdk_swap_remove: d_keys is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    RECSDK_LAUNCH(k_swap_remove, dim3((unsigned)cdiv(n, kBlock)), dim3(kBlock), s, h->map, d_keys, n, h->cacheKey,
                  h->cacheVer);
    return RECSDK_OK;
}
