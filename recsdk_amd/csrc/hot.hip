// Hot-key staging of the restore vector.
//
// Sequential definition (training/tf_rec_v1/src/core/key_process/key_process.cpp: HotHashSplit :1218-1293,
// ComputeHotPos :963-985, UpdateHotMap :1334-1356): every table keeps a set of "hot" keys, refreshed every
// hotEmbUpdateStep batches to the hotCount most frequent keys of that batch.  Walking the batch in order, the first
// occurrence of a hot key takes the next hot position h = 0, 1, ... and hotPos[h] records where the key sits among
// the table's distinct keys; every occurrence of a hot key gets restore = h, every other key
// restore = (index among the distinct keys) + hotCount.  The hot rows can then be staged in a small dense prefix.
// Parallel form: the distinct keys come in first-occurrence order from the dedup kernels, so h is a scan over the
// "is hot" flags of the distinct keys, restarted at every table.
#include <algorithm>
#include <vector>

#include "common.h"
#include "dedup.h"
#include "hashmap.h"

namespace recsdk {

struct HotTable {
    MapRef set;        // hot keys of the table (value unused)
    int32_t hotCount;  // hotEmbTotCount: size of the hot prefix
    int32_t posOff;    // start of this table's entries in hot_pos
};

// hot flags of the distinct keys + per-tile counts
__global__ __launch_bounds__(kBlock) void k_hot_flag(const HotTable* __restrict__ tabs,
                                                     const int64_t* __restrict__ uniq,
                                                     const int64_t* __restrict__ uoff, int T,
                                                     const int64_t* __restrict__ total, uint8_t* __restrict__ flag,
                                                     uint32_t* __restrict__ tileH)
{
    __shared__ uint32_t red[kBlock / kWave];
    __shared__ int sT0;
    const int64_t U = total[0];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= U) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(uoff, T, tile0);
    }
    __syncthreads();
    int t = sT0;
    uint32_t f = 0;
    uint8_t fl[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t R = tile0 + (int64_t)threadIdx.x * kItems + k;
        fl[k] = 0;
        if (R < U) {
            t = advance_segment(uoff, t, R);
            const HotTable& h = tabs[t];
            if (h.hotCount > 0 && map_find(h.set, uniq[R]) >= 0) {
                fl[k] = 1;
                f += 1;
            }
        }
    }
    *reinterpret_cast<uchar4*>(flag + tile0 + (int64_t)threadIdx.x * kItems) = make_uchar4(fl[0], fl[1], fl[2], fl[3]);
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
        tileH[blockIdx.x] = s;
    }
}

// single block: exclusive scan of the tile counts; hotBase[t] = hot keys before table t; hot_pos starts as zeros
__global__ __launch_bounds__(kBlock) void k_hot_scan(uint32_t* tileH, const uint8_t* __restrict__ flag,
                                                     const int64_t* __restrict__ uoff, int T,
                                                     const int64_t* __restrict__ total, int64_t* __restrict__ hotBase,
                                                     int32_t* __restrict__ hotPos, int64_t hotPosLen)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carry;
    const int64_t U = total[0];
    const int64_t ntiles = (U + kTile - 1) / kTile;
    if (threadIdx.x == 0) {
        carry = 0;
    }
    __syncthreads();
    for (int64_t b = 0; b < ntiles; b += kBlock) {
        const int64_t j = b + threadIdx.x;
        const uint32_t v = (j < ntiles) ? tileH[j] : 0;
        uint32_t tot;
        const uint32_t e = block_exclusive_scan(v, smem, &tot);
        if (j < ntiles) {
            tileH[j] = carry + e;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            carry += tot;
        }
        __syncthreads();
    }
    segment_start_ranks(flag, tileH, uoff, T, U, carry, hotBase);
    for (int64_t j = threadIdx.x; j < hotPosLen; j += kBlock) {
        hotPos[j] = 0;
    }
}

// hot index of every distinct key (-1 = not hot) and hot_pos
__global__ __launch_bounds__(kBlock) void k_hot_emit(const HotTable* __restrict__ tabs,
                                                     const int64_t* __restrict__ uoff, int T,
                                                     const int64_t* __restrict__ total,
                                                     const uint8_t* __restrict__ flag,
                                                     const uint32_t* __restrict__ tileH,
                                                     const int64_t* __restrict__ hotBase,
                                                     int32_t* __restrict__ hotIdx, int32_t* __restrict__ hotPos)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ int sT0;
    const int64_t U = total[0];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= U) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(uoff, T, tile0);
    }
    const int64_t R0 = tile0 + (int64_t)threadIdx.x * kItems;
    const uchar4 f4 = *reinterpret_cast<const uchar4*>(flag + R0);
    const uint8_t fl[kItems] = {f4.x, f4.y, f4.z, f4.w};
    const uint32_t f = fl[0] + fl[1] + fl[2] + fl[3];
    uint32_t tot;
    int64_t r = (int64_t)block_exclusive_scan(f, smem, &tot) + tileH[blockIdx.x];  // includes a barrier: sT0 is set
    int t = sT0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t R = R0 + k;
        if (R >= U) {
            break;
        }
        int32_t h = -1;
        if (fl[k]) {
            t = advance_segment(uoff, t, R);
            const HotTable& tab = tabs[t];
            const int64_t hi = r - hotBase[t];
            // a table never holds more hot keys than its hot set, which is at most hotCount keys
            if (hi < tab.hotCount) {
                h = (int32_t)hi;
                hotPos[tab.posOff + hi] = (int32_t)(R - uoff[t]);
            }
            r += 1;
        }
        hotIdx[R] = h;
    }
}

__global__ __launch_bounds__(kBlock) void k_hot_restore(const HotTable* __restrict__ tabs,
                                                        const int64_t* __restrict__ off, int T,
                                                        const int32_t* __restrict__ grank,
                                                        const int32_t* __restrict__ inverse,
                                                        const int32_t* __restrict__ hotIdx,
                                                        int32_t* __restrict__ restore, int64_t n)
{
    __shared__ int sT0;
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, tile0);
    }
    __syncthreads();
    int t = sT0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t i = tile0 + k * kBlock + threadIdx.x;
        if (i >= n) {
            break;
        }
        const int32_t R = grank[i];
        int32_t v = -1;
        if (R >= 0) {
            t = advance_segment(off, t, i);
            const int32_t h = hotIdx[R];
            v = h >= 0 ? h : inverse[i] + tabs[t].hotCount;
        }
        restore[i] = v;
    }
}

__global__ __launch_bounds__(kBlock) void k_hot_set_clear(TableEntry* entries, int64_t count)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < count) {
        TableEntry e;
        e.key = kEmptyKey;
        e.slot = -1;
        entries[i] = e;
    }
}

__global__ __launch_bounds__(kBlock) void k_hot_set_fill(const HotTable* __restrict__ tabs,
                                                         const int64_t* __restrict__ keys,
                                                         const int32_t* __restrict__ tableOf, int64_t count)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < count) {
        map_insert(tabs[tableOf[i]].set, keys[i], 0);
    }
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_hot {
    int32_t T = 0;
    int64_t maxKeys = 0;
    int64_t hotTotal = 0;
    std::vector<HotTable> host;
    std::vector<int64_t> entryOff;  // start of each table's set inside `entries`
    int64_t entryCount = 0;
    HotTable* tabs = nullptr;
    TableEntry* entries = nullptr;
    uint8_t* flag = nullptr;
    uint32_t* tileH = nullptr;
    int64_t* hotBase = nullptr;
    int32_t* hotIdx = nullptr;
    int64_t* newKeys = nullptr;   // refresh staging (device)
    int32_t* newTable = nullptr;
};

extern "C" int recsdk_hot_destroy(recsdk_hot_t* h)
{
    if (h == nullptr) {
        return RECSDK_OK;
    }
    void* ptrs[] = {h->tabs, h->entries, h->flag, h->tileH, h->hotBase, h->hotIdx, h->newKeys, h->newTable};
    for (void* p : ptrs) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_hot_create(int32_t T, const int32_t* h_hot_counts, int64_t max_keys, recsdk_hot_t** out)
{
    RECSDK_REQUIRE(out != nullptr && h_hot_counts != nullptr, RECSDK_ENULL, "recsdk_hot_create: NULL argument");
    RECSDK_REQUIRE(T > 0 && T <= 65536 && max_keys > 0 && max_keys <= (int64_t(1) << 28), RECSDK_EINVAL,
                   "recsdk_hot_create: T must be in (0, 65536] and max_keys in (0, 2^28]");
    auto* h = new recsdk_hot();
    h->T = T;
    h->maxKeys = max_keys;
    h->host.resize(T);
    h->entryOff.resize(T);
    for (int t = 0; t < T; ++t) {
        if (h_hot_counts[t] < 0) {
            delete h;
            set_error("recsdk_hot_create: negative hot count");
            return RECSDK_EINVAL;
        }
        uint64_t cap = 16;
        while (cap < 2 * (uint64_t)h_hot_counts[t]) {
            cap <<= 1;
        }
        h->entryOff[t] = h->entryCount;
        h->entryCount += (int64_t)cap + 1;
        h->host[t].set.mask = cap - 1;
        h->host[t].hotCount = h_hot_counts[t];
        h->host[t].posOff = (int32_t)h->hotTotal;
        h->hotTotal += h_hot_counts[t];
    }
    bool ok = true;
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes ? bytes : 16) != hipSuccess) {
            ok = false;
        }
    };
    const int64_t padded = cdiv(max_keys, kTile) * kTile;
    alloc(&h->tabs, sizeof(HotTable) * T);
    alloc(&h->entries, sizeof(TableEntry) * h->entryCount);
    alloc(&h->flag, padded);
    alloc(&h->tileH, sizeof(uint32_t) * (padded / kTile + 1));
    alloc(&h->hotBase, sizeof(int64_t) * (T + 1));
    alloc(&h->hotIdx, sizeof(int32_t) * padded);
    alloc(&h->newKeys, sizeof(int64_t) * std::max<int64_t>(h->hotTotal, 1));
    alloc(&h->newTable, sizeof(int32_t) * std::max<int64_t>(h->hotTotal, 1));
    if (ok) {
        for (int t = 0; t < T; ++t) {
            h->host[t].set.entries = h->entries + h->entryOff[t];
        }
        // all-ones bytes: empty sets (no key is hot before the first refresh, hotKey starts empty)
        ok = hipMemset(h->entries, 0xFF, sizeof(TableEntry) * h->entryCount) == hipSuccess &&
             hipMemcpy(h->tabs, h->host.data(), sizeof(HotTable) * T, hipMemcpyHostToDevice) == hipSuccess;
    }
    if (!ok) {
        (void)hipGetLastError();
        recsdk_hot_destroy(h);
        set_error("recsdk_hot_create: allocation failed");
        return RECSDK_ENOMEM;
    }
    *out = h;
    return RECSDK_OK;
}

extern "C" int recsdk_hot_split(recsdk_hot_t* h, recsdk_unique_t* u, int32_t* d_restore, int32_t* d_hot_pos,
                                int32_t refresh, void* stream)
{
    RECSDK_REQUIRE(h != nullptr && u != nullptr && d_restore != nullptr && (h->hotTotal == 0 || d_hot_pos != nullptr),
                   RECSDK_ENULL, "recsdk_hot_split: NULL argument");
    const UniqueView* v = recsdk_unique_view(u);
    RECSDK_REQUIRE(v->T == h->T, RECSDK_EINVAL, "recsdk_hot_split: table count of the hot sets and the unique run differ");
    RECSDK_REQUIRE(v->n <= h->maxKeys, RECSDK_ECAPACITY, "recsdk_hot_split: the unique run is larger than max_keys");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t n = v->n;
    const unsigned grid = (unsigned)std::max<int64_t>(cdiv(n, kTile), 1);
    if (n > 0) {
        RECSDK_LAUNCH(k_hot_flag, dim3(grid), dim3(kBlock), s, h->tabs, v->uniq, v->uoff, v->T, v->total, h->flag,
                      h->tileH);
    }
    RECSDK_LAUNCH(k_hot_scan, dim3(1), dim3(kBlock), s, h->tileH, h->flag, v->uoff, v->T, v->total, h->hotBase, d_hot_pos,
                  h->hotTotal);
    if (n > 0) {
        RECSDK_LAUNCH(k_hot_emit, dim3(grid), dim3(kBlock), s, h->tabs, v->uoff, v->T, v->total, h->flag, h->tileH,
                      h->hotBase, h->hotIdx, d_hot_pos);
        RECSDK_LAUNCH(k_hot_restore, dim3(grid), dim3(kBlock), s, h->tabs, v->off, v->T, v->grank, v->inverse, h->hotIdx,
                      d_restore, n);
    }
    if (!refresh || h->hotTotal == 0) {
        return RECSDK_OK;
    }
    // UpdateHotMap: the hotCount most frequent keys of this batch, ties to the smaller key.  Rare (every
    // hotEmbUpdateStep batches) and small: selected on the host, like the reference does.
    int64_t U = 0;
    RECSDK_HIP_TRY(recsdk_unique_wait_counts(v, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(&U, v->total, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    std::vector<int64_t> keys((size_t)U);
    std::vector<uint32_t> counts((size_t)U);
    std::vector<int64_t> uoff((size_t)h->T + 1);
    if (U > 0) {
        RECSDK_HIP_TRY(hipMemcpyAsync(keys.data(), v->uniq, sizeof(int64_t) * U, hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipMemcpyAsync(counts.data(), v->ucount, sizeof(uint32_t) * U, hipMemcpyDeviceToHost, s));
    }
    RECSDK_HIP_TRY(hipMemcpyAsync(uoff.data(), v->uoff, sizeof(int64_t) * (h->T + 1), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    std::vector<int64_t> newKeys;
    std::vector<int32_t> newTable;
    std::vector<int64_t> order;
    for (int t = 0; t < h->T; ++t) {
        const int64_t b = uoff[t];
        const int64_t e = uoff[t + 1];
        const int64_t want = std::min<int64_t>(h->host[t].hotCount, e - b);
        if (want <= 0) {
            continue;
        }
        order.resize((size_t)(e - b));
        for (int64_t j = 0; j < e - b; ++j) {
            order[(size_t)j] = b + j;
        }
        auto better = [&](int64_t x, int64_t y) {
            return counts[(size_t)x] != counts[(size_t)y] ? counts[(size_t)x] > counts[(size_t)y]
                                                           : keys[(size_t)x] < keys[(size_t)y];
        };
        std::partial_sort(order.begin(), order.begin() + want, order.end(), better);
        for (int64_t j = 0; j < want; ++j) {
            newKeys.push_back(keys[(size_t)order[(size_t)j]]);
            newTable.push_back(t);
        }
    }
    RECSDK_LAUNCH(k_hot_set_clear, dim3((unsigned)cdiv(h->entryCount, kBlock)), dim3(kBlock), s, h->entries,
                  h->entryCount);
    const int64_t m = (int64_t)newKeys.size();
    if (m > 0) {
        RECSDK_HIP_TRY(hipMemcpyAsync(h->newKeys, newKeys.data(), sizeof(int64_t) * m, hipMemcpyHostToDevice, s));
        RECSDK_HIP_TRY(hipMemcpyAsync(h->newTable, newTable.data(), sizeof(int32_t) * m, hipMemcpyHostToDevice, s));
        RECSDK_LAUNCH(k_hot_set_fill, dim3((unsigned)cdiv(m, kBlock)), dim3(kBlock), s, h->tabs, h->newKeys, h->newTable,
                      m);
        RECSDK_HIP_TRY(hipStreamSynchronize(s));  // the staging vectors go out of scope
    }
    return RECSDK_OK;
}
