// Multi-table key dedup in first-occurrence order (unique + inverse + counts) and the
// per-distinct-key position lists used by the gradient segment-reduce.
//
// Algorithm (all tables in one set of launches, n = total keys):
//   plan     per table: scratch hash region of pow2 >= 2*n_t slots (+1 side slot for the key that equals
//            the empty marker)
//   insert   every key CAS-claims a scratch slot; atomicMin keeps the smallest global index ("first"),
//            atomicAdd the multiplicity
//   flags    is_first[i] = (first(slot_i) == i); per-tile sums of flags and of multiplicities
//   tilescan single block: exclusive scan of the tile sums; unique_offsets[t] = rank at the table start
//   emit     per tile rescan: rank R of every first occurrence -> unique_keys[R], counts[R], seg_start[R];
//            the rank is written back into the scratch slot; keys seen more than kListMax times are
//            appended to the long list
//   inverse  inverse[i] = R(slot_i) - unique_offsets[t]; positions of keys seen 2..kListMax times are
//            appended (unordered) to pos_list[seg_start[R] ...]
//   finalize one wave per key seen at least twice puts its position list in ascending order
// Ranks come from a scan over key positions, so the order of distinct keys is the order of first
// occurrence regardless of how the CAS races resolve.
#include <algorithm>

#include "common.h"
#include "dedup.h"

namespace recsdk {

struct __attribute__((aligned(16))) DedupEntry {
    long long key;
    uint32_t first;
    uint32_t count;
};

__global__ __launch_bounds__(kBlock) void k_dedup_plan(const int64_t* __restrict__ off, int T, int64_t* sbase,
                                                       uint32_t* smask, uint32_t* counters)
{
    // single thread; T is small
    if (threadIdx.x == 0) {
        counters[0] = 0;  // number of keys seen more than kListMax times
        counters[1] = 0;  // number of keys seen 2..kListMax times
        int64_t base = 0;
        for (int t = 0; t < T; ++t) {
            int64_t nt = off[t + 1] - off[t];
            uint64_t cap = 64;
            while ((int64_t)cap < 2 * nt) {
                cap <<= 1;
            }
            sbase[t] = base;
            smask[t] = (uint32_t)(cap - 1);
            base += (int64_t)cap + 1;
        }
        sbase[T] = base;
    }
}

__global__ __launch_bounds__(kBlock) void k_dedup_clear(DedupEntry* S, const int64_t* __restrict__ sbase, int T)
{
    int64_t total = sbase[T];
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * kBlock;
    DedupEntry e;
    e.key = kEmptyKey;
    e.first = 0xFFFFFFFFu;
    e.count = 0;
    for (; i < total; i += stride) {
        S[i] = e;
    }
}

// Device-wide claim of a scratch slot for `key` in region R (capacity mask+1, side slot at mask+1).
__device__ __forceinline__ uint32_t scratch_claim(DedupEntry* R, uint32_t mask, long long key)
{
    if (key == kEmptyKey) {
        return mask + 1;  // side slot: only this key lands here, no claim needed
    }
    uint32_t pos = (uint32_t)hash64((uint64_t)key) & mask;
    while (true) {
        long long cur = __hip_atomic_load(&R[pos].key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (cur == key) {
            return pos;
        }
        if (cur == kEmptyKey) {
            unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&R[pos].key),
                                                (unsigned long long)kEmptyKey, (unsigned long long)key);
            if ((long long)prev == kEmptyKey || (long long)prev == key) {
                return pos;
            }
        }
        pos = (pos + 1) & mask;
    }
}

constexpr int kLdsSlots = 2 * kTile;  // block-local hash: load factor <= 0.5

// A block first merges its 1024 keys in an LDS hash (first index, multiplicity), then touches the device-wide
// scratch once per distinct key of the block.  A key seen thousands of times therefore costs one pair of
// device atomics per block instead of one pair per occurrence.
__global__ __launch_bounds__(kBlock) void k_dedup_insert(const int64_t* __restrict__ keys,
                                                         const uint32_t* __restrict__ inCounts,
                                                         const int64_t* __restrict__ off, int T,
                                                         const int64_t* __restrict__ sbase,
                                                         const uint32_t* __restrict__ smask, DedupEntry* S,
                                                         int32_t* __restrict__ sslot, int64_t nMax, int skipEnabled,
                                                         long long skipKey)
{
    __shared__ DedupEntry L[kLdsSlots + 1];
    __shared__ int sT0;
    __shared__ int sT1;
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, tile0);
        int64_t last = tile0 + kTile - 1 < n ? tile0 + kTile - 1 : n - 1;
        sT1 = find_segment(off, T, last);
    }
    for (int e = threadIdx.x; e <= kLdsSlots; e += kBlock) {
        L[e].key = kEmptyKey;
        L[e].first = 0xFFFFFFFFu;
        L[e].count = 0;
    }
    __syncthreads();
    int t = sT0;
    if (sT0 != sT1) {
        // the tile straddles tables: every key goes to the device-wide scratch directly
#pragma unroll
        for (int k = 0; k < kItems; ++k) {
            int64_t i = tile0 + k * kBlock + threadIdx.x;
            if (i >= n) {
                break;
            }
            long long key = keys[i];
            if (skipEnabled && key == skipKey) {
                sslot[i] = -1;
                continue;
            }
            t = advance_segment(off, t, i);
            DedupEntry* R = S + sbase[t];
            uint32_t pos = scratch_claim(R, smask[t], key);
            atomicMin(&R[pos].first, (uint32_t)i);
            atomicAdd(&R[pos].count, inCounts ? inCounts[i] : 1u);
            sslot[i] = (int32_t)(sbase[t] + pos);
        }
        return;
    }
    // phase 1: merge in LDS
    int lpos[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t i = tile0 + k * kBlock + threadIdx.x;
        lpos[k] = -1;
        if (i >= n) {
            continue;
        }
        long long key = keys[i];
        if (skipEnabled && key == skipKey) {
            continue;
        }
        uint32_t pos;
        if (key == kEmptyKey) {
            pos = kLdsSlots;
        } else {
            pos = (uint32_t)(hash64((uint64_t)key) >> 32) & (kLdsSlots - 1);
            while (true) {
                unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&L[pos].key),
                                                    (unsigned long long)kEmptyKey, (unsigned long long)key);
                if ((long long)prev == kEmptyKey || (long long)prev == key) {
                    break;
                }
                pos = (pos + 1) & (kLdsSlots - 1);
            }
        }
        atomicMin(&L[pos].first, (uint32_t)i);
        atomicAdd(&L[pos].count, inCounts ? inCounts[i] : 1u);
        lpos[k] = (int)pos;
    }
    __syncthreads();
    // phase 2: one device-wide update per distinct key of the block; the LDS entry then holds the scratch slot
    {
        DedupEntry* R = S + sbase[t];
        const uint32_t mask = smask[t];
        const int64_t base = sbase[t];
        for (int e = threadIdx.x; e <= kLdsSlots; e += kBlock) {
            const uint32_t first = L[e].first;
            if (first == 0xFFFFFFFFu) {
                continue;
            }
            const long long key = (e == kLdsSlots) ? kEmptyKey : L[e].key;
            uint32_t pos = scratch_claim(R, mask, key);
            atomicMin(&R[pos].first, first);
            atomicAdd(&R[pos].count, L[e].count);
            L[e].first = (uint32_t)(base + pos);
        }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t i = tile0 + k * kBlock + threadIdx.x;
        if (i < n) {
            sslot[i] = (lpos[k] >= 0) ? (int32_t)L[lpos[k]].first : -1;
        }
    }
}

// flags + tile sums.  Items are thread-contiguous here (4 consecutive keys per thread) to match k_dedup_emit.
__global__ __launch_bounds__(kBlock) void k_dedup_flags(const DedupEntry* __restrict__ S,
                                                        const int32_t* __restrict__ sslot,
                                                        const int64_t* __restrict__ off, int T,
                                                        uint8_t* __restrict__ isFirst, uint32_t* __restrict__ tileF,
                                                        uint32_t* __restrict__ tileC, int64_t nMax)
{
    __shared__ uint32_t red[2 * kBlock / kWave];
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    uint32_t f = 0;
    uint32_t c = 0;
    uint8_t fl[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t i = tile0 + (int64_t)threadIdx.x * kItems + k;
        fl[k] = 0;
        if (i < n) {
            int32_t pos = sslot[i];
            if (pos >= 0) {
                DedupEntry e = S[pos];
                if (e.first == (uint32_t)i) {
                    fl[k] = 1;
                    f += 1;
                    c += e.count;
                }
            }
        }
    }
    *reinterpret_cast<uchar4*>(isFirst + tile0 + (int64_t)threadIdx.x * kItems) = make_uchar4(fl[0], fl[1], fl[2], fl[3]);
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
        f += __shfl_down(f, d, kWave);
        c += __shfl_down(c, d, kWave);
    }
    int w = threadIdx.x >> 6;
    if (lane_id() == 0) {
        red[w] = f;
        red[kBlock / kWave + w] = c;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t sf = 0;
        uint32_t sc = 0;
        for (int k = 0; k < kBlock / kWave; ++k) {
            sf += red[k];
            sc += red[kBlock / kWave + k];
        }
        tileF[blockIdx.x] = sf;
        tileC[blockIdx.x] = sc;
    }
}

// single block: exclusive scan of the tile sums (in place) and unique_offsets.
__global__ __launch_bounds__(kBlock) void k_dedup_tilescan(uint32_t* tileF, uint32_t* tileC,
                                                           const uint8_t* __restrict__ isFirst,
                                                           const int64_t* __restrict__ off, int T, int64_t* uoff,
                                                           int64_t* totals, int64_t nMax)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carryF;
    __shared__ uint32_t carryC;
    const int64_t n = off[T] < nMax ? off[T] : nMax;
    const int64_t ntiles = (n + kTile - 1) / kTile;
    if (threadIdx.x == 0) {
        carryF = 0;
        carryC = 0;
    }
    __syncthreads();
    for (int64_t b = 0; b < ntiles; b += kBlock) {
        int64_t j = b + threadIdx.x;
        uint32_t vf = (j < ntiles) ? tileF[j] : 0;
        uint32_t vc = (j < ntiles) ? tileC[j] : 0;
        uint32_t tf;
        uint32_t tc;
        uint32_t ef = block_exclusive_scan(vf, smem, &tf);
        uint32_t ec = block_exclusive_scan(vc, smem, &tc);
        if (j < ntiles) {
            tileF[j] = carryF + ef;
            tileC[j] = carryC + ec;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            carryF += tf;
            carryC += tc;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        totals[0] = carryF;  // U
    }
    // rank at each table's first key: tile base + flags before it inside its tile (one wave per table)
    for (int t = threadIdx.x >> 6; t <= T; t += kBlock / kWave) {
        const int64_t o = off[t];
        int64_t r;
        if (o >= n) {
            r = carryF;
        } else {
            const int64_t tile = o / kTile;
            uint32_t part = 0;
            for (int64_t i = tile * kTile + lane_id(); i < o; i += kWave) {
                part += isFirst[i];
            }
#pragma unroll
            for (int dlt = kWave / 2; dlt > 0; dlt >>= 1) {
                part += __shfl_down(part, dlt, kWave);
            }
            r = (int64_t)tileF[tile] + __shfl(part, 0, kWave);
        }
        if (lane_id() == 0) {
            uoff[t] = r;
        }
    }
}

__global__ __launch_bounds__(kBlock) void k_dedup_emit(DedupEntry* S, const int32_t* __restrict__ sslot,
                                                       const int64_t* __restrict__ keys,
                                                       const int64_t* __restrict__ off, int T,
                                                       const uint8_t* __restrict__ isFirst,
                                                       const uint32_t* __restrict__ tileF,
                                                       const uint32_t* __restrict__ tileC,
                                                       int64_t* __restrict__ uniq, uint32_t* __restrict__ ucount,
                                                       uint32_t* __restrict__ useg, int32_t* __restrict__ longList,
                                                       int32_t* __restrict__ midList, uint32_t* counters,
                                                       int64_t nMax, int buildLists)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t sBase[2];
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    const int64_t i0 = tile0 + (int64_t)threadIdx.x * kItems;
    uchar4 f4 = *reinterpret_cast<const uchar4*>(isFirst + i0);
    uint8_t fl[kItems] = {f4.x, f4.y, f4.z, f4.w};
    uint32_t cnt[kItems];
    int32_t pos[kItems];
    uint32_t f = 0;
    uint32_t c = 0;
    uint32_t lm = 0;  // low 16 bits: keys seen 2..kListMax times, high 16 bits: keys seen more often
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        cnt[k] = 0;
        pos[k] = -1;
        if (fl[k]) {
            pos[k] = sslot[i0 + k];
            cnt[k] = S[pos[k]].count;
            f += 1;
            c += cnt[k];
            if (cnt[k] > (uint32_t)kListMax) {
                lm += 1u << 16;
            } else if (cnt[k] > 1) {
                lm += 1u;
            }
        }
    }
    uint32_t tf;
    uint32_t tc;
    uint32_t tl;
    uint32_t rf = block_exclusive_scan(f, smem, &tf) + tileF[blockIdx.x];
    uint32_t rc = block_exclusive_scan(c, smem, &tc) + tileC[blockIdx.x];
    uint32_t rl = buildLists ? block_exclusive_scan(lm, smem, &tl) : 0;
    if (buildLists) {
        if (threadIdx.x == 0) {
            sBase[0] = (tl >> 16) ? atomicAdd(&counters[0], tl >> 16) : 0;
            sBase[1] = (tl & 0xffffu) ? atomicAdd(&counters[1], tl & 0xffffu) : 0;
        }
        __syncthreads();
    }
    uint32_t longAt = buildLists ? sBase[0] + (rl >> 16) : 0;
    uint32_t midAt = buildLists ? sBase[1] + (rl & 0xffffu) : 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (fl[k]) {
            uniq[rf] = keys[i0 + k];
            ucount[rf] = cnt[k];
            useg[rf] = rc;
            S[pos[k]].first = rf;
            if (buildLists) {
                if (cnt[k] > (uint32_t)kListMax) {
                    longList[longAt++] = (int32_t)rf;
                } else if (cnt[k] > 1) {
                    midList[midAt++] = (int32_t)rf;
                }
            }
            rf += 1;
            rc += cnt[k];
        }
    }
}

__global__ __launch_bounds__(kBlock) void k_dedup_inverse(DedupEntry* S, const int32_t* __restrict__ sslot,
                                                          const int64_t* __restrict__ off, int T,
                                                          const int64_t* __restrict__ uoff,
                                                          const uint32_t* __restrict__ ucount,
                                                          const uint32_t* __restrict__ useg,
                                                          int32_t* __restrict__ inverse, int32_t* __restrict__ grank,
                                                          int32_t* __restrict__ posList, int64_t nMax, int buildLists)
{
    __shared__ int sT0;
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, tile0);
    }
    __syncthreads();
    int t = sT0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t i = tile0 + k * kBlock + threadIdx.x;
        if (i >= n) {
            break;
        }
        int32_t pos = sslot[i];
        if (pos < 0) {
            inverse[i] = -1;
            grank[i] = -1;
            continue;
        }
        t = advance_segment(off, t, i);
        uint32_t R = S[pos].first;
        inverse[i] = (int32_t)((int64_t)R - uoff[t]);
        grank[i] = (int32_t)R;
        if (buildLists) {
            uint32_t c = ucount[R];
            if (c == 1) {
                posList[useg[R]] = (int32_t)i;
            } else if (c <= (uint32_t)kListMax) {
                uint32_t old = atomicSub(&S[pos].count, 1u);
                posList[useg[R] + old - 1] = (int32_t)i;
            }
        }
    }
}

// Puts every key's position list in ascending order.  A block takes either
//   one key seen more than kListMax times: its four waves each count the key's occurrences in a quarter of the
//     table's rank array, exchange the counts, then compact the matching positions in index order into
//     pos_list[seg_start[R] ...] (nothing was appended for these keys before); or
//   four keys seen 2..kListMax times: each wave sorts the unordered list it finds (rank + scatter).
__global__ __launch_bounds__(kBlock) void k_dedup_finalize_lists(const int32_t* __restrict__ longList,
                                                                 const int32_t* __restrict__ midList,
                                                                 const uint32_t* __restrict__ counters,
                                                                 const int64_t* __restrict__ off, int T,
                                                                 const int64_t* __restrict__ uoff,
                                                                 const uint32_t* __restrict__ ucount,
                                                                 const uint32_t* __restrict__ useg,
                                                                 const int32_t* __restrict__ grank,
                                                                 int32_t* __restrict__ posList)
{
    constexpr int kWaves = kBlock / kWave;
    constexpr int kUn = 8;
    __shared__ uint32_t sCnt[kWaves];
    const uint32_t nLong = counters[0];
    const uint32_t nMid = counters[1];
    const uint32_t items = nLong + (nMid + kWaves - 1) / kWaves;
    const int lane = lane_id();
    const int w = threadIdx.x >> 6;
    for (uint32_t item = blockIdx.x; item < items; item += gridDim.x) {
        if (item < nLong) {
            const int32_t R = longList[item];
            const int t = find_segment(uoff, T, (int64_t)R);
            const int64_t o = off[t];
            const int64_t nt = off[t + 1] - o;
            const int32_t* src = grank + o;
            // quarter [qb, qe) of the table, in whole steps of kUn*64 positions
            const int64_t step = kUn * kWave;
            const int64_t stepsTotal = (nt + step - 1) / step;
            const int64_t qb = (stepsTotal * w / kWaves) * step;
            const int64_t qe = min(nt, (stepsTotal * (w + 1) / kWaves) * step);
            uint32_t mine = 0;
            for (int64_t base = qb; base < qe; base += step) {
                int32_t v[kUn];
#pragma unroll
                for (int k = 0; k < kUn; ++k) {
                    int64_t j = base + k * kWave + lane;
                    v[k] = (j < qe) ? src[j] : -2;
                }
#pragma unroll
                for (int k = 0; k < kUn; ++k) {
                    mine += (v[k] == R) ? 1u : 0u;
                }
            }
#pragma unroll
            for (int d = kWave / 2; d > 0; d >>= 1) {
                mine += __shfl_down(mine, d, kWave);
            }
            if (lane == 0) {
                sCnt[w] = mine;
            }
            __syncthreads();
            uint32_t cursor = 0;
            for (int k = 0; k < w; ++k) {
                cursor += sCnt[k];
            }
            __syncthreads();
            int32_t* dst = posList + useg[R];
            for (int64_t base = qb; base < qe; base += step) {
                int32_t v[kUn];
#pragma unroll
                for (int k = 0; k < kUn; ++k) {
                    int64_t j = base + k * kWave + lane;
                    v[k] = (j < qe) ? src[j] : -2;
                }
#pragma unroll
                for (int k = 0; k < kUn; ++k) {
                    const bool hit = (v[k] == R);
                    const unsigned long long m = __ballot(hit);
                    if (hit) {
                        uint32_t before = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                                                    __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                        dst[cursor + before] = (int32_t)(o + base + k * kWave + lane);
                    }
                    cursor += (uint32_t)__popcll(m);
                }
            }
        } else {
            const uint32_t mi = (item - nLong) * kWaves + w;
            if (mi < nMid) {
                const int32_t R = midList[mi];
                const uint32_t c = ucount[R];
                int32_t* list = posList + useg[R];
                int32_t p = (lane < (int)c) ? list[lane] : 0x7fffffff;
                int rank = 0;
                for (uint32_t j = 0; j < c; ++j) {
                    int32_t pj = __builtin_amdgcn_readlane(p, __builtin_amdgcn_readfirstlane(j));
                    rank += (pj < p) ? 1 : 0;
                }
                if (lane < (int)c) {
                    list[rank] = p;
                }
            }
        }
    }
}

// out[i] = values[index of key i among the distinct keys] (fill for skipped keys)
__global__ __launch_bounds__(kBlock) void k_dedup_expand(const int32_t* __restrict__ grank,
                                                         const int64_t* __restrict__ values, long long fill,
                                                         int64_t* __restrict__ out, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) {
        const int32_t R = grank[i];
        out[i] = (R >= 0) ? values[R] : fill;
    }
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_unique {
    int64_t maxKeys = 0;
    int32_t maxTables = 0;
    // workspace
    DedupEntry* S = nullptr;
    int32_t* sslot = nullptr;
    uint8_t* isFirst = nullptr;
    uint32_t* tileF = nullptr;
    uint32_t* tileC = nullptr;
    int64_t* sbase = nullptr;
    uint32_t* smask = nullptr;
    uint32_t* counters = nullptr;
    int64_t* totals = nullptr;
    // results
    UniqueView view;
};

static void unique_free(recsdk_unique* u)
{
    void* ptrs[] = {u->S, u->sslot, u->isFirst, u->tileF, u->tileC, u->sbase, u->smask, u->counters, u->totals,
                    (void*)u->view.uniq, (void*)u->view.uoff, (void*)u->view.inverse, (void*)u->view.grank,
                    (void*)u->view.ucount, (void*)u->view.useg, (void*)u->view.posList, (void*)u->view.longList, (void*)u->view.midList};
    for (void* p : ptrs) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
}

extern "C" int recsdk_unique_create(int64_t max_keys, int32_t max_tables, recsdk_unique_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_unique_create: out is NULL");
    RECSDK_REQUIRE(max_keys > 0 && max_keys <= (int64_t(1) << 28), RECSDK_EINVAL,
                   "recsdk_unique_create: max_keys must be in (0, 2^28]");
    RECSDK_REQUIRE(max_tables > 0 && max_tables <= 65536, RECSDK_EINVAL,
                   "recsdk_unique_create: max_tables must be in (0, 65536]");
    auto* u = new recsdk_unique();
    u->maxKeys = max_keys;
    u->maxTables = max_tables;
    const int64_t padded = cdiv(max_keys, kTile) * kTile;
    const int64_t ntiles = padded / kTile;
    const int64_t entries = 4 * max_keys + 65 * (int64_t)max_tables;
    bool ok = true;
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes ? bytes : 16) != hipSuccess) {
            ok = false;
        }
    };
    alloc(&u->S, sizeof(DedupEntry) * entries);
    alloc(&u->sslot, sizeof(int32_t) * padded);
    alloc(&u->isFirst, padded);
    alloc(&u->tileF, sizeof(uint32_t) * (ntiles + 1));
    alloc(&u->tileC, sizeof(uint32_t) * (ntiles + 1));
    alloc(&u->sbase, sizeof(int64_t) * (max_tables + 1));
    alloc(&u->smask, sizeof(uint32_t) * (max_tables + 1));
    alloc(&u->counters, sizeof(uint32_t) * 4);
    alloc(&u->totals, sizeof(int64_t) * 4);
    alloc(&u->view.uniq, sizeof(int64_t) * padded);
    alloc(&u->view.uoff, sizeof(int64_t) * (max_tables + 1));
    alloc(&u->view.inverse, sizeof(int32_t) * padded);
    alloc(&u->view.grank, sizeof(int32_t) * padded);
    alloc(&u->view.ucount, sizeof(uint32_t) * padded);
    alloc(&u->view.useg, sizeof(uint32_t) * padded);
    alloc(&u->view.posList, sizeof(int32_t) * padded);
    alloc(&u->view.longList, sizeof(int32_t) * (max_keys / kListMax + 2));
    alloc(&u->view.midList, sizeof(int32_t) * (max_keys / 2 + 2));
    if (!ok) {
        (void)hipGetLastError();
        unique_free(u);
        delete u;
        set_error("recsdk_unique_create: hipMalloc failed for %lld keys", (long long)max_keys);
        return RECSDK_ENOMEM;
    }
    u->view.nLong = u->counters;
    u->view.total = u->totals;
    *out = u;
    return RECSDK_OK;
}

extern "C" int recsdk_unique_destroy(recsdk_unique_t* u)
{
    if (u == nullptr) {
        return RECSDK_OK;
    }
    unique_free(u);
    delete u;
    return RECSDK_OK;
}

extern "C" int recsdk_unique_run(recsdk_unique_t* u, const int64_t* d_keys, const uint32_t* d_in_counts,
                                 const int64_t* d_offsets, int32_t T, int64_t n, int32_t skip_key_enabled,
                                 int64_t skip_key, void* stream)
{
    RECSDK_REQUIRE(u != nullptr && d_offsets != nullptr, RECSDK_ENULL, "recsdk_unique_run: NULL argument");
    RECSDK_REQUIRE(T > 0 && T <= u->maxTables, RECSDK_ECAPACITY, "recsdk_unique_run: T exceeds the handle's max_tables");
    RECSDK_REQUIRE(n >= 0 && n <= u->maxKeys, RECSDK_ECAPACITY, "recsdk_unique_run: n exceeds the handle's max_keys");
    RECSDK_REQUIRE(n == 0 || d_keys != nullptr, RECSDK_ENULL, "recsdk_unique_run: d_keys is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    UniqueView& v = u->view;
    v.keys = d_keys;
    v.off = d_offsets;
    v.T = T;
    v.n = n;
    v.hasLists = (d_in_counts == nullptr);
    const int64_t ntiles = cdiv(n, kTile);
    const unsigned grid = (unsigned)(ntiles > 0 ? ntiles : 1);
    RECSDK_LAUNCH(k_dedup_plan, dim3(1), dim3(kBlock), s, d_offsets, T, u->sbase, u->smask, u->counters);
    RECSDK_LAUNCH_CHECK();
    {
        int64_t entries = 4 * n + 65 * (int64_t)T;
        unsigned cg = (unsigned)std::min<int64_t>(cdiv(entries, kBlock), 256 * 32);
        RECSDK_LAUNCH(k_dedup_clear, dim3(cg), dim3(kBlock), s, u->S, u->sbase, T);
        RECSDK_LAUNCH_CHECK();
    }
    if (n > 0) {
        RECSDK_LAUNCH(k_dedup_insert, dim3(grid), dim3(kBlock), s, d_keys, d_in_counts, d_offsets, T, u->sbase,
                           u->smask, u->S, u->sslot, n, skip_key_enabled, (long long)skip_key);
        RECSDK_LAUNCH_CHECK();
        RECSDK_LAUNCH(k_dedup_flags, dim3(grid), dim3(kBlock), s, u->S, u->sslot, d_offsets, T, u->isFirst,
                           u->tileF, u->tileC, n);
        RECSDK_LAUNCH_CHECK();
    }
    RECSDK_LAUNCH(k_dedup_tilescan, dim3(1), dim3(kBlock), s, u->tileF, u->tileC, u->isFirst, d_offsets, T,
                       v.uoff, u->totals, n);
    RECSDK_LAUNCH_CHECK();
    if (n > 0) {
        RECSDK_LAUNCH(k_dedup_emit, dim3(grid), dim3(kBlock), s, u->S, u->sslot, d_keys, d_offsets, T,
                           u->isFirst, u->tileF, u->tileC, v.uniq, v.ucount, v.useg, v.longList, v.midList, u->counters, n, v.hasLists ? 1 : 0);
        RECSDK_LAUNCH_CHECK();
        RECSDK_LAUNCH(k_dedup_inverse, dim3(grid), dim3(kBlock), s, u->S, u->sslot, d_offsets, T, v.uoff,
                           v.ucount, v.useg, v.inverse, v.grank, v.posList, n, v.hasLists ? 1 : 0);
        RECSDK_LAUNCH_CHECK();
        if (v.hasLists && n > 1) {
            unsigned lg = (unsigned)std::min<int64_t>(n / kListMax + 1 + cdiv(n / 2 + 1, kBlock / kWave), 8192);
            RECSDK_LAUNCH(k_dedup_finalize_lists, dim3(lg), dim3(kBlock), s, v.longList, v.midList, u->counters,
                          d_offsets, T, v.uoff, v.ucount, v.useg, v.grank, v.posList);
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_unique_results(recsdk_unique_t* u, const int64_t** d_unique_keys,
                                     const int64_t** d_unique_offsets, const int32_t** d_inverse,
                                     const uint32_t** d_counts)
{
    RECSDK_REQUIRE(u != nullptr, RECSDK_ENULL, "recsdk_unique_results: NULL handle");
    if (d_unique_keys) {
        *d_unique_keys = u->view.uniq;
    }
    if (d_unique_offsets) {
        *d_unique_offsets = u->view.uoff;
    }
    if (d_inverse) {
        *d_inverse = u->view.inverse;
    }
    if (d_counts) {
        *d_counts = u->view.ucount;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_unique_fetch(recsdk_unique_t* u, int64_t* d_unique_keys, int64_t* d_unique_offsets,
                                   int32_t* d_inverse, uint32_t* d_counts, void* stream)
{
    RECSDK_REQUIRE(u != nullptr, RECSDK_ENULL, "recsdk_unique_fetch: NULL handle");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const UniqueView& v = u->view;
    if (d_unique_offsets) {
        RECSDK_HIP_TRY(hipMemcpyAsync(d_unique_offsets, v.uoff, sizeof(int64_t) * (v.T + 1), hipMemcpyDeviceToDevice, s));
    }
    if (v.n == 0) {
        return RECSDK_OK;
    }
    if (d_unique_keys) {
        RECSDK_HIP_TRY(hipMemcpyAsync(d_unique_keys, v.uniq, sizeof(int64_t) * v.n, hipMemcpyDeviceToDevice, s));
    }
    if (d_inverse) {
        RECSDK_HIP_TRY(hipMemcpyAsync(d_inverse, v.inverse, sizeof(int32_t) * v.n, hipMemcpyDeviceToDevice, s));
    }
    if (d_counts) {
        RECSDK_HIP_TRY(hipMemcpyAsync(d_counts, v.ucount, sizeof(uint32_t) * v.n, hipMemcpyDeviceToDevice, s));
    }
    return RECSDK_OK;
}

extern "C" int recsdk_unique_expand(recsdk_unique_t* u, const int64_t* d_values, int64_t fill, int64_t* d_out,
                                    void* stream)
{
    RECSDK_REQUIRE(u != nullptr, RECSDK_ENULL, "recsdk_unique_expand: NULL handle");
    const UniqueView& v = u->view;
    if (v.n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_values != nullptr && d_out != nullptr, RECSDK_ENULL, "recsdk_unique_expand: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    RECSDK_LAUNCH(k_dedup_expand, dim3((unsigned)cdiv(v.n, kBlock)), dim3(kBlock), s, v.grank, d_values, (long long)fill,
                  d_out, v.n);
    return RECSDK_OK;
}

extern "C" int recsdk_unique_total(recsdk_unique_t* u, void* stream, int64_t* h_total)
{
    RECSDK_REQUIRE(u != nullptr && h_total != nullptr, RECSDK_ENULL, "recsdk_unique_total: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    RECSDK_HIP_TRY(hipMemcpyAsync(h_total, u->totals, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    return RECSDK_OK;
}

const recsdk::UniqueView* recsdk_unique_view(const recsdk_unique* u) { return &u->view; }
