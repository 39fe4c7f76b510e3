// Multi-table key dedup in first-occurrence order (unique + inverse + counts) and the
// per-distinct-key position lists used by the gradient segment-reduce.
//
// Algorithm (all tables in one set of launches, n = total keys):
//   plan     per table: scratch hash region of pow2 >= 2*n_t slots (+1 side slot for the key that equals
//            the empty marker); the same launch clears the scratch
//   insert   every key CAS-claims a scratch slot; atomicMin keeps the smallest global index ("first"); when the
//            caller wants the multiplicities before the lists exist, atomicAdd collects them as well
//   flags    is_first[i] = (first(slot_i) == i); per-tile sums of the flags
//   tilescan single block: exclusive scan of the tile sums; unique_offsets[t] = rank at the table start
//   emit     per tile rescan: rank R of every first occurrence -> unique_keys[R]; the rank is written back into
//            the scratch slot
//   inverse  inverse[i] = R(slot_i) - unique_offsets[t]; every position gets the sort key R (skipped keys a
//            sentinel above every rank)
//   lists    (own stream) stable radix sort of (R, position): posList then holds, rank after rank, the ascending
//            position list of every distinct key; run heads give list starts, their differences the multiplicities;
//            keys seen more than kListMax times ("long" keys) are listed, and split at kHugeMin occurrences
// Ranks come from a scan over key positions, so the order of distinct keys is the order of first
// occurrence regardless of how the CAS races resolve.  Lists and multiplicities need no atomics at all: one
// multiplicity per distinct key of a block used to cost a device atomic each, a third of the insert kernel's.
#include <string.h>

#include <algorithm>
#include <mutex>

#include <hip/hip_runtime.h>

#include "common.h"
#include "dedup.h"
#include "radix_sort.h"

namespace recsdk {

constexpr int kCounterSegError = 7;  // counters[7]: set when a table exceeds the promised number of keys

struct __attribute__((aligned(16))) DedupEntry {
    long long key;
    uint32_t first;
    uint32_t count;
};

// Plan + clear in one launch.  Every block derives the scratch layout from the offsets (per table a region of
// pow2 >= 2*n_t slots plus one side slot); block 0 also publishes it (sbase, smask) and zeroes the counters.
// Then all blocks clear the scratch.
__global__ __launch_bounds__(kBlock) void k_dedup_plan_clear(const int64_t* __restrict__ off, int T, int64_t* sbase,
                                                             uint32_t* smask, uint32_t* counters, DedupEntry* S,
                                                             int64_t segBound)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ unsigned long long carry;
    if (threadIdx.x == 0) {
        carry = 0;
        if (blockIdx.x == 0) {
            counters[kCounterSegError] = 0;  // a table holds more keys than the caller promised
        }
    }
    __syncthreads();
    for (int t0 = 0; t0 < T; t0 += kBlock) {
        const int t = t0 + threadIdx.x;
        uint32_t region = 0;
        uint64_t cap = 64;
        if (t < T) {
            const int64_t nt = off[t + 1] - off[t];
            while ((int64_t)cap < 2 * nt) {
                cap <<= 1;
            }
            region = (uint32_t)cap + 1;
            if (blockIdx.x == 0 && nt > segBound) {
                atomicOr(&counters[kCounterSegError], 1u);
            }
        }
        uint32_t tot;
        const uint32_t ex = block_exclusive_scan(region, smem, &tot);
        if (blockIdx.x == 0 && t < T) {
            sbase[t] = (int64_t)(carry + ex);
            smask[t] = (uint32_t)(cap - 1);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            carry += tot;
        }
        __syncthreads();
    }
    const int64_t total = (int64_t)carry;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        sbase[T] = total;
        counters[0] = 0;  // number of keys seen more than kListMax times (long keys)
        counters[1] = 0;  // number of keys seen 2..kListMax times
        counters[2] = 0;  // long keys seen more than kHugeMin times
        counters[3] = 0;  // the other long keys
        counters[4] = 0;  // of counters[2]: keys seen more than kVeryHugeMin times
        counters[5] = 0;  // chunks of the two-level sums (the gradient reduce counts and resets it)
        counters[6] = 0;  // stays 0
    }
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    DedupEntry e;
    e.key = kEmptyKey;
    e.first = 0xFFFFFFFFu;
    e.count = 0;
    for (; i < total; i += stride) {
        S[i] = e;
    }
}

// One ordinary (cached) 16-byte load of a scratch entry.  What it returns may be older than what the entry holds by
// now - entries change under device atomics of other compute units while the launch runs - and the callers only draw
// conclusions that stay true: a key, once in an entry, never changes, and a first index only ever decreases.
__device__ __forceinline__ DedupEntry scratch_peek(const DedupEntry* R, uint32_t pos)
{
    const uint4 raw = *reinterpret_cast<const uint4*>(R + pos);
    DedupEntry e;
    e.key = (long long)(((unsigned long long)raw.y << 32) | raw.x);
    e.first = raw.z;
    e.count = raw.w;
    return e;
}

// Device-wide claim of a scratch slot for `key` in region R (capacity mask+1, side slot at mask+1) and
// first[slot] = min(first[slot], first).  A probe is one cached load: an entry that shows another key is passed by,
// one that shows our key with a first index at or below ours needs nothing more, an empty one is claimed by a
// compare-and-swap (which tells what it really holds).  A key that every block of the launch holds thus costs its
// claim, one minimum per block that lowers the index (about ln(blocks) of them) and cache hits otherwise: device
// atomics and coherent loads of ONE entry are served one after the other, about 12 ns each, which made a key present
// in all 512 blocks of a 131072-key run cost 25 us by itself.
__device__ __forceinline__ uint32_t scratch_claim_min(DedupEntry* R, uint32_t mask, long long key, uint32_t first)
{
    if (key == kEmptyKey) {
        if (scratch_peek(R, mask + 1).first > first) {
            atomicMin(&R[mask + 1].first, first);  // side slot: only this key lands here, no claim needed
        }
        return mask + 1;
    }
    uint32_t pos = (uint32_t)hash64((uint64_t)key) & mask;
    while (true) {
        const DedupEntry e = scratch_peek(R, pos);
        if (e.key == key) {
            if (e.first > first) {
                atomicMin(&R[pos].first, first);
            }
            return pos;
        }
        if (e.key == kEmptyKey) {
            unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&R[pos].key),
                                                (unsigned long long)kEmptyKey, (unsigned long long)key);
            if ((long long)prev == kEmptyKey || (long long)prev == key) {
                atomicMin(&R[pos].first, first);
                return pos;
            }
        }
        pos = (pos + 1) & mask;
    }
}

// A block first merges its keys in an LDS hash (first index, multiplicity), then touches the device-wide
// scratch once per distinct key of the block.  A key seen thousands of times therefore costs one pair of
// device atomics per block instead of one pair per occurrence.  ITEMS keys per thread: 4 (1024 keys per block) for
// large batches; 1 for small ones, whose few blocks would otherwise each walk eight dependent rounds of device
// atomics per thread while most of the device idles (4096 keys: 47 -> 15 us).
template <int ITEMS, bool COUNT>
__global__ __launch_bounds__(kBlock) void k_dedup_insert(const int64_t* __restrict__ keys,
                                                         const uint32_t* __restrict__ inCounts,
                                                         const int64_t* __restrict__ off, int T,
                                                         const int64_t* __restrict__ sbase,
                                                         const uint32_t* __restrict__ smask, DedupEntry* S,
                                                         int32_t* __restrict__ sslot, int64_t nMax, int skipEnabled,
                                                         long long skipKey)
{
    constexpr int kKeysPerBlock = kBlock * ITEMS;
    // Block-local hash, load factor <= 0.57, in separate arrays so that a run without multiplicities pays 12 bytes
    // per slot: 1792 slots are 21.5 KB, seven blocks share a CU's LDS and the 1664 blocks of a 1.7 M-key batch are
    // resident at once (2048 slots of 16 bytes: four per CU, the launch took 1.6 rounds of blocks).
    constexpr int kLdsSlots = (ITEMS == 4) ? 1792 : 2 * kKeysPerBlock;
    __shared__ long long Lkey[kLdsSlots + 1];
    __shared__ uint32_t Lfirst[kLdsSlots + 1];
    __shared__ uint32_t Lcount[COUNT ? kLdsSlots + 1 : 1];
    __shared__ int sT0;
    __shared__ int sT1;
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kKeysPerBlock;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, tile0);
        int64_t last = tile0 + kKeysPerBlock - 1 < n ? tile0 + kKeysPerBlock - 1 : n - 1;
        sT1 = find_segment(off, T, last);
    }
    for (int e = threadIdx.x; e <= kLdsSlots; e += kBlock) {
        Lkey[e] = kEmptyKey;
        Lfirst[e] = 0xFFFFFFFFu;
        if (COUNT) {
            Lcount[e] = 0;
        }
    }
    __syncthreads();
    int t = sT0;
    if (sT0 != sT1) {
        // the tile straddles tables: every key goes to the device-wide scratch directly
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
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
            uint32_t pos = scratch_claim_min(R, smask[t], key, (uint32_t)i);
            if (COUNT) {
                atomicAdd(&R[pos].count, inCounts ? inCounts[i] : 1u);
            }
            sslot[i] = (int32_t)(sbase[t] + pos);
        }
        return;
    }
    // phase 1: merge in LDS
    int lpos[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
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
            pos = (uint32_t)(((hash64((uint64_t)key) >> 32) * (uint64_t)kLdsSlots) >> 32);
            while (true) {
                unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&Lkey[pos]),
                                                    (unsigned long long)kEmptyKey, (unsigned long long)key);
                if ((long long)prev == kEmptyKey || (long long)prev == key) {
                    break;
                }
                pos = (pos + 1 == (uint32_t)kLdsSlots) ? 0u : pos + 1;
            }
        }
        atomicMin(&Lfirst[pos], (uint32_t)i);
        if (COUNT) {
            atomicAdd(&Lcount[pos], inCounts ? inCounts[i] : 1u);
        }
        lpos[k] = (int)pos;
    }
    __syncthreads();
    // phase 2: one device-wide update per distinct key of the block; the LDS entry then holds the scratch slot.
    // The update of an entry is done by the thread that holds the key's first occurrence in the block (the position
    // the entry's minimum names): a thread has at most ITEMS of those, against up to seven entries of a walk over the
    // LDS table, almost half of them empty - and every update is a chain of device round trips that the lanes of a
    // wave wait out together.
    DedupEntry* R = S + sbase[t];
    const uint32_t mask = smask[t];
    const int64_t base = sbase[t];
    bool own[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const int64_t i = tile0 + k * kBlock + threadIdx.x;
        own[k] = lpos[k] >= 0 && Lfirst[lpos[k]] == (uint32_t)i;
    }
    __syncthreads();   // every owner is known before the first entry is overwritten with its scratch slot
    // With few blocks (ITEMS == 1) or with multiplicities a thread works on a group of its entries at once - probe
    // loads together, then the claims of those that found an empty slot, then the minima and the counts; entries that
    // met another key move one slot on and take part in the next round of their group: a block is a chain of dependent
    // device round trips.  Without multiplicities the large-block variant is fastest one entry after the other (1.7 M
    // keys in 26 tables: in groups of four 110 us against 75, all at once 129 us, at the same residency).
    if constexpr (ITEMS == 1 || COUNT) {
        constexpr int kGroup = ITEMS < 2 ? 1 : 2;
#pragma unroll 1
        for (int g0 = 0; g0 < ITEMS; g0 += kGroup) {
            long long key[kGroup];
            uint32_t first[kGroup];
            uint32_t pos[kGroup];
            int ent[kGroup];
            bool live[kGroup];
            bool any = false;
#pragma unroll
            for (int k = 0; k < kGroup; ++k) {
                live[k] = false;
                key[k] = 0;
                first[k] = 0xFFFFFFFFu;
                pos[k] = 0;
                ent[k] = 0;
                // lpos and own are indexed with compile-time constants only (they live in registers)
#pragma unroll
                for (int q = 0; q < ITEMS; ++q) {
                    if (q == g0 + k && own[q]) {
                        ent[k] = lpos[q];
                        live[k] = true;
                    }
                }
                if (live[k]) {
                    const int e = ent[k];
                    first[k] = Lfirst[e];
                    if (e == kLdsSlots) {
                        // the key that equals the empty marker: its own slot behind the region, no claim
                        if (scratch_peek(R, mask + 1).first > first[k]) {
                            atomicMin(&R[mask + 1].first, first[k]);
                        }
                        if (COUNT) {
                            atomicAdd(&R[mask + 1].count, Lcount[e]);
                        }
                        Lfirst[e] = (uint32_t)(base + mask + 1);
                        live[k] = false;
                    } else {
                        key[k] = Lkey[e];
                        pos[k] = (uint32_t)hash64((uint64_t)key[k]) & mask;
                        any = true;
                    }
                }
            }
            while (any) {
                long long cur[kGroup];
                uint32_t seen[kGroup];
#pragma unroll
                for (int k = 0; k < kGroup; ++k) {
                    if (live[k]) {
                        const DedupEntry e = scratch_peek(R, pos[k]);
                        cur[k] = e.key;
                        seen[k] = e.first;
                    }
                }
#pragma unroll
                for (int k = 0; k < kGroup; ++k) {
                    if (live[k] && cur[k] == kEmptyKey) {
                        cur[k] = (long long)atomicCAS(reinterpret_cast<unsigned long long*>(&R[pos[k]].key),
                                                      (unsigned long long)kEmptyKey, (unsigned long long)key[k]);
                        if (cur[k] == kEmptyKey) {
                            cur[k] = key[k];
                        }
                        seen[k] = 0xFFFFFFFFu;   // whatever it holds by now, lower it
                    }
                }
                any = false;
#pragma unroll
                for (int k = 0; k < kGroup; ++k) {
                    if (live[k]) {
                        if (cur[k] == key[k]) {
                            // a first index at or below ours needs no atomic (a stale value is safe: it only decreases)
                            if (seen[k] > first[k]) {
                                atomicMin(&R[pos[k]].first, first[k]);
                            }
                            if (COUNT) {
                                atomicAdd(&R[pos[k]].count, Lcount[ent[k]]);
                            }
                            Lfirst[ent[k]] = (uint32_t)(base + pos[k]);
                            live[k] = false;
                        } else {
                            pos[k] = (pos[k] + 1) & mask;
                            any = true;
                        }
                    }
                }
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            if (own[k]) {
                const int e = lpos[k];
                const long long key = (e == kLdsSlots) ? kEmptyKey : Lkey[e];
                Lfirst[e] = (uint32_t)(base + scratch_claim_min(R, mask, key, Lfirst[e]));
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        int64_t i = tile0 + k * kBlock + threadIdx.x;
        if (i < n) {
            sslot[i] = (lpos[k] >= 0) ? (int32_t)Lfirst[lpos[k]] : -1;
        }
    }
}

// First-occurrence flags, tile sums and, for every distinct key, where its rank comes from: the scratch entry's
// `first` (the index of the key's first occurrence until now) becomes kRankPacked | tile << 10 | rank of that first
// occurrence inside its tile; the key's rank is then tileBase[tile] + the low ten bits, for every position of the key,
// once the tile sums are scanned.  The marker bit keeps the new value apart from every index that another thread of
// this launch may still be comparing with (indices stay below 2^31).
constexpr uint32_t kRankPacked = 0x80000000u;
static_assert(kTile == 1024, "ten bits of in-tile rank");
__global__ __launch_bounds__(kBlock) void k_dedup_flags(DedupEntry* S, const int32_t* __restrict__ sslot,
                                                        const int64_t* __restrict__ off, int T,
                                                        uint8_t* __restrict__ isFirst, uint32_t* __restrict__ tileF,
                                                        int64_t nMax)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    uint32_t f = 0;
    uint8_t fl[kItems];
    int32_t pos[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t i = tile0 + (int64_t)threadIdx.x * kItems + k;
        fl[k] = 0;
        pos[k] = -1;
        if (i < n) {
            pos[k] = sslot[i];
        }
    }
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t i = tile0 + (int64_t)threadIdx.x * kItems + k;
        if (pos[k] >= 0 && S[pos[k]].first == (uint32_t)i) {
            fl[k] = 1;
            f += 1;
        }
    }
    *reinterpret_cast<uchar4*>(isFirst + tile0 + (int64_t)threadIdx.x * kItems) = make_uchar4(fl[0], fl[1], fl[2], fl[3]);
    uint32_t total;
    uint32_t rank = block_exclusive_scan(f, smem, &total);
    const uint32_t packed = kRankPacked | ((uint32_t)blockIdx.x << 10);
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (fl[k]) {
            S[pos[k]].first = packed | rank;
            rank += 1;
        }
    }
    if (threadIdx.x == 0) {
        tileF[blockIdx.x] = total;
    }
}

// single block: exclusive scan of the tile sums (in place) and unique_offsets.
__global__ __launch_bounds__(kBlock) void k_dedup_tilescan(uint32_t* tileF, const uint8_t* __restrict__ isFirst,
                                                           const int64_t* __restrict__ off, int T, int64_t* uoff,
                                                           int64_t* totals, int64_t nMax)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carryF;
    const int64_t n = off[T] < nMax ? off[T] : nMax;
    const int64_t ntiles = (n + kTile - 1) / kTile;
    // every thread owns a run of consecutive tiles: local sum, one block scan, local prefixes
    const int64_t per = (ntiles + kBlock - 1) / kBlock;
    const int64_t first = (int64_t)threadIdx.x * per;
    const int64_t last = first + per < ntiles ? first + per : ntiles;
    uint32_t sf = 0;
    for (int64_t j = first; j < last; ++j) {
        sf += tileF[j];
    }
    uint32_t tf;
    uint32_t ef = block_exclusive_scan(sf, smem, &tf);
    for (int64_t j = first; j < last; ++j) {
        const uint32_t vf = tileF[j];
        tileF[j] = ef;
        ef += vf;
    }
    if (threadIdx.x == 0) {
        carryF = tf;
        totals[0] = tf;  // U
        totals[1] = 0;
        totals[2] = n;   // end of the position lists; lowered by the list kernels when keys were skipped
    }
    __syncthreads();
    segment_start_ranks(isFirst, tileF, off, T, n, carryF, uoff);
}

// Rank of every position's key (tile base of the key's first occurrence + its rank inside that tile), the inverse
// index and, at the first occurrences themselves, unique_keys (and the multiplicities when the insert kernel
// collected them: ucount != NULL).  sortKey == NULL: no lists wanted.
__global__ __launch_bounds__(kTile) void k_dedup_inverse(const DedupEntry* __restrict__ S,
                                                          const int32_t* __restrict__ sslot,
                                                          const int64_t* __restrict__ keys,
                                                          const int64_t* __restrict__ off, int T,
                                                          const uint8_t* __restrict__ isFirst,
                                                          const uint32_t* __restrict__ tileBase,
                                                          const int64_t* __restrict__ uoff,
                                                          int64_t* __restrict__ uniq, uint32_t* __restrict__ ucount,
                                                          int32_t* __restrict__ inverse, int32_t* __restrict__ grank,
                                                          uint32_t* __restrict__ sortKey, uint32_t* __restrict__ sortVal,
                                                          uint32_t sentinel, int64_t nMax)
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
    // one position per thread, a tile per block: the rank comes through a chain of three dependent loads
    const int64_t i = tile0 + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int32_t pos = sslot[i];
    uint32_t sk = sentinel;
    if (pos < 0) {
        inverse[i] = -1;
        grank[i] = -1;
    } else {
        const int t = advance_segment(off, sT0, i);
        const uint32_t packed = S[pos].first;
        const uint32_t R = tileBase[(packed & ~kRankPacked) >> 10] + (packed & 1023u);
        const int32_t local = (int32_t)((int64_t)R - uoff[t]);
        inverse[i] = local;
        grank[i] = (int32_t)R;
        sk = (uint32_t)local & sentinel;  // sentinel = all ones in the sorted bits
        if (isFirst[i]) {
            uniq[R] = keys[i];
            if (ucount != nullptr) {
                ucount[R] = S[pos].count;
            }
        }
    }
    if (sortKey != nullptr) {
        sortKey[i] = sk;
        sortVal[i] = (uint32_t)i;
    }
}

// ---- position lists from the sorted positions ------------------------------------------------------------------
// The positions were sorted (stably) by the index of their key inside its table, so the positions of one distinct key
// are adjacent and ascending; keys of different tables with the same index follow one another in table order.  Where
// the lists lie in posList is free: a list starts where the rank of the position's key changes.  Skipped positions
// (rank -1) belong to no list.
// STAGED (at most kBoundsTables tables): the rank of a sorted entry comes from its sorted key (the index of its key
// inside the table) and the table of its position, found in a copy of the offsets in LDS, instead of a random read
// of the rank array per entry.  An entry whose key equals the sentinel may be a skipped position: only those look
// their rank up.
constexpr int kBoundsTables = 1023;
template <bool STAGED>
__global__ __launch_bounds__(kBlock) void k_lists_bounds(const uint32_t* __restrict__ sortedKey,
                                                         const int32_t* __restrict__ posList,
                                                         const int32_t* __restrict__ grank,
                                                         const int64_t* __restrict__ off,
                                                         const int64_t* __restrict__ uoff, int T, uint32_t sentinel,
                                                         int64_t n, uint32_t* __restrict__ useg,
                                                         uint32_t* __restrict__ uend)
{
    __shared__ int32_t sOff[STAGED ? kBoundsTables + 1 : 1];   // positions and ranks fit 31 bits
    __shared__ int32_t sUoff[STAGED ? kBoundsTables + 1 : 1];
    if (STAGED) {
        for (int t = threadIdx.x; t <= T; t += kBlock) {
            sOff[t] = (int32_t)off[t];
            sUoff[t] = (int32_t)uoff[t];
        }
        __syncthreads();
    }
    const int64_t i0 = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * kItems;
    if (i0 >= n) {
        return;
    }
    int32_t pos[kItems + 2];
    uint32_t key[kItems + 2];
#pragma unroll
    for (int k = 0; k < kItems + 2; ++k) {
        const int64_t j = i0 - 1 + k;
        const bool in = j >= 0 && j < n;
        pos[k] = in ? posList[j] : -1;
        key[k] = (STAGED && in) ? sortedKey[j] : 0u;
    }
    int32_t R[kItems + 2];
#pragma unroll
    for (int k = 0; k < kItems + 2; ++k) {
        int32_t r = -1;
        if (pos[k] >= 0) {
            if (!STAGED) {
                r = grank[pos[k]];
            } else if (key[k] == sentinel && grank[pos[k]] < 0) {
                r = -1;
            } else {
                int lo = 0;
                int hi = T;   // sOff[lo] <= pos < sOff[hi]
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (sOff[mid] <= pos[k]) {
                        lo = mid;
                    } else {
                        hi = mid;
                    }
                }
                r = (int32_t)key[k] + sUoff[lo];
            }
        }
        R[k] = r;
    }
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t i = i0 + k;
        const int32_t cur = R[k + 1];
        if (i < n && cur >= 0) {
            if (i == 0 || cur != R[k]) {
                useg[cur] = (uint32_t)i;
            }
            if (i == n - 1 || cur != R[k + 2]) {
                uend[cur] = (uint32_t)(i + 1);
            }
        }
    }
}

// multiplicity of every distinct key = length of its list; keys seen more than kListMax times get a long id.  The
// long ids of a block collect in LDS and take their places with one device atomic per flush (thousands of atomics on
// the one counter would serialise).  When a table held more keys than the sort was sized for, every list is empty.
__global__ __launch_bounds__(kBlock) void k_lists_finish(const int64_t* __restrict__ totals,
                                                         const uint32_t* __restrict__ useg,
                                                         const uint32_t* __restrict__ uend,
                                                         uint32_t* __restrict__ ucount, uint32_t* counters,
                                                         int32_t* __restrict__ longList, uint32_t* __restrict__ longSeg,
                                                         uint32_t* __restrict__ longCnt)
{
    constexpr int kCap = 4 * kBlock;
    __shared__ int32_t sR[kCap];
    __shared__ uint32_t sSeg[kCap];
    __shared__ uint32_t sCnt[kCap];
    __shared__ uint32_t sCount;
    __shared__ uint32_t sBase;
    const int64_t U = totals[0];
    const bool bad = counters[kCounterSegError] != 0;
    if (threadIdx.x == 0) {
        sCount = 0;
    }
    __syncthreads();
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t R0 = (int64_t)blockIdx.x * kBlock; R0 < U; R0 += stride) {  // uniform trip count per block
        const int64_t R = R0 + threadIdx.x;
        if (R < U) {
            const uint32_t start = useg[R];
            const uint32_t c = bad ? 0u : uend[R] - start;
            ucount[R] = c;
            if (c > (uint32_t)kListMax) {
                const uint32_t at = atomicAdd(&sCount, 1u);
                sR[at] = (int32_t)R;
                sSeg[at] = start;
                sCnt[at] = c;
            }
        }
        __syncthreads();
        const bool last = R0 + stride >= U;
        if (sCount + kBlock > (uint32_t)kCap || last) {
            const uint32_t m = sCount;
            if (m != 0) {
                if (threadIdx.x == 0) {
                    sBase = atomicAdd(&counters[0], m);
                }
                __syncthreads();
                for (uint32_t j = threadIdx.x; j < m; j += kBlock) {
                    longList[sBase + j] = sR[j];
                    longSeg[sBase + j] = sSeg[j];
                    longCnt[sBase + j] = sCnt[j];
                }
                __syncthreads();
                if (threadIdx.x == 0) {
                    sCount = 0;
                }
            }
            __syncthreads();
        }
    }
}

// Single block: splits the long ids into those of keys seen more than kHugeMin times (hugeIds, longest list
// first) and the rest (longIds, ascending).  longCnt[id] = multiplicity of the long id's key, written by the kernel
// that handed out the ids.
// One block does it all, NT threads of it: 1024 where the kernel runs alone and the long lists are many (the pooled
// backward: 11 k of them, 63 -> 29 us), 256 on the list stream beside the forward gather, where a block of 1024 threads
// waits for half a CU to fall free at once (15 -> 27 us).
template <int kClassBlock>
__global__ __launch_bounds__(kClassBlock) void k_dedup_classify(const uint32_t* __restrict__ longCnt,
                                                           uint32_t* __restrict__ counters,
                                                           int32_t* __restrict__ hugeIds, int32_t* __restrict__ longIds)
{
    constexpr int kWaves = kClassBlock / kWave;
    constexpr int kSortCap = 4096;
    __shared__ uint32_t smem[kWaves + 1];
    __shared__ unsigned long long sortBuf[kSortCap];
    const uint32_t nLong = counters[0];
    uint32_t hugeBase = 0;
    uint32_t restBase = 0;
    uint32_t nVeryHuge = 0;   // this thread's share of the keys seen more than kVeryHugeMin times
    constexpr int kPer = 16;  // long ids per thread and round, loaded together so their latencies overlap
    for (uint32_t b = 0; b < nLong; b += kClassBlock * kPer) {
        const uint32_t first = b + threadIdx.x * kPer;
        uint32_t cnt[kPer];
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            cnt[k] = (first + k < nLong) ? longCnt[first + k] : 0u;
        }
        uint32_t nh = 0;
        uint32_t nl = 0;
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            nh += cnt[k] > (uint32_t)kHugeMin ? 1u : 0u;
            nl += cnt[k] > 0u ? 1u : 0u;
            nVeryHuge += cnt[k] > (uint32_t)kVeryHugeMin ? 1u : 0u;
        }
        uint32_t th;
        uint32_t tl;
        uint32_t eh = block_exclusive_scan_n<kClassBlock>(nh, smem, &th);
        uint32_t el = block_exclusive_scan_n<kClassBlock>(nl, smem, &tl);
        uint32_t er = el - eh;
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            if (cnt[k] > (uint32_t)kHugeMin) {
                // (count, id) stays in LDS for the sort below: no second walk through ucount[longList[...]]
                if (hugeBase + eh < (uint32_t)kSortCap) {
                    sortBuf[hugeBase + eh] = ((unsigned long long)cnt[k] << 32) | (0xffffffffu - (first + k));
                }
                hugeIds[hugeBase + eh++] = (int32_t)(first + k);
            } else if (cnt[k] > 0u) {
                longIds[restBase + er++] = (int32_t)(first + k);
            }
        }
        hugeBase += th;
        restBase += tl - th;
    }
    if (threadIdx.x == 0) {
        counters[2] = hugeBase;
        counters[3] = restBase;
    }
    // longest lists first: the kernels that walk these lists start their longest chains at once and fill
    // the tail of the launch with short ones.  Bitonic sort in LDS on (count, id); larger sets stay as they are.
    __syncthreads();
    __shared__ uint32_t veryHuge;
    if (threadIdx.x == 0) {
        veryHuge = 0;
    }
    __syncthreads();
    // how many of them are seen more than kVeryHugeMin times (they lead the list once it is sorted)
    if (nVeryHuge != 0) {
        atomicAdd(&veryHuge, nVeryHuge);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        // unsorted lists (more than kSortCap entries) take the narrow slices throughout
        counters[4] = hugeBase <= (uint32_t)kSortCap ? veryHuge : hugeBase;
    }
    if (hugeBase > 1 && hugeBase <= 256u) {
        // a handful: every entry is ranked against all others by a thread of its own, no barriers
        if (threadIdx.x < hugeBase) {
            const unsigned long long mine = sortBuf[threadIdx.x];
            uint32_t rank = 0;
#pragma unroll 4
            for (uint32_t k = 0; k < hugeBase; ++k) {
                rank += sortBuf[k] > mine ? 1u : 0u;
            }
            hugeIds[rank] = (int32_t)(0xffffffffu - (uint32_t)mine);
        }
    } else if (hugeBase > 1 && hugeBase <= (uint32_t)kSortCap) {
        uint32_t m = 2;
        while (m < hugeBase) {
            m <<= 1;
        }
        for (uint32_t j = hugeBase + threadIdx.x; j < m; j += kClassBlock) {
            sortBuf[j] = 0;  // padding sorts last
        }
        __syncthreads();
        for (uint32_t k = 2; k <= m; k <<= 1) {
            for (uint32_t j = k >> 1; j > 0; j >>= 1) {
                for (uint32_t i = threadIdx.x; i < m; i += kClassBlock) {
                    const uint32_t partner = i ^ j;
                    if (partner > i) {
                        const unsigned long long a = sortBuf[i];
                        const unsigned long long b = sortBuf[partner];
                        const bool descending = (i & k) == 0;
                        if (descending ? (a < b) : (a > b)) {
                            sortBuf[i] = b;
                            sortBuf[partner] = a;
                        }
                    }
                }
                __syncthreads();
            }
        }
        for (uint32_t j = threadIdx.x; j < hugeBase; j += kClassBlock) {
            hugeIds[j] = (int32_t)(0xffffffffu - (uint32_t)sortBuf[j]);
        }
    }
}

// ---- a small batch in one launch ----------------------------------------------------------------------------
// At most kSmallKeys keys and kSmallTables tables: one block builds the distinct keys in first-occurrence order, the
// inverse index and the multiplicities entirely in LDS (hash of 4 * kSmallKeys entries that hold the smallest position
// of their key; keys are compared through the positions).  No scratch, no position lists: the gradient reduce of so
// few keys scans the inverse index instead (k_apply_small).  Seven dependent launches of 4096 keys cost 40 us, this
// one 8.  Results are those of the large path, bit for bit.

__global__ __launch_bounds__(kSmallBlock) void k_dedup_small(const int64_t* __restrict__ keys,
                                                        const uint32_t* __restrict__ inCounts,
                                                        const int64_t* __restrict__ off, int T, int skipEnabled,
                                                        long long skipKey, int64_t* __restrict__ uniq,
                                                        int64_t* __restrict__ uoff, int32_t* __restrict__ inverse,
                                                        int32_t* __restrict__ grank, uint32_t* __restrict__ ucount,
                                                        int64_t* __restrict__ totals, uint32_t* __restrict__ counters, int nHost)
{
    constexpr int kPer = kSmallKeys / kSmallBlock;
    constexpr int kSlots = 4 * kSmallKeys;
    static_assert(kSlots <= 65536, "sSlot holds an entry index in 16 bits");
    constexpr uint32_t kNone = 0xFFFFFFFFu;
    static_assert(kSmallKeys % kSmallBlock == 0, "whole rounds of the block");
    __shared__ uint32_t smem[kSmallBlock / kWave];
    __shared__ long long sKey[kSmallKeys];
    __shared__ __align__(16) uint32_t hEnt[kSlots];          // smallest position of the key that owns the slot
    __shared__ uint16_t sSlot[kSmallKeys];     // hash slot of position i, then its key's first position
    __shared__ uint8_t sTab[kSmallKeys];
    __shared__ uint8_t sSkip[kSmallKeys];
    __shared__ uint16_t sPre[kSmallKeys + 1];  // first occurrences before position i
    __shared__ __align__(16) uint32_t sCnt[kSmallKeys];
    __shared__ int64_t sOff[kSmallTables + 1];
    __shared__ int64_t sUoff[kSmallTables + 1];
    // All of a thread's keys are fetched before the first is used, and before the offsets are known: the one block is
    // all the parallelism there is.  nHost, the caller's count of keys, bounds what may be read.
    long long mine[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const int i = k * kSmallBlock + (int)threadIdx.x;
        mine[k] = i < nHost ? keys[i] : 0;
    }
    for (int t = threadIdx.x; t <= T; t += kSmallBlock) {
        sOff[t] = off[t];
    }
    {
        const uint4 none4 = make_uint4(kNone, kNone, kNone, kNone);
        const uint4 zero4 = make_uint4(0, 0, 0, 0);
        for (int e = threadIdx.x; e < kSlots / 4; e += kSmallBlock) {
            reinterpret_cast<uint4*>(hEnt)[e] = none4;
        }
        for (int e = threadIdx.x; e < kSmallKeys / 4; e += kSmallBlock) {
            reinterpret_cast<uint4*>(sCnt)[e] = zero4;
        }
    }
    __syncthreads();
    const int nDev = (int)(sOff[T] < kSmallKeys ? sOff[T] : kSmallKeys);
    const int n = nDev < nHost ? nDev : nHost;
    // insert: the slot of a key holds the smallest position seen so far; any position in it names the key.  A thread's
    // keys take their first probe together, as blind compare-and-swaps (most find their entry empty): one after the
    // other, each a read, a swap and a compare in turn, the four chains of a thread took half of the kernel.
    {
        uint32_t pos[kPer];
        uint32_t cur[kPer];
        uint8_t tab[kPer];
        bool pend[kPer];
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            const int i = k * kSmallBlock + (int)threadIdx.x;
            pend[k] = false;
            pos[k] = 0;
            cur[k] = kNone;
            tab[k] = 0;
            if (i < n) {
                const bool skip = skipEnabled && mine[k] == skipKey;
                tab[k] = (uint8_t)find_segment(sOff, T, i);
                sKey[i] = mine[k];
                sTab[i] = tab[k];
                sSkip[i] = skip ? 1 : 0;
                pend[k] = !skip;
                pos[k] = (uint32_t)(hash64((uint64_t)mine[k] ^ ((uint64_t)tab[k] << 56)) >> 40) & (uint32_t)(kSlots - 1);
            }
        }
        __syncthreads();  // a probe compares with the keys of other positions
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            if (pend[k]) {
                cur[k] = atomicCAS(&hEnt[pos[k]], kNone, (uint32_t)(k * kSmallBlock + (int)threadIdx.x));
            }
        }
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            if (!pend[k]) {
                continue;
            }
            const int i = k * kSmallBlock + (int)threadIdx.x;
            const long long key = mine[k];
            const uint8_t t = tab[k];
            uint32_t at = pos[k];
            uint32_t c = cur[k];
            while (c != kNone) {  // kNone: the entry was empty and is this position's now
                if (sKey[c] == key && sTab[c] == t) {
                    atomicMin(&hEnt[at], (uint32_t)i);
                    break;
                }
                at = (at + 1) & (uint32_t)(kSlots - 1);
                c = atomicCAS(&hEnt[at], kNone, (uint32_t)i);
            }
            sSlot[i] = (uint16_t)at;
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += kSmallBlock) {
        if (!sSkip[i]) {
            sSlot[i] = (uint16_t)hEnt[sSlot[i]];  // first position of the key
        }
    }
    __syncthreads();
    // ranks of the first occurrences: scan over positions, kPer consecutive positions per thread
    const int i0 = (int)threadIdx.x * kPer;
    uint32_t f = 0;
    bool fl[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const int i = i0 + k;
        fl[k] = i < n && !sSkip[i] && sSlot[i] == (uint16_t)i;
        f += fl[k] ? 1u : 0u;
    }
    uint32_t U;
    uint32_t r = block_exclusive_scan_n<kSmallBlock>(f, smem, &U);
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const int i = i0 + k;
        sPre[i] = (uint16_t)r;
        if (fl[k]) {
            uniq[r] = sKey[i];
            r += 1;
        }
    }
    if (threadIdx.x == 0) {
        sPre[kSmallKeys] = (uint16_t)U;
        totals[0] = U;
        totals[1] = 0;
        totals[2] = 0;
        for (int c = 0; c < 8; ++c) {
            counters[c] = 0;
        }
    }
    __syncthreads();
    for (int t = threadIdx.x; t <= T; t += kSmallBlock) {
        const int64_t u = sOff[t] >= n ? (int64_t)U : (int64_t)sPre[sOff[t]];
        sUoff[t] = u;
        uoff[t] = u;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += kSmallBlock) {
        if (sSkip[i]) {
            inverse[i] = -1;
            grank[i] = -1;
        } else {
            const uint32_t R = sPre[sSlot[i]];
            inverse[i] = (int32_t)((int64_t)R - sUoff[sTab[i]]);
            grank[i] = (int32_t)R;
            atomicAdd(&sCnt[R], inCounts ? inCounts[i] : 1u);
        }
    }
    __syncthreads();
    for (uint32_t R = threadIdx.x; R < U; R += kSmallBlock) {
        ucount[R] = sCnt[R];
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

// ---- grouping by a stable sort (row indices of known range, order of the distinct keys free) -----------------
// The pooled lookup's backward pass needs, per touched row, the list of gradient rows to add in ascending position
// order, but not the first-occurrence order of the distinct rows.  With row indices bounded by the table sizes a
// stable radix sort of (table base + row, value of the position) over few bits delivers every list at once: equal
// keys end up adjacent, their values in position order.  No hash table, no atomics per key.
__global__ __launch_bounds__(kBlock) void k_group_keys(const int64_t* __restrict__ rows, const int64_t* __restrict__ tb,
                                                       const int64_t* __restrict__ cumsum, int T,
                                                       const int32_t* __restrict__ values,
                                                       uint32_t* __restrict__ sortKey, uint32_t* __restrict__ sortVal,
                                                       int64_t n, uint32_t sentinel)
{
    __shared__ int sT0;
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(tb, T, tile0);
    }
    __syncthreads();
    int t = sT0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t i = tile0 + k * kBlock + threadIdx.x;
        if (i >= n) {
            break;
        }
        t = advance_segment(tb, t, i);
        const int64_t base = cumsum[t];
        const int64_t row = rows[i];
        // rows outside their table take the sentinel: they sort behind every key and belong to no list
        sortKey[i] = (row >= 0 && row < cumsum[t + 1] - base) ? (uint32_t)(base + row) : sentinel;
        sortVal[i] = (uint32_t)values[i];
    }
}

__global__ __launch_bounds__(kBlock) void k_group_heads(const uint32_t* __restrict__ key, int64_t n, uint32_t sentinel,
                                                        uint8_t* __restrict__ isFirst, uint32_t* __restrict__ tileF)
{
    __shared__ uint32_t red[kBlock / kWave];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n) {
        return;
    }
    const int64_t i0 = tile0 + (int64_t)threadIdx.x * kItems;
    uint32_t prev = (i0 > 0 && i0 <= n) ? key[i0 - 1] : sentinel;
    uint8_t fl[kItems];
    uint32_t f = 0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t i = i0 + k;
        fl[k] = 0;
        if (i < n) {
            const uint32_t cur = key[i];
            fl[k] = (cur != sentinel && (i == 0 || cur != prev)) ? 1 : 0;
            prev = cur;
        }
        f += fl[k];
    }
    *reinterpret_cast<uchar4*>(isFirst + i0) = make_uchar4(fl[0], fl[1], fl[2], fl[3]);
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) {
        f += __shfl_down(f, d, kWave);
    }
    if (lane_id() == 0) {
        red[threadIdx.x >> 6] = f;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t sum = 0;
        for (int k = 0; k < kBlock / kWave; ++k) {
            sum += red[k];
        }
        tileF[blockIdx.x] = sum;
    }
}

// single block: exclusive scan of the tile counts in place; totals[0] = distinct keys; counters cleared
__global__ __launch_bounds__(kBlock) void k_group_scan(uint32_t* tileF, int64_t ntiles, int64_t* totals,
                                                       uint32_t* counters, int64_t n)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carry;
    if (threadIdx.x == 0) {
        carry = 0;
    }
    if (threadIdx.x < 8) {
        counters[threadIdx.x] = 0;
    }
    __syncthreads();
    // kItems tiles per thread and round
    for (int64_t b = 0; b < ntiles; b += kTile) {
        uint32_t v[kItems];
        uint32_t sum = 0;
#pragma unroll
        for (int k = 0; k < kItems; ++k) {
            const int64_t j = b + (int64_t)threadIdx.x * kItems + k;
            v[k] = j < ntiles ? tileF[j] : 0;
            sum += v[k];
        }
        uint32_t tot;
        uint32_t e = block_exclusive_scan(sum, smem, &tot) + carry;
#pragma unroll
        for (int k = 0; k < kItems; ++k) {
            const int64_t j = b + (int64_t)threadIdx.x * kItems + k;
            if (j < ntiles) {
                tileF[j] = e;
            }
            e += v[k];
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            carry += tot;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        totals[0] = carry;
        totals[1] = 0;
        totals[2] = n;  // end of the last list; lowered by the emit kernel when rows were left out
    }
}

__global__ __launch_bounds__(kBlock) void k_group_emit(const uint32_t* __restrict__ key,
                                                       const uint8_t* __restrict__ isFirst,
                                                       const uint32_t* __restrict__ tileF, int64_t n, uint32_t sentinel,
                                                       int64_t* __restrict__ uniq, uint32_t* __restrict__ useg,
                                                       int64_t* __restrict__ totals)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n) {
        return;
    }
    const int64_t i0 = tile0 + (int64_t)threadIdx.x * kItems;
    const uchar4 f4 = *reinterpret_cast<const uchar4*>(isFirst + i0);
    const uint8_t fl[kItems] = {f4.x, f4.y, f4.z, f4.w};
    uint32_t tot;
    uint32_t r = block_exclusive_scan((uint32_t)(fl[0] + fl[1] + fl[2] + fl[3]), smem, &tot) + tileF[blockIdx.x];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const int64_t i = i0 + k;
        if (i >= n) {
            break;
        }
        const uint32_t cur = key[i];
        if (fl[k]) {
            uniq[r] = (int64_t)cur;
            useg[r] = (uint32_t)i;
            r += 1;
        } else if (cur == sentinel && (i == 0 || key[i - 1] != sentinel)) {
            totals[2] = i;  // the first left-out row ends the last list
        }
    }
}

// per distinct key: multiplicity, row inside its table; keys seen more than kListMax times get a long id
__global__ __launch_bounds__(kBlock) void k_group_finish(const int64_t* __restrict__ totals,
                                                         const int64_t* __restrict__ uniq,
                                                         const uint32_t* __restrict__ useg,
                                                         const int64_t* __restrict__ cumsum, int T,
                                                         uint32_t* __restrict__ ucount, int64_t* __restrict__ slots,
                                                         uint32_t* counters, int32_t* __restrict__ longList,
                                                         uint32_t* __restrict__ longSeg, uint32_t* __restrict__ longCnt)
{
    const int64_t U = totals[0];
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R >= U) {
        return;
    }
    const uint32_t start = useg[R];
    const uint32_t end = (R + 1 < U) ? useg[R + 1] : (uint32_t)totals[2];
    const uint32_t c = end - start;
    const int64_t k = uniq[R];
    const int t = find_segment(cumsum, T, k);
    ucount[R] = c;
    slots[R] = k - cumsum[t];
    if (c > (uint32_t)kListMax) {
        const uint32_t lid = atomicAdd(&counters[0], 1u);
        longList[lid] = (int32_t)R;
        longSeg[lid] = start;
        longCnt[lid] = c;
    }
}

// uoff[t] = number of distinct keys below table t's first row (keys are ascending)
__global__ void k_group_uoff(const int64_t* __restrict__ totals, const int64_t* __restrict__ uniq,
                             const int64_t* __restrict__ cumsum, int T, int64_t* __restrict__ uoff)
{
    const int64_t U = totals[0];
    for (int t = threadIdx.x; t <= T; t += blockDim.x) {
        const int64_t want = cumsum[t];
        int64_t lo = 0;
        int64_t hi = U;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (uniq[mid] < want) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        uoff[t] = lo;
    }
}

}  // namespace recsdk

using namespace recsdk;

// Device buffers the dedup kernels work in (beyond the caller's keys and the results).
struct DedupWorkspace {
    DedupEntry* S;       // 4 n + 65 T entries
    int32_t* sslot;      // n rounded up to a whole tile
    uint8_t* isFirst;    // n rounded up to a whole tile
    uint32_t* tileF;     // tiles + 1
    int64_t* sbase;      // T + 1
    uint32_t* smask;     // T + 1
    uint32_t* counters;  // 8
    int64_t* totals;     // 4
};

// The launches from the scratch clear to the inverse index: they fill v.uniq, v.uoff, v.inverse, v.grank, with
// `counts` also v.ucount, and with sortKey the (rank, position) pairs that the list kernels sort.
static int dedup_core(const DedupWorkspace& w, const UniqueView& v, const int64_t* d_keys, const uint32_t* d_in_counts,
                      const int64_t* d_offsets, int32_t T, int64_t n, int32_t skip_key_enabled, int64_t skip_key,
                      bool counts, uint32_t* sortKey, uint32_t* sortVal, uint32_t sentinel, int64_t segBound,
                      hipStream_t s)
{
    const int64_t ntiles = cdiv(n, kTile);
    const unsigned grid = (unsigned)(ntiles > 0 ? ntiles : 1);
    {
        int64_t entries = 4 * n + 65 * (int64_t)T;
        unsigned cg = (unsigned)std::min<int64_t>(cdiv(entries, kBlock), 256 * 32);
        RECSDK_LAUNCH(k_dedup_plan_clear, dim3(cg), dim3(kBlock), s, d_offsets, T, w.sbase, w.smask, w.counters, w.S,
                      segBound);
    }
    if (n > 0) {
        // a small batch: four times as many, smaller blocks
        const bool small = ntiles < 2 * 256;
        const dim3 ig(small ? (unsigned)cdiv(n, kBlock) : grid);
#define RECSDK_DEDUP_INSERT(ITEMS, COUNT)                                                                         \
    RECSDK_LAUNCH_AS("k_dedup_insert", (k_dedup_insert<ITEMS, COUNT>), ig, dim3(kBlock), s, d_keys, d_in_counts,   \
                     d_offsets, T, w.sbase, w.smask, w.S, w.sslot, n, skip_key_enabled, (long long)skip_key)
        if (small && counts) {
            RECSDK_DEDUP_INSERT(1, true);
        } else if (small) {
            RECSDK_DEDUP_INSERT(1, false);
        } else if (counts) {
            RECSDK_DEDUP_INSERT(kItems, true);
        } else {
            RECSDK_DEDUP_INSERT(kItems, false);
        }
#undef RECSDK_DEDUP_INSERT
        RECSDK_LAUNCH(k_dedup_flags, dim3(grid), dim3(kBlock), s, w.S, w.sslot, d_offsets, T, w.isFirst, w.tileF, n);
    }
    RECSDK_LAUNCH(k_dedup_tilescan, dim3(1), dim3(kBlock), s, w.tileF, w.isFirst, d_offsets, T, v.uoff, w.totals, n);
    if (n > 0) {
        RECSDK_LAUNCH(k_dedup_inverse, dim3(grid), dim3(kTile), s, w.S, w.sslot, d_keys, d_offsets, T, w.isFirst,
                      w.tileF, v.uoff, v.uniq, counts ? v.ucount : (uint32_t*)nullptr, v.inverse, v.grank, sortKey,
                      sortVal, sentinel, n);
    }
    return RECSDK_OK;
}

struct recsdk_unique {
    int64_t maxKeys = 0;
    int32_t maxTables = 0;
    bool wantLists = true;   // build the per-key position lists (only the gradient reduce reads them)
    bool wantCounts = true;  // collect the multiplicities in the insert kernel, so that they exist before the lists
    int64_t maxTableKeys = 0;  // promised bound of the keys of one table per run (0 = unknown): sizes the sort's key
    // The list kernels after `inverse` (sort of the positions by rank, list starts, split of the long ids) feed only
    // the gradient reduce.  They run on the handle's own stream so that the caller's stream can go on to the
    // key -> slot kernels and the forward gather; list readers wait for evLists.
    hipStream_t listStream = nullptr;
    hipEvent_t evFork = nullptr;
    hipEvent_t evLists = nullptr;
    bool listsPending = false;
    // workspace
    DedupEntry* S = nullptr;
    int32_t* sslot = nullptr;
    uint8_t* isFirst = nullptr;
    uint32_t* tileF = nullptr;
    uint32_t* sortKey = nullptr;     // per position: rank of its key, or a sentinel
    uint32_t* sortKeyOut = nullptr;
    uint32_t* longCnt = nullptr;     // long id -> multiplicity of its key (what k_dedup_classify sorts by)
    uint32_t* sortVal = nullptr;     // per position: the position
    void* sortTmp = nullptr;         // the radix sort's workspace, cut up in sortWs
    rsort::Workspace sortWs;
    int64_t* sbase = nullptr;
    uint32_t* smask = nullptr;
    uint32_t* counters = nullptr;
    int64_t* totals = nullptr;
    // results
    UniqueView view;
};

// Stable sort of the handle's n (sortKey, sortVal) pairs by keys that hold nothing above their low `bits` bits: the
// library's own one-sweep radix sort (radix_sort.h), kernels only, so that a captured stream records no memset node.
static int sort_pairs_stable(recsdk_unique* u, const char* name, uint32_t* keysOut, uint32_t* valsOut, int64_t n, int bits,
                             hipStream_t s)
{
    return rsort::sort_pairs<uint32_t>(u->sortWs, name, u->sortKey, keysOut, u->sortVal, valsOut, n, bits, s);
}

static void unique_free(recsdk_unique* u)
{
    if (u->listStream != nullptr) {
        (void)hipStreamSynchronize(u->listStream);
        (void)hipStreamDestroy(u->listStream);
    }
    if (u->evFork != nullptr) {
        (void)hipEventDestroy(u->evFork);
    }
    if (u->evLists != nullptr) {
        (void)hipEventDestroy(u->evLists);
    }
    void* ptrs[] = {u->S, u->sslot, u->isFirst, u->tileF, u->sbase, u->smask, u->counters, u->totals,
                    u->sortKey, u->sortKeyOut, u->sortVal, u->sortTmp, u->longCnt,
                    (void*)u->view.longSeg, (void*)u->view.hugeIds, (void*)u->view.longIds, u->view.longMeta,
                    u->view.chunkMeta, (void*)u->view.chunkSums, (void*)u->view.chunkList, (void*)u->view.chunkIds,
                    (void*)u->view.uniq, (void*)u->view.uoff, (void*)u->view.inverse, (void*)u->view.grank,
                    (void*)u->view.ucount, (void*)u->view.useg, (void*)u->view.posList, (void*)u->view.longList};
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
    alloc(&u->sortKey, sizeof(uint32_t) * padded);
    alloc(&u->sortKeyOut, sizeof(uint32_t) * padded);
    alloc(&u->sortVal, sizeof(uint32_t) * padded);
    alloc(&u->sortTmp, rsort::workspace_bytes(max_keys, sizeof(uint32_t)));
    if (ok) {
        u->sortWs = rsort::workspace_carve(u->sortTmp, max_keys, sizeof(uint32_t));
    }
    alloc(&u->sbase, sizeof(int64_t) * (max_tables + 1));
    alloc(&u->smask, sizeof(uint32_t) * (max_tables + 1));
    alloc(&u->counters, sizeof(uint32_t) * 8);
    alloc(&u->totals, sizeof(int64_t) * 4);
    alloc(&u->view.uniq, sizeof(int64_t) * padded);
    alloc(&u->view.uoff, sizeof(int64_t) * (max_tables + 1));
    alloc(&u->view.inverse, sizeof(int32_t) * padded);
    alloc(&u->view.grank, sizeof(int32_t) * padded);
    alloc(&u->view.ucount, sizeof(uint32_t) * padded);
    alloc(&u->view.useg, sizeof(uint32_t) * (padded + 1));
    alloc(&u->view.posList, sizeof(int32_t) * padded);
    alloc(&u->view.longList, sizeof(int32_t) * (max_keys / kListMax + 2));
    alloc(&u->view.longSeg, sizeof(uint32_t) * (max_keys / kListMax + 2));
    alloc(&u->longCnt, sizeof(uint32_t) * (max_keys / kListMax + 2));
    alloc(&u->view.hugeIds, sizeof(int32_t) * (max_keys / kListMax + 2));
    alloc(&u->view.longIds, sizeof(int32_t) * (max_keys / kListMax + 2));
    u->view.longPos = u->view.posList;  // every list, long or short, is a stretch of the sorted positions
    alloc(&u->view.longMeta, (size_t)64 * (max_keys / kListMax + 2));
    if (!ok) {
        (void)hipGetLastError();
        unique_free(u);
        delete u;
        set_error("recsdk_unique_create: hipMalloc failed for %lld keys", (long long)max_keys);
        return RECSDK_ENOMEM;
    }
    // RECSDK_SERIAL_LISTS=1 keeps the list kernels on the caller's stream (per-kernel measurements)
    if (getenv("RECSDK_SERIAL_LISTS") == nullptr) {
        if (hipStreamCreateWithFlags(&u->listStream, hipStreamNonBlocking) != hipSuccess ||
            hipEventCreateWithFlags(&u->evFork, hipEventDisableTiming) != hipSuccess ||
            hipEventCreateWithFlags(&u->evLists, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            unique_free(u);
            delete u;
            set_error("recsdk_unique_create: could not create the list stream");
            return RECSDK_EHIP;
        }
    }
    u->view.nChunks = u->counters + 5;
    u->view.zero = u->counters + 6;
    u->view.nLong = u->counters;
    u->view.nHuge = u->counters + 2;
    u->view.nLongRest = u->counters + 3;
    u->view.nVeryHuge = u->counters + 4;
    u->view.total = u->totals;
    *out = u;
    return RECSDK_OK;
}

extern "C" int recsdk_unique_set_lists(recsdk_unique_t* u, int32_t enable)
{
    RECSDK_REQUIRE(u != nullptr, RECSDK_ENULL, "recsdk_unique_set_lists: NULL handle");
    u->wantLists = enable != 0;
    return RECSDK_OK;
}

extern "C" int recsdk_unique_set_counts(recsdk_unique_t* u, int32_t enable)
{
    RECSDK_REQUIRE(u != nullptr, RECSDK_ENULL, "recsdk_unique_set_counts: NULL handle");
    u->wantCounts = enable != 0;
    return RECSDK_OK;
}

extern "C" int recsdk_unique_set_max_table_keys(recsdk_unique_t* u, int64_t max_table_keys)
{
    RECSDK_REQUIRE(u != nullptr, RECSDK_ENULL, "recsdk_unique_set_max_table_keys: NULL handle");
    RECSDK_REQUIRE(max_table_keys >= 0, RECSDK_EINVAL, "recsdk_unique_set_max_table_keys: negative bound");
    u->maxTableKeys = max_table_keys;
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
    return recsdk_unique_run_lists(u, d_keys, d_in_counts, d_offsets, T, n, skip_key_enabled, skip_key, true, stream);
}

int recsdk_unique_run_lists(recsdk_unique* u, const int64_t* d_keys, const uint32_t* d_in_counts,
                            const int64_t* d_offsets, int32_t T, int64_t n, int32_t skip_key_enabled, int64_t skip_key,
                            bool allow_small, void* stream)
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
    v.hasLists = (d_in_counts == nullptr) && u->wantLists;
    v.listsReady = nullptr;
    v.classesReady = nullptr;
    v.longPos = v.posList;
    v.scanReduce = false;
    if (allow_small && n <= small_batch_keys() && T <= kSmallTables) {
        // one launch; the gradient reduce of this run scans the inverse index instead of reading position lists
        if (u->listsPending) {
            RECSDK_HIP_TRY(hipStreamWaitEvent(s, u->evLists, 0));
            u->listsPending = false;
        }
        v.countsWithLists = false;
        v.scanReduce = v.hasLists;
        RECSDK_LAUNCH(k_dedup_small, dim3(1), dim3(kSmallBlock), s, d_keys, d_in_counts, d_offsets, T,
                      skip_key_enabled ? 1 : 0, (long long)skip_key, v.uniq, v.uoff, v.inverse, v.grank, v.ucount,
                      u->totals, u->counters, (int)n);
        return RECSDK_OK;
    }
    // the multiplicities come from the insert kernel when the caller wants them early or brings input counts to sum,
    // and always when no lists are built; otherwise the list kernels deliver them as list lengths
    const bool counts = u->wantCounts || d_in_counts != nullptr || !v.hasLists;
    v.countsWithLists = !counts;
    if (u->listsPending) {
        // the previous run's list kernels still own the list buffers this run rewrites
        RECSDK_HIP_TRY(hipStreamWaitEvent(s, u->evLists, 0));
        u->listsPending = false;
    }
    // sort keys are the keys' indices inside their tables (below the largest number of keys a table can hold); skipped
    // positions take all ones in the sorted bits and are told apart later by their rank of -1
    const bool lists = v.hasLists && n > 0;
    const int64_t segBound = (u->maxTableKeys > 0 && u->maxTableKeys < n) ? u->maxTableKeys : std::max<int64_t>(n, 1);
    int bits = 1;
    while ((int64_t(1) << bits) < segBound) {
        ++bits;
    }
    const uint32_t sentinel = (uint32_t)((int64_t(1) << bits) - 1);
    DedupWorkspace ws;
    ws.S = u->S;
    ws.sslot = u->sslot;
    ws.isFirst = u->isFirst;
    ws.tileF = u->tileF;
    ws.sbase = u->sbase;
    ws.smask = u->smask;
    ws.counters = u->counters;
    ws.totals = u->totals;
    {
        const int rc = dedup_core(ws, v, d_keys, d_in_counts, d_offsets, T, n, skip_key_enabled, skip_key, counts,
                                  lists ? u->sortKey : (uint32_t*)nullptr, u->sortVal, sentinel, segBound, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    if (lists) {
        hipStream_t ls = s;
        const bool fork = u->listStream != nullptr;
        if (fork) {
            ls = u->listStream;
            RECSDK_HIP_TRY(hipEventRecord(u->evFork, s));
            RECSDK_HIP_TRY(hipStreamWaitEvent(ls, u->evFork, 0));
        }
        {
            const int rc = sort_pairs_stable(u, "sort_positions_by_rank", u->sortKeyOut,
                                             reinterpret_cast<uint32_t*>(v.posList), n, bits, ls);
            if (rc != RECSDK_OK) {
                return rc;
            }
        }
        uint32_t* uend = u->sortKey;  // the sort's input keys are dead by now
        if (T <= kBoundsTables) {
            RECSDK_LAUNCH_AS("k_lists_bounds", (k_lists_bounds<true>), dim3((unsigned)cdiv(n, kTile)), dim3(kBlock), ls,
                             u->sortKeyOut, v.posList, v.grank, d_offsets, v.uoff, T, sentinel, n, v.useg, uend);
        } else {
            RECSDK_LAUNCH_AS("k_lists_bounds", (k_lists_bounds<false>), dim3((unsigned)cdiv(n, kTile)), dim3(kBlock), ls,
                             u->sortKeyOut, v.posList, v.grank, d_offsets, v.uoff, T, sentinel, n, v.useg, uend);
        }
        {
            const unsigned fg = (unsigned)std::min<int64_t>(cdiv(n, kBlock), 256);
            RECSDK_LAUNCH(k_lists_finish, dim3(fg), dim3(kBlock), ls, u->totals, v.useg, uend, v.ucount, u->counters,
                          v.longList, v.longSeg, u->longCnt);
        }
        if (n > kListMax) {
            RECSDK_LAUNCH_AS("k_dedup_classify", k_dedup_classify<256>, dim3(1), dim3(256), ls, u->longCnt, u->counters, v.hugeIds, v.longIds);
        }
        if (fork) {
            RECSDK_HIP_TRY(hipEventRecord(u->evLists, ls));
            u->listsPending = true;
            v.listsReady = u->evLists;
        }
    }
    return RECSDK_OK;
}

// ---- the dedup without allocation: the workspace is a static device array ---------------------------------------
namespace recsdk {
constexpr int64_t kNoAllocMaxKeys = RECSDK_UNIQUE_NOALLOC_MAX_KEYS;
constexpr int32_t kNoAllocMaxTables = RECSDK_UNIQUE_NOALLOC_MAX_TABLES;
constexpr int64_t kNoAllocPadded = (kNoAllocMaxKeys + kTile - 1) / kTile * kTile;
constexpr int64_t kNoAllocTiles = kNoAllocPadded / kTile + 1;
constexpr size_t align256(size_t x) { return (x + 255) / 256 * 256; }
// carve-up of the static array, every piece 256-byte aligned
constexpr size_t kNaS = 0;
constexpr size_t kNaSslot = kNaS + align256(sizeof(DedupEntry) * (4 * kNoAllocMaxKeys + 65 * (int64_t)kNoAllocMaxTables));
constexpr size_t kNaIsFirst = kNaSslot + align256(sizeof(int32_t) * kNoAllocPadded);
constexpr size_t kNaTileF = kNaIsFirst + align256(kNoAllocPadded);
constexpr size_t kNaSbase = kNaTileF + align256(sizeof(uint32_t) * kNoAllocTiles);
constexpr size_t kNaSmask = kNaSbase + align256(sizeof(int64_t) * (kNoAllocMaxTables + 1));
constexpr size_t kNaCounters = kNaSmask + align256(sizeof(uint32_t) * (kNoAllocMaxTables + 1));
constexpr size_t kNaTotals = kNaCounters + align256(sizeof(uint32_t) * 8);
constexpr size_t kNaGrank = kNaTotals + align256(sizeof(int64_t) * 4);
constexpr size_t kNaUcount = kNaGrank + align256(sizeof(int32_t) * kNoAllocPadded);
constexpr size_t kNaBytes = kNaUcount + align256(sizeof(uint32_t) * kNoAllocPadded);
}  // namespace recsdk

// Workspace of recsdk_unique_run_noalloc (about 5 MB per device, held until the process ends).  In host code this
// name is only a handle for hipGetSymbolAddress: kernels get the address that call returns for the current device.
static __device__ __align__(256) unsigned char scratch[recsdk::kNaBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratchMutex;
unsigned char* g_scratchPtr[kMaxDevices] = {};
}  // namespace

// Address of `scratch` on the current device (looked up once per device).
static int noalloc_scratch(unsigned char** out)
{
    int dev = 0;
    RECSDK_HIP_TRY(hipGetDevice(&dev));
    RECSDK_REQUIRE(dev >= 0 && dev < kMaxDevices, RECSDK_EINVAL, "recsdk_unique_run_noalloc: device index out of range");
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if (g_scratchPtr[dev] == nullptr) {
        void* p = nullptr;
        RECSDK_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        RECSDK_REQUIRE(p != nullptr, RECSDK_EHIP, "recsdk_unique_run_noalloc: the static workspace has no device address");
        g_scratchPtr[dev] = static_cast<unsigned char*>(p);
    }
    *out = g_scratchPtr[dev];
    return RECSDK_OK;
}

extern "C" int recsdk_unique_run_noalloc(const int64_t* d_keys, const uint32_t* d_in_counts, const int64_t* d_offsets,
                                         int32_t T, int64_t n, int32_t skip_key_enabled, int64_t skip_key,
                                         int64_t* d_unique_keys, int64_t* d_unique_offsets, int32_t* d_inverse,
                                         uint32_t* d_counts, void* stream)
{
    RECSDK_REQUIRE(d_offsets != nullptr && d_unique_offsets != nullptr, RECSDK_ENULL,
                   "recsdk_unique_run_noalloc: NULL argument");
    RECSDK_REQUIRE(T > 0 && T <= kNoAllocMaxTables, RECSDK_ECAPACITY,
                   "recsdk_unique_run_noalloc: T exceeds RECSDK_UNIQUE_NOALLOC_MAX_TABLES");
    RECSDK_REQUIRE(n >= 0 && n <= kNoAllocMaxKeys, RECSDK_ECAPACITY,
                   "recsdk_unique_run_noalloc: n exceeds RECSDK_UNIQUE_NOALLOC_MAX_KEYS");
    RECSDK_REQUIRE(n == 0 || (d_keys != nullptr && d_unique_keys != nullptr && d_inverse != nullptr), RECSDK_ENULL,
                   "recsdk_unique_run_noalloc: NULL key, unique-key or inverse buffer");
    unsigned char* base = nullptr;
    {
        const int rc = noalloc_scratch(&base);
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    DedupWorkspace ws;
    ws.S = reinterpret_cast<DedupEntry*>(base + kNaS);
    ws.sslot = reinterpret_cast<int32_t*>(base + kNaSslot);
    ws.isFirst = base + kNaIsFirst;
    ws.tileF = reinterpret_cast<uint32_t*>(base + kNaTileF);
    ws.sbase = reinterpret_cast<int64_t*>(base + kNaSbase);
    ws.smask = reinterpret_cast<uint32_t*>(base + kNaSmask);
    ws.counters = reinterpret_cast<uint32_t*>(base + kNaCounters);
    ws.totals = reinterpret_cast<int64_t*>(base + kNaTotals);
    UniqueView v;
    v.keys = d_keys;
    v.off = d_offsets;
    v.T = T;
    v.n = n;
    v.hasLists = false;
    v.uniq = d_unique_keys;
    v.uoff = d_unique_offsets;
    v.inverse = d_inverse;
    v.grank = reinterpret_cast<int32_t*>(base + kNaGrank);
    v.ucount = d_counts != nullptr ? d_counts : reinterpret_cast<uint32_t*>(base + kNaUcount);
    return dedup_core(ws, v, d_keys, d_in_counts, d_offsets, T, n, skip_key_enabled, skip_key, true, nullptr, nullptr,
                      0u, std::max<int64_t>(n, 1), static_cast<hipStream_t>(stream));
}

int recsdk_unique_group_input(recsdk_unique* u, uint32_t** key, uint32_t** value)
{
    RECSDK_REQUIRE(u != nullptr && key != nullptr && value != nullptr, RECSDK_ENULL,
                   "recsdk_unique_group_input: NULL argument");
    *key = u->sortKey;
    *value = u->sortVal;
    return RECSDK_OK;
}

int recsdk_unique_run_grouped(recsdk_unique* u, const int64_t* d_rows, const int64_t* d_tb,
                              const int64_t* d_row_base, int32_t T, int64_t n, int64_t total_rows,
                              const int32_t* d_values, int64_t* d_slots, hipStream_t s)
{
    RECSDK_REQUIRE(u != nullptr && d_rows != nullptr && d_tb != nullptr && d_row_base != nullptr && d_slots != nullptr,
                   RECSDK_ENULL, "recsdk_unique_run_grouped: NULL argument");
    RECSDK_REQUIRE(T > 0 && T <= u->maxTables && n > 0 && n <= u->maxKeys, RECSDK_ECAPACITY,
                   "recsdk_unique_run_grouped: T or n exceeds what the handle was created for");
    RECSDK_REQUIRE(total_rows > 0 && total_rows < (int64_t)0xFFFFFFFFLL, RECSDK_EINVAL,
                   "recsdk_unique_run_grouped: the tables hold 2^32 rows or more");
    UniqueView& v = u->view;
    v.keys = d_rows;
    v.off = d_tb;
    v.T = T;
    v.n = n;
    v.hasLists = true;
    v.listsReady = nullptr;
    v.classesReady = nullptr;
    v.longPos = v.posList;  // every list, long or short, is a stretch of the sorted values
    if (u->listsPending) {
        RECSDK_HIP_TRY(hipStreamWaitEvent(s, u->evLists, 0));
        u->listsPending = false;
    }
    const uint32_t sentinel = (uint32_t)total_rows;  // above every table base + row
    int bits = 1;
    while ((int64_t(1) << bits) <= total_rows) {
        ++bits;
    }
    const int64_t ntiles = cdiv(n, kTile);
    const unsigned grid = (unsigned)ntiles;
    if (d_values != nullptr) {
        RECSDK_LAUNCH(k_group_keys, dim3(grid), dim3(kBlock), s, d_rows, d_tb, d_row_base, T, d_values, u->sortKey,
                      u->sortVal, n, sentinel);
    }
    {
        const int rc = sort_pairs_stable(u, "sort_rows", u->sortKeyOut, reinterpret_cast<uint32_t*>(v.posList), n,
                                         bits, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    RECSDK_LAUNCH(k_group_heads, dim3(grid), dim3(kBlock), s, u->sortKeyOut, n, sentinel, u->isFirst, u->tileF);
    RECSDK_LAUNCH(k_group_scan, dim3(1), dim3(kBlock), s, u->tileF, ntiles, u->totals, u->counters, n);
    RECSDK_LAUNCH(k_group_emit, dim3(grid), dim3(kBlock), s, u->sortKeyOut, u->isFirst, u->tileF, n, sentinel, v.uniq,
                  v.useg, u->totals);
    RECSDK_LAUNCH(k_group_finish, dim3((unsigned)cdiv(n, kBlock)), dim3(kBlock), s, u->totals, v.uniq, v.useg,
                  d_row_base, T, v.ucount, d_slots, u->counters, v.longList, v.longSeg, u->longCnt);
    RECSDK_LAUNCH(k_group_uoff, dim3(1), dim3(kBlock), s, u->totals, v.uniq, d_row_base, T, v.uoff);
    if (n > kListMax) {
        // The classes of the long lists (one block's work) are read by the long-list kernels only: on the handle's own
        // stream they run beside whatever the caller enqueues next, normally the short-list kernel.
        hipStream_t cs = s;
        if (u->listStream != nullptr) {
            cs = u->listStream;
            RECSDK_HIP_TRY(hipEventRecord(u->evFork, s));
            RECSDK_HIP_TRY(hipStreamWaitEvent(cs, u->evFork, 0));
        }
        RECSDK_LAUNCH_AS("k_dedup_classify", k_dedup_classify<1024>, dim3(1), dim3(1024), cs, u->longCnt, u->counters,
                         v.hugeIds, v.longIds);
        if (cs != s) {
            RECSDK_HIP_TRY(hipEventRecord(u->evLists, cs));
            u->listsPending = true;  // the next run waits for it before it touches the counters
            v.classesReady = u->evLists;
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
        if (v.countsWithLists && v.listsReady != nullptr) {
            RECSDK_HIP_TRY(hipStreamWaitEvent(s, v.listsReady, 0));  // the multiplicities are the list lengths
        }
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
    uint32_t segError = 0;
    RECSDK_HIP_TRY(hipMemcpyAsync(h_total, u->totals, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipMemcpyAsync(&segError, u->counters + kCounterSegError, sizeof(uint32_t), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    RECSDK_REQUIRE(segError == 0 || !u->view.hasLists, RECSDK_ECAPACITY,
                   "recsdk_unique_run: a table held more keys than recsdk_unique_set_max_table_keys promised; the "
                   "position lists of this run are empty");
    return RECSDK_OK;
}

namespace recsdk {
__global__ __launch_bounds__(kBlock) void k_iota(int32_t* out, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) {
        out[i] = (int32_t)i;
    }
}
}  // namespace recsdk

int recsdk_unique_chunk_buffers(recsdk_unique* u, int32_t dim)
{
    UniqueView& v = u->view;
    const int32_t pitch = (dim + 3) / 4 * 4;
    if (v.chunkCap > 0 && v.chunkPitch >= pitch) {
        return RECSDK_OK;
    }
    // a key seen c > kTwoLevelMin times has ceil(c / kChunkRows) chunks; all such keys of a run of n positions
    // together have fewer than n / kChunkRows + n / kTwoLevelMin + 1
    const int64_t cap = u->maxKeys / kChunkRows + u->maxKeys / kTwoLevelMin + 2;
    if (v.chunkSums != nullptr) {
        RECSDK_HIP_TRY(hipFree(v.chunkSums));  // waits for the device: no kernel still reads it
        v.chunkSums = nullptr;
    }
    RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&v.chunkSums), sizeof(float) * cap * pitch));
    if (v.chunkMeta == nullptr) {
        RECSDK_HIP_TRY(hipMalloc(&v.chunkMeta, (size_t)64 * cap));
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&v.chunkList), sizeof(int32_t) * cap));
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&v.chunkIds), sizeof(int32_t) * cap));
        hipLaunchKernelGGL(k_iota, dim3((unsigned)cdiv(cap, kBlock)), dim3(kBlock), 0, (hipStream_t) nullptr, v.chunkIds,
                           cap);
        RECSDK_HIP_TRY(hipGetLastError());
        RECSDK_HIP_TRY(hipStreamSynchronize(nullptr));
    }
    v.chunkCap = cap;
    v.chunkPitch = pitch;
    return RECSDK_OK;
}

const recsdk::UniqueView* recsdk_unique_view(const recsdk_unique* u) { return &u->view; }
