// key -> slot / address tables on the device: open addressing, 64-bit keys, 16-byte {key, slot} slots,
// linear probing, CAS insertion.  Slot numbers are assigned from a scan over the "is new" flags in array
// order, so they do not depend on how the insertion races resolve:
//   new key with rank r among the table's new keys of this call takes
//     evicted[evictCount-1-r]           while r < evictCount   (last evicted first)
//     maxOffset + (r - evictCount)      afterwards.
#include <string.h>

#include <algorithm>
#include <vector>

#include <rocprim/rocprim.hpp>

#include "common.h"
#include "hashmap.h"
#include "tables.h"

namespace recsdk {

struct TableDesc {
    TableEntry* entries;   // capacity + 1 entries; the last one is the side slot of the key equal to kTombKey
    uint64_t mask;         // capacity - 1
    int64_t vocab;
    int64_t maxOffset;
    int64_t live;
    int64_t evictCount;
    int64_t* evictPos;
    int64_t evictCap;
    int64_t arenaBase;
    int64_t rowBytes;
    int32_t dynamic;
    int32_t overflow;      // bit flags, sticky: kTableVocabOverflow | kTableDupKey | kTableMapFull
    int64_t tombs;         // entries erased since the map was last rebuilt (an upper bound of the erased entries it
                           // still holds: insertions that reuse one are not taken off); counted on the device, so that
                           // evictions replayed from a graph are counted too
};
constexpr int32_t kTableVocabOverflow = 1;
constexpr int32_t kTableDupKey = 2;
constexpr int32_t kTableMapFull = 4;

__device__ __forceinline__ MapRef map_of(const TableDesc& d) { return MapRef{d.entries, d.mask}; }

// ---- key2offset ---------------------------------------------------------------------------------
// pass 1: resolve existing keys in place, flag new ones, per-tile counts of new keys
__global__ __launch_bounds__(kTile) void k_table_probe(const TableDesc* __restrict__ descs, int64_t* keys,
                                                       const int64_t* __restrict__ off, int T, int channel,
                                                       uint8_t* __restrict__ isNew, uint32_t* __restrict__ tileN,
                                                       int64_t nMax)
{
    __shared__ uint32_t red[kTile / kWave];
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
    const int64_t i = tile0 + (int64_t)threadIdx.x;  // one key per thread, a tile per block
    uint32_t f = 0;
    if (i < n) {
        const TableDesc& d = descs[advance_segment(off, sT0, i)];
        const long long key = keys[i];
        if (key == kEmptyKey) {
            if (d.dynamic) {
                keys[i] = 0;
            }
        } else {
            const int64_t pos = map_find(map_of(d), key);
            if (pos >= 0) {
                keys[i] = d.entries[pos].slot;
            } else if (channel == RECSDK_CHANNEL_TRAIN) {
                f = 1;
            } else {
                keys[i] = d.dynamic ? 0 : -1;
            }
        }
    }
    isNew[i] = (uint8_t)f;  // whole tiles of flags
#pragma unroll
    for (int dlt = kWave / 2; dlt > 0; dlt >>= 1) {
        f += __shfl_down(f, dlt, kWave);
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
        tileN[blockIdx.x] = s;
    }
}

// pass 2 (single block): scan tile counts; per table: rank base of its new keys, snapshot of
// maxOffset/evictCount for pass 3, then the table counters are advanced.
__global__ __launch_bounds__(kBlock) void k_table_scan(TableDesc* descs, uint32_t* tileN,
                                                       const uint8_t* __restrict__ flags,
                                                       const int64_t* __restrict__ off, int T, int64_t* newBase,
                                                       int64_t* snapMax, int64_t* snapEv, int64_t nMax, int evictMode)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ uint32_t carry;
    const int64_t n = off[T] < nMax ? off[T] : nMax;
    const int64_t ntiles = (n + kTile - 1) / kTile;
    if (threadIdx.x == 0) {
        carry = 0;
    }
    __syncthreads();
    for (int64_t b = 0; b < ntiles; b += kBlock) {
        int64_t j = b + threadIdx.x;
        uint32_t v = (j < ntiles) ? tileN[j] : 0;
        uint32_t tot;
        uint32_t e = block_exclusive_scan(v, smem, &tot);
        if (j < ntiles) {
            tileN[j] = carry + e;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            carry += tot;
        }
        __syncthreads();
    }
    segment_start_ranks(flags, tileN, off, T, n, carry, newBase);
    __syncthreads();
    for (int t = threadIdx.x; t < T; t += kBlock) {
        TableDesc& d = descs[t];
        int64_t cnt = newBase[t + 1] - newBase[t];
        snapMax[t] = d.maxOffset;
        snapEv[t] = d.evictCount;
        if (evictMode) {
            d.evictCount += cnt;
            d.live -= cnt;
            d.tombs += cnt;
        } else if (d.dynamic) {
            int64_t room = d.vocab - d.maxOffset;
            if (cnt > room) {
                d.overflow |= kTableVocabOverflow;
            }
            d.maxOffset += cnt;
            d.live += cnt < room ? cnt : (room > 0 ? room : 0);
        } else {
            int64_t reuse = cnt < d.evictCount ? cnt : d.evictCount;
            int64_t fresh = cnt - reuse;
            int64_t room = d.vocab - d.maxOffset;
            d.evictCount -= reuse;
            d.maxOffset += fresh;
            if (fresh > room) {
                d.overflow |= kTableVocabOverflow;
                fresh = room > 0 ? room : 0;
            }
            d.live += reuse + fresh;
        }
    }
}

// pass 3: rank new keys, mint their slot / address, insert, write the result in place.  One key per thread, a tile
// per block of 1024 threads: an insert is a chain of two or three dependent trips to memory (load, compare-and-swap,
// store), and with four keys per thread one after the other a step that creates 80 k keys spent 27 us here.
constexpr int kAssignBlock = 1024;
static_assert(kAssignBlock == kTile, "the ranks of the new keys are counted per tile");
__global__ __launch_bounds__(kAssignBlock) void k_table_assign(const TableDesc* __restrict__ descs, int64_t* keys,
                                                               const int64_t* __restrict__ off, int T,
                                                               const uint8_t* __restrict__ isNew,
                                                               const uint32_t* __restrict__ tileN,
                                                               const int64_t* __restrict__ newBase,
                                                               const int64_t* __restrict__ snapMax,
                                                               const int64_t* __restrict__ snapEv, int64_t nMax,
                                                               int64_t* __restrict__ newRank)
{
    __shared__ uint32_t smem[kAssignBlock / kWave];
    __shared__ int sT0;
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, tile0);
    }
    const int64_t i = tile0 + (int64_t)threadIdx.x;
    const uint32_t f = isNew[i];  // the flags are written for whole tiles
    uint32_t tot;
    const int64_t r = (int64_t)block_exclusive_scan_n<kAssignBlock>(f, smem, &tot) + tileN[blockIdx.x];
    if (f == 0) {
        return;
    }
    const int t = advance_segment(off, sT0, i);
    const TableDesc& d = descs[t];
    const int64_t rt = r - newBase[t];
    const long long key = keys[i];
    long long value;
    bool ok = true;
    if (d.dynamic) {
        const int64_t seq = snapMax[t] + rt;
        ok = seq < d.vocab;
        value = ok ? d.arenaBase + seq * d.rowBytes : 0;
    } else {
        const int64_t ev = snapEv[t];
        if (rt < ev) {
            value = d.evictPos[ev - 1 - rt];
        } else {
            value = snapMax[t] + (rt - ev);
            ok = value < d.vocab;
            if (!ok) {
                value = -1;
            }
        }
    }
    if (ok) {
        const int st = map_insert(map_of(d), key, value);
        if (st != 0) {
            // a key listed twice in one call (the caller did not dedup) or a map without room: the slot
            // counters have been advanced for it already, so the call is reported as failed
            atomicOr(const_cast<int32_t*>(&d.overflow), st == 1 ? kTableDupKey : kTableMapFull);
        }
    }
    keys[i] = value;
    if (newRank != nullptr) {
        newRank[i] = rt;  // the key is the rt-th key its table created in this call
    }
}

// ---- key2offset of a small batch in one launch ---------------------------------------------------
// At most kSmallKeys keys and kSmallTables tables: one block does the three passes above with its flags and prefixes
// in LDS.  A batch of a few thousand keys is bound by the launches it takes, not by its traffic (three dependent
// launches of 4096 keys: 18 us, one: 6).  Slots come out exactly as from the three-kernel path.

__global__ __launch_bounds__(kSmallBlock) void k_table_small(TableDesc* descs, int64_t* keys,
                                                        const int64_t* __restrict__ off, int T, int channel,
                                                        int64_t* __restrict__ snapMaxOut, int64_t* __restrict__ newRank)
{
    constexpr int kPer = kSmallKeys / kSmallBlock;  // consecutive keys per thread
    __shared__ uint32_t smem[kSmallBlock / kWave];
    __shared__ int64_t sOff[kSmallTables + 1];
    __shared__ uint16_t sPre[kSmallKeys + 1];  // new keys before position i
    __shared__ int64_t sBase[kSmallTables + 1];
    __shared__ int64_t sSnapMax[kSmallTables];
    __shared__ int64_t sSnapEv[kSmallTables];
    __shared__ TableDesc sDesc[kSmallTables];  // the tables' descriptors: read by every key, so fetched once
    for (int t = threadIdx.x; t <= T; t += kSmallBlock) {
        sOff[t] = off[t];
        if (t < T) {
            sDesc[t] = descs[t];
        }
    }
    __syncthreads();
    const int64_t n = sOff[T] < kSmallKeys ? sOff[T] : kSmallKeys;
    // pass 1: resolve existing keys in place, flag new ones
    const int64_t i0 = (int64_t)threadIdx.x * kPer;
    bool isNew[kPer];
    uint32_t f = 0;
    int t = (i0 < n) ? find_segment(sOff, T, i0) : 0;
    // the thread's keys and the first entry each of them hashes to are fetched together: one block holds all the
    // parallelism there is, so a thread that probed its keys one after the other would pay kPer memory round trips
    long long kk[kPer];
    int tab[kPer];
    TableEntry first[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const int64_t i = i0 + k;
        kk[k] = (i < n) ? keys[i] : kEmptyKey;
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const int64_t i = i0 + k;
        tab[k] = 0;
        first[k].key = kEmptyKey;
        first[k].slot = -1;
        if (i < n) {
            t = advance_segment(sOff, t, i);
            tab[k] = t;
            if (kk[k] != kEmptyKey && kk[k] != kTombKey) {
                const TableDesc& d = sDesc[t];
                const uint4 raw = *reinterpret_cast<const uint4*>(&d.entries[hash64((uint64_t)kk[k]) & d.mask]);
                first[k].key = (long long)(((unsigned long long)raw.y << 32) | raw.x);
                first[k].slot = (long long)(((unsigned long long)raw.w << 32) | raw.z);
            }
        }
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const int64_t i = i0 + k;
        isNew[k] = false;
        if (i < n) {
            const TableDesc& d = sDesc[tab[k]];
            if (kk[k] == kEmptyKey) {
                if (d.dynamic) {
                    keys[i] = 0;
                }
            } else {
                long long slot = -1;
                bool found = false;
                if (first[k].key == kk[k] && kk[k] != kTombKey) {
                    found = true;
                    slot = first[k].slot;
                } else if (first[k].key != kEmptyKey || kk[k] == kTombKey) {
                    const int64_t pos = map_find(map_of(d), kk[k]);  // a longer probe chain, or the side slot
                    if (pos >= 0) {
                        found = true;
                        slot = d.entries[pos].slot;
                    }
                }
                if (found) {
                    keys[i] = slot;
                } else if (channel == RECSDK_CHANNEL_TRAIN) {
                    isNew[k] = true;
                    f += 1;
                } else {
                    keys[i] = d.dynamic ? 0 : -1;
                }
            }
        }
    }
    if (channel != RECSDK_CHANNEL_TRAIN) {
        return;
    }
    uint32_t total;
    uint32_t r = block_exclusive_scan_n<kSmallBlock>(f, smem, &total);
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        sPre[i0 + k] = (uint16_t)r;
        r += isNew[k] ? 1u : 0u;
    }
    if (threadIdx.x == 0) {
        sPre[kSmallKeys] = (uint16_t)total;
    }
    __syncthreads();
    // pass 2: per table the rank of its first new key, a snapshot of its counters, then the counters advance
    for (int tt = threadIdx.x; tt <= T; tt += kSmallBlock) {
        sBase[tt] = sOff[tt] >= n ? (int64_t)total : (int64_t)sPre[sOff[tt]];
    }
    __syncthreads();
    for (int tt = threadIdx.x; tt < T; tt += kSmallBlock) {
        TableDesc& d = descs[tt];  // the counters advance in the table itself; the block keeps using its copy
        const int64_t cnt = sBase[tt + 1] - sBase[tt];
        sSnapMax[tt] = d.maxOffset;
        sSnapEv[tt] = d.evictCount;
        snapMaxOut[tt] = d.maxOffset;
        if (d.dynamic) {
            const int64_t room = d.vocab - d.maxOffset;
            if (cnt > room) {
                d.overflow |= kTableVocabOverflow;
            }
            d.maxOffset += cnt;
            d.live += cnt < room ? cnt : (room > 0 ? room : 0);
        } else {
            const int64_t reuse = cnt < d.evictCount ? cnt : d.evictCount;
            int64_t fresh = cnt - reuse;
            const int64_t room = d.vocab - d.maxOffset;
            d.evictCount -= reuse;
            d.maxOffset += fresh;
            if (fresh > room) {
                d.overflow |= kTableVocabOverflow;
                fresh = room > 0 ? room : 0;
            }
            d.live += reuse + fresh;
        }
    }
    __syncthreads();
    if (f == 0) {
        return;
    }
    // pass 3: mint the slot of every new key, insert, write the result in place.  A key whose first entry was empty
    // in pass 1 claims it with a compare-and-swap issued together with those of the thread's other keys; only where
    // that fails (another new key took the entry meanwhile) does the key walk its probe chain.
    long long value[kPer];
    bool ok[kPer];
    unsigned long long claimed[kPer];
    bool tried[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        value[k] = 0;
        ok[k] = false;
        if (!isNew[k]) {
            continue;
        }
        const TableDesc& d = sDesc[tab[k]];
        const int64_t rt = (int64_t)sPre[i0 + k] - sBase[tab[k]];
        ok[k] = true;
        if (d.dynamic) {
            const int64_t seq = sSnapMax[tab[k]] + rt;
            ok[k] = seq < d.vocab;
            value[k] = ok[k] ? d.arenaBase + seq * d.rowBytes : 0;
        } else {
            const int64_t ev = sSnapEv[tab[k]];
            if (rt < ev) {
                value[k] = d.evictPos[ev - 1 - rt];
            } else {
                value[k] = sSnapMax[tab[k]] + (rt - ev);
                ok[k] = value[k] < d.vocab;
                if (!ok[k]) {
                    value[k] = -1;
                }
            }
        }
        if (newRank != nullptr) {
            newRank[i0 + k] = rt;
        }
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        claimed[k] = 0;
        tried[k] = isNew[k] && ok[k] && first[k].key == kEmptyKey && kk[k] != kTombKey;
        if (tried[k]) {
            const TableDesc& d = sDesc[tab[k]];
            claimed[k] = atomicCAS(reinterpret_cast<unsigned long long*>(&d.entries[hash64((uint64_t)kk[k]) & d.mask].key),
                                   (unsigned long long)kEmptyKey, (unsigned long long)kk[k]);
        }
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        if (!isNew[k]) {
            continue;
        }
        const TableDesc& d = sDesc[tab[k]];
        if (ok[k]) {
            int st;
            if (tried[k] && (long long)claimed[k] == kEmptyKey) {
                d.entries[hash64((uint64_t)kk[k]) & d.mask].slot = value[k];
                st = 0;
            } else if (tried[k] && (long long)claimed[k] == kk[k]) {
                st = 1;  // the same key was inserted by another position of this call
            } else {
                st = map_insert(map_of(d), kk[k], value[k]);
            }
            if (st != 0) {
                atomicOr(&descs[tab[k]].overflow, st == 1 ? kTableDupKey : kTableMapFull);
            }
        }
        keys[i0 + k] = value[k];
    }
}

// ---- key2offset of a small batch of ONE table on several compute units ---------------------------------
// The one-block kernel above moves 4096 random lines three times (probe, claim, slot) through one compute unit's
// path to L2, which is what its 29 us are made of.  With one table there is one thing the blocks must agree on, the number
// of new keys in front of each block, so the batch is spread over blocks of BLOCK keys: a block takes a ticket (the
// order of its keys), publishes how many new keys it found, adds up what the tickets before it published, and mints
// its slots from there.  The words live in the handle and are all zero between launches: the block with the last
// ticket waits until every block has read what it needs, advances the table's counters and clears them.  Every word
// that one block waits for is written with one atomic store that carries the value itself, so no fence is needed; a
// block waits only for tickets lower than its own, which belong to blocks that are running.  Slots come out exactly as
// from the one-block kernel and from the three-kernel path.  (The same kernel with blocks of 1024 keys for batches of
// up to 262144 keys took 12 us where probe, scan and assign take 17 in three launches, and left the step of 131072
// keys where it was: the position sort runs beside it and is as long.  Not kept.)
constexpr int kSpreadSmallBlock = 256;
constexpr int kSpreadMaxBlocks = kSmallKeys / kSpreadSmallBlock;
constexpr uint32_t kSpreadValid = 1u << 31;
struct SpreadWords {
    uint32_t ticket;
    uint32_t done;
    uint32_t found[kSpreadMaxBlocks];   // kSpreadValid | new keys of the block with that ticket
};

template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void k_table_spread(TableDesc* descs, int64_t* keys,
                                                        const int64_t* __restrict__ off, int channel,
                                                        int64_t* __restrict__ snapMaxOut, int64_t* __restrict__ newRank,
                                                        SpreadWords* words, int64_t nMax)
{
    __shared__ uint32_t smem[BLOCK / kWave];
    __shared__ TableDesc sDesc;
    __shared__ uint32_t sTicket;
    __shared__ uint32_t sBefore;
    if (threadIdx.x == 0) {
        sDesc = descs[0];
        sTicket = atomicAdd(&words->ticket, 1u);
    }
    __syncthreads();   // the descriptor has been read before anything below is published
    const TableDesc& d = sDesc;
    const int64_t n = off[1] < nMax ? off[1] : nMax;
    const uint32_t blocks = gridDim.x;
    const uint32_t ticket = sTicket;
    const int64_t i = (int64_t)ticket * BLOCK + threadIdx.x;
    // pass 1: resolve an existing key in place, flag a new one
    long long kk = kEmptyKey;
    TableEntry first;
    first.key = kEmptyKey;
    first.slot = -1;
    bool isNew = false;
    if (i < n) {
        kk = keys[i];
        if (kk == kEmptyKey) {
            if (d.dynamic) {
                keys[i] = 0;
            }
        } else {
            long long slot = -1;
            bool found = false;
            if (kk != kTombKey) {
                const uint4 raw = *reinterpret_cast<const uint4*>(&d.entries[hash64((uint64_t)kk) & d.mask]);
                first.key = (long long)(((unsigned long long)raw.y << 32) | raw.x);
                first.slot = (long long)(((unsigned long long)raw.w << 32) | raw.z);
            }
            if (first.key == kk && kk != kTombKey) {
                found = true;
                slot = first.slot;
            } else if (first.key != kEmptyKey || kk == kTombKey) {
                const int64_t pos = map_find(map_of(d), kk);  // a longer probe chain, or the side slot
                if (pos >= 0) {
                    found = true;
                    slot = d.entries[pos].slot;
                }
            }
            if (found) {
                keys[i] = slot;
            } else if (channel == RECSDK_CHANNEL_TRAIN) {
                isNew = true;
            } else {
                keys[i] = d.dynamic ? 0 : -1;
            }
        }
    }
    uint32_t mine;
    const uint32_t r0 = block_exclusive_scan_n<BLOCK>(isNew ? 1u : 0u, smem, &mine);
    // publish this block's count, add up the counts of the tickets before it
    if (threadIdx.x == 0) {
        __hip_atomic_store(&words->found[ticket], kSpreadValid | mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (threadIdx.x < kWave) {
        uint32_t sum = 0;
        for (uint32_t j = threadIdx.x; j < ticket; j += kWave) {
            uint32_t v;
            do {
                v = __hip_atomic_load(&words->found[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } while ((v & kSpreadValid) == 0);
            sum += v & ~kSpreadValid;
        }
#pragma unroll
        for (int dlt = kWave / 2; dlt > 0; dlt >>= 1) {
            sum += __shfl_down(sum, dlt, kWave);
        }
        if (threadIdx.x == 0) {
            sBefore = sum;
            atomicAdd(&words->done, 1u);
        }
    }
    __syncthreads();
    const int64_t rt = (int64_t)sBefore + r0;   // the key is the rt-th key the table creates in this call
    // pass 3 first (it needs the counters as they were): mint the slot, insert, write the result in place
    if (isNew) {
        long long value;
        bool ok = true;
        if (d.dynamic) {
            const int64_t seq = d.maxOffset + rt;
            ok = seq < d.vocab;
            value = ok ? d.arenaBase + seq * d.rowBytes : 0;
        } else {
            const int64_t ev = d.evictCount;
            if (rt < ev) {
                value = d.evictPos[ev - 1 - rt];
            } else {
                value = d.maxOffset + (rt - ev);
                ok = value < d.vocab;
                if (!ok) {
                    value = -1;
                }
            }
        }
        if (newRank != nullptr) {
            newRank[i] = rt;
        }
        if (ok) {
            int st;
            unsigned long long claimed = 1;
            const bool tried = first.key == kEmptyKey && kk != kTombKey;
            if (tried) {
                claimed = atomicCAS(reinterpret_cast<unsigned long long*>(&d.entries[hash64((uint64_t)kk) & d.mask].key),
                                    (unsigned long long)kEmptyKey, (unsigned long long)kk);
            }
            if (tried && (long long)claimed == kEmptyKey) {
                d.entries[hash64((uint64_t)kk) & d.mask].slot = value;
                st = 0;
            } else if (tried && (long long)claimed == kk) {
                st = 1;  // the same key was inserted by another position of this call
            } else {
                st = map_insert(map_of(d), kk, value);
            }
            if (st != 0) {
                atomicOr(&descs[0].overflow, st == 1 ? kTableDupKey : kTableMapFull);
            }
        }
        keys[i] = value;
    }
    // pass 2, by the block with the last ticket: the table's counters advance by what the call created, and the
    // words go back to zero once every block has added up what it needed
    if (ticket + 1 == blocks && threadIdx.x == 0) {
        const int64_t cnt = (int64_t)sBefore + mine;
        TableDesc& g = descs[0];
        if (channel == RECSDK_CHANNEL_TRAIN) {
            snapMaxOut[0] = d.maxOffset;
            if (d.dynamic) {
                const int64_t room = d.vocab - d.maxOffset;
                if (cnt > room) {
                    atomicOr(&g.overflow, kTableVocabOverflow);
                }
                g.maxOffset = d.maxOffset + cnt;
                g.live = d.live + (cnt < room ? cnt : (room > 0 ? room : 0));
            } else {
                const int64_t reuse = cnt < d.evictCount ? cnt : d.evictCount;
                int64_t fresh = cnt - reuse;
                const int64_t room = d.vocab - d.maxOffset;
                g.evictCount = d.evictCount - reuse;
                g.maxOffset = d.maxOffset + fresh;
                if (fresh > room) {
                    atomicOr(&g.overflow, kTableVocabOverflow);
                    fresh = room > 0 ? room : 0;
                }
                g.live = d.live + reuse + fresh;
            }
        }
        while (__hip_atomic_load(&words->done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != blocks) {
        }
        for (uint32_t b = 0; b < blocks; ++b) {
            __hip_atomic_store(&words->found[b], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __hip_atomic_store(&words->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&words->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- evict --------------------------------------------------------------------------------------
// one key per thread (an erase is a chain of dependent trips to memory: probe, value, compare-and-swap), a tile per
// block of 1024 threads
__global__ __launch_bounds__(kAssignBlock) void k_table_erase(const TableDesc* __restrict__ descs,
                                                              const int64_t* __restrict__ keys,
                                                              const int64_t* __restrict__ off, int T,
                                                              uint8_t* __restrict__ flags, uint32_t* __restrict__ tileN,
                                                              int64_t* __restrict__ tmpSlot, int64_t nMax)
{
    __shared__ uint32_t red[kAssignBlock / kWave];
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
    const int64_t i = tile0 + (int64_t)threadIdx.x;
    uint32_t f = 0;
    if (i < n) {
        const TableDesc& d = descs[advance_segment(off, sT0, i)];
        const long long key = keys[i];
        if (key != kEmptyKey) {
            long long slot = 0;
            if (map_erase(map_of(d), key, &slot)) {
                f = 1;
                tmpSlot[i] = slot;
            }
        }
    }
    flags[i] = (uint8_t)f;  // whole tiles of flags
#pragma unroll
    for (int dlt = kWave / 2; dlt > 0; dlt >>= 1) {
        f += __shfl_down(f, dlt, kWave);
    }
    if (lane_id() == 0) {
        red[threadIdx.x >> 6] = f;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t s = 0;
        for (int k = 0; k < kAssignBlock / kWave; ++k) {
            s += red[k];
        }
        tileN[blockIdx.x] = s;
    }
}

__global__ __launch_bounds__(kBlock) void k_table_push_evicted(const TableDesc* __restrict__ descs,
                                                               const int64_t* __restrict__ off, int T,
                                                               const uint8_t* __restrict__ flags,
                                                               const uint32_t* __restrict__ tileN,
                                                               const int64_t* __restrict__ newBase,
                                                               const int64_t* __restrict__ snapEv,
                                                               const int64_t* __restrict__ tmpSlot, int64_t nMax)
{
    __shared__ uint32_t smem[kBlock / kWave + 1];
    __shared__ int sT0;
    const int64_t n = off[T];
    const int64_t tile0 = (int64_t)blockIdx.x * kTile;
    if (tile0 >= n || tile0 >= nMax) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, tile0);
    }
    const int64_t i0 = tile0 + (int64_t)threadIdx.x * kItems;
    uchar4 f4 = *reinterpret_cast<const uchar4*>(flags + i0);
    uint8_t fl[kItems] = {f4.x, f4.y, f4.z, f4.w};
    uint32_t f = fl[0] + fl[1] + fl[2] + fl[3];
    uint32_t tot;
    int64_t r = (int64_t)block_exclusive_scan(f, smem, &tot) + tileN[blockIdx.x];
    if (f == 0) {
        return;
    }
    int t = sT0;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (!fl[k]) {
            continue;
        }
        int64_t i = i0 + k;
        t = advance_segment(off, t, i);
        const TableDesc& d = descs[t];
        int64_t idx = snapEv[t] + (r - newBase[t]);
        if (idx < d.evictCap) {
            d.evictPos[idx] = tmpSlot[i];
        }
        r += 1;
    }
}

// Re-insert the live entries of `src` into the empty table `dst` (compaction after many evictions).
__global__ __launch_bounds__(kBlock) void k_table_rehash(const TableEntry* __restrict__ src, uint64_t srcCap,
                                                         TableDesc dst)
{
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (; i < srcCap; i += stride) {
        TableEntry e = src[i];
        if (e.key != kEmptyKey && e.key != kTombKey) {
            map_insert(map_of(dst), e.key, e.slot);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        dst.entries[dst.mask + 1].slot = src[srcCap].slot;
    }
}

// Export: live (key, value) pairs of one table compacted in table order (sorted by value afterwards).
__global__ __launch_bounds__(kBlock) void k_table_export(const TableDesc* __restrict__ descs, int t,
                                                         unsigned long long* __restrict__ values,
                                                         int64_t* __restrict__ keys, unsigned long long* counter,
                                                         int64_t cap)
{
    const TableDesc& d = descs[t];
    const uint64_t slots = d.mask + 2;
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (; i < slots; i += stride) {
        const TableEntry e = d.entries[i];
        const bool side = (i == d.mask + 1);
        const bool occupied = side ? (e.slot != -1) : (e.key != kEmptyKey && e.key != kTombKey);
        const unsigned long long at = wave_take(counter, occupied);
        if (occupied && (int64_t)at < cap) {
            keys[at] = side ? kTombKey : e.key;
            values[at] = (unsigned long long)e.slot;
        }
    }
}

__global__ __launch_bounds__(kBlock) void k_table_clear(TableDesc* descs, int t)
{
    TableDesc& d = descs[t];
    const uint64_t slots = d.mask + 2;
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (; i < slots; i += stride) {
        TableEntry e;
        e.key = kEmptyKey;
        e.slot = -1;
        d.entries[i] = e;
    }
}

// Load: key i of the file takes value i (static) or arenaBase + i*rowBytes (dynamic); a key that occurs more than
// once keeps the value of its last occurrence (what assigning into a map in file order leaves behind).
__global__ __launch_bounds__(kBlock) void k_table_load(TableDesc* descs, int t, const int64_t* __restrict__ keys,
                                                       int64_t n, unsigned long long* distinct)
{
    TableDesc& d = descs[t];
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    bool fresh = false;  // this thread created the key's entry
    if (i < n) {
        const long long key = keys[i];
        const long long value = d.dynamic ? d.arenaBase + i * d.rowBytes : i;
        if (key == kTombKey) {
            const long long prev = __hip_atomic_fetch_max(&d.entries[d.mask + 1].slot, value, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT);
            fresh = prev == -1;
        } else {
            uint64_t pos = hash64((uint64_t)key) & d.mask;
            for (uint64_t probes = 0; probes <= d.mask; ++probes) {
                long long cur = load_key(&d.entries[pos]);
                if (cur == kEmptyKey) {
                    const unsigned long long prev =
                        atomicCAS(reinterpret_cast<unsigned long long*>(&d.entries[pos].key),
                                  (unsigned long long)kEmptyKey, (unsigned long long)key);
                    if ((long long)prev == kEmptyKey) {
                        fresh = true;
                        cur = key;
                    } else {
                        cur = (long long)prev;
                    }
                }
                if (cur == key) {
                    // cleared slots hold -1, values are >= 0
                    __hip_atomic_fetch_max(&d.entries[pos].slot, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                pos = (pos + 1) & d.mask;
            }
        }
    }
    wave_count_add(distinct, 0, fresh);
}

__global__ void k_table_load_finish(TableDesc* descs, int t, int64_t n, const unsigned long long* distinct)
{
    TableDesc& d = descs[t];
    const int64_t u = (int64_t)*distinct;
    d.live = u;
    d.maxOffset = d.dynamic ? n : u;
    d.evictCount = 0;
    d.overflow = 0;
    d.tombs = 0;
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_tables {
    int32_t T = 0;
    int64_t maxKeys = 0;
    std::vector<TableDesc> host;      // host mirror (pointers and constants only; counters live on the device)
    std::vector<int64_t> tombBound;   // upper bound of erased slots since the last compaction
    TableDesc* descs = nullptr;       // device
    uint8_t* flags = nullptr;
    uint32_t* tileN = nullptr;
    int64_t* newBase = nullptr;
    int64_t* snapMax = nullptr;
    int64_t* snapEv = nullptr;
    int64_t* tmpSlot = nullptr;
    SpreadWords* spread = nullptr;    // zero between launches
};

static void tables_free(recsdk_tables* tg)
{
    for (auto& d : tg->host) {
        if (d.entries) {
            (void)hipFree(d.entries);
        }
        if (d.evictPos) {
            (void)hipFree(d.evictPos);
        }
    }
    void* ptrs[] = {tg->descs, tg->flags, tg->tileN, tg->newBase, tg->snapMax, tg->snapEv, tg->tmpSlot, tg->spread};
    for (void* p : ptrs) {
        if (p) {
            (void)hipFree(p);
        }
    }
}

extern "C" int recsdk_tables_create(int32_t T, const int64_t* h_dev_vocab_size, const int32_t* h_dynamic,
                                    const int64_t* h_arena_base, const int64_t* h_row_bytes, int64_t max_keys,
                                    recsdk_tables_t** out)
{
    RECSDK_REQUIRE(out != nullptr && h_dev_vocab_size != nullptr, RECSDK_ENULL, "recsdk_tables_create: NULL argument");
    RECSDK_REQUIRE(T > 0 && T <= 65536, RECSDK_EINVAL, "recsdk_tables_create: T must be in (0, 65536]");
    RECSDK_REQUIRE(max_keys > 0 && max_keys <= (int64_t(1) << 28), RECSDK_EINVAL,
                   "recsdk_tables_create: max_keys must be in (0, 2^28]");
    auto* tg = new recsdk_tables();
    tg->T = T;
    tg->maxKeys = max_keys;
    tg->host.resize(T);
    tg->tombBound.assign(T, 0);
    bool ok = true;
    for (int t = 0; t < T && ok; ++t) {
        TableDesc& d = tg->host[t];
        d = TableDesc{};
        int64_t vocab = h_dev_vocab_size[t];
        if (vocab <= 0) {
            ok = false;
            break;
        }
        uint64_t cap = 64;
        while (cap < 2 * (uint64_t)vocab) {
            cap <<= 1;
        }
        d.mask = cap - 1;
        d.vocab = vocab;
        d.dynamic = (h_dynamic != nullptr) ? h_dynamic[t] : 0;
        d.arenaBase = (h_arena_base != nullptr) ? h_arena_base[t] : 0;
        d.rowBytes = (h_row_bytes != nullptr) ? h_row_bytes[t] : 0;
        if (hipMalloc(reinterpret_cast<void**>(&d.entries), sizeof(TableEntry) * (cap + 1)) != hipSuccess) {
            d.entries = nullptr;
            ok = false;
            break;
        }
        if (hipMemset(d.entries, 0xFF, sizeof(TableEntry) * (cap + 1)) != hipSuccess) {
            ok = false;
        }
    }
    const int64_t padded = cdiv(max_keys, kTile) * kTile;
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes) != hipSuccess) {
            ok = false;
        }
    };
    alloc(&tg->descs, sizeof(TableDesc) * T);
    alloc(&tg->flags, padded);
    alloc(&tg->tileN, sizeof(uint32_t) * (padded / kTile + 1));
    alloc(&tg->newBase, sizeof(int64_t) * (T + 1));
    alloc(&tg->snapMax, sizeof(int64_t) * T);
    alloc(&tg->snapEv, sizeof(int64_t) * T);
    alloc(&tg->tmpSlot, sizeof(int64_t) * padded);
    alloc(&tg->spread, sizeof(SpreadWords));
    if (ok && hipMemset(tg->spread, 0, sizeof(SpreadWords)) != hipSuccess) {
        ok = false;
    }
    if (ok && hipMemcpy(tg->descs, tg->host.data(), sizeof(TableDesc) * T, hipMemcpyHostToDevice) != hipSuccess) {
        ok = false;
    }
    if (!ok) {
        (void)hipGetLastError();
        tables_free(tg);
        delete tg;
        set_error("recsdk_tables_create: invalid vocabulary size or hipMalloc failed");
        return RECSDK_ENOMEM;
    }
    *out = tg;
    return RECSDK_OK;
}

extern "C" int recsdk_tables_destroy(recsdk_tables_t* tg)
{
    if (tg == nullptr) {
        return RECSDK_OK;
    }
    tables_free(tg);
    delete tg;
    return RECSDK_OK;
}

extern "C" int recsdk_tables_key2offset(recsdk_tables_t* tg, int64_t* d_keys, const int64_t* d_offsets, int32_t T,
                                        int64_t n, int32_t channel, void* stream)
{
    return recsdk_tables_key2offset_ranked(tg, d_keys, d_offsets, T, n, channel, nullptr, stream);
}

const int64_t* recsdk_tables_frontier_snapshot(const recsdk_tables* tg) { return tg->snapMax; }

int recsdk_tables_key2offset_ranked(recsdk_tables* tg, int64_t* d_keys, const int64_t* d_offsets, int32_t T, int64_t n,
                                    int32_t channel, int64_t* d_new_rank, void* stream)
{
    RECSDK_REQUIRE(tg != nullptr && d_offsets != nullptr, RECSDK_ENULL, "recsdk_tables_key2offset: NULL argument");
    RECSDK_REQUIRE(T == tg->T, RECSDK_EINVAL, "recsdk_tables_key2offset: T differs from the group's table count");
    RECSDK_REQUIRE(n >= 0 && n <= tg->maxKeys, RECSDK_ECAPACITY, "recsdk_tables_key2offset: n exceeds max_keys");
    RECSDK_REQUIRE(channel == RECSDK_CHANNEL_TRAIN || channel == RECSDK_CHANNEL_EVAL, RECSDK_EINVAL,
                   "recsdk_tables_key2offset: bad channel");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_keys != nullptr, RECSDK_ENULL, "recsdk_tables_key2offset: d_keys is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (T == 1 && n > kSpreadSmallBlock && n <= small_batch_keys()) {
        // the grid covers the caller's n, an upper bound of the keys the offsets name; blocks beyond them find nothing
        RECSDK_LAUNCH_AS("k_table_spread", (k_table_spread<kSpreadSmallBlock>), dim3((unsigned)cdiv(n, kSpreadSmallBlock)),
                         dim3(kSpreadSmallBlock), s, tg->descs, d_keys, d_offsets, channel, tg->snapMax, d_new_rank,
                         tg->spread, n);
        return RECSDK_OK;
    }
    if (n <= small_batch_keys() && T <= kSmallTables) {
        RECSDK_LAUNCH(k_table_small, dim3(1), dim3(kSmallBlock), s, tg->descs, d_keys, d_offsets, T, channel, tg->snapMax,
                      d_new_rank);
        return RECSDK_OK;
    }
    const unsigned grid = (unsigned)cdiv(n, kTile);
    RECSDK_LAUNCH(k_table_probe, dim3(grid), dim3(kTile), s, tg->descs, d_keys, d_offsets, T, channel,
                       tg->flags, tg->tileN, n);
    RECSDK_LAUNCH_CHECK();
    if (channel == RECSDK_CHANNEL_TRAIN) {
        RECSDK_LAUNCH(k_table_scan, dim3(1), dim3(kBlock), s, tg->descs, tg->tileN, tg->flags, d_offsets, T,
                           tg->newBase, tg->snapMax, tg->snapEv, n, 0);
        RECSDK_LAUNCH_CHECK();
        RECSDK_LAUNCH(k_table_assign, dim3(grid), dim3(kAssignBlock), s, tg->descs, d_keys, d_offsets, T, tg->flags,
                           tg->tileN, tg->newBase, tg->snapMax, tg->snapEv, n, d_new_rank);
        RECSDK_LAUNCH_CHECK();
    }
    return RECSDK_OK;
}

// Compaction: rebuild table t without erased slots.  Synchronises `s`.
static int tables_compact(recsdk_tables* tg, int t, hipStream_t s)
{
    TableDesc& h = tg->host[t];
    const uint64_t cap = h.mask + 1;
    TableEntry* fresh = nullptr;
    RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&fresh), sizeof(TableEntry) * (cap + 1)));
    RECSDK_HIP_TRY(hipMemsetAsync(fresh, 0xFF, sizeof(TableEntry) * (cap + 1), s));
    TableDesc dst = h;
    dst.entries = fresh;
    unsigned grid = (unsigned)std::min<uint64_t>((cap + kBlock - 1) / kBlock, 256 * 16);
    RECSDK_LAUNCH(k_table_rehash, dim3(grid), dim3(kBlock), s, h.entries, cap, dst);
    RECSDK_LAUNCH_CHECK();
    // swing the device descriptor's pointer; the other counters stay as they are on the device
    RECSDK_HIP_TRY(hipMemcpyAsync(reinterpret_cast<char*>(tg->descs + t) + offsetof(TableDesc, entries), &fresh,
                                  sizeof(fresh), hipMemcpyHostToDevice, s));
    static const int64_t kNoTombs = 0;
    RECSDK_HIP_TRY(hipMemcpyAsync(reinterpret_cast<char*>(tg->descs + t) + offsetof(TableDesc, tombs), &kNoTombs,
                                  sizeof(kNoTombs), hipMemcpyHostToDevice, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    RECSDK_HIP_TRY(hipFree(h.entries));
    h.entries = fresh;
    tg->tombBound[t] = 0;
    return RECSDK_OK;
}

extern "C" int recsdk_tables_evict(recsdk_tables_t* tg, const int64_t* d_keys, const int64_t* d_offsets, int32_t T,
                                   int64_t n, void* stream)
{
    RECSDK_REQUIRE(tg != nullptr && d_offsets != nullptr, RECSDK_ENULL, "recsdk_tables_evict: NULL argument");
    RECSDK_REQUIRE(T == tg->T, RECSDK_EINVAL, "recsdk_tables_evict: T differs from the group's table count");
    RECSDK_REQUIRE(n >= 0 && n <= tg->maxKeys, RECSDK_ECAPACITY, "recsdk_tables_evict: n exceeds max_keys");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_keys != nullptr, RECSDK_ENULL, "recsdk_tables_evict: d_keys is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    // evicted-slot stacks are allocated on first use
    for (int t = 0; t < T; ++t) {
        TableDesc& h = tg->host[t];
        if (h.evictPos == nullptr) {
            RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&h.evictPos), sizeof(int64_t) * h.vocab));
            h.evictCap = h.vocab;
            RECSDK_HIP_TRY(hipMemcpyAsync(reinterpret_cast<char*>(tg->descs + t) + offsetof(TableDesc, evictPos),
                                          &h.evictPos, sizeof(h.evictPos), hipMemcpyHostToDevice, s));
            RECSDK_HIP_TRY(hipMemcpyAsync(reinterpret_cast<char*>(tg->descs + t) + offsetof(TableDesc, evictCap),
                                          &h.evictCap, sizeof(h.evictCap), hipMemcpyHostToDevice, s));
        }
    }
    const unsigned grid = (unsigned)cdiv(n, kTile);
    RECSDK_LAUNCH(k_table_erase, dim3(grid), dim3(kAssignBlock), s, tg->descs, d_keys, d_offsets, T, tg->flags,
                       tg->tileN, tg->tmpSlot, n);
    RECSDK_LAUNCH_CHECK();
    RECSDK_LAUNCH(k_table_scan, dim3(1), dim3(kBlock), s, tg->descs, tg->tileN, tg->flags, d_offsets, T,
                       tg->newBase, tg->snapMax, tg->snapEv, n, 1);
    RECSDK_LAUNCH_CHECK();
    RECSDK_LAUNCH(k_table_push_evicted, dim3(grid), dim3(kBlock), s, tg->descs, d_offsets, T, tg->flags,
                       tg->tileN, tg->newBase, tg->snapEv, tg->tmpSlot, n);
    RECSDK_LAUNCH_CHECK();
    // erased slots lengthen probe chains; compact a table once they may fill a quarter of it.  Not while the stream
    // is being recorded into a graph (the rebuild allocates and waits): insertions reuse erased slots anyway.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusNone;
    }
    for (int t = 0; t < T && capturing == hipStreamCaptureStatusNone; ++t) {
        tg->tombBound[t] += n;  // per-table split is only known on the device: conservative bound
        if ((uint64_t)tg->tombBound[t] > (tg->host[t].mask + 1) / 4) {
            int rc = tables_compact(tg, t, s);
            if (rc != RECSDK_OK) {
                return rc;
            }
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_tables_maintain(recsdk_tables_t* tg, void* stream, int32_t* h_rebuilt)
{
    RECSDK_REQUIRE(tg != nullptr, RECSDK_ENULL, "recsdk_tables_maintain: NULL handle");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusNone;
    }
    RECSDK_REQUIRE(capturing == hipStreamCaptureStatusNone, RECSDK_EINVAL,
                   "recsdk_tables_maintain: the stream is being captured (the call waits for it and may allocate)");
    std::vector<TableDesc> tmp(tg->T);
    RECSDK_HIP_TRY(hipMemcpyAsync(tmp.data(), tg->descs, sizeof(TableDesc) * tg->T, hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    int32_t rebuilt = 0;
    for (int t = 0; t < tg->T; ++t) {
        if ((uint64_t)tmp[t].tombs > (tg->host[t].mask + 1) / 4) {
            const int rc = tables_compact(tg, t, s);
            if (rc != RECSDK_OK) {
                return rc;
            }
            ++rebuilt;
        }
    }
    if (h_rebuilt != nullptr) {
        *h_rebuilt = rebuilt;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_tables_stats(recsdk_tables_t* tg, void* stream, int64_t* h_max_offset, int64_t* h_live,
                                   int64_t* h_evicted)
{
    RECSDK_REQUIRE(tg != nullptr, RECSDK_ENULL, "recsdk_tables_stats: NULL handle");
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::vector<TableDesc> tmp(tg->T);
    RECSDK_HIP_TRY(hipMemcpyAsync(tmp.data(), tg->descs, sizeof(TableDesc) * tg->T, hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    int rc = RECSDK_OK;
    for (int t = 0; t < tg->T; ++t) {
        if (h_max_offset) {
            h_max_offset[t] = tmp[t].maxOffset;
        }
        if (h_live) {
            h_live[t] = tmp[t].live;
        }
        if (h_evicted) {
            h_evicted[t] = tmp[t].evictCount;
        }
        if (tmp[t].overflow & (kTableDupKey | kTableMapFull)) {
            set_error("recsdk_tables_key2offset: table %d was given a key twice in one call (keys must be distinct per "
                      "table, e.g. the output of recsdk_unique_run) or its map ran out of slots; the table is corrupt",
                      t);
            return RECSDK_EINVAL;
        }
        if (tmp[t].overflow) {
            rc = RECSDK_EOVERFLOW;
        }
    }
    if (rc != RECSDK_OK) {
        set_error("device vocabulary overflow: a table's max_offset exceeded its device_vocabulary_size");
    }
    return rc;
}

extern "C" int recsdk_tables_evict_pos(recsdk_tables_t* tg, int32_t t, void* stream, int64_t* h_out, int64_t cap,
                                       int64_t* h_count)
{
    RECSDK_REQUIRE(tg != nullptr && h_count != nullptr, RECSDK_ENULL, "recsdk_tables_evict_pos: NULL argument");
    RECSDK_REQUIRE(t >= 0 && t < tg->T, RECSDK_EINVAL, "recsdk_tables_evict_pos: bad table index");
    hipStream_t s = static_cast<hipStream_t>(stream);
    TableDesc d;
    RECSDK_HIP_TRY(hipMemcpyAsync(&d, tg->descs + t, sizeof(TableDesc), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    *h_count = d.evictCount;
    int64_t m = std::min<int64_t>(d.evictCount, cap);
    if (m > 0 && h_out != nullptr) {
        RECSDK_HIP_TRY(hipMemcpy(h_out, d.evictPos, sizeof(int64_t) * m, hipMemcpyDeviceToHost));
    }
    return RECSDK_OK;
}

extern "C" int recsdk_tables_export(recsdk_tables_t* tg, int32_t t, int64_t* d_keys, int64_t* d_values, int64_t cap,
                                    void* stream, int64_t* h_count)
{
    RECSDK_REQUIRE(tg != nullptr && h_count != nullptr, RECSDK_ENULL, "recsdk_tables_export: NULL argument");
    RECSDK_REQUIRE(t >= 0 && t < tg->T, RECSDK_EINVAL, "recsdk_tables_export: bad table index");
    RECSDK_REQUIRE(cap >= 0 && (cap == 0 || (d_keys != nullptr && d_values != nullptr)), RECSDK_ENULL,
                   "recsdk_tables_export: NULL output buffer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    TableDesc d;
    RECSDK_HIP_TRY(hipMemcpyAsync(&d, tg->descs + t, sizeof(TableDesc), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    *h_count = d.live;
    if (cap < d.live) {
        set_error("recsdk_tables_export: table %d holds %ld keys, the buffers take %ld", t, (long)d.live, (long)cap);
        return RECSDK_ECAPACITY;
    }
    if (d.live == 0) {
        return RECSDK_OK;
    }
    const size_t m = (size_t)d.live;
    unsigned long long* counter = nullptr;
    unsigned long long* valIn = nullptr;
    int64_t* keyIn = nullptr;
    void* tmp = nullptr;
    size_t tmpBytes = 0;
    (void)rocprim::radix_sort_pairs(nullptr, tmpBytes, valIn, valIn, keyIn, keyIn, m, 0, 64, s);
    int rc = RECSDK_OK;
    auto body = [&]() -> int {
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&counter), sizeof(unsigned long long)));
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&valIn), sizeof(unsigned long long) * m));
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&keyIn), sizeof(int64_t) * m));
        RECSDK_HIP_TRY(hipMalloc(&tmp, tmpBytes ? tmpBytes : 16));
        RECSDK_HIP_TRY(hipMemsetAsync(counter, 0, sizeof(unsigned long long), s));
        const uint64_t slots = tg->host[t].mask + 2;
        const unsigned grid = (unsigned)std::min<uint64_t>((slots + kBlock - 1) / kBlock, 256 * 32);
        RECSDK_LAUNCH(k_table_export, dim3(grid), dim3(kBlock), s, tg->descs, t, valIn, keyIn, counter, (int64_t)m);
        // ascending value: slot numbers / addresses are unique per table, so the order is fully determined
        RECSDK_HIP_TRY(rocprim::radix_sort_pairs(tmp, tmpBytes, valIn, reinterpret_cast<unsigned long long*>(d_values),
                                                 keyIn, d_keys, m, 0, 64, s));
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
        return RECSDK_OK;
    };
    rc = body();
    void* ptrs[] = {counter, valIn, keyIn, tmp};
    for (void* p : ptrs) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    return rc;
}

extern "C" int recsdk_tables_load_keys(recsdk_tables_t* tg, int32_t t, const int64_t* d_keys, int64_t n, void* stream)
{
    RECSDK_REQUIRE(tg != nullptr && (n == 0 || d_keys != nullptr), RECSDK_ENULL, "recsdk_tables_load_keys: NULL argument");
    RECSDK_REQUIRE(t >= 0 && t < tg->T && n >= 0, RECSDK_EINVAL, "recsdk_tables_load_keys: bad table index or size");
    if (n > tg->host[t].vocab) {
        set_error("Load keys failed, table:%d, load key size:%ld exceeds device vocab size:%ld.", t, (long)n,
                  (long)tg->host[t].vocab);
        return RECSDK_EOVERFLOW;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned long long* distinct = nullptr;
    RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&distinct), sizeof(unsigned long long)));
    auto body = [&]() -> int {
        RECSDK_HIP_TRY(hipMemsetAsync(distinct, 0, sizeof(unsigned long long), s));
        const uint64_t slots = tg->host[t].mask + 2;
        const unsigned cgrid = (unsigned)std::min<uint64_t>((slots + kBlock - 1) / kBlock, 256 * 32);
        RECSDK_LAUNCH(k_table_clear, dim3(cgrid), dim3(kBlock), s, tg->descs, t);
        if (n > 0) {
            RECSDK_LAUNCH(k_table_load, dim3((unsigned)cdiv(n, kBlock)), dim3(kBlock), s, tg->descs, t, d_keys, n,
                          distinct);
        }
        RECSDK_LAUNCH(k_table_load_finish, dim3(1), dim3(1), s, tg->descs, t, n, distinct);
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
        return RECSDK_OK;
    };
    const int rc = body();
    (void)hipFree(distinct);
    tg->tombBound[t] = 0;
    return rc;
}
