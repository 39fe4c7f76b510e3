// Feature admission and eviction history on the device: per table an open-addressing map
//   key -> { count, lastTime }   (16-byte slots: key 8 B, count 4 B, lastTime 4 B relative to the table's first
//   timestamp), linear probing, CAS insertion, erased slots reusable.
// Every operation first merges repeated keys with the dedup kernels (summing their counts), so the history kernels
// see each key once per call and need no atomics on the record fields.
// Evicted keys are emitted in ascending (lastTime, key) order: two stable radix sorts (rocPRIM) over the compacted
// candidates.  Eviction is a rare, host-driven operation and synchronises the stream.
#include <string.h>

#include <rocprim/rocprim.hpp>

#include <algorithm>
#include <vector>

#include "common.h"
#include "dedup.h"

namespace recsdk {

constexpr uint32_t kNoCount = 0xFFFFFFFFu;            // record has no count yet
constexpr int32_t kNoTime = (int32_t)0x80000000;      // record has no timestamp yet
constexpr uint32_t kCountMax = 0xFFFFFFFEu;           // counts saturate here

struct __attribute__((aligned(16))) HistEntry {
    long long key;
    uint32_t count;
    int32_t lastTime;
};

struct HistDesc {
    HistEntry* entries;  // capacity + 1 (side slot of the key equal to kTombKey)
    int32_t* stamp;      // stamp[i] = entries[i].lastTime while slot i holds a record with a timestamp, else kNoTime:
                         // a quarter of the bytes for the eviction scan, which looks at nothing else of most slots
    uint64_t mask;
    int64_t live;
    int64_t timeBase;    // absolute timestamp of relative time 0 (set by the first timestamp seen)
    int64_t latest;      // largest timestamp seen
    int32_t hasBase;
    int32_t full;        // an insertion found no free slot
    int32_t countThreshold;
    int32_t timeThreshold;
    int32_t coef;
    int32_t enableSum;
};

__device__ __forceinline__ int64_t hist_find(const HistDesc& d, long long key)
{
    if (key == kTombKey) {
        int64_t side = (int64_t)d.mask + 1;
        return d.entries[side].key == kTombKey ? side : -1;  // side slot holds kTombKey when occupied, -1 when not
    }
    uint64_t pos = hash64((uint64_t)key) & d.mask;
    for (uint64_t probes = 0; probes <= d.mask; ++probes) {
        long long cur = __hip_atomic_load(&d.entries[pos].key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (cur == key) {
            return (int64_t)pos;
        }
        if (cur == kEmptyKey) {
            return -1;
        }
        pos = (pos + 1) & d.mask;
    }
    return -1;
}

// Find the record of `key` or create an empty one.  Keys are distinct within a call.
__device__ __forceinline__ int64_t hist_find_or_insert(HistDesc& d, long long key, bool* created)
{
    *created = false;
    int64_t pos = hist_find(d, key);
    if (pos >= 0) {
        return pos;
    }
    if (key == kTombKey) {
        int64_t side = (int64_t)d.mask + 1;
        d.entries[side].key = kTombKey;
        d.entries[side].count = kNoCount;
        d.entries[side].lastTime = kNoTime;
        d.stamp[side] = kNoTime;
        *created = true;
        return side;
    }
    uint64_t p = hash64((uint64_t)key) & d.mask;
    for (uint64_t probes = 0; probes <= d.mask; ++probes) {
        long long cur = __hip_atomic_load(&d.entries[p].key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (cur == kEmptyKey || cur == kTombKey) {
            unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&d.entries[p].key),
                                                (unsigned long long)cur, (unsigned long long)key);
            if ((long long)prev == cur) {
                d.entries[p].count = kNoCount;
                d.entries[p].lastTime = kNoTime;
                d.stamp[p] = kNoTime;
                *created = true;
                return (int64_t)p;
            }
        }
        p = (p + 1) & d.mask;
    }
    atomicOr(&d.full, 1);
    return -1;
}

__device__ __forceinline__ uint32_t sat_add(uint32_t a, uint64_t b)
{
    uint64_t s = (uint64_t)a + b;
    return s > kCountMax ? kCountMax : (uint32_t)s;
}

// per-table timestamp bookkeeping of a call, for the tables that have keys in it: latest = max(latest, ts[t]);
// the first timestamp becomes the base
__global__ void k_hist_begin(HistDesc* descs, const int64_t* __restrict__ ts, const int64_t* __restrict__ off, int T)
{
    for (int t = threadIdx.x; t < T; t += blockDim.x) {
        if (off[t + 1] <= off[t]) {
            continue;
        }
        HistDesc& d = descs[t];
        if (!d.hasBase) {
            d.timeBase = ts[t];
            d.latest = ts[t];
            d.hasBase = 1;
        } else if (ts[t] > d.latest) {
            d.latest = ts[t];
        }
    }
}

// FeatureAdmit on distinct keys (feature_admit_and_evict.cpp:46-145).  ukeys[U] are the distinct keys of the call,
// ucount[U] their merged counts; verdict[R] = 1 keeps the key.
__global__ __launch_bounds__(kBlock) void k_hist_admit(HistDesc* descs, const int64_t* __restrict__ ukeys,
                                                       const uint32_t* __restrict__ ucount,
                                                       const int64_t* __restrict__ uoff, int T,
                                                       const int64_t* __restrict__ total, int channel,
                                                       uint8_t* __restrict__ verdict, int64_t* liveDelta)
{
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R >= total[0]) {
        return;
    }
    const int t = find_segment(uoff, T, R);
    HistDesc& d = descs[t];
    const long long key = ukeys[R];
    if (key == kEmptyKey) {
        verdict[R] = 1;  // invalid keys pass through untouched
        return;
    }
    uint32_t curr = 0;
    if (channel == RECSDK_CHANNEL_EVAL || !d.enableSum) {
        int64_t pos = hist_find(d, key);
        if (pos >= 0 && d.entries[pos].count != kNoCount) {
            curr = d.entries[pos].count;
        }
    } else {
        bool created;
        int64_t pos = hist_find_or_insert(d, key, &created);
        if (pos >= 0) {
            HistEntry& e = d.entries[pos];
            // the reference multiplies in 32-bit unsigned arithmetic (uint32 count, int coefficient)
            const uint32_t add = (uint32_t)d.coef * (ucount != nullptr ? ucount[R] : 1u);
            e.count = (created || e.count == kNoCount) ? add : e.count + add;
            e.lastTime = (int32_t)(d.latest - d.timeBase);
            d.stamp[pos] = e.lastTime;
            curr = e.count;
            wave_count_add(reinterpret_cast<unsigned long long*>(liveDelta), t, created);
        }
    }
    verdict[R] = (curr >= (uint32_t)d.countThreshold) ? 1 : 0;
}

// keys[i] = -1 where the verdict of its distinct key is 0
__global__ __launch_bounds__(kBlock) void k_hist_expand(int64_t* keys, const int32_t* __restrict__ grank,
                                                        const uint8_t* __restrict__ verdict, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int32_t R = grank[i];
    if (R >= 0 && !verdict[R]) {
        keys[i] = kEmptyKey;
    }
}

// distinct keys: the verdicts apply in place
__global__ __launch_bounds__(kBlock) void k_hist_blank(int64_t* keys, const uint8_t* __restrict__ verdict,
                                                       const int64_t* __restrict__ total, HistDesc* descs,
                                                       int64_t* liveDelta, int T)
{
    // the first block also books the records the admit kernel created (one launch less in the device-side loop)
    if (blockIdx.x == 0) {
        for (int t = threadIdx.x; t < T; t += kBlock) {
            descs[t].live += liveDelta[t];
            liveDelta[t] = 0;
        }
    }
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R < total[0] && !verdict[R]) {
        keys[R] = kEmptyKey;
    }
}

// StatisticsKeyCount (feature_filter.cpp:112-138) on distinct keys with merged counts
__global__ __launch_bounds__(kBlock) void k_hist_count_add(HistDesc* descs, const int64_t* __restrict__ ukeys,
                                                           const uint32_t* __restrict__ ucount,
                                                           const int64_t* __restrict__ uoff, int T,
                                                           const int64_t* __restrict__ total, int64_t* liveDelta)
{
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R >= total[0]) {
        return;
    }
    const int t = find_segment(uoff, T, R);
    HistDesc& d = descs[t];
    bool created;
    int64_t pos = hist_find_or_insert(d, ukeys[R], &created);
    if (pos < 0) {
        return;
    }
    HistEntry& e = d.entries[pos];
    e.count = (e.count == kNoCount) ? sat_add(0, ucount[R]) : sat_add(e.count, ucount[R]);
    wave_count_add(reinterpret_cast<unsigned long long*>(liveDelta), t, created);
}

// CountFilter (feature_filter.cpp:140-160): a key with a count record below the threshold becomes -1
__global__ __launch_bounds__(kBlock) void k_hist_count_filter(const HistDesc* __restrict__ descs, int64_t* keys,
                                                              const int64_t* __restrict__ off, int T, int64_t nMax)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= off[T] || i >= nMax) {
        return;
    }
    const int t = find_segment(off, T, i);
    const HistDesc& d = descs[t];
    if (d.countThreshold < 0 || keys[i] == kEmptyKey) {
        return;  // admission disabled for this table / invalid key
    }
    int64_t pos = hist_find(d, keys[i]);
    if (pos >= 0) {
        uint32_t c = d.entries[pos].count;
        if (c != kNoCount && c < (uint32_t)d.countThreshold) {
            keys[i] = kEmptyKey;
        }
    }
}

// RecordTimestamp (feature_filter.cpp:27-50): the timestamp of a key's last occurrence wins.
// pass 1 per occurrence: best[R] = max over occurrences of (index << 32 | low word of index) -> the last index
__global__ __launch_bounds__(kBlock) void k_hist_last_occurrence(const int32_t* __restrict__ grank, int64_t n,
                                                                 unsigned long long* best)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int32_t R = grank[i];
    if (R >= 0) {
        atomicMax(&best[R], (unsigned long long)i + 1ull);
    }
}

__global__ void k_hist_ts_begin(HistDesc* descs, const int64_t* __restrict__ ts, const int64_t* __restrict__ off, int T)
{
    // base and latest from the timestamps of this call (one wave per table)
    for (int t = threadIdx.x >> 6; t < T; t += blockDim.x >> 6) {
        long long mx = (long long)0x8000000000000000ULL;
        for (int64_t i = off[t] + lane_id(); i < off[t + 1]; i += kWave) {
            mx = ts[i] > mx ? ts[i] : mx;
        }
#pragma unroll
        for (int dlt = kWave / 2; dlt > 0; dlt >>= 1) {
            long long o = __shfl_down(mx, dlt, kWave);
            mx = o > mx ? o : mx;
        }
        if (lane_id() == 0 && off[t + 1] > off[t]) {
            HistDesc& d = descs[t];
            if (!d.hasBase) {
                d.timeBase = ts[off[t]];
                d.latest = mx;
                d.hasBase = 1;
            } else if (mx > d.latest) {
                d.latest = mx;
            }
        }
    }
}

__global__ __launch_bounds__(kBlock) void k_hist_record_ts(HistDesc* descs, const int64_t* __restrict__ ukeys,
                                                           const int64_t* __restrict__ uoff, int T,
                                                           const int64_t* __restrict__ total,
                                                           const unsigned long long* __restrict__ best,
                                                           const int64_t* __restrict__ ts, int64_t* liveDelta)
{
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R >= total[0]) {
        return;
    }
    const int t = find_segment(uoff, T, R);
    HistDesc& d = descs[t];
    bool created;
    int64_t pos = hist_find_or_insert(d, ukeys[R], &created);
    if (pos < 0) {
        return;
    }
    const int64_t last = (int64_t)best[R] - 1;
    d.entries[pos].lastTime = (int32_t)(ts[last] - d.timeBase);
    d.stamp[pos] = d.entries[pos].lastTime;
    wave_count_add(reinterpret_cast<unsigned long long*>(liveDelta), t, created);
}

__global__ void k_hist_commit_live(HistDesc* descs, int64_t* liveDelta, int T)
{
    for (int t = threadIdx.x; t < T; t += blockDim.x) {
        descs[t].live += liveDelta[t];
        liveDelta[t] = 0;
    }
}

// Eviction scan of table t: erase the records idle for at least / more than the threshold and append them to
// (outKey, outTime).  strict: now - lastTime > thr (feature_filter.cpp:64), else >= (feature_admit_and_evict.cpp:179).
__global__ __launch_bounds__(kBlock) void k_hist_evict_scan(HistDesc* descs, int t, int64_t now, int64_t thr,
                                                            int strict, uint64_t* __restrict__ outKey,
                                                            uint32_t* __restrict__ outTime,
                                                            unsigned long long* counter, int64_t cap)
{
    __shared__ BlockAppend<2048> found;
    HistDesc& d = descs[t];
    HistEntry* entries = d.entries;
    int32_t* stamp = d.stamp;
    const uint64_t mask = d.mask;
    const int64_t timeBase = d.timeBase;
    const uint64_t groups = (mask + 2 + 3) / 4;  // four stamps per 16-byte load; the array is padded with kNoTime
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    found.init();
    for (uint64_t base = (uint64_t)blockIdx.x * kBlock; base < groups; base += stride) {
        const uint64_t g = base + threadIdx.x;
        int4 st = make_int4(kNoTime, kNoTime, kNoTime, kNoTime);
        if (g < groups) {
            st = reinterpret_cast<const int4*>(stamp)[g];
        }
        const int32_t sv[4] = {st.x, st.y, st.z, st.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint64_t i = g * 4 + c;
            const int64_t idle = now - (timeBase + (int64_t)sv[c]);
            const bool evict = sv[c] != kNoTime && (strict ? (idle > thr) : (idle >= thr));
            long long key = 0;
            if (evict) {
                key = entries[i].key;
                entries[i].key = (i == mask + 1) ? kEmptyKey : kTombKey;
                stamp[i] = kNoTime;
            }
            // order-preserving unsigned images of the signed key and time
            found.push(evict, (unsigned long long)key ^ 0x8000000000000000ULL, (uint32_t)sv[c] ^ 0x80000000u);
        }
        found.maybe_flush(counter, reinterpret_cast<unsigned long long*>(outKey), outTime, cap, 4);
    }
    found.flush(counter, reinterpret_cast<unsigned long long*>(outKey), outTime, cap);
}

// ---- eviction without the host in the loop -------------------------------------------------------------------
// The same scan with everything it needs read from the table itself, the evicted keys appended (in no particular
// order) straight to the caller's buffer behind the tables before it, and the count left on the device.  The counter
// these kernels share is the handle's own for this path: zero when the handle is made, and set back to zero by the
// kernel that closes a table, so no launch has to clear it first.
constexpr int kEvictBlock = 1024;
__global__ __launch_bounds__(kEvictBlock) void k_hist_evict_dev_scan(HistDesc* descs, int t, int strict,
                                                                     int64_t* __restrict__ outKeys,
                                                                     const int64_t* __restrict__ outOff, int64_t cap,
                                                                     unsigned long long* counter)
{
    __shared__ uint32_t smem[kEvictBlock / kWave];
    __shared__ unsigned long long sBase;
    HistDesc& d = descs[t];
    if (d.timeThreshold < 0 || !d.hasBase || d.live <= 0) {
        return;
    }
    HistEntry* entries = d.entries;
    int32_t* stamp = d.stamp;
    const uint64_t mask = d.mask;
    const int64_t timeBase = d.timeBase;
    const int64_t now = d.latest;
    const int64_t thr = d.timeThreshold;
    const uint64_t groups = (mask + 2 + 3) / 4;  // four stamps per 16-byte load; the array is padded with kNoTime
    const uint64_t stride = (uint64_t)gridDim.x * kEvictBlock;
    const int64_t begin = t == 0 ? 0 : outOff[t];  // outOff[0] is written when table 0 is closed
    int64_t* out = outKeys + begin;
    const int64_t room = cap - begin;
    // Only the stamps are read (4 bytes per slot, the records themselves 16): a slot's record is touched when it is
    // evicted.  Few, large blocks with several loads per thread in flight together: a history of 8 M slots is one
    // round of 512 blocks.  Per round a block counts what its threads found, takes room for all of it with one atomic
    // on the shared counter (atomics on one address are served one after the other, about 12 ns each) and every
    // thread writes its keys straight behind those of the threads before it.
    constexpr int kPer = 4;
    for (uint64_t base = (uint64_t)blockIdx.x * kEvictBlock; base < groups; base += stride * kPer) {
        int4 st[kPer];
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            const uint64_t g = base + q * stride + threadIdx.x;
            st[q] = make_int4(kNoTime, kNoTime, kNoTime, kNoTime);
            if (g < groups) {
                st[q] = reinterpret_cast<const int4*>(stamp)[g];
            }
        }
        // the records of all slots this thread evicts in this round are fetched together: one after the other, each
        // would cost a memory round trip of its own (a wave of 64 lanes x 16 slots finds several per round)
        bool hit[kPer][4];
        long long key[kPer][4];
        uint32_t mine = 0;
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            const uint64_t g = base + q * stride + threadIdx.x;
            const int32_t sv[4] = {st[q].x, st[q].y, st[q].z, st[q].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int64_t idle = now - (timeBase + (int64_t)sv[c]);
                hit[q][c] = sv[c] != kNoTime && (strict ? (idle > thr) : (idle >= thr));
                key[q][c] = 0;
                if (hit[q][c]) {
                    key[q][c] = entries[g * 4 + c].key;
                    mine += 1;
                }
            }
        }
        uint32_t total;
        uint32_t at = block_exclusive_scan_n<kEvictBlock>(mine, smem, &total);
        if (total == 0) {
            continue;  // uniform: every thread sees the same total
        }
        if (threadIdx.x == 0) {
            sBase = atomicAdd(counter, (unsigned long long)total);
        }
        __syncthreads();
        const int64_t first = (int64_t)sBase + at;
        int64_t w = first;
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            const uint64_t g = base + q * stride + threadIdx.x;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint64_t i = g * 4 + c;
                if (hit[q][c]) {
                    entries[i].key = (i == mask + 1) ? kEmptyKey : kTombKey;
                    stamp[i] = kNoTime;
                    if (w < room) {
                        out[w] = key[q][c];
                    }
                    w += 1;
                }
            }
        }
        __syncthreads();  // sBase is rewritten in the next round
    }
}

// closes table t: its keys end where the next table's begin; the table lost as many records as the scan found
__global__ void k_hist_evict_dev_end(HistDesc* descs, int t, int64_t* outOff, int64_t cap, unsigned long long* counter)
{
    const int64_t m = (int64_t)*counter;
    const int64_t begin = t == 0 ? 0 : outOff[t];
    const int64_t room = cap - begin;
    if (t == 0) {
        outOff[0] = 0;
    }
    outOff[t + 1] = begin + (m < room ? m : room);
    descs[t].live -= m;
    if (m > room) {
        descs[t].full |= 2;  // sticky: recsdk_faae_stats reports that evicted keys did not fit the caller's buffer
    }
    *counter = 0;
}

__global__ __launch_bounds__(kBlock) void k_hist_evict_finish(const uint64_t* __restrict__ sortedKey, int64_t m,
                                                              int64_t* __restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < m) {
        out[i] = (int64_t)(sortedKey[i] ^ 0x8000000000000000ULL);
    }
}

// dump of one table (tests / checkpoints): occupied records compacted in table order
__global__ __launch_bounds__(kBlock) void k_hist_dump(const HistDesc* __restrict__ descs, int t, int64_t* keys,
                                                      uint32_t* counts, int64_t* times, unsigned long long* counter,
                                                      int64_t cap)
{
    const HistDesc& d = descs[t];
    const uint64_t slots = d.mask + 2;
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (; i < slots; i += stride) {
        HistEntry e = d.entries[i];
        const bool side = (i == d.mask + 1);
        const bool occupied = side ? (e.key == kTombKey) : (e.key != kEmptyKey && e.key != kTombKey);
        const unsigned long long at = wave_take(counter, occupied);
        if (occupied && (int64_t)at < cap) {
            keys[at] = e.key;
            counts[at] = e.count;
            times[at] = (e.lastTime == kNoTime) ? (int64_t)0x8000000000000000ULL : d.timeBase + (int64_t)e.lastTime;
        }
    }
}

// ---- load of saved records (checkpoints) ------------------------------------------------------------------
// best[i] = 0 for i < n (a kernel, not a memset: the call may sit in a stream under capture)
__global__ __launch_bounds__(kBlock) void k_hist_zero_words(unsigned long long* __restrict__ p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) {
        p[i] = 0ull;
    }
}

__global__ __launch_bounds__(kBlock) void k_hist_clear(HistDesc* descs, int t)
{
    HistDesc& d = descs[t];
    const uint64_t slots = d.mask + 2;
    uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (; i < slots; i += stride) {
        HistEntry e;
        e.key = kEmptyKey;
        e.count = kNoCount;
        e.lastTime = kNoTime;
        d.entries[i] = e;
        d.stamp[i] = kNoTime;
    }
}

// one wave: reset the bookkeeping when the records are replaced; the table time becomes tableTime when given
// (INT64_MIN = not given: the largest loaded time then), the time base is set when the table has none
__global__ void k_hist_load_begin(HistDesc* descs, int t, int replace, long long tableTime,
                                  const int64_t* __restrict__ times, int64_t n)
{
    const long long none = (long long)0x8000000000000000ULL;
    long long mx = none;
    if (times != nullptr) {
        for (int64_t i = threadIdx.x; i < n; i += kWave) {
            mx = (times[i] != none && times[i] > mx) ? times[i] : mx;
        }
    }
#pragma unroll
    for (int dlt = kWave / 2; dlt > 0; dlt >>= 1) {
        const long long o = __shfl_down(mx, dlt, kWave);
        mx = o > mx ? o : mx;
    }
    if (threadIdx.x != 0) {
        return;
    }
    HistDesc& d = descs[t];
    if (replace) {
        d.live = 0;
        d.hasBase = 0;
        d.full = 0;
    }
    const long long now = tableTime != none ? tableTime : mx;
    if (now == none) {
        return;  // nothing that carries a time
    }
    if (!d.hasBase) {
        d.timeBase = now;
        d.latest = now;
        d.hasBase = 1;
    } else if (replace || now > d.latest) {
        d.latest = now;
    }
}

__global__ __launch_bounds__(kBlock) void k_hist_load(HistDesc* descs, int t, const int64_t* __restrict__ keys,
                                                      const uint32_t* __restrict__ counts,
                                                      const int64_t* __restrict__ times, int64_t n, int64_t* liveDelta)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) {
        return;
    }
    HistDesc& d = descs[t];
    bool created;
    const int64_t pos = hist_find_or_insert(d, keys[i], &created);
    if (pos < 0) {
        return;
    }
    if (counts != nullptr) {
        d.entries[pos].count = counts[i];
    }
    if (times != nullptr && times[i] != (int64_t)0x8000000000000000ULL) {
        d.entries[pos].lastTime = (int32_t)(times[i] - d.timeBase);
        d.stamp[pos] = d.entries[pos].lastTime;
    }
    wave_count_add(reinterpret_cast<unsigned long long*>(liveDelta), t, created);
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_faae {
    int32_t T = 0;
    int64_t maxKeys = 0;
    std::vector<HistDesc> host;
    HistDesc* descs = nullptr;
    recsdk_unique_t* uq = nullptr;
    uint8_t* verdict = nullptr;
    int64_t* liveDelta = nullptr;
    int64_t* tsStage = nullptr;            // [T] per-call table timestamps
    unsigned long long* best = nullptr;    // [maxKeys]
    unsigned long long* counter = nullptr;
    unsigned long long* devCounter = nullptr;  // of the device-side eviction: zero between calls
    // eviction scratch (candidates and their sort buffers), grown on demand
    uint64_t* evKeyA = nullptr;
    uint64_t* evKeyB = nullptr;
    uint32_t* evTimeA = nullptr;
    uint32_t* evTimeB = nullptr;
    void* evTmp = nullptr;
    size_t evTmpBytes = 0;
    int64_t evRoom = 0;
};

static void evict_scratch_free(recsdk_faae* f)
{
    void* ps[] = {f->evKeyA, f->evKeyB, f->evTimeA, f->evTimeB, f->evTmp};
    for (void* p : ps) {
        if (p != nullptr) {
            (void)hipFree(p);  // waits for the device: no kernel still uses the buffers
        }
    }
    f->evKeyA = f->evKeyB = nullptr;
    f->evTimeA = f->evTimeB = nullptr;
    f->evTmp = nullptr;
    f->evTmpBytes = 0;
    f->evRoom = 0;
}

// buffers for up to `room` eviction candidates
static int evict_scratch(recsdk_faae* f, int64_t room)
{
    if (room <= f->evRoom) {
        return RECSDK_OK;
    }
    evict_scratch_free(f);
    int64_t want = 1 << 16;
    while (want < room) {
        want <<= 1;
    }
    size_t bytes1 = 0;
    size_t bytes2 = 0;
    (void)rocprim::radix_sort_pairs(nullptr, bytes1, (uint64_t*)nullptr, (uint64_t*)nullptr, (uint32_t*)nullptr,
                                    (uint32_t*)nullptr, (size_t)want, 0, 64, (hipStream_t) nullptr);
    (void)rocprim::radix_sort_pairs(nullptr, bytes2, (uint32_t*)nullptr, (uint32_t*)nullptr, (uint64_t*)nullptr,
                                    (uint64_t*)nullptr, (size_t)want, 0, 32, (hipStream_t) nullptr);
    const size_t tmpBytes = std::max(bytes1, bytes2) + 256;
    if (hipMalloc(reinterpret_cast<void**>(&f->evKeyA), 8 * want) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&f->evKeyB), 8 * want) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&f->evTimeA), 4 * want) != hipSuccess ||
        hipMalloc(reinterpret_cast<void**>(&f->evTimeB), 4 * want) != hipSuccess ||
        hipMalloc(&f->evTmp, tmpBytes) != hipSuccess) {
        (void)hipGetLastError();
        evict_scratch_free(f);
        set_error("recsdk_faae_evict: hipMalloc failed");
        return RECSDK_ENOMEM;
    }
    f->evTmpBytes = tmpBytes;
    f->evRoom = want;
    return RECSDK_OK;
}

extern "C" int recsdk_faae_destroy(recsdk_faae_t* f)
{
    if (f == nullptr) {
        return RECSDK_OK;
    }
    for (auto& d : f->host) {
        if (d.entries) {
            (void)hipFree(d.entries);
        }
        if (d.stamp) {
            (void)hipFree(d.stamp);
        }
    }
    recsdk_unique_destroy(f->uq);
    evict_scratch_free(f);
    void* ptrs[] = {f->descs, f->verdict, f->liveDelta, f->tsStage, f->best, f->counter, f->devCounter};
    for (void* p : ptrs) {
        if (p) {
            (void)hipFree(p);
        }
    }
    delete f;
    return RECSDK_OK;
}

extern "C" int recsdk_faae_create(int32_t T, const int64_t* h_capacity, const int32_t* h_count_threshold,
                                  const int32_t* h_time_threshold, const int32_t* h_coef,
                                  const int32_t* h_enable_sum, int64_t max_keys, recsdk_faae_t** out)
{
    RECSDK_REQUIRE(out != nullptr && h_capacity != nullptr && h_count_threshold != nullptr, RECSDK_ENULL,
                   "recsdk_faae_create: NULL argument");
    RECSDK_REQUIRE(T > 0 && T <= 65536 && max_keys > 0, RECSDK_EINVAL, "recsdk_faae_create: bad sizes");
    auto* f = new recsdk_faae();
    f->T = T;
    f->maxKeys = max_keys;
    f->host.resize(T);
    bool ok = true;
    for (int t = 0; t < T && ok; ++t) {
        HistDesc& d = f->host[t];
        d = HistDesc{};
        if (h_capacity[t] <= 0) {
            ok = false;
            break;
        }
        uint64_t cap = 64;
        while (cap < 2 * (uint64_t)h_capacity[t]) {
            cap <<= 1;
        }
        d.mask = cap - 1;
        d.countThreshold = h_count_threshold[t];
        d.timeThreshold = h_time_threshold ? h_time_threshold[t] : -1;
        d.coef = h_coef ? h_coef[t] : 1;
        d.enableSum = h_enable_sum ? h_enable_sum[t] : 1;
        if (hipMalloc(reinterpret_cast<void**>(&d.entries), sizeof(HistEntry) * (cap + 1)) != hipSuccess) {
            d.entries = nullptr;
            ok = false;
            break;
        }
        if (hipMalloc(reinterpret_cast<void**>(&d.stamp), sizeof(int32_t) * (cap + 4)) != hipSuccess) {
            d.stamp = nullptr;
            ok = false;
            break;
        }
        // empty slots: key = -1 (all ones); count/lastTime are written when a record is created; no stamp anywhere
        ok = hipMemset(d.entries, 0xFF, sizeof(HistEntry) * (cap + 1)) == hipSuccess &&
             hipMemsetD32(reinterpret_cast<hipDeviceptr_t>(d.stamp), (int)kNoTime, cap + 4) == hipSuccess;
    }
    if (ok) {
        ok = recsdk_unique_create(max_keys, T, &f->uq) == RECSDK_OK && recsdk_unique_set_lists(f->uq, 0) == RECSDK_OK;
    }
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes) != hipSuccess) {
            ok = false;
        }
    };
    alloc(&f->descs, sizeof(HistDesc) * T);
    alloc(&f->verdict, (size_t)max_keys);
    alloc(&f->liveDelta, sizeof(int64_t) * T);
    alloc(&f->tsStage, sizeof(int64_t) * T);
    alloc(&f->best, sizeof(unsigned long long) * max_keys);
    alloc(&f->counter, sizeof(unsigned long long));
    alloc(&f->devCounter, sizeof(unsigned long long));
    if (ok) {
        ok = hipMemcpy(f->descs, f->host.data(), sizeof(HistDesc) * T, hipMemcpyHostToDevice) == hipSuccess &&
             hipMemset(f->liveDelta, 0, sizeof(int64_t) * T) == hipSuccess &&
             hipMemset(f->devCounter, 0, sizeof(unsigned long long)) == hipSuccess;
    }
    if (!ok) {
        (void)hipGetLastError();
        recsdk_faae_destroy(f);
        set_error("recsdk_faae_create: invalid capacity or allocation failed");
        return RECSDK_ENOMEM;
    }
    *out = f;
    return RECSDK_OK;
}

static int faae_check(recsdk_faae_t* f, const void* d_keys, const int64_t* d_offsets, int32_t T, int64_t n,
                      const char* who)
{
    if (f == nullptr || d_offsets == nullptr || (n > 0 && d_keys == nullptr)) {
        set_error("%s: NULL argument", who);
        return RECSDK_ENULL;
    }
    if (T != f->T) {
        set_error("%s: T differs from the handle's table count", who);
        return RECSDK_EINVAL;
    }
    if (n < 0 || n > f->maxKeys) {
        set_error("%s: n exceeds max_keys", who);
        return RECSDK_ECAPACITY;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_faae_admit(recsdk_faae_t* f, int32_t channel, int64_t* d_keys, const uint32_t* d_counts,
                                 const int64_t* d_offsets, int32_t T, int64_t n, const int64_t* h_timestamps,
                                 void* stream)
{
    int rc = faae_check(f, d_keys, d_offsets, T, n, "recsdk_faae_admit");
    if (rc != RECSDK_OK) {
        return rc;
    }
    RECSDK_REQUIRE(h_timestamps != nullptr, RECSDK_ENULL, "recsdk_faae_admit: h_timestamps is NULL");
    RECSDK_REQUIRE(channel == RECSDK_CHANNEL_TRAIN || channel == RECSDK_CHANNEL_EVAL, RECSDK_EINVAL,
                   "recsdk_faae_admit: bad channel");
    hipStream_t s = static_cast<hipStream_t>(stream);
    RECSDK_HIP_TRY(hipMemcpyAsync(f->tsStage, h_timestamps, sizeof(int64_t) * T, hipMemcpyHostToDevice, s));
    RECSDK_LAUNCH(k_hist_begin, dim3(1), dim3(kBlock), s, f->descs, f->tsStage, d_offsets, T);
    if (n == 0) {
        return RECSDK_OK;
    }
    // merge repeated keys and their counts (PreProcessKeys, feature_admit_and_evict.cpp:218-233); -1 is skipped
    rc = recsdk_unique_run(f->uq, d_keys, d_counts, d_offsets, T, n, 1, -1, stream);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const UniqueView* v = recsdk_unique_view(f->uq);
    const unsigned grid = (unsigned)cdiv(n, kBlock);
    RECSDK_LAUNCH(k_hist_admit, dim3(grid), dim3(kBlock), s, f->descs, v->uniq, v->ucount, v->uoff, T, v->total, channel,
                  f->verdict, f->liveDelta);
    RECSDK_LAUNCH(k_hist_commit_live, dim3(1), dim3(kBlock), s, f->descs, f->liveDelta, T);
    RECSDK_LAUNCH(k_hist_expand, dim3(grid), dim3(kBlock), s, d_keys, v->grank, f->verdict, n);
    return RECSDK_OK;
}

// timestamps on the host (copied to the device first) or already on the device
static int faae_admit_distinct(recsdk_faae_t* f, int32_t channel, int64_t* d_keys, const uint32_t* d_counts,
                               const int64_t* d_offsets, int32_t T, int64_t n, const int64_t* h_timestamps,
                               const int64_t* d_timestamps, void* stream)
{
    int rc = faae_check(f, d_keys, d_offsets, T, n, "recsdk_faae_admit_distinct");
    if (rc != RECSDK_OK) {
        return rc;
    }
    RECSDK_REQUIRE(h_timestamps != nullptr || d_timestamps != nullptr, RECSDK_ENULL,
                   "recsdk_faae_admit_distinct: the timestamps are NULL");
    RECSDK_REQUIRE(channel == RECSDK_CHANNEL_TRAIN || channel == RECSDK_CHANNEL_EVAL, RECSDK_EINVAL,
                   "recsdk_faae_admit_distinct: bad channel");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (d_timestamps == nullptr) {
        RECSDK_HIP_TRY(hipMemcpyAsync(f->tsStage, h_timestamps, sizeof(int64_t) * T, hipMemcpyHostToDevice, s));
        d_timestamps = f->tsStage;
    }
    RECSDK_LAUNCH(k_hist_begin, dim3(1), dim3(kBlock), s, f->descs, d_timestamps, d_offsets, T);
    if (n == 0) {
        return RECSDK_OK;
    }
    // the keys are what a unique run delivered: no merge needed, the table offsets are their segment offsets
    const unsigned grid = (unsigned)cdiv(n, kBlock);
    RECSDK_LAUNCH(k_hist_admit, dim3(grid), dim3(kBlock), s, f->descs, d_keys, d_counts, d_offsets, T, d_offsets + T,
                  channel, f->verdict, f->liveDelta);
    RECSDK_LAUNCH(k_hist_blank, dim3(grid), dim3(kBlock), s, d_keys, f->verdict, d_offsets + T, f->descs, f->liveDelta,
                  T);
    return RECSDK_OK;
}

extern "C" int recsdk_faae_admit_distinct(recsdk_faae_t* f, int32_t channel, int64_t* d_keys, const uint32_t* d_counts,
                                          const int64_t* d_offsets, int32_t T, int64_t n, const int64_t* h_timestamps,
                                          void* stream)
{
    RECSDK_REQUIRE(h_timestamps != nullptr, RECSDK_ENULL, "recsdk_faae_admit_distinct: h_timestamps is NULL");
    return faae_admit_distinct(f, channel, d_keys, d_counts, d_offsets, T, n, h_timestamps, nullptr, stream);
}

extern "C" int recsdk_faae_admit_distinct_dev(recsdk_faae_t* f, int32_t channel, int64_t* d_keys,
                                              const uint32_t* d_counts, const int64_t* d_offsets, int32_t T, int64_t n,
                                              const int64_t* d_timestamps, void* stream)
{
    RECSDK_REQUIRE(d_timestamps != nullptr, RECSDK_ENULL, "recsdk_faae_admit_distinct_dev: d_timestamps is NULL");
    return faae_admit_distinct(f, channel, d_keys, d_counts, d_offsets, T, n, nullptr, d_timestamps, stream);
}

extern "C" int recsdk_faae_evict_dev(recsdk_faae_t* f, int32_t strict, int64_t* d_out_keys, int64_t cap,
                                     int64_t* d_out_offsets, void* stream)
{
    RECSDK_REQUIRE(f != nullptr && d_out_offsets != nullptr, RECSDK_ENULL, "recsdk_faae_evict_dev: NULL argument");
    RECSDK_REQUIRE(cap >= 0 && (cap == 0 || d_out_keys != nullptr), RECSDK_EINVAL,
                   "recsdk_faae_evict_dev: bad output buffer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (int t = 0; t < f->T; ++t) {
        const unsigned grid = (unsigned)std::min<uint64_t>(((f->host[t].mask + 5) / 4 + kEvictBlock - 1) / kEvictBlock, 256 * 2);
        RECSDK_LAUNCH(k_hist_evict_dev_scan, dim3(grid), dim3(kEvictBlock), s, f->descs, t, strict, d_out_keys, d_out_offsets,
                      cap, f->devCounter);
        RECSDK_LAUNCH(k_hist_evict_dev_end, dim3(1), dim3(1), s, f->descs, t, d_out_offsets, cap, f->devCounter);
    }
    return RECSDK_OK;
}

extern "C" int recsdk_faae_count_add(recsdk_faae_t* f, const int64_t* d_keys, const uint32_t* d_counts,
                                     const int64_t* d_offsets, int32_t T, int64_t n, void* stream)
{
    int rc = faae_check(f, d_keys, d_offsets, T, n, "recsdk_faae_count_add");
    if (rc != RECSDK_OK || n == 0) {
        return rc;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    rc = recsdk_unique_run(f->uq, d_keys, d_counts, d_offsets, T, n, 1, -1, stream);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const UniqueView* v = recsdk_unique_view(f->uq);
    const unsigned grid = (unsigned)cdiv(n, kBlock);
    RECSDK_LAUNCH(k_hist_count_add, dim3(grid), dim3(kBlock), s, f->descs, v->uniq, v->ucount, v->uoff, T, v->total,
                  f->liveDelta);
    RECSDK_LAUNCH(k_hist_commit_live, dim3(1), dim3(kBlock), s, f->descs, f->liveDelta, T);
    return RECSDK_OK;
}

extern "C" int recsdk_faae_count_filter(recsdk_faae_t* f, int64_t* d_keys, const int64_t* d_offsets, int32_t T,
                                        int64_t n, void* stream)
{
    int rc = faae_check(f, d_keys, d_offsets, T, n, "recsdk_faae_count_filter");
    if (rc != RECSDK_OK || n == 0) {
        return rc;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned grid = (unsigned)cdiv(n, kBlock);
    RECSDK_LAUNCH(k_hist_count_filter, dim3(grid), dim3(kBlock), s, f->descs, d_keys, d_offsets, T, n);
    return RECSDK_OK;
}

extern "C" int recsdk_faae_record_timestamp(recsdk_faae_t* f, const int64_t* d_keys, const int64_t* d_timestamps,
                                            const int64_t* d_offsets, int32_t T, int64_t n, void* stream)
{
    int rc = faae_check(f, d_keys, d_offsets, T, n, "recsdk_faae_record_timestamp");
    if (rc != RECSDK_OK || n == 0) {
        return rc;
    }
    RECSDK_REQUIRE(d_timestamps != nullptr, RECSDK_ENULL, "recsdk_faae_record_timestamp: d_timestamps is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    RECSDK_LAUNCH(k_hist_ts_begin, dim3(1), dim3(kBlock), s, f->descs, d_timestamps, d_offsets, T);
    rc = recsdk_unique_run(f->uq, d_keys, nullptr, d_offsets, T, n, 1, -1, stream);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const UniqueView* v = recsdk_unique_view(f->uq);
    const unsigned grid = (unsigned)cdiv(n, kBlock);
    RECSDK_LAUNCH(k_hist_zero_words, dim3(grid), dim3(kBlock), s, f->best, n);
    RECSDK_LAUNCH(k_hist_last_occurrence, dim3(grid), dim3(kBlock), s, v->grank, n, f->best);
    RECSDK_LAUNCH(k_hist_record_ts, dim3(grid), dim3(kBlock), s, f->descs, v->uniq, v->uoff, T, v->total, f->best,
                  d_timestamps, f->liveDelta);
    RECSDK_LAUNCH(k_hist_commit_live, dim3(1), dim3(kBlock), s, f->descs, f->liveDelta, T);
    return RECSDK_OK;
}

extern "C" int recsdk_faae_stats(recsdk_faae_t* f, void* stream, int64_t* h_live, int64_t* h_latest)
{
    RECSDK_REQUIRE(f != nullptr, RECSDK_ENULL, "recsdk_faae_stats: NULL handle");
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::vector<HistDesc> tmp(f->T);
    RECSDK_HIP_TRY(hipMemcpyAsync(tmp.data(), f->descs, sizeof(HistDesc) * f->T, hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    int rc = RECSDK_OK;
    for (int t = 0; t < f->T; ++t) {
        if (h_live) {
            h_live[t] = tmp[t].live;
        }
        if (h_latest) {
            h_latest[t] = tmp[t].latest;
        }
        if (tmp[t].full & 2) {
            set_error("recsdk_faae_evict_dev: evicted keys of table %d did not fit the output buffer (their records "
                      "were erased)", t);
            return RECSDK_ECAPACITY;
        }
        if (tmp[t].full) {
            rc = RECSDK_EOVERFLOW;
        }
    }
    if (rc != RECSDK_OK) {
        set_error("feature history is full: create the handle with a larger capacity");
    }
    return rc;
}

extern "C" int recsdk_faae_evict(recsdk_faae_t* f, int32_t strict, int64_t* d_out_keys, int64_t cap,
                                 int64_t* h_out_offsets, void* stream)
{
    RECSDK_REQUIRE(f != nullptr && h_out_offsets != nullptr, RECSDK_ENULL, "recsdk_faae_evict: NULL argument");
    RECSDK_REQUIRE(cap >= 0 && (cap == 0 || d_out_keys != nullptr), RECSDK_EINVAL, "recsdk_faae_evict: bad output buffer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::vector<HistDesc> cur(f->T);
    RECSDK_HIP_TRY(hipMemcpyAsync(cur.data(), f->descs, sizeof(HistDesc) * f->T, hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    int64_t written = 0;
    h_out_offsets[0] = 0;
    int rc = RECSDK_OK;
    for (int t = 0; t < f->T; ++t) {
        const HistDesc& d = cur[t];
        int64_t evicted = 0;
        if (d.timeThreshold >= 0 && d.hasBase && d.live > 0) {
            const int64_t room = d.live;  // at most every live record
            const int src = evict_scratch(f, room);
            if (src != RECSDK_OK) {
                return src;
            }
            uint64_t* kA = f->evKeyA;
            uint64_t* kB = f->evKeyB;
            uint32_t* tA = f->evTimeA;
            uint32_t* tB = f->evTimeB;
            RECSDK_HIP_TRY(hipMemsetAsync(f->counter, 0, sizeof(unsigned long long), s));
            const unsigned grid = (unsigned)std::min<uint64_t>(((d.mask + 5) / 4 + kBlock - 1) / kBlock, 256 * 8);
            RECSDK_LAUNCH(k_hist_evict_scan, dim3(grid), dim3(kBlock), s, f->descs, t, d.latest, (int64_t)d.timeThreshold,
                          strict, kA, tA, f->counter, room);
            unsigned long long m = 0;
            RECSDK_HIP_TRY(hipMemcpyAsync(&m, f->counter, sizeof(m), hipMemcpyDeviceToHost, s));
            RECSDK_HIP_TRY(hipStreamSynchronize(s));
            evicted = (int64_t)m;
            if (evicted > 0) {
                // ascending (lastTime, key): stable sort by key, then stable sort by time
                size_t bytes1 = f->evTmpBytes;
                size_t bytes2 = f->evTmpBytes;
                RECSDK_HIP_TRY(rocprim::radix_sort_pairs(f->evTmp, bytes1, kA, kB, tA, tB, (size_t)evicted, 0, 64, s));
                RECSDK_HIP_TRY(rocprim::radix_sort_pairs(f->evTmp, bytes2, tB, tA, kB, kA, (size_t)evicted, 0, 32, s));
                const int64_t fit = std::min<int64_t>(evicted, cap - written);
                if (fit > 0) {
                    const unsigned g2 = (unsigned)cdiv(fit, kBlock);
                    RECSDK_LAUNCH(k_hist_evict_finish, dim3(g2), dim3(kBlock), s, kA, fit, d_out_keys + written);
                }
                if (fit < evicted) {
                    rc = RECSDK_ECAPACITY;
                }
                written += std::max<int64_t>(fit, 0);
                // the table lost `evicted` records
                const int64_t live = d.live - evicted;
                RECSDK_HIP_TRY(hipMemcpyAsync(reinterpret_cast<char*>(f->descs + t) + offsetof(HistDesc, live), &live,
                                              sizeof(live), hipMemcpyHostToDevice, s));
            }
            RECSDK_HIP_TRY(hipStreamSynchronize(s));  // `live` above is copied from this stack frame
        }
        h_out_offsets[t + 1] = written;
    }
    if (rc != RECSDK_OK) {
        set_error("recsdk_faae_evict: output buffer too small for the evicted keys (records were erased)");
    }
    return rc;
}

extern "C" int recsdk_faae_dump(recsdk_faae_t* f, int32_t t, int64_t* d_keys, uint32_t* d_counts, int64_t* d_times,
                                int64_t cap, int64_t* h_count, void* stream)
{
    RECSDK_REQUIRE(f != nullptr && h_count != nullptr, RECSDK_ENULL, "recsdk_faae_dump: NULL argument");
    RECSDK_REQUIRE(t >= 0 && t < f->T, RECSDK_EINVAL, "recsdk_faae_dump: bad table index");
    hipStream_t s = static_cast<hipStream_t>(stream);
    RECSDK_HIP_TRY(hipMemsetAsync(f->counter, 0, sizeof(unsigned long long), s));
    const uint64_t slots = f->host[t].mask + 2;
    const unsigned grid = (unsigned)std::min<uint64_t>((slots + kBlock - 1) / kBlock, 256 * 32);
    RECSDK_LAUNCH(k_hist_dump, dim3(grid), dim3(kBlock), s, f->descs, t, d_keys, d_counts, d_times, f->counter, cap);
    unsigned long long m = 0;
    RECSDK_HIP_TRY(hipMemcpyAsync(&m, f->counter, sizeof(m), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    *h_count = (int64_t)m;
    return RECSDK_OK;
}

extern "C" int recsdk_faae_load(recsdk_faae_t* f, int32_t t, const int64_t* d_keys, const uint32_t* d_counts,
                                const int64_t* d_times, int64_t n, int32_t replace, int64_t table_time, void* stream)
{
    RECSDK_REQUIRE(f != nullptr && (n == 0 || d_keys != nullptr), RECSDK_ENULL, "recsdk_faae_load: NULL argument");
    RECSDK_REQUIRE(t >= 0 && t < f->T && n >= 0, RECSDK_EINVAL, "recsdk_faae_load: bad table index or size");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (replace) {
        const uint64_t slots = f->host[t].mask + 2;
        const unsigned grid = (unsigned)std::min<uint64_t>((slots + kBlock - 1) / kBlock, 256 * 32);
        RECSDK_LAUNCH(k_hist_clear, dim3(grid), dim3(kBlock), s, f->descs, t);
    }
    RECSDK_LAUNCH(k_hist_load_begin, dim3(1), dim3(kWave), s, f->descs, t, replace, (long long)table_time, d_times, n);
    if (n > 0) {
        RECSDK_LAUNCH(k_hist_load, dim3((unsigned)cdiv(n, kBlock)), dim3(kBlock), s, f->descs, t, d_keys, d_counts,
                      d_times, n, f->liveDelta);
    }
    RECSDK_LAUNCH(k_hist_commit_live, dim3(1), dim3(kBlock), s, f->descs, f->liveDelta, f->T);
    return RECSDK_OK;
}
