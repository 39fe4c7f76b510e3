// 64-bit key -> 64-bit value open-addressing map on the device: 16-byte {key, value} slots, linear probing,
// CAS insertion, erased slots (tombstones) reusable.  Key -1 marks an empty slot and is never stored; the key
// whose value equals the tombstone marker lives in a side slot at index capacity.
#ifndef RECSDK_CSRC_HASHMAP_H
#define RECSDK_CSRC_HASHMAP_H

#include "common.h"

namespace recsdk {

struct __attribute__((aligned(16))) TableEntry {
    long long key;
    long long slot;
};

struct MapRef {
    TableEntry* entries;  // capacity + 1 entries
    uint64_t mask;        // capacity - 1
};

#ifdef __HIPCC__

__device__ __forceinline__ long long load_key(const TableEntry* e)
{
    return __hip_atomic_load(&e->key, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Returns the entry index of `key`, or -1.
__device__ __forceinline__ int64_t map_find(const MapRef& d, long long key)
{
    if (key == kTombKey) {
        int64_t side = (int64_t)d.mask + 1;
        return d.entries[side].slot != -1 ? side : -1;
    }
    uint64_t pos = hash64((uint64_t)key) & d.mask;
    for (uint64_t probes = 0; probes <= d.mask; ++probes) {
        long long cur = load_key(&d.entries[pos]);
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

// Insert a key expected to be absent (distinct keys may be inserted concurrently).  Returns 0 when the key was
// inserted, 1 when the probe met the key already in the map (a duplicate in the caller's list: nothing is written),
// 2 when the probe found no free slot.
__device__ __forceinline__ int map_insert(const MapRef& d, long long key, long long value)
{
    if (key == kTombKey) {
        const unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&d.entries[d.mask + 1].slot),
                                                  (unsigned long long)-1LL, (unsigned long long)value);
        return (long long)prev == -1 ? 0 : 1;
    }
    uint64_t pos = hash64((uint64_t)key) & d.mask;
    for (uint64_t probes = 0; probes <= d.mask; ++probes) {
        long long cur = load_key(&d.entries[pos]);
        if (cur == key) {
            return 1;
        }
        if (cur == kEmptyKey || cur == kTombKey) {
            unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&d.entries[pos].key),
                                                (unsigned long long)cur, (unsigned long long)key);
            if ((long long)prev == cur) {
                d.entries[pos].slot = value;
                return 0;
            }
            if ((long long)prev == key) {
                return 1;
            }
        }
        pos = (pos + 1) & d.mask;
    }
    return 2;
}

// Erase `key`; returns true for the one caller that removed it and stores its value in *value.
__device__ __forceinline__ bool map_erase(const MapRef& d, long long key, long long* value)
{
    int64_t pos = map_find(d, key);
    if (pos < 0) {
        return false;
    }
    if (key == kTombKey) {
        // the side slot has no key word to claim: the caller that swaps the value out is the one that erased it
        const unsigned long long prev =
            atomicExch(reinterpret_cast<unsigned long long*>(&d.entries[pos].slot), (unsigned long long)-1LL);
        *value = (long long)prev;
        return (long long)prev != -1;
    }
    *value = d.entries[pos].slot;
    unsigned long long prev = atomicCAS(reinterpret_cast<unsigned long long*>(&d.entries[pos].key),
                                        (unsigned long long)key, (unsigned long long)kTombKey);
    return (long long)prev == key;
}

#endif  // __HIPCC__

}  // namespace recsdk

#endif
