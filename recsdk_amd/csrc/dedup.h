// Internal view of a unique handle's device results, shared by the kernels that consume them.
#ifndef RECSDK_CSRC_DEDUP_H
#define RECSDK_CSRC_DEDUP_H

#include <stdint.h>

#include <hip/hip_runtime.h>

struct recsdk_unique;

namespace recsdk {

struct UniqueView {
    // inputs of the last run (caller-owned device memory)
    const int64_t* keys = nullptr;
    const int64_t* off = nullptr;  // [T+1]
    int32_t T = 0;
    int64_t n = 0;                 // total keys (host copy)
    bool hasLists = false;         // posList/longList valid (run without input counts)
    bool countsWithLists = false;  // ucount is written by the list kernels: its readers wait for listsReady too
    bool scanReduce = false;       // a small run: no position lists, the gradient reduce scans grank instead
    hipEvent_t listsReady = nullptr;  // when set: readers of the lists below make their stream wait for it first
    hipEvent_t classesReady = nullptr;  // when set: readers of hugeIds / longIds and their counts wait for it first
    // results (handle-owned device memory)
    int64_t* uniq = nullptr;       // [U] distinct keys
    int64_t* uoff = nullptr;       // [T+1]
    int32_t* inverse = nullptr;    // [n] index inside the table's slice, -1 = skipped
    int32_t* grank = nullptr;      // [n] index into uniq (all tables), -1 = skipped
    uint32_t* ucount = nullptr;    // [U] multiplicity
    uint32_t* useg = nullptr;      // [U] start of the key's position list
    int32_t* posList = nullptr;    // [n] per distinct key: the positions (global key index) where it occurs,
                                   // ascending, at useg[R]
    int32_t* longList = nullptr;   // long id -> index into uniq, for the keys seen more than kListMax times ("long"
                                   // keys), in no particular order
    uint32_t* longSeg = nullptr;   // long id -> start of the key's ascending position list in longPos
    int32_t* longPos = nullptr;    // = posList
    int32_t* hugeIds = nullptr;    // long ids of keys seen more than kHugeMin times, longest list first
    int32_t* longIds = nullptr;    // the other long ids, ascending
    void* longMeta = nullptr;      // workspace of the gradient reduce: one 64-byte record per long id
    // workspace of the two-level sums of the keys seen more than kTwoLevelMin times (recsdk_unique_chunk_buffers)
    void* chunkMeta = nullptr;     // one 64-byte record per chunk
    float* chunkSums = nullptr;    // [chunkCap, chunkPitch] the chunk sums
    int32_t* chunkList = nullptr;  // per chunk: its row in chunkSums as a list entry of the gradient source
    int32_t* chunkIds = nullptr;   // 0, 1, 2, ...
    int64_t chunkCap = 0;
    int32_t chunkPitch = 0;        // floats per row of chunkSums
    uint32_t* nChunks = nullptr;   // device counter
    uint32_t* zero = nullptr;      // device word that stays 0
    uint32_t* nLong = nullptr;     // device counter: number of long keys
    uint32_t* nHuge = nullptr;     // device counter: length of hugeIds
    uint32_t* nLongRest = nullptr; // device counter: length of longIds
    uint32_t* nVeryHuge = nullptr; // device counter: leading entries of hugeIds seen more than kVeryHugeMin times
    int64_t* total = nullptr;      // device: U
};

}  // namespace recsdk

const recsdk::UniqueView* recsdk_unique_view(const recsdk_unique* u);

// Makes sure the handle owns the chunk workspace of the two-level sums for rows of up to `dim` floats (allocates on
// the first call and when a wider row comes; not in steady state).
int recsdk_unique_chunk_buffers(recsdk_unique* u, int32_t dim);

// Readers of view.ucount call this first: when the multiplicities are delivered by the list kernels (which run on the
// handle's own stream) it makes `s` wait for them.
inline hipError_t recsdk_unique_wait_counts(const recsdk::UniqueView* v, hipStream_t s)
{
    if (v->countsWithLists && v->listsReady != nullptr) {
        return hipStreamWaitEvent(s, v->listsReady, 0);
    }
    return hipSuccess;
}

// recsdk_unique_run with a say in the small-batch path: allow_small == false always builds the position lists (for
// callers that read them directly instead of going through apply_launch).
int recsdk_unique_run_lists(recsdk_unique* u, const int64_t* d_keys, const uint32_t* d_in_counts,
                            const int64_t* d_offsets, int32_t T, int64_t n, int32_t skip_key_enabled, int64_t skip_key,
                            bool allow_small, void* stream);

// Grouping by a stable sort for callers that need the per-key lists but not the first-occurrence order of the
// distinct keys (the pooled lookup's backward pass).  d_rows[n]: row index of each position, table t's positions are
// d_tb[t]..d_tb[t+1]; table t's rows are numbered d_row_base[t]..d_row_base[t+1] in one range of total_rows < 2^32
// rows.  Fills the view's uoff, ucount, useg, posList (per key: d_values of its positions in position order), the
// long-key lists and counters, and d_slots[R] = row of the R-th distinct key inside its table.  Rows outside their
// table are left out.  Everything runs on `s`; inverse / grank are not produced.
// d_values == NULL: the caller has written the sort's input itself, on `s`, into the buffers that
// recsdk_unique_group_input returns: key[i] = d_row_base[t] + row of position i (total_rows for a row outside its
// table), value[i] = what d_values[i] would hold.
int recsdk_unique_group_input(recsdk_unique* u, uint32_t** key, uint32_t** value);
int recsdk_unique_run_grouped(recsdk_unique* u, const int64_t* d_rows, const int64_t* d_tb, const int64_t* d_row_base,
                              int32_t T, int64_t n, int64_t total_rows, const int32_t* d_values, int64_t* d_slots,
                              hipStream_t s);

#endif
