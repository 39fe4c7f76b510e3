// Internal view of a unique handle's device results, shared by the kernels that consume them.
#ifndef RECSDK_CSRC_DEDUP_H
#define RECSDK_CSRC_DEDUP_H

#include <stdint.h>

struct recsdk_unique;

namespace recsdk {

struct UniqueView {
    // inputs of the last run (caller-owned device memory)
    const int64_t* keys = nullptr;
    const int64_t* off = nullptr;  // [T+1]
    int32_t T = 0;
    int64_t n = 0;                 // total keys (host copy)
    bool hasLists = false;         // posList/longList valid (run without input counts)
    // results (handle-owned device memory)
    int64_t* uniq = nullptr;       // [U] distinct keys
    int64_t* uoff = nullptr;       // [T+1]
    int32_t* inverse = nullptr;    // [n] index inside the table's slice, -1 = skipped
    int32_t* grank = nullptr;      // [n] index into uniq (all tables), -1 = skipped
    uint32_t* ucount = nullptr;    // [U] multiplicity
    uint32_t* useg = nullptr;      // [U] start of the key's position list
    int32_t* posList = nullptr;    // [n] per distinct key: the positions (global key index) where it occurs, ascending
    int32_t* longList = nullptr;   // distinct keys seen more than kListMax times (index into uniq), unordered
    int32_t* midList = nullptr;    // distinct keys seen 2..kListMax times (index into uniq), unordered
    uint32_t* nLong = nullptr;     // device counter: length of longList
    int64_t* total = nullptr;      // device: U
};

}  // namespace recsdk

const recsdk::UniqueView* recsdk_unique_view(const recsdk_unique* u);

#endif
