// Internal additions to the key -> slot tables for other parts of the library.
#ifndef RECSDK_CSRC_TABLES_H
#define RECSDK_CSRC_TABLES_H

#include "common.h"

struct recsdk_tables;

// recsdk_tables_key2offset that also reports which keys it created: d_new_rank[i] = r when key i is the r-th key its
// table created in this call (array order), untouched otherwise (the caller pre-fills it, e.g. with -1).
int recsdk_tables_key2offset_ranked(recsdk_tables* tg, int64_t* d_keys, const int64_t* d_offsets, int32_t T, int64_t n,
                                    int32_t channel, int64_t* d_new_rank, void* stream);

// Device array, one entry per table: the first row of table t that had never been handed out when the latest
// recsdk_tables_key2offset(_ranked) / recsdk_tables_evict call on the group began.  Valid for kernels queued on that
// call's stream before the next such call.
const int64_t* recsdk_tables_frontier_snapshot(const recsdk_tables* tg);

#endif
