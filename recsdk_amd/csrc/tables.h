// Internal additions to the key -> slot tables for other parts of the library.
#ifndef RECSDK_CSRC_TABLES_H
#define RECSDK_CSRC_TABLES_H

#include "common.h"

struct recsdk_tables;

// recsdk_tables_key2offset that also reports which keys it created: d_new_rank[i] = r when key i is the r-th key its
// table created in this call (array order), untouched otherwise (the caller pre-fills it, e.g. with -1).
int recsdk_tables_key2offset_ranked(recsdk_tables* tg, int64_t* d_keys, const int64_t* d_offsets, int32_t T, int64_t n,
                                    int32_t channel, int64_t* d_new_rank, void* stream);

#endif
