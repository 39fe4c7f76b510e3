/*
 * recsdk_hip.h - C ABI of the MI355X (gfx950) sparse-embedding hot path.
 *
 * The library behind this header (librecsdk_hip.so) implements, as hand-written HIP kernels, the
 * data-parallel path   key dedup -> admission -> key->slot hash table -> row gather / pooled lookup ->
 * gradient segment-reduce -> sparse optimizer update,   and nothing else.
 *
 * Conventions
 *   - plain pointers and sizes only; `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - pointers named d_* are device pointers, h_* host pointers;
 *   - every function returns 0 (RECSDK_OK) or a negative RECSDK_E* code, never throws, and never
 *     synchronises the stream unless its comment says "synchronous";
 *   - all kernels of one call are enqueued on `stream`; calls on one handle must be stream-ordered;
 *   - key value -1 is the reference's INVALID_KEY_VALUE (training/tf_rec_v1/src/core/utils/common.h:82).
 *
 * Each entry point cites the reference interface it replaces (paths relative to the reference checkout).
 */
#ifndef RECSDK_HIP_H
#define RECSDK_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RECSDK_API __attribute__((visibility("default")))

/* error codes (0 = ok).  Positive CTRCode values of the reference
 * (training/tf_rec_v1/src/AccCTR/src/common/util/error_code.h:20-47) are reported negated where they apply. */
#define RECSDK_OK 0
#define RECSDK_EINVAL (-1)        /* H_ERROR: bad argument                                  */
#define RECSDK_ENULL (-3)         /* H_ADDRESS_NULL                                         */
#define RECSDK_ENOMEM (-10)       /* H_MEMORY_ALLOC_ERROR: hipMalloc failed                  */
#define RECSDK_EOVERFLOW (-16)    /* H_MAX_CACHESIZE_TOO_SMALL / device vocabulary overflow */
#define RECSDK_EHIP (-100)        /* a HIP runtime call failed                              */
#define RECSDK_ENOTFOUND (-101)   /* key must exist (DP lookup) but does not                */
#define RECSDK_EIO (-103)         /* a checkpoint file could not be created, read or written */
#define RECSDK_ECAPACITY (-102)   /* call larger than the handle was created for            */

/* element types of the by-address ops (cust_op/.../cust_op_by_addr/v220/emb_custom.json:22-25) */
#define RECSDK_DT_F32 0
#define RECSDK_DT_F16 1
#define RECSDK_DT_I32 2
#define RECSDK_DT_BF16 3
#define RECSDK_DT_I64 4

/* optimizers */
#define RECSDK_OPT_SGD 0
#define RECSDK_OPT_ADAGRAD 1
#define RECSDK_OPT_ADAM 2

/* pooling modes of the split-embedding ops */
#define RECSDK_POOL_SUM 0
#define RECSDK_POOL_MEAN 1
#define RECSDK_POOL_NONE 2

/* channels (training/tf_rec_v1/src/core/utils/common.h:49-50) */
#define RECSDK_CHANNEL_TRAIN 0
#define RECSDK_CHANNEL_EVAL 1

/* library / device info.  Returns the version (>0). */
RECSDK_API int recsdk_version(void);
/* Last error text of the calling thread (static storage, never NULL). */
RECSDK_API const char* recsdk_last_error(void);

/* Batches of at most max_keys keys (and at most 64 tables) take one-launch paths in recsdk_unique_run,
 * recsdk_tables_key2offset, recsdk_gather_unique and recsdk_sparse_apply: one block dedups in LDS, one block resolves
 * the slots, and the gradient reduce scans the inverse index instead of reading position lists.  Such a batch is
 * bound by the launches it takes (the reference's smallest configuration has 4096 keys per step), and the results are
 * those of the general path bit for bit.  Default and maximum: 4096; 0 sends every batch down the general path.
 * Process-wide; set it while no call is in flight.  No counterpart in the reference. */
RECSDK_API int recsdk_set_small_batch_keys(int64_t max_keys);
/* Optional per-kernel timing (off by default).  Between start() and stop() every kernel whose name begins
 * with kernel_prefix (NULL or "" = all kernels) is bracketed by a HIP event pair on its launch stream.
 * stop() returns the number of distinct kernel names seen; get() synchronises the events of name `index` and
 * returns its launch count and summed duration.  At most 65536 launches are recorded per session. */
RECSDK_API int recsdk_profile_start(const char* kernel_prefix);
RECSDK_API int recsdk_profile_stop(void);
RECSDK_API int recsdk_profile_get(int32_t index, char* name, int32_t name_cap, int64_t* launches, double* total_ms);
/* Calibration: a plain device-to-device streaming copy of `bytes` (a multiple of 16, buffers 16-byte aligned) with the
 * fastest plain shape found on MI355X (16 bytes per lane, two requests in flight per lane, past the caches).  Timing
 * it gives the rate the memory system sustains on the device at hand, to set beside the row kernels' rates.  No counterpart in the
 * reference. */
RECSDK_API int recsdk_calib_copy(void* d_dst, const void* d_src, int64_t bytes, void* stream);
/* What a captured HIP graph holds: the type of every node of `hip_graph` (a hipGraph_t; values of hipGraphNodeType:
 * 0 kernel, 1 memcpy, 2 memset, 3 host, 4 child graph, 5 empty, 6 wait event, 7 event record, ...) into h_kinds[0..cap)
 * and the number of nodes into *h_count.  For callers that capture this library's steps and want to hold only kernel
 * nodes (and the event nodes of the library's side streams), as the tests do.  No counterpart in the reference. */
RECSDK_API int recsdk_graph_node_kinds(void* hip_graph, int32_t* h_kinds, int64_t cap, int64_t* h_count);

/* ------------------------------------------------------------------------------------------------
 * Stable radix sort of (key, 32-bit value) pairs: the sorter behind the position lists of the gradient reduce
 * (recsdk_unique_run), the row grouping of the split-embedding backward (recsdk_tbe_backward) and the shard
 * regrouping (recsdk_unique_sharded).  Where the reference sorts at all it calls a library routine
 *   (torch.unique in hybrid_torchrec/.../unique.cpp:55-118, std::sort of evicted records in
 *   training/tf_rec_v1/src/core/key_process/feature_admit_and_evict.cpp:148-200);
 * this one is written for gfx950: one counting kernel over all digits, then one kernel per digit of 8, 9 or 10 bits
 * (decoupled look-back between tiles, wave-wide ballots for the ranks inside a tile), kernels only: a stream under
 * capture records no memset node.
 *   key_bytes     4 (uint32 keys) or 8 (uint64 keys)
 *   bits          the keys hold nothing above their low `bits` bits (fewer bits, fewer passes)
 *   descending    0: ascending; else descending; pairs with equal keys keep their input order either way
 * The outputs must not alias the inputs, which are left as they are.  Calls on one sorter must be stream-ordered. */
typedef struct recsdk_sorter recsdk_sorter_t;
RECSDK_API int recsdk_sorter_create(int64_t max_pairs, int32_t key_bytes, recsdk_sorter_t** out);
RECSDK_API int recsdk_sorter_destroy(recsdk_sorter_t* h);
RECSDK_API int recsdk_sort_pairs(recsdk_sorter_t* h, const void* d_keys_in, void* d_keys_out,
                                 const uint32_t* d_values_in, uint32_t* d_values_out, int64_t n, int32_t bits,
                                 int32_t descending, void* stream);

/* ------------------------------------------------------------------------------------------------
 * By-address row ops.
 * Replaces the device entry points of the TF custom ops
 *   EmbeddingLookupByAddress  cust_op/framework/tf_plugin/src/cust_embedding_by_address.cpp:19-33
 *                             kernel cust_op/ascendc_op/ai_core_op/cust_op_by_addr/v220/op_kernel/embedding_lookup_by_address.cpp:117-132
 *   EmbeddingUpdateByAddress  cust_op/framework/tf_plugin/src/cust_embedding_by_address.cpp:36-51
 *                             kernel .../op_kernel/embedding_update_by_address.cpp:107-144,158-188
 * d_address[i] is a raw device address minted by the key->address table (0 = skip: lookup writes a zero row,
 * update does nothing).  update_type 0 = atomic add (duplicates accumulate), 1 = overwrite. */
RECSDK_API int recsdk_lookup_by_addr(const int64_t* d_address, int64_t n, int32_t dim, int32_t dtype, void* d_y,
                                     void* stream);
RECSDK_API int recsdk_update_by_addr(const int64_t* d_address, int64_t n, int32_t dim, int32_t dtype,
                                     const void* d_embedding, int32_t update_type, void* stream);

/* LazyAdam fused op: cust_op/framework/tf_plugin/src/lazy_adam.cpp:20-34,
 * kernel cust_op/ascendc_op/ai_core_op/fused_lazy_adam/v220/op_kernel/lazy_adam.cpp:138-205.
 * Rows d_indices[i] >= 0 of m, v, var ([rows, dim] fp32) are updated in place; indices must be distinct
 * (as the reference assumes).  lr is the caller's bias-corrected rate. */
RECSDK_API int recsdk_lazy_adam(const float* d_grad, const int32_t* d_indices, int64_t n, int32_t dim, float* d_m,
                                float* d_v, float* d_var, float lr, float beta1, float beta2, float epsilon,
                                void* stream);
/* Sgd fused op: cust_op/framework/tf_plugin/src/sgd.cpp:19-26,
 * kernel cust_op/ascendc_op/ai_core_op/fused_sgd/v220/op_kernel/sgd_kernel.h:72-95,151-196.
 * var[idx] += -lr * (g + weight_decay * var[idx]) with an atomic add. */
RECSDK_API int recsdk_sgd(const float* d_grad, const int32_t* d_indices, int64_t n, int32_t dim, float* d_var,
                          float lr, float weight_decay, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Key dedup (unique + inverse), multi-table, first-occurrence order.
 * Replaces  KeyProcess::HashSplit / HashSplitWithFAAE (rankSize 1)  training/tf_rec_v1/src/core/key_process/key_process.cpp:1134-1216
 *           KeyProcess::GlobalUnique                                training/tf_rec_v1/src/core/key_process/key_process.h:114-145
 *           IdsMapper::UniqueAndLookupOut (unique/inverse part)     training/torch_rec_v1/hybrid_torchrec/src/ids_process/ids_mapper.cpp:63-113
 *           ock::ctr::Unique::DoUnique / DoEnhancedUnique           training/tf_rec_v1/src/AccCTR/src/include/unique.h:85-125
 * A handle owns the workspace (like ock::ctr::Unique::Initialize); one handle per stream.
 *
 * run(): d_keys[n] holds T tables' keys back to back, table t at [d_offsets[t], d_offsets[t+1]).
 * Results stay in the handle (device memory) until the next run():
 *   unique_keys[U]     distinct keys, table by table, each table in first-occurrence order
 *   unique_offsets[T+1] start of each table's slice in unique_keys; unique_offsets[T] = U
 *   inverse[n]         index of keys[i] inside its table's slice ("restore vector"), -1 for skipped keys
 *   counts[U]          multiplicity of each distinct key (sum of d_in_counts when given)
 * skip_key_enabled != 0: keys equal to skip_key are not deduplicated (inverse = -1), as GlobalUnique does
 * for padding keys under useStatic. */
typedef struct recsdk_unique recsdk_unique_t;

RECSDK_API int recsdk_unique_create(int64_t max_keys, int32_t max_tables, recsdk_unique_t** out);
RECSDK_API int recsdk_unique_destroy(recsdk_unique_t* u);
/* enable == 0: later runs skip the per-key position lists (the ordered occurrence lists that only
 * recsdk_sparse_apply and recsdk_tbe_backward read); unique keys, inverse and counts are unaffected.  Default: on. */
RECSDK_API int recsdk_unique_set_lists(recsdk_unique_t* u, int32_t enable);
/* enable == 0: later runs that build position lists do not collect the multiplicities in their hashing pass (a third of
 * its device atomics); `counts` is then written by the list kernels, as the list lengths, on the handle's own stream:
 * recsdk_unique_fetch and the library's own readers order themselves after it, a caller that reads the pointer of
 * recsdk_unique_results itself must not read counts before the gradient reduce (recsdk_sparse_apply) has been
 * enqueued.  This is KeyProcess::HashSplit, which has no counts (key_process.cpp:1134-1156); the default, on, is
 * HashSplitWithFAAE, whose keyCount feeds the admission that follows at once (:1170-1216).  Runs with d_in_counts or
 * without lists always collect them.  Default: on. */
RECSDK_API int recsdk_unique_set_counts(recsdk_unique_t* u, int32_t enable);
/* A promise that no table holds more than max_table_keys keys in any later run (0 = no promise).  The position lists
 * come from a stable radix sort of the positions by the index of their key inside its table; the promise bounds that
 * index and so the number of radix passes (65536 keys per table: 2 passes of 8 bits, against 3 for 1.7 M keys of
 * unknown split).  With static shapes the caller knows it: one key per sample and field makes it the batch size
 * (the reference pads to static shapes for the same reason, key_process.cpp:1158-1168).  A run that breaks the
 * promise builds empty lists and recsdk_unique_total reports RECSDK_ECAPACITY; unique keys, inverse and early counts
 * are unaffected.  No counterpart in the reference. */
RECSDK_API int recsdk_unique_set_max_table_keys(recsdk_unique_t* u, int64_t max_table_keys);
RECSDK_API int recsdk_unique_run(recsdk_unique_t* u, const int64_t* d_keys, const uint32_t* d_in_counts,
                                 const int64_t* d_offsets, int32_t T, int64_t n, int32_t skip_key_enabled,
                                 int64_t skip_key, void* stream);
/* Device pointers of the results of the last run() (valid until the next run or destroy). */
RECSDK_API int recsdk_unique_results(recsdk_unique_t* u, const int64_t** d_unique_keys,
                                     const int64_t** d_unique_offsets, const int32_t** d_inverse,
                                     const uint32_t** d_counts);
/* Copies the results of the last run() into caller-allocated device buffers (any may be NULL):
 * d_unique_keys[n], d_unique_offsets[T+1], d_inverse[n], d_counts[n]; entries past U are unspecified. */
RECSDK_API int recsdk_unique_fetch(recsdk_unique_t* u, int64_t* d_unique_keys, int64_t* d_unique_offsets,
                                   int32_t* d_inverse, uint32_t* d_counts, void* stream);
/* d_out[i] = d_values[j] where j is the position of key i among ALL distinct keys of the last run (table slices
 * back to back), or `fill` for skipped keys: turns per-distinct-key results (slots, offsets) into per-key ones. */
RECSDK_API int recsdk_unique_expand(recsdk_unique_t* u, const int64_t* d_values, int64_t fill, int64_t* d_out,
                                    void* stream);
/* Synchronous: waits for `stream`, returns U = number of distinct keys of the last run. */
RECSDK_API int recsdk_unique_total(recsdk_unique_t* u, void* stream, int64_t* h_total);

/* recsdk_unique_run for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  The call takes no handle: its workspace is one
 * static device array inside the library (about 5 MB, held by every GPU the library runs on until the process ends),
 * so it calls no hipMalloc / hipFree; its kernels clear what they need of the array themselves.  Limits:
 * n <= RECSDK_UNIQUE_NOALLOC_MAX_KEYS and T <= RECSDK_UNIQUE_NOALLOC_MAX_TABLES, RECSDK_ECAPACITY beyond them.
 * The results go straight to caller-allocated device buffers, with the meaning they have in recsdk_unique_run /
 * recsdk_unique_fetch: d_unique_keys[n], d_unique_offsets[T+1] (entry T = number of distinct keys), d_inverse[n],
 * d_counts[n] (may be NULL).  No position lists are built.  All calls on one GPU share the one array: calls that
 * overlap on a GPU (two streams, two threads) race; order them on one stream or with events. */
#define RECSDK_UNIQUE_NOALLOC_MAX_KEYS 65536
#define RECSDK_UNIQUE_NOALLOC_MAX_TABLES 64
RECSDK_API int recsdk_unique_run_noalloc(const int64_t* d_keys, const uint32_t* d_in_counts, const int64_t* d_offsets,
                                         int32_t T, int64_t n, int32_t skip_key_enabled, int64_t skip_key,
                                         int64_t* d_unique_keys, int64_t* d_unique_offsets, int32_t* d_inverse,
                                         uint32_t* d_counts, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Re-ordered views of a unique run over ONE table (offsets of length 2): the distinct keys grouped by shard and
 * the distinct keys in ascending order.  A regroup handle owns the sort workspace for up to max_keys input keys.
 * Replaces  ock::ctr::Unique::DoEnhancedUnique  training/tf_rec_v1/src/AccCTR/src/unique/unique_impl.cpp:89-148
 *             (ShardedDedup::Compute unique_func.h:271-329, TileAndFill :400-453, HandleFill :455-468,
 *              GetFillOffset unique_func.cpp:173-180; configuration struct include/unique.h:49-65)
 *           hybrid::UniqueParallel             training/torch_rec_v1/hybrid_torchrec/src/ids_process/unique.cpp:55-118
 * ------------------------------------------------------------------------------------------------ */
typedef struct recsdk_regroup recsdk_regroup_t;
RECSDK_API int recsdk_regroup_create(int64_t max_keys, recsdk_regroup_t** out);
RECSDK_API int recsdk_regroup_destroy(recsdk_regroup_t* g);
/* The enhanced outputs of the reference's unique with sharding.  shard(key) = (uint64)key % shards, or
 * (uint64)key & (shards-1) when use_mask != 0 (the reference's `performance` mode; shards a power of two).
 * Inside a shard the keys keep first-occurrence order (the reference's order inside a shard is hash-bucket order;
 * its tests assert the order-free properties only).  With c[s] = distinct keys of shard s, b[s] = c[0]+..+c[s-1]:
 *   padding_size == 0:  d_unique_id[b[s]+r] = r-th key of shard s                      (U entries)
 *                       d_id_cnt[b[s]+r] = its multiplicity (NULL = not wanted)
 *                       *h_unique_id_cnt = U
 *   padding_size  > 0:  d_unique_id[s*padding_size + r] = r-th key of shard s, the rest padding_val
 *                       (shards*padding_size entries); d_id_cnt_fill likewise with 0 in the padding (NULL = not
 *                       wanted); d_id_cnt[b[s]+r] as above; *h_unique_id_cnt = shards*padding_size;
 *                       RECSDK_ECAPACITY (the reference's H_PADDING_SMALL) when some c[s] > padding_size.
 *   d_index[i]               = place of key i's value in d_unique_id             (n entries)
 *   d_unique_in_bucket[b[s]+r] = r-th key of shard s (NULL = not wanted)         (U entries)
 *   d_cnt_in_bucket[s]       = c[s]                                              (shards entries)
 * Synchronous: returns after `stream` has finished.  A run with input counts reports their sums as multiplicity. */
RECSDK_API int recsdk_unique_sharded(recsdk_regroup_t* g, recsdk_unique_t* u, int32_t shards, int32_t use_mask,
                                     int32_t padding_size, int64_t padding_val, int64_t* d_unique_id,
                                     uint32_t* d_index, int64_t* d_unique_in_bucket, int32_t* d_cnt_in_bucket,
                                     int32_t* d_id_cnt, int32_t* d_id_cnt_fill, void* stream,
                                     int32_t* h_unique_id_cnt);
/* d_sorted[0..U) = the distinct keys ascending (signed), d_inverse[i] = place of key i in d_sorted (-1 for a
 * skipped key).  Waits once on `stream` (the sort covers the U distinct keys over the bits in which they differ, and
 * the host needs both numbers to launch it); the result kernels are then queued on `stream`.  U from
 * recsdk_unique_total. */
RECSDK_API int recsdk_unique_sorted(recsdk_regroup_t* g, recsdk_unique_t* u, int64_t* d_sorted, int64_t* d_inverse,
                                    void* stream);

/* ------------------------------------------------------------------------------------------------
 * key -> slot / address tables (a group of T tables, the counterpart of EmbeddingMgmt's table map).
 * Replaces  EmbeddingStatic::Key2Offset   training/tf_rec_v1/src/core/emb_table/embedding_static.cpp:38-99
 *           EmbeddingDynamic::Key2Offset  training/tf_rec_v1/src/core/emb_table/embedding_dynamic.cpp:59-85
 *           EmbeddingTable::EvictKeys     training/tf_rec_v1/src/core/emb_table/embedding_table.cpp:66-85
 *           EmbeddingMgmt::Key2Offset     training/tf_rec_v1/src/core/emb_table/embedding_mgmt.h:47
 * h_dev_vocab_size[t]: capacity in rows.  h_dynamic[t] != 0: the table mints device addresses
 * h_arena_base[t] + seq * h_row_bytes[t] instead of slot numbers, never reuses them, maps -1 to address 0. */
typedef struct recsdk_tables recsdk_tables_t;

RECSDK_API int recsdk_tables_create(int32_t T, const int64_t* h_dev_vocab_size, const int32_t* h_dynamic,
                                    const int64_t* h_arena_base, const int64_t* h_row_bytes, int64_t max_keys,
                                    recsdk_tables_t** out);
RECSDK_API int recsdk_tables_destroy(recsdk_tables_t* tg);
/* In place: d_keys (distinct per table except -1, laid out by d_offsets[T+1]) -> slots / addresses.
 * New keys take slots in array order: evicted slots last-evicted-first, then max_offset++ (train channel);
 * on the eval channel new keys map to -1 (static) / 0 (dynamic).  `n` is an upper bound of d_offsets[T]
 * (the exact total may live only on the device). */
RECSDK_API int recsdk_tables_key2offset(recsdk_tables_t* tg, int64_t* d_keys, const int64_t* d_offsets, int32_t T,
                                        int64_t n, int32_t channel, void* stream);
/* Erase d_keys (distinct per table) and push their slots on the table's evicted-slot stack in array order.
 * Erased entries lengthen probe chains, so once they may fill a quarter of a table's map the call rebuilds that map:
 * it then allocates, waits for `stream` and frees the old map.  Work on OTHER streams that resolves keys against
 * this table group must therefore have finished (or be ordered after this call) whenever evict runs.  On a stream
 * under capture the call records its kernels and never rebuilds; the erased entries are counted on the device, so a
 * loop that replays evictions from a graph calls recsdk_tables_maintain now and then instead. */
RECSDK_API int recsdk_tables_evict(recsdk_tables_t* tg, const int64_t* d_keys, const int64_t* d_offsets, int32_t T,
                                   int64_t n, void* stream);
/* Synchronous housekeeping for callers whose evictions run from a replayed graph (host code never sees them): reads
 * the device-side count of erased entries of every table and rebuilds the maps in which they may fill a quarter.
 * *h_rebuilt (may be NULL) gets the number of tables rebuilt.  Not on a stream under capture.  The reference erases
 * from a host hash map (embedding_table.cpp:66-85) and has nothing to maintain. */
RECSDK_API int recsdk_tables_maintain(recsdk_tables_t* tg, void* stream, int32_t* h_rebuilt);
/* Synchronous: per-table max_offset (EmbeddingTable::size), live key count and evicted-stack depth.
 * Returns RECSDK_EOVERFLOW if any static table's max_offset exceeded its vocabulary
 * (embedding_static.cpp:90-98 throws there), RECSDK_EINVAL if a key2offset call since creation listed one new key
 * twice in a table (the precondition above; the table is corrupt then). Any output pointer may be NULL. */
RECSDK_API int recsdk_tables_stats(recsdk_tables_t* tg, void* stream, int64_t* h_max_offset, int64_t* h_live,
                                   int64_t* h_evicted);
/* Synchronous: copy table t's evicted-slot stack (bottom first) to h_out[cap]; returns depth in *h_count. */
RECSDK_API int recsdk_tables_evict_pos(recsdk_tables_t* tg, int32_t t, void* stream, int64_t* h_out, int64_t cap,
                                       int64_t* h_count);

/* Checkpoint of one table's map.  Export: the live (key, value) pairs in ascending value order (the reference walks its
 * hash map, embedding_static.cpp:163-167 / embedding_dynamic.cpp:203-207, in no defined order) into device buffers of
 * `cap` entries; *h_count = their number; RECSDK_ECAPACITY when cap is too small.  Synchronous.
 * Load (EmbeddingStatic::LoadKey, embedding_static.cpp:190-239; EmbeddingDynamic::LoadKey, embedding_dynamic.cpp:327-387):
 * the table is emptied, then key i of d_keys maps to slot i (dynamic: h_arena_base + i * h_row_bytes), max_offset = n;
 * RECSDK_EOVERFLOW when n exceeds the table's vocabulary ("load key size exceeds device vocab size").  Synchronous. */
RECSDK_API int recsdk_tables_export(recsdk_tables_t* tg, int32_t t, int64_t* d_keys, int64_t* d_values, int64_t cap,
                                    void* stream, int64_t* h_count);
RECSDK_API int recsdk_tables_load_keys(recsdk_tables_t* tg, int32_t t, const int64_t* d_keys, int64_t n, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Checkpoint files in the reference's layout (raw little-endian arrays; parent directories are created).
 *   key file   <savePath>/<table>/key/slice_<rank>.data            int64 keys
 *   row files  <savePath>/<table>/embedding/slice_<rank>.data      embSize floats per key, in key-file order
 *              <savePath>/<table>/<optimName>_<param>/slice_<rank>.data   the same for each optimizer state
 * recsdk_ckpt_write_keys  = the file body of EmbeddingStatic/Dynamic::SaveKey (embedding_static.cpp:137-187).
 * recsdk_ckpt_read_keys   = the filter of ::LoadKey (embedding_static.cpp:216-225): of the file's keys, this rank keeps
 *                           those with key % rank_size == rank_id (all when is_dp); h_load_offset[j] = index in the
 *                           file of the j-th kept key.  *h_count = kept keys; RECSDK_ECAPACITY when cap is too small.
 * recsdk_ckpt_write_rows  = LocalFileSystem::WriteEmbedding (local_file_system.cpp:165-224): row i = emb_size floats
 *                           at device address d_addr[i] + byte_offset (byte_offset = p * emb_size * 4 selects
 *                           optimizer state p, embedding_dynamic.cpp:236-245).
 * recsdk_ckpt_read_rows   = LocalFileSystem::ReadEmbedding (local_file_system.cpp:317-381): file row h_load_offset[i]
 *                           (i when NULL) -> d_first + i * ext_emb_size floats.
 * All four are synchronous on `stream`.  RECSDK_EIO = the reference's IO_ERROR exceptions. */
RECSDK_API int recsdk_ckpt_write_keys(const char* path, const int64_t* d_keys, int64_t n, void* stream);
RECSDK_API int recsdk_ckpt_read_keys(const char* path, int32_t rank_id, int32_t rank_size, int32_t is_dp,
                                     int64_t* h_keys, int64_t* h_load_offset, int64_t cap, int64_t* h_count);
RECSDK_API int recsdk_ckpt_write_rows(const char* path, const int64_t* d_addr, int64_t n, int32_t emb_size,
                                      int64_t byte_offset, void* stream);
RECSDK_API int recsdk_ckpt_read_rows(const char* path, const int64_t* h_load_offset, int64_t n, int32_t emb_size,
                                     float* d_first, int64_t ext_emb_size, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Row storage description used by gather / sparse update: table t's row r lives at
 *   w: h_w[t] + r*h_stride[t]   s1: h_s1[t] + r*h_stride[t]   s2: h_s2[t] + r*h_stride[t]    (fp32 elements)
 * which covers both split variables (stride = dim) and the extended-row layout [w|s1|s2]
 * (training/tf_rec_v1/src/core/emb_table/embedding_dynamic.cpp:131,140: stride = (1+slots)*dim). */
typedef struct recsdk_rows recsdk_rows_t;

RECSDK_API int recsdk_rows_create(int32_t T, int32_t dim, float* const* h_w, float* const* h_s1, float* const* h_s2,
                                  const int64_t* h_stride, recsdk_rows_t** out);
RECSDK_API int recsdk_rows_destroy(recsdk_rows_t* rows);

/* Forward of the sparse lookup: d_out[i, :] = w_t[slot(unique index of key i)], zero row when the key was
 * skipped or its slot is negative.  Replaces tf.gather(table, id_offsets) + gather(unique_emb, restore_vector)
 * (training/tf_rec_v1/python/core/emb/base_sparse_embedding.py:596-609, core/emb/sparse_embedding.py:49-50).
 * d_slots[U] is parallel to the unique keys of `u`'s last run. */
RECSDK_API int recsdk_gather_unique(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots, float* d_out,
                                    void* stream);
/* Backward + optimizer: G[j] = sum of d_grad[i,:] over lookups i of distinct key j (unsorted_segment_sum by restore
 * vector, base_sparse_embedding.py:546-573, optimizers/base.py:87-115), in a fixed order (the reference's atomic adds
 * have none): in ascending i from zero; for a key with more than 1024 lookups, every 256 consecutive lookups of it are
 * summed like that first and the partial sums are then added in order from zero.  Results are reproducible bit for
 * bit.  dim: a multiple of 4, at most 2048.  Then one fused row update per distinct key with slot >= 0:
 *   RECSDK_OPT_ADAM    m,v,w as LazyAdam (lazy_adam.cpp:168-185; lazy_adam_by_addr.py:126-157), lr = bias-corrected rate
 *   RECSDK_OPT_ADAGRAD s += g*g; w += -lr*g/sqrt(s+eps) (adagrad_by_addr.py:101-125)
 *   RECSDK_OPT_SGD     w += -lr*(g + weight_decay*w) (gradient_descent_by_addr.py:86-109) */
RECSDK_API int recsdk_sparse_apply(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots,
                                   const float* d_grad, int32_t optim, float lr, float beta1, float beta2, float eps,
                                   float weight_decay, void* stream);
/* The same with the rate read from device memory (*d_lr, one float) when the kernels run: for a step recorded into a
 * HIP graph, whose launch arguments are fixed at capture - the caller writes the rate of the step (Adam's
 * bias-corrected one changes every step) into *d_lr on the stream before each replay.  Results equal those of
 * recsdk_sparse_apply called with the same value.  No counterpart in the reference, whose TF optimizers take the rate
 * as a tensor already (lazy_adam_by_addr.py:126-157). */
RECSDK_API int recsdk_sparse_apply_lr_dev(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots,
                                          const float* d_grad, int32_t optim, const float* d_lr, float beta1,
                                          float beta2, float eps, float weight_decay, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Feature admission and eviction history (count threshold admission, idle-time eviction), T tables per handle.
 * Replaces  FeatureAdmitAndEvict::FeatureAdmit / FeatureEvict   training/tf_rec_v1/src/core/key_process/feature_admit_and_evict.cpp:46-145,148-200
 *           FeatureFilter::{StatisticsKeyCount,CountFilter,RecordTimestamp,FeatureEvict}
 *                                                               training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/feature_filter/feature_filter.cpp:27-80,112-160
 * Per table (ThresholdValue, training/tf_rec_v1/src/core/utils/common.h:238-255): count threshold (-1 = admission
 * off), time threshold (-1 = eviction off), count coefficient, enable-sum flag; h_capacity[t] bounds the number of
 * live records.  Keys may repeat within a call (their counts are merged); key -1 is ignored.  Timestamps must stay
 * within +-2^31 of the first one a table sees; counts saturate at 2^32-2. */
typedef struct recsdk_faae recsdk_faae_t;
RECSDK_API int recsdk_faae_create(int32_t T, const int64_t* h_capacity, const int32_t* h_count_threshold,
                                  const int32_t* h_time_threshold, const int32_t* h_coef,
                                  const int32_t* h_enable_sum, int64_t max_keys, recsdk_faae_t** out);
RECSDK_API int recsdk_faae_destroy(recsdk_faae_t* f);
/* FeatureAdmit: for every table with keys in the call, table time = max(table time, h_timestamps[t]); on the train channel with enable-sum the record of
 * every distinct key gets count += coef * (its merged d_counts) and lastTime = table time; every occurrence of a
 * key whose count is below the threshold becomes -1 in d_keys.  Eval channel / enable-sum off: look up only. */
RECSDK_API int recsdk_faae_admit(recsdk_faae_t* f, int32_t channel, int64_t* d_keys, const uint32_t* d_counts,
                                 const int64_t* d_offsets, int32_t T, int64_t n, const int64_t* h_timestamps,
                                 void* stream);
/* The same for keys that are already distinct inside each table (the output of recsdk_unique_run with its counts, as
 * KeyProcess hands splitKeys and keyCount to FeatureAdmit, key_process.cpp:1170-1216): no second merge pass.
 * d_counts may be NULL (every key counts once); d_offsets[T] on the device bounds the keys, n is an upper bound. */
RECSDK_API int recsdk_faae_admit_distinct(recsdk_faae_t* f, int32_t channel, int64_t* d_keys, const uint32_t* d_counts,
                                          const int64_t* d_offsets, int32_t T, int64_t n, const int64_t* h_timestamps,
                                          void* stream);
/* recsdk_faae_admit_distinct with the table timestamps in device memory (d_timestamps[T]): nothing is copied from the
 * host, so the call can be recorded into a HIP graph whose replays read the timestamps the caller has put there.  No
 * counterpart in the reference, whose FeatureAdmit takes the batch timestamp from the host-side batch. */
RECSDK_API int recsdk_faae_admit_distinct_dev(recsdk_faae_t* f, int32_t channel, int64_t* d_keys,
                                              const uint32_t* d_counts, const int64_t* d_offsets, int32_t T, int64_t n,
                                              const int64_t* d_timestamps, void* stream);
/* StatisticsKeyCount: count += d_counts[i] (1 when d_counts is NULL) per occurrence. */
RECSDK_API int recsdk_faae_count_add(recsdk_faae_t* f, const int64_t* d_keys, const uint32_t* d_counts,
                                     const int64_t* d_offsets, int32_t T, int64_t n, void* stream);
/* CountFilter: keys that have a count record below the threshold become -1. */
RECSDK_API int recsdk_faae_count_filter(recsdk_faae_t* f, int64_t* d_keys, const int64_t* d_offsets, int32_t T,
                                        int64_t n, void* stream);
/* RecordTimestamp: lastTime[key] = d_timestamps[last occurrence of key]; table time = max over the call. */
RECSDK_API int recsdk_faae_record_timestamp(recsdk_faae_t* f, const int64_t* d_keys, const int64_t* d_timestamps,
                                            const int64_t* d_offsets, int32_t T, int64_t n, void* stream);
/* Synchronous.  Erases every record with tableTime - lastTime >= timeThreshold (strict != 0: >) and writes the
 * evicted keys of table t to d_out_keys[h_out_offsets[t] .. h_out_offsets[t+1]) in ascending (lastTime, key) order.
 * Returns RECSDK_ECAPACITY when `cap` was too small (the records are erased nonetheless). */
RECSDK_API int recsdk_faae_evict(recsdk_faae_t* f, int32_t strict, int64_t* d_out_keys, int64_t cap,
                                 int64_t* h_out_offsets, void* stream);
/* The same eviction without the host in the loop: nothing waits for the stream, the evicted keys of table t go to
 * d_out_keys[d_out_offsets[t] .. d_out_offsets[t+1]) with the offsets ([T+1]) written on the device, in NO particular
 * order (the reference's is hash-map order; recsdk_faae_evict's ascending (lastTime, key) needs two sorts whose sizes
 * must come back to the host).  The lists feed recsdk_tables_evict as they are (it takes device offsets and an upper
 * bound of the key count).  Tables whose evicted-slot stack is reused (static tables) hand out slots in that order
 * afterwards, so runs are reproducible only with recsdk_faae_evict; dynamic tables never reuse.  Keys beyond `cap`
 * are dropped (their records are erased all the same) and recsdk_faae_stats reports RECSDK_ECAPACITY.  Calls
 * no allocator: it can be recorded into a HIP graph.  No counterpart in the reference. */
RECSDK_API int recsdk_faae_evict_dev(recsdk_faae_t* f, int32_t strict, int64_t* d_out_keys, int64_t cap,
                                     int64_t* d_out_offsets, void* stream);
/* Synchronous: live record count and table time per table; RECSDK_EOVERFLOW when a history ran out of slots. */
RECSDK_API int recsdk_faae_stats(recsdk_faae_t* f, void* stream, int64_t* h_live, int64_t* h_latest);
/* Synchronous: copies table t's records (unordered) into device buffers of `cap` entries; a record without
 * count reads 0xFFFFFFFF, without timestamp INT64_MIN. */
RECSDK_API int recsdk_faae_dump(recsdk_faae_t* f, int32_t t, int64_t* d_keys, uint32_t* d_counts, int64_t* d_times,
                                int64_t cap, int64_t* h_count, void* stream);
/* Loads saved records into table t (FeatureAdmitAndEvict::LoadHistoryRecords, feature_admit_and_evict.cpp:323-327,
 * replace != 0: the table's records are dropped first and the table time becomes table_time; FeatureFilter::
 * LoadFeatureRecords / LoadTimestampRecords, feature_filter.cpp:92-110, replace == 0: the given fields are assigned
 * to the records of the keys, which are created when absent).  d_keys must be distinct; d_counts / d_times may be
 * NULL (field left alone), a time of INT64_MIN means "none".  table_time INT64_MIN = the largest loaded time. */
RECSDK_API int recsdk_faae_load(recsdk_faae_t* f, int32_t t, const int64_t* d_keys, const uint32_t* d_counts,
                                const int64_t* d_times, int64_t n, int32_t replace, int64_t table_time, void* stream);

/* ------------------------------------------------------------------------------------------------
 * HBM-cache planner with a version clock.
 * Replaces  SwapManager::ComputeSwapInfo / RemoveKeys
 *           training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/embedding_cache/swap_manager.cpp:32-159
 * cache_size slots, the first mem_start_offset of them never used.  compute(): d_keys[n] need not be distinct,
 * -1 maps to offset 0.  Hits keep their slot (and are stamped with the current version); misses, in batch order,
 * take never-used slots while there are any, then the slots of a clock sweep that were used neither in this nor
 * in the previous batch.  Outputs (caller-allocated, n entries each): swap-out keys/offsets (victims that were not
 * removed before), swap-in keys/offsets (every distinct missed key, batch order), and the slot of every key.
 * counts() is synchronous and returns RECSDK_EOVERFLOW when the last batch did not fit ("cacheSize_ too small");
 * such a batch changes nothing but the hit stamps. */
typedef struct recsdk_swap recsdk_swap_t;
RECSDK_API int recsdk_swap_create(int64_t cache_size, int64_t mem_start_offset, int64_t max_keys, recsdk_swap_t** out);
RECSDK_API int recsdk_swap_destroy(recsdk_swap_t* h);
RECSDK_API int recsdk_swap_compute(recsdk_swap_t* h, const int64_t* d_keys, int64_t n, int64_t* d_swapout_keys,
                                   int64_t* d_swapout_offs, int64_t* d_swapin_keys, int64_t* d_swapin_offs,
                                   int64_t* d_batch_offs, void* stream);
RECSDK_API int recsdk_swap_counts(recsdk_swap_t* h, void* stream, int64_t* h_swapouts, int64_t* h_swapins,
                                  int64_t* h_occupied);
RECSDK_API int recsdk_swap_remove(recsdk_swap_t* h, const int64_t* d_keys, int64_t n, void* stream);
/* d_cache_keys[cache_size] = the key each slot holds, -1 after RemoveKeys (the reference's SwapManager::GetKey,
 * swap_manager.cpp:161-165, which EmbcacheManager walks slot by slot when it saves, embcache_manager.cpp:296-306);
 * slots at or past the occupied count are unspecified.  Asynchronous on `stream`. */
RECSDK_API int recsdk_swap_export(recsdk_swap_t* h, int64_t* d_cache_keys, void* stream);

/* ------------------------------------------------------------------------------------------------
 * HBM-cache planner of the TF path: which slot of the device cache each key of a batch uses, which keys must be
 * brought in and which are pushed out to make room.
 * Replaces  EmbCache::OffsetMapper::GetSwapPairsAndKey2Offset
 *             training/tf_rec_v1/src/AccCTR/src/embedding_cache/offset_mapper/offset_mapper.h:135-171
 *             (FilterKeys :273-295, FindInUsedPos :178-244, FindInOffsetMapper :246-271, Remove :107-119,
 *              LimitedSet limited_set.h:25-140), reached through EmbCacheManager::GetSwapPairsAndKey2Offset
 *             (include/embedding_cache.h) from HybridMgmt (core/hybrid_mgmt/hybrid_mgmt.cpp:983-1056).
 * One handle per table.  The slot sequence is the reference's, bit for bit: keys that are not cached take, in input
 * order, slots freed by remove (latest first), then - only when the cache cannot hold them all - slots whose key
 * neither this call nor the previous one used (most recently released first; their keys are the swap-out list),
 * then never-used slots.
 * ------------------------------------------------------------------------------------------------ */
typedef struct recsdk_om recsdk_om_t;
RECSDK_API int recsdk_om_create(int64_t max_cache_size, int64_t max_keys, recsdk_om_t** out);
RECSDK_API int recsdk_om_destroy(recsdk_om_t* h);
/* d_keys[n] (distinct apart from -1, which is left alone) are replaced in place by their slots.  The keys brought
 * in and their slots go to d_swapin_keys / d_swapin_pos, the keys pushed out and their slots to d_swapout_keys /
 * d_swapout_pos (all device, n entries each); their lengths come from recsdk_om_counts.  Asynchronous on `stream`.
 * When the cache is too small for the batch nothing but the hit stamps changes and recsdk_om_counts reports it
 * (the reference leaves its state half updated in that case and the caller aborts). */
RECSDK_API int recsdk_om_compute(recsdk_om_t* h, int64_t* d_keys, int64_t n, int64_t* d_swapin_keys,
                                 int64_t* d_swapin_pos, int64_t* d_swapout_keys, int64_t* d_swapout_pos,
                                 void* stream);
/* Synchronous: lengths of the lists of the last compute, slots ever used and freed slots waiting for reuse (any
 * pointer may be NULL).  RECSDK_EOVERFLOW = the reference's H_MAX_CACHESIZE_TOO_SMALL for the last compute. */
RECSDK_API int recsdk_om_counts(recsdk_om_t* h, void* stream, int64_t* h_swapins, int64_t* h_swapouts,
                                int64_t* h_use_length, int64_t* h_evict_size);
/* OffsetMapper::Remove for each of d_keys[n] (distinct; keys that are not cached are ignored), in input order. */
RECSDK_API int recsdk_om_remove(recsdk_om_t* h, const int64_t* d_keys, int64_t n, void* stream);
/* d_pos2key[max_cache_size] = key held by each slot, -1 for a slot that is free or was never used
 * (the content of ExportSortedKVPairs, offset_mapper.h:121-126). */
RECSDK_API int recsdk_om_export(recsdk_om_t* h, int64_t* d_pos2key, void* stream);
/* dst takes over the whole state of src (both created with the same max_cache_size): the copy a caller keeps across
 * an evaluation phase.  Replaces the mapper copies of EmbCacheManagerImpl::BackUpTrainStatus / RecoverTrainStatus
 * (training/tf_rec_v1/src/AccCTR/src/embedding_cache/cache_manager/cache_manager.cpp:300-352).  Asynchronous. */
RECSDK_API int recsdk_om_copy_state(recsdk_om_t* dst, const recsdk_om_t* src, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Row initializers and the host-DRAM row store behind the HBM cache (host memory, host key map; the rows move to
 * and from the device cache through two kernels that access the pinned host rows directly).
 * Replaces  ConstantInitializer / RandomNormalInitializer / TruncatedNormalInitializer
 *             training/tf_rec_v1/src/AccCTR/src/embedding_cache/initializer/constant_initializer/constant_initializer.cpp:25-63
 *             .../random_normal_initializer/random_normal_initializer.cpp:24-79
 *             .../truncated_normal_initializer/truncated_normal_initializer.cpp:23-95
 *           EmbLocalTable::{Gather,Scatter,GatherAddrs,GatherAndRemove,RemoveByKeys}
 *             .../embedding_local_table/emb_local_table.cpp:106-335, pool address_mapper.h:72-231
 *           the row movement of HybridMgmt::EmbeddingLookUpAndSendDDR / EmbeddingReceiveAndUpdateDDR
 *             training/tf_rec_v1/src/core/hybrid_mgmt/hybrid_mgmt.cpp:1272-1333, 1606-1822
 * Values: every random initializer owns a std::default_random_engine seeded once and a
 * std::normal_distribution<float>, as in the reference; the j-th row ever created gets the j-th row of that stream
 * (what the reference's pool produces with one refill thread).
 * ------------------------------------------------------------------------------------------------ */
enum { RECSDK_INIT_CONSTANT = 0, RECSDK_INIT_RANDOM_NORMAL = 1, RECSDK_INIT_TRUNCATED_NORMAL = 2 };
typedef struct recsdk_initializer_desc {
    int32_t kind;         /* RECSDK_INIT_* */
    uint32_t start;       /* first column of the row this initializer fills */
    uint32_t len;         /* number of columns */
    float value_or_mean;  /* constant value, or mean of the normal */
    float stddev;         /* normal kinds only */
    uint32_t seed;        /* normal kinds only */
    float init_k;         /* every value is multiplied by init_k */
} recsdk_initializer_desc_t;
typedef struct recsdk_initializer recsdk_initializer_t;
RECSDK_API int recsdk_initializer_create(const recsdk_initializer_desc_t* descs, int32_t n_descs,
                                         recsdk_initializer_t** out);
RECSDK_API int recsdk_initializer_destroy(recsdk_initializer_t* h);
/* Fills `rows` consecutive host rows of ext_dim floats: for each row every initializer writes its column range
 * (columns no initializer covers are left untouched).  The generators keep their state between calls. */
RECSDK_API int recsdk_initializer_generate(recsdk_initializer_t* h, float* h_rows, int64_t rows, int32_t ext_dim);

typedef struct recsdk_hostrows recsdk_hostrows_t;
/* vocab_size rows of ext_dim floats (a multiple of 4) in pinned host memory.  When every initializer is a constant
 * the call also writes that one initial row into every host row (a device kernel over the host link, about a second
 * per 50 GB), so that a later swap-in of a new key whose row was never used writes its cache row only. */
RECSDK_API int recsdk_hostrows_create(int64_t vocab_size, int32_t ext_dim, const recsdk_initializer_desc_t* descs,
                                      int32_t n_descs, recsdk_hostrows_t** out);
RECSDK_API int recsdk_hostrows_destroy(recsdk_hostrows_t* h);
/* EmbLocalTable::Gather / Scatter: find-or-create the row of each key (new rows initialised in input order), copy it
 * to / from h_dst / h_src (n rows of ext_dim floats).  RECSDK_ECAPACITY = H_HOST_VOCAB_SIZE_TOO_SMALL. */
RECSDK_API int recsdk_hostrows_gather(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, float* h_dst,
                                      int32_t threads);
RECSDK_API int recsdk_hostrows_scatter(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const float* h_src,
                                       int32_t threads);
/* EmbLocalTable::GatherAndRemove: a stored key's row is copied out and the key removed; a key without a row gets
 * fresh initial values and is not stored. */
RECSDK_API int recsdk_hostrows_gather_and_remove(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, float* h_dst);
RECSDK_API int recsdk_hostrows_remove(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n);
/* EmbLocalTable::GatherAddrs with row indices in place of addresses; create == 0 reports absent keys as -1. */
RECSDK_API int recsdk_hostrows_find_rows(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, int32_t create,
                                         int64_t* h_rows);
RECSDK_API int recsdk_hostrows_size(recsdk_hostrows_t* h, int64_t* h_live);
/* First row of the pinned host arena: row r (as recsdk_hostrows_find_rows reports it) starts at *h_base + r * ext_dim.
 * These are the addresses EmbLocalTable::GatherAddrs hands out (emb_local_table.cpp:157-199). */
RECSDK_API int recsdk_hostrows_arena(recsdk_hostrows_t* h, float** h_base);
/* All stored (key, row) pairs in ascending key order (h_keys[cap], h_rows[cap*ext_dim]); *h_count = their number
 * (nothing is copied when cap is too small or a buffer is NULL). */
RECSDK_API int recsdk_hostrows_export(recsdk_hostrows_t* h, int64_t* h_keys, float* h_rows, int64_t cap,
                                      int64_t* h_count);
/* EmbLocalTable::Serialize / Deserialize (emb_local_table.cpp:361-402): records [key u64 | ext_dim floats], here in
 * ascending key order.  serialize: *h_bytes = size needed; nothing is written when h_buf is NULL or cap too small.
 * deserialize: each key's row is found or created, then overwritten; a cut record -> RECSDK_EINVAL "get data failed!". */
RECSDK_API int recsdk_hostrows_serialize(recsdk_hostrows_t* h, char* h_buf, int64_t cap, int64_t* h_bytes);
RECSDK_API int recsdk_hostrows_deserialize(recsdk_hostrows_t* h, const char* h_buf, int64_t bytes);
/* EmbcacheManager::Save / Load for one table (training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/
 * embedding_cache/embcache_manager.cpp:342-458,460-527): under prefix = <path>/<table>/rank<rank>
 *   key/slice.data int64 keys, key/slice.attribute {8, count};
 *   embedding/slice.data, momentum1/, momentum2/ (optim_num 0..2): emb_dim floats per key, slice.attribute
 *   {4, count, emb_dim}; a row is [embedding | momentum1 | momentum2].  Keys are written in ascending order (the
 * reference walks its map).  load checks the attributes like the reference (count, dim, file sizes) and assigns
 * the rows (InsertOrAssign). */
RECSDK_API int recsdk_hostrows_save(recsdk_hostrows_t* h, const char* prefix, int32_t emb_dim, int32_t optim_num);
RECSDK_API int recsdk_hostrows_load(recsdk_hostrows_t* h, const char* prefix, int32_t emb_dim, int32_t optim_num);
/* Swap-out: device cache rows d_cache[d_slots[i]*cache_stride ...] -> host rows of h_keys[i] (found or created).
 * Swap-in : host rows of h_keys[i] (found, or created with initial values) -> device cache rows.
 * h_keys is host memory (uploaded in pieces after `stream` has drained), d_slots device memory; the row copies are
 * asynchronous on `stream`: synchronise it before the host reads rows a swap-out wrote.  Issue the swap-out of a
 * batch before its swap-in: they reuse the same cache slots.  Key -1 is reserved and has no row. */
RECSDK_API int recsdk_hostrows_swap_out(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots,
                                        const float* d_cache, int64_t cache_stride, void* stream);
RECSDK_API int recsdk_hostrows_swap_in(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots,
                                       float* d_cache, int64_t cache_stride, void* stream);
/* The same with the keys in device memory (distinct, as the cache planners emit them): the key -> row map of the
 * store lives on the device, so nothing waits for the host (with non-constant initializers the call first waits for
 * `stream` to learn how far the initializer stream has been consumed, and generates the next n rows of it).  Keys
 * that find the store full are skipped: a swap-out drops their rows, a swap-in leaves their cache rows as they were,
 * and the call itself still returns RECSDK_OK because it does not wait for the device.  The condition is sticky on
 * the device and recsdk_hostrows_size (one 8-byte read after a stream wait) reports it as RECSDK_ECAPACITY: a caller
 * whose store may fill up checks it once per step, before it trusts the rows of that step.  No counterpart in the
 * reference, whose planner and row store exchange key lists through the host. */
RECSDK_API int recsdk_hostrows_swap_out_dev(recsdk_hostrows_t* h, const int64_t* d_keys, int64_t n,
                                            const int64_t* d_slots, const float* d_cache, int64_t cache_stride,
                                            void* stream);
RECSDK_API int recsdk_hostrows_swap_in_dev(recsdk_hostrows_t* h, const int64_t* d_keys, int64_t n,
                                           const int64_t* d_slots, float* d_cache, int64_t cache_stride, void* stream);
/* recsdk_hostrows_swap_out_dev(out ...) followed by recsdk_hostrows_swap_in_dev(in ...), with the rows that go out
 * and the rows that come in crossing the host link at the same time: the outgoing cache rows are first copied aside in
 * HBM (the store keeps a buffer for them, grown on demand), so the incoming rows may take their slots at once.  The
 * result equals that of the two calls when no key is in both lists, which holds for the lists of one planner call
 * (a key a batch needs is never that batch's victim).  No counterpart in the reference, whose EmbCacheManager moves
 * the two lists one after the other with host threads. */
RECSDK_API int recsdk_hostrows_swap_dev(recsdk_hostrows_t* h, const int64_t* d_out_keys, int64_t n_out,
                                        const int64_t* d_out_slots, const int64_t* d_in_keys, int64_t n_in,
                                        const int64_t* d_in_slots, float* d_cache, int64_t cache_stride, void* stream);

/* `event` (a hipEvent_t of the caller, NULL = none): every later recsdk_hostrows_swap_dev records it on its stream
 * after the kernels that prepare the move (host rows of the keys, the copy aside of the rows that go out) and right
 * before the kernel that crosses the host link.  For callers that run other work beside the link kernel but not
 * beside the preparation: the kernels before the link kernel are short and bound by latency, and next to a
 * bandwidth-bound kernel they take twice as long while the link waits for them.  A call that has rows for one
 * direction only, or more than one device call holds, moves them one direction after the other and records nothing.
 * The caller keeps the event alive until it hands over another or NULL.  No counterpart in the reference. */
RECSDK_API int recsdk_hostrows_on_link_start(recsdk_hostrows_t* h, void* event);

/* ------------------------------------------------------------------------------------------------
 * Batch ingestion (the step before the dedup).
 * Replaces ReadEmbKeyV2::EnqueueBatchData and ::ParseTimestampAndCheck
 * (training/tf_rec_v1/src/ops_tf/hybrid_dataset_ops.cpp:467-531).  d_sample is the batch tensor of the input
 * pipeline, data_size elements of sample_dtype (RECSDK_DT_I32 or RECSDK_DT_I64): with is_timestamp one leading
 * element whose first 8 bytes are a unix time, then h_splits[i] keys for table i = 0..n_tables-1.  Tables with
 * h_table_used[i] == 0 are skipped (NULL = all used).  The keys of the used tables are written back to back, widened
 * to int64, to d_keys; their offsets [used+1] go to d_offsets (device) and h_offsets (host), either may be NULL.
 * Errors, as the reference: is_timestamp and data_size - field_num != 1 -> RECSDK_EINVAL "Timestamp field not found";
 * timestamp <= 0 -> RECSDK_EINVAL; also RECSDK_EINVAL when the splits exceed the tensor.  *h_timestamp = the time, or
 * -1 without is_timestamp.  Reading the timestamp synchronises `stream`; the copy itself is asynchronous. */
RECSDK_API int recsdk_read_emb_key(const void* d_sample, int32_t sample_dtype, int64_t data_size,
                                   const int64_t* h_splits, const uint8_t* h_table_used, int32_t n_tables,
                                   int32_t is_timestamp, int64_t field_num, int64_t* d_keys, int64_t* d_offsets,
                                   int64_t* h_offsets, int64_t* h_timestamp, void* stream);
/* KeyProcess::PushPaddingKeysTensors (key_process.cpp:1808-1827) and HybridMgmt::SendPaddingKeysMaskVecDDRL3
 * (hybrid_mgmt.cpp:2520-2540): d_mask[i] = 0 when d_values[i] is one of the n_padding host values, else 1.  The
 * reference tests offsets against the offsets recorded for the padding keys (EmbeddingTable::RecordPaddingKeysOffset,
 * embedding_table.cpp:263-272); testing the keys against the padding keys before the key->offset step gives the same
 * mask and needs no recorded set. */
RECSDK_API int recsdk_padding_keys_mask(const int64_t* d_values, int64_t n, const int64_t* h_padding, int32_t n_padding,
                                        int32_t* d_mask, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Hot-key staging of the restore vector, on top of a unique run.
 * Replaces KeyProcess::HotHashSplit (training/tf_rec_v1/src/core/key_process/key_process.cpp:1218-1293),
 * KeyProcess::ComputeHotPos (:963-985) and KeyProcess::UpdateHotMap / UpdateHotMapForUnique (:1310-1356) for one
 * rank.  Each table t keeps a set of at most h_hot_counts[t] (hotEmbTotCount) hot keys, empty at creation.
 * recsdk_hot_split, after recsdk_unique_run on `u`:
 *   d_restore[i] (i over all keys of the run) = h, when key i is the h-th distinct hot key of its table in order of
 *                first occurrence; otherwise (index of the key among the table's distinct keys) + h_hot_counts[t];
 *                -1 for keys the run skipped
 *   d_hot_pos   [sum of h_hot_counts], table after table: entry h of table t = index, among the table's distinct keys,
 *                of that h-th hot key; entries past the hot keys seen in this batch are 0
 *   refresh != 0 (the reference does it when batchId % hotEmbUpdateStep == 0): afterwards each table's hot set
 *                becomes the h_hot_counts[t] most frequent keys of this batch (ties: the smaller key); this part
 *                synchronises `stream` and selects on the host. */
typedef struct recsdk_hot recsdk_hot_t;
RECSDK_API int recsdk_hot_create(int32_t T, const int32_t* h_hot_counts, int64_t max_keys, recsdk_hot_t** out);
RECSDK_API int recsdk_hot_destroy(recsdk_hot_t* h);
RECSDK_API int recsdk_hot_split(recsdk_hot_t* h, recsdk_unique_t* u, int32_t* d_restore, int32_t* d_hot_pos,
                                int32_t refresh, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Split-embedding (table-batched) pooled lookup and its exact backward with fused optimizer.
 * Replaces the device side of the torch operators
 *   fbgemm::split_embedding_codegen_forward_unweighted_cuda
 *       cust_op/framework/torch_plugin/torch_library/2.6.0/split_embedding_codegen_forward_unweighted/split_embedding_codegen_forward_unweighted.cpp:77-96
 *       spec cust_op/ascendc_op/ai_core_op/split_embedding_codegen_forward_unweighted/v220/README.md:81-127
 *   fbgemm::split_embedding_backward_codegen_{adagrad,adam,sgd}_unweighted_exact_cuda
 *       .../backward_codegen_adam_unweighted_exact.cpp:469-508
 *       spec cust_op/ascendc_op/ai_core_op/backward_codegen_adagrad_unweighted_exact/v220/README.md:101-160,233-303,358-416
 * Layout as in the reference: table t's rows start at element d_weights_offsets[t] of d_dev_weights and are
 * D_t = d_D_offsets[t+1]-d_D_offsets[t] wide; d_offsets[T*B+1] is feature-major (bag (t,b) at t*B+b);
 * d_out is [B, total_D] fp32 (pooling NONE: [nnz, total_D/T]).  weights_dtype is RECSDK_DT_F32 or RECSDK_DT_BF16
 * (bf16 rows are widened to fp32 for the sums; an extension, the reference op is fp32 only).  nnz is the length
 * of d_indices (= d_offsets[T*B]).  Rows outside the weight buffer / the table contribute nothing.  Row widths are
 * multiples of 4 up to 2048 (the reference's operator test goes to 1536). */
RECSDK_API int recsdk_tbe_forward(const void* d_dev_weights, int32_t weights_dtype, int64_t weights_numel,
                                  const int64_t* d_weights_offsets, const int32_t* d_D_offsets, int64_t total_D,
                                  int32_t max_D, const int64_t* d_indices, const int64_t* d_offsets, int32_t T,
                                  int64_t B, int64_t nnz, int32_t pooling_mode, float* d_out, void* stream);

/* Backward workspace (dedup scratch, per-position sample map); one handle per stream. */
typedef struct recsdk_tbe recsdk_tbe_t;
RECSDK_API int recsdk_tbe_create(int32_t max_tables, int64_t max_nnz, recsdk_tbe_t** out);
RECSDK_API int recsdk_tbe_destroy(recsdk_tbe_t* h);
/* G[row] = sum, over the positions that name `row`, of the position's gradient row, in the fixed order of
 * recsdk_sparse_apply (ascending position; more than 1024 positions: 256 at a time, then the partial sums):
 *   sum / mean pooling  d_grad_output[b, D-slice of t] for a position of bag (t, b) (mean: times 1/len of the bag);
 *                       d_grad_output is [B, total_D]
 *   RECSDK_POOL_NONE    d_grad_output[k, :] for position k; d_grad_output is [nnz, max_D], total_D = T * max_D
 * Features (entries of d_weights_offsets / d_D_offsets / segments of d_offsets) that read one table carry the same
 * d_hash_size_cumsum entry and must be adjacent; their positions are summed into the same rows, as the reference's kernel
 * does by accumulating at hash_size_cumsum[t] + row (op_kernel/backward_codegen_unweighted_exact_kernel.h:314-316,373-378).
 * Then one update per touched row, in place:
 *   RECSDK_OPT_ADAGRAD  m1 += G*G; w += -(lr/(sqrt(m1)+eps))*G
 *   RECSDK_OPT_ADAM     m1 = b1*m1+(1-b1)*G; m2 = b2*m2+(1-b2)*G*G; w += (-lr*sqrt(1-b2^iter)/(1-b1^iter)) * m1/(sqrt(m2)+eps)
 *   RECSDK_OPT_SGD      w += -lr*G
 * momenta are fp32 arrays laid out like the weights.  The touched rows are grouped by a stable radix sort of
 * (first row of the table + row, gradient row) when all tables together hold fewer than 2^32 rows (by hashing otherwise);
 * d_hash_size_cumsum[T] is read back once per handle for that, on the first call (a handle serves one set of tables).
 * The reference reads rows by hash_indices when its caller passes that tensor (op_kernel/...exact_kernel.h:314,373-374):
 * such a caller passes hash_indices as d_indices here (and to recsdk_tbe_forward, ...forward_unweighted_kernel.h:103-107). */
RECSDK_API int recsdk_tbe_backward(recsdk_tbe_t* h, int32_t optim, const float* d_grad_output, void* d_dev_weights,
                                   int32_t weights_dtype, const int64_t* d_weights_offsets, const int32_t* d_D_offsets,
                                   int64_t total_D, int32_t max_D, const int64_t* d_hash_size_cumsum,
                                   const int64_t* d_indices, const int64_t* d_offsets, int32_t T, int64_t B,
                                   int64_t nnz, int32_t pooling_mode, float* d_momentum1, float* d_momentum2, float lr,
                                   float eps, float beta1, float beta2, int64_t iter, void* stream);
/* The unique variant of the same operators: the caller brings the distinct rows and the inverse index instead of
 * having the operator find them.  Replaces the kernels selected when unique_ids is given
 *   cust_op/ascendc_op/ai_core_op/backward_codegen_adagrad_unweighted_exact/v220/op_kernel/backward_codegen_unweighted_exact_kernel_unique.h:47-95,115-270
 *   .../backward_codegen_adam_unweighted_exact_kernel_unique.h:52-66,110-160, op_host/...cpp:69-120,178-204
 *   (operator arguments unique_ids, unique_offsets, unique_inverse: torch_library/2.6.0/.../backward_codegen_adam_unweighted_exact.cpp:383-409).
 * d_unique_ids[num_unique]: the distinct rows, table after table; d_unique_offsets[T+1]: start of feature t's table in
 * it (features of one table carry the same start; entry T = num_unique); d_unique_inverse[nnz]: place of position k's
 * row inside its table's slice.  G[j] is summed at j = unique_offsets[t] + unique_inverse[k] in ascending k, then row
 * d_unique_ids[j] of its table gets one update.  The positions are grouped by a stable sort on log2(num_unique) bits
 * (the plain form sorts on log2(rows of all tables) bits); indices are not read.  Positions whose inverse lies outside
 * their table's slice, and distinct rows outside their table, are left out.  The reference runs the Adagrad kernel for
 * SGD in this variant (op_host/...cpp:113-119); here SGD is SGD. */
RECSDK_API int recsdk_tbe_backward_unique(recsdk_tbe_t* h, int32_t optim, const float* d_grad_output,
                                          void* d_dev_weights, int32_t weights_dtype, const int64_t* d_weights_offsets,
                                          const int32_t* d_D_offsets, int64_t total_D, int32_t max_D,
                                          const int64_t* d_hash_size_cumsum, const int64_t* d_offsets, int32_t T,
                                          int64_t B, int64_t nnz, int32_t pooling_mode, const int64_t* d_unique_ids,
                                          const int64_t* d_unique_offsets, const int64_t* d_unique_inverse,
                                          int64_t num_unique, float* d_momentum1, float* d_momentum2, float lr,
                                          float eps, float beta1, float beta2, int64_t iter, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RECSDK_HIP_H */
