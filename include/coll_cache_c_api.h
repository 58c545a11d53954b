/*
 * coll_cache_c_api.h — the drop-in C boundary of the embedding-extraction path (libcoll_cache.so).
 *
 * Section 1 is, name for name and argument for argument, the extern "C" surface of the reference's shim
 * (SJTU-IPADS/ugache python/collcache/common/operation.h:31-61 and operation.cc:205-209), which its ctypes
 * loader (python/collcache/common/__init__.py:173-262) and its PyTorch / TensorFlow bindings call.
 * Section 2 holds C-callable forms of what the reference exposes only as C++ (the std::function allocator of
 * coll_cache_init, the refresh driven by the TF LookupManager) plus wide-key siblings; each names what it
 * stands for.
 *
 * Errors follow the reference: no return codes; a violated precondition or a failed GPU call prints a message
 * and abort()s (coll_cache_lib/logging.h:32-34, logging.cc:69-73).
 * Threading: one replica <-> one GPU <-> one caller thread; coll_cache_lookup is blocking and not re-entrant per
 * replica; coll_cache_refresh may run on another thread concurrently with lookups.
 * All key / output pointers of lookups are device pointers; `stream` is a hipStream_t passed as void*.
 */
#ifndef COLL_CACHE_C_API_H_
#define COLL_CACHE_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *StreamHandle; /* coll_cache_lib/common.h:137 */

/* ---------------- Section 1: the reference's extern "C" surface ---------------- */

/* operation.h:35-36, operation.cc:154-167.  Required keys (operation.cc:72-78): cache_percentage, _cache_policy,
 * num_device, num_global_step_per_epoch, num_epoch, num_total_item, omp_thread_num.  Once per process. */
void coll_cache_config(const char **config_keys, const char **config_values, const size_t num_config_items);
/* operation.h:42, operation.cc:177-180 */
void coll_cache_log_step_by_key(uint64_t key, int item, double val);
/* operation.h:44, operation.cc:182-186 */
void coll_cache_report_step_by_key(uint64_t key);
/* operation.h:46, operation.cc:188-202 */
void coll_cache_report_step_average_by_key(uint64_t key);
/* operation.h:49, operation.cc:211-213 */
void coll_cache_train_barrier(void);
/* operation.h:53, operation.cc:219-230: waitpid(-1); 1 if a child exited non-zero or by signal, else 0 */
int coll_cache_wait_one_child(void);
/* operation.h:55, operation.cc:258-261 */
void coll_cache_print_memory_usage(void);
/* operation.h:57, operation.cc:232-236: output[i, :] = table[key[i], :]; step key = steps[replica] * num_device + replica */
void coll_cache_lookup(int replica_id, uint32_t *key, size_t num_keys, void *output, StreamHandle stream);
/* operation.h:59, operation.cc:241-244: host pointer; counts hotness and tracks the largest batch */
void coll_cache_record(int replica_id, uint32_t *key, size_t num_keys);
/* operation.cc:205-209 (declared by the ctypes loader, __init__.py:201-202) */
void coll_cache_record_init(int replica_id);

/* ---------------- Section 2: C forms of the reference's C++-only entry points ---------------- */

/* Device allocator callback pair standing for std::function<MemHandle(size_t)> (operation.h:28;
 * coll_cache_lib/common.h:140-149): alloc returns device memory of at least nbytes, release frees it.
 * Passing alloc == NULL makes the library use its own device allocator. */
typedef void *(*coll_cache_alloc_fn)(size_t nbytes, void *user);
typedef void (*coll_cache_release_fn)(void *ptr, void *user);

/* coll_cache_init (operation.h:28, operation.cc:129-150): combine + rank the recorded hotness, place, build the
 * cache of replica_id.  dtype is the DataType code of coll_cache_lib/common.h:39-49 (kF32 = 0, kF16 = 2 ...);
 * fp16 tables may be passed as kF16 with their true dim.  cpu_data must be pinned GPU-mapped host memory
 * (coll_cache_alloc_host_table) unless cache_percentage == 1. */
void coll_cache_init_c(int replica_id, size_t key_space_size, coll_cache_alloc_fn alloc, coll_cache_release_fn release,
                       void *user, void *cpu_data, int dtype, size_t dim, double cache_percentage,
                       StreamHandle stream);
/* the build_v2 overload taking an explicit rank list + frequency list over all keys
 * (coll_cache_lib/facade.h:56-60) instead of recorded hotness */
void coll_cache_init_ranked_c(int replica_id, size_t key_space_size, const uint32_t *rank_keys,
                              const uint32_t *rank_freq, coll_cache_alloc_fn alloc, coll_cache_release_fn release,
                              void *user, void *cpu_data, int dtype, size_t dim, double cache_percentage,
                              StreamHandle stream);
/* CollCache::build (coll_cache_lib/facade.h:52-54, facade.cc:38-72) for C callers: builds every replica from the
 * placement the library already holds, with an allocator made per replica from the callback pair.  A cache of 0 % or
 * 100 % needs no placement; a partial one needs an earlier coll_cache_init* to have solved (build places nothing). */
void coll_cache_build_all_c(coll_cache_alloc_fn alloc, coll_cache_release_fn release, void *user, void *cpu_data,
                            int dtype, size_t dim, double cache_percentage, StreamHandle stream);
/* 64-bit (dense) keys: siblings of coll_cache_lookup / coll_cache_record.  The reference is uint32 end to end
 * (coll_cache_lib/constant.h:28). */
void coll_cache_lookup_i64(int replica_id, const int64_t *key, size_t num_keys, void *output, StreamHandle stream);
void coll_cache_record_i64(int replica_id, const int64_t *key, size_t num_keys);
/* The distinct keys of a batch looked up once (extension; the "unique -> lookup -> gather(idx)" of the TF2 binding's
 * sparse layer, python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:196-209, with the unique done on the
 * GPU inside the call): output[u, :] = row of the u-th distinct key (in order of first claim, not sorted),
 * inverse_out[i] = which distinct key position i holds, so output[inverse_out[i], :] is the row of key[i].  output
 * (device) needs room for num_keys rows, inverse_out (device) for num_keys words.  Blocking.  Returns the number of
 * distinct keys. */
size_t coll_cache_lookup_unique(int replica_id, const uint32_t *key, size_t num_keys, void *output,
                                uint32_t *inverse_out, StreamHandle stream);
size_t coll_cache_lookup_unique_i64(int replica_id, const int64_t *key, size_t num_keys, void *output,
                                    uint32_t *inverse_out, StreamHandle stream);
/* Lookup and per-sample combination of a multi-hot feature in one call (extension; what the TF2 sparse layer does in
 * three steps, python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:196-265: look the ids up, gather,
 * embedding_lookup_sparse).  Segment r = key[seg_off[r] .. seg_off[r + 1]); output[r, :] = sum of weights[j] x row(key[j])
 * over the segment (weights NULL: 1), as it is (combiner 0 "sum"), divided by the sum of the weights (1 "mean") or by
 * the root of the sum of their squares (2 "sqrtn"); a zero denominator or an empty segment gives a zero row.  Elements
 * are fp32 (elem_bytes 4), fp16 (elem_bytes 2: the rows of a table configured as half) or bfloat16 (elem_bytes 0x102,
 * UGK_ELEM_BF16 of ugache_hip.h: such a table is configured as half too), added in fp32 in the order of
 * the ids.  key, seg_off (num_rows + 1 ascending int64 offsets, the last one num_keys), weights: device memory;
 * output: device [num_rows, dim], caller-allocated; blocking, like coll_cache_lookup.  Rows must be a multiple of 16
 * bytes and at most 4096 bytes long.  coll_cache_last_group_offset afterwards counts keys, not output rows. */
void coll_cache_lookup_pooled(int replica_id, const uint32_t *key, const int64_t *seg_off, const float *weights,
                              size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                              StreamHandle stream);
void coll_cache_lookup_pooled_i64(int replica_id, const int64_t *key, const int64_t *seg_off, const float *weights,
                                  size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                                  StreamHandle stream);
/* the same as one step of the serving loop (coll_cache_forward*: a prefix of the keys recorded, a background refresh
 * at the configured step) */
void coll_cache_forward_pooled(int replica_id, const uint32_t *key, const int64_t *seg_off, const float *weights,
                               size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                               StreamHandle stream);
void coll_cache_forward_pooled_i64(int replica_id, const int64_t *key, const int64_t *seg_off, const float *weights,
                                   size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                                   StreamHandle stream);
/* Stream-ordered lookups (extension; the reference's lookup always blocks, facade.cc:74-88 and the synchronisations
 * of cache_context.cu:1199-1794).  coll_cache_lookup_async* enqueue the batch on `stream` and return: `output` is
 * complete for anything enqueued on the same stream afterwards, which is all a framework op needs; about 10 us of
 * blocking round trip per batch disappear.  `key` and `output` must stay valid until the work has run.  The
 * stream-ordered lookups of a replica that are in flight together must use one stream (they report through the same
 * words); a refresh may run on any stream and in any thread: it waits for the lookups in flight wherever they were
 * enqueued before it reuses a slot.  coll_cache_lookup_wait blocks until
 * everything enqueued so far has finished, aborts if a key was outside its table, and makes
 * coll_cache_last_group_offset describe the last batch; any blocking lookup does the same first.  No per-step profiler
 * values are logged for stream-ordered batches.  Such a call is kernel launches only (no synchronisation, no
 * allocation, no memset), so it may be recorded into a HIP graph by a caller that captures its stream; while a stream
 * records, the library enqueues kernels on that stream and nothing else, and with the hotness counted on the device
 * (COLL_GPU_RECORD=1) the counting is one more kernel of the recorded lookup, so every replay counts the keys it
 * reads.  Batches the
 * one-kernel paths cannot take (COLL_DEDUP_KEYS, a factored
 * SAMGRAPH_COLL_CACHE_CONCURRENT_LINK_IMPL, rows not multiples of 16 bytes with a partial cache) block as usual. */
void coll_cache_lookup_async(int replica_id, const uint32_t *key, size_t num_keys, void *output, StreamHandle stream);
void coll_cache_lookup_async_i64(int replica_id, const int64_t *key, size_t num_keys, void *output,
                                 StreamHandle stream);
/* The pooled lookup in the same stream-ordered form (no counterpart in the reference either): enqueued and left, the
 * group sizes (of ids) and the status arrive with coll_cache_lookup_wait. */
void coll_cache_lookup_pooled_async(int replica_id, const uint32_t *key, const int64_t *seg_off, const float *weights,
                                    size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                                    StreamHandle stream);
void coll_cache_lookup_pooled_async_i64(int replica_id, const int64_t *key, const int64_t *seg_off,
                                        const float *weights, size_t num_rows, size_t num_keys, int combiner,
                                        int elem_bytes, void *output, StreamHandle stream);
/* The max_norm of the sparse layer (python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:95-140, handed to
 * embedding_lookup_sparse): the pooled lookups of the replica that follow clip every looked-up row to this l2 norm
 * before it is weighted, x * max_norm / max(||x||_2, max_norm), inside the same kernel.  0 (the default) turns it
 * off.  No counterpart as an entry point in the reference, where TensorFlow clips. */
void coll_cache_set_pooled_max_norm(int replica_id, float max_norm);
/* The seg_off a pooled lookup takes, made on the device from the row of every entry of a sparse feature in row-major
 * order (extension; the indices[:, 0] of the SparseTensor of sparse_lookup_layer.py:196-265): seg_off[r] = number of
 * entries whose row is below r, r = 0 .. num_rows (num_rows + 1 device words).  One kernel on `stream`, no wait.
 * Entries out of order or outside [0, num_rows) make the next lookup's status check abort with a message. */
void coll_cache_segment_offsets(int replica_id, const int64_t *sorted_rows, size_t num_entries, size_t num_rows,
                                int64_t *seg_off, StreamHandle stream);
void coll_cache_lookup_wait(int replica_id, StreamHandle stream);
/* Sparse-id mode (extension; call after coll_cache_config and before recording or building): the caller's id of
 * host row r is (r * mul) mod 2^bits with mul odd, so 64-bit hashed ids from a 2^bits space address a dense host table
 * of num_total_item rows.  Cached ids live in the open-addressing GPU table; a missed id is turned back into its row
 * with the modular inverse.  mul == 0 restores plain row-number keys.  Lookups and records then take int64 ids. */
void coll_cache_set_key_map(uint64_t mul, int bits);
/* LookupManager::refresh (python_tf2/collcache_tf2/collcache_tf2/core/lookup_manager.cc:317-333) ->
 * CollCache::refresh (coll_cache_lib/facade.cc:513-557): re-rank by the hotness recorded since the last
 * build/refresh, evict and insert.  foreground != 0 skips the wait for an in-flight lookup and the throttling. */
void coll_cache_refresh(int replica_id, StreamHandle stream, int foreground);
/* pinned, GPU-mapped host memory for the embedding table; stands for Tensor::CreateShm + cudaHostRegister
 * (python/collcache/torch/adapter.cc:239-268; coll_cache_lib/facade.cc:476) */
void *coll_cache_alloc_host_table(size_t nbytes);
void coll_cache_free_host_table(void *ptr);
/* `extern size_t max_num_keys` of operation.h:29 */
size_t coll_cache_max_num_keys(void);
void coll_cache_set_max_num_keys(size_t n);
/* {0, #rows served from the GPU cache, num_keys} of the last lookup: the reference's group_offset
 * (coll_cache_lib/cache_context.cu:825-847) */
void coll_cache_last_group_offset(int replica_id, uint32_t out[3]);
/* out[0] cache capacity in rows, [1] cached rows, [2] lookup table kind (0 none/direct, 1 flat, 2 open addressing),
 * [3] row bytes, [4] key space, [5] completed lookups, [6] free cache slots, [7] lookup-table rebuilds so far */
void coll_cache_get_info(int replica_id, uint64_t out[8]);
/* With COLL_MISS_STAGE_ROWS=n the fused extraction also files every row it takes from the host table in a
 * direct-mapped set of n rows in HBM, and a refresh takes the rows it inserts from there when it finds them
 * (the reference copies them over the host link again, cache_context.cu:4054-4090).  Returns how many rows the refreshes
 * of replica_id have taken from that set so far (blocks on the refresh stream; call while no refresh runs). */
uint64_t coll_cache_rows_from_stage(int replica_id);
/* cached keys of replica_id (ascending): copies up to `capacity` keys, returns the number cached */
size_t coll_cache_get_cached_keys(int replica_id, uint32_t *out, size_t capacity);
/* value of one profiler item of the reference's LogStepItem enum at a step key (0 when not logged) */
double coll_cache_get_step_value(uint64_t key, int item);
/* host-only pieces of the build, callable without a GPU:
 * rank the hotness recorded so far exactly as coll_cache_init_c would (LocalCombineToShared + GlobalCombine + Sort,
 * operation.cc:138-147; this consumes the recorded counts): distinct keys in rank order with their counts, up to
 * `capacity` entries are copied; returns the number of distinct keys */
size_t coll_cache_rank_hotness(int replica_id, uint32_t *keys_out, uint32_t *cnts_out, size_t capacity);
/* place num_node ranked keys for one GPU (the solver step of build_v2, facade.cc:93-160): nid_to_block_out[key] = 0
 * (cached) or 1 (host); returns the number of cached keys */
uint32_t coll_cache_place_ranked(const uint32_t *rank_keys, const uint32_t *rank_freq, uint32_t num_node,
                                 double cache_percentage, uint32_t *nid_to_block_out);
/* the two steps above in one, as coll_cache_init_c and coll_cache_refresh run them (ranking consumed from the
 * recorder, solver fed with the observed keys only: solve_impl_master(ContFreqBuf*), facade.cc:161-236); keys never
 * recorded rank behind all recorded ones in ascending order.  num_node must equal num_total_item. */
uint32_t coll_cache_place_recorded(int replica_id, uint32_t num_node, double cache_percentage,
                                   uint32_t *nid_to_block_out);
/* ---- serving loop: LookupManager::forward (python_tf2/collcache_tf2/collcache_tf2_cc/collcache_tf2_cc_infra/src/
 *      lookup_manager.cc:158-213, record thread :291-312, refresh :317-333) without TensorFlow -------------------
 * coll_cache_forward_config: enable_refresh and refresh_iter are ps_config's coll_cache_enable_refresh and
 * coll_cache_refresh_iter (inference_utils.cpp:62-140); record_fraction is the share of each batch whose hotness is
 * recorded, a prefix of the batch (the reference records the first 5 %: 0.05); periodic != 0 starts a refresh every
 * refresh_iter steps instead of once at step refresh_iter.
 * coll_cache_forward_*: one step = record the prefix (on the device when COLL_GPU_RECORD=1, else a copy of the prefix
 * to the host and coll_cache_record: by a thread of the library beside the lookup, or, for a prefix of up to
 * COLL_RECORD_INLINE_BYTES = 64 KB, by a kernel in front of the lookup and the calling thread after it), blocking
 * lookup, and at the configured step a refresh started on a background thread (skipped with a log line while the
 * previous one still runs).  output as in coll_cache_lookup. */
void coll_cache_forward_config(int enable_refresh, uint64_t refresh_iter, double record_fraction, int periodic);
void coll_cache_forward(int replica_id, uint32_t *key, size_t num_keys, void *output, StreamHandle stream);
void coll_cache_forward_i64(int replica_id, const int64_t *key, size_t num_keys, void *output, StreamHandle stream);
/* A serving step that does not block (no counterpart in the reference: LookupManager::forward returns when the
 * lookup has): the lookup is enqueued on `stream` like coll_cache_lookup_async* / coll_cache_lookup_pooled_async* and
 * completed by coll_cache_lookup_wait; the prefix is recorded and the refresh started as in any step.  Where the
 * hotness is counted on the host, a prefix of up to COLL_RECORD_INLINE_BYTES is copied into pinned memory by a kernel
 * on `stream` and counted later — by a later step that finds the copy complete, or by whatever needs the counts (a
 * ranking, coll_cache_lookup_wait, coll_cache_shutdown), which waits for it; a longer prefix makes the step block like
 * coll_cache_forward*, because it is copied out of the caller's key buffer while the step knows that buffer to be
 * alive.  A step that is being recorded into a HIP graph records no prefix. */
void coll_cache_forward_async(int replica_id, const uint32_t *key, size_t num_keys, void *output,
                              StreamHandle stream);
void coll_cache_forward_async_i64(int replica_id, const int64_t *key, size_t num_keys, void *output,
                                  StreamHandle stream);
void coll_cache_forward_pooled_async(int replica_id, const uint32_t *key, const int64_t *seg_off,
                                     const float *weights, size_t num_rows, size_t num_keys, int combiner,
                                     int elem_bytes, void *output, StreamHandle stream);
void coll_cache_forward_pooled_async_i64(int replica_id, const int64_t *key, const int64_t *seg_off,
                                         const float *weights, size_t num_rows, size_t num_keys, int combiner,
                                         int elem_bytes, void *output, StreamHandle stream);
/* 1 while a background refresh started by coll_cache_forward runs */
int coll_cache_forward_refresh_ongoing(void);
/* waits for it; returns the number of refreshes coll_cache_forward has completed so far */
uint64_t coll_cache_forward_join(void);
/* drop every global object so that coll_cache_config may be called again (the reference has no teardown) */
void coll_cache_shutdown(void);

#ifdef __cplusplus
}
#endif
#endif /* COLL_CACHE_C_API_H_ */
