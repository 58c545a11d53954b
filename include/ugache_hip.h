/*
 * ugache_hip.h — the thin C-ABI over the hand-written gfx950 kernels of the embedding-extraction path.
 *
 * Everything above this header (the coll_cache_lib-compatible facade, CacheContext, ExtractSession,
 * RefreshSession, the collcache Python package) is host code that never includes a HIP header: it sees
 * plain pointers, sizes and opaque `void*` streams/events.  Each entry point names the piece of the
 * reference (SJTU-IPADS/ugache, paths relative to its root) whose job it takes over.
 *
 * Conventions
 *   - every function returns 0 on success, non-zero on failure; ugk_last_error() then describes it
 *     (thread-local, valid until the next failing call on the same thread);
 *   - all launches are asynchronous on `stream` (NULL = the null stream) unless stated otherwise;
 *   - `status_dev` is a device word the kernels OR error bits into instead of faulting (UGK_ST_*);
 *   - `host_mirror` (per-batch entry points only, may be NULL) points at 4 words of pinned host memory that
 *     the kernels write with ordinary stores so the caller needs no device-to-host copy after its one
 *     synchronisation: [0] = non-zero if any error bit was raised (details are in status_dev),
 *     [1] / [2] = size of the local / host group as seen by ugk_gather_group; the caller clears [0];
 *   - pointers named *_dev must be device-accessible (HBM, or pinned host memory from ugk_host_malloc).
 */
#ifndef UGACHE_HIP_H_
#define UGACHE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status bits written by kernels -------------------------------------------------------------- */
#define UGK_ST_KEY_OUT_OF_RANGE 0x1u /* a key / source row index beyond the source's row count: row skipped */
#define UGK_ST_TABLE_FULL 0x2u       /* hash insert found no free bucket */
#define UGK_ST_DUP_KEY 0x4u          /* insert of a key that is already present (the reference asserts) */
#define UGK_ST_EVICT_ABSENT 0x8u     /* evict of a key that is not present */
#define UGK_ST_BAD_SEGMENT 0x10u     /* pooled extraction: offsets that leave [0, nnz], run backwards or do not span [0, nnz] */
#define UGK_ST_PLACE_PROMISE 0x20u   /* ugk_rank_place_observed: k or more rows were observed; nothing was placed */

/* element code of the pooled extraction for bfloat16 rows (fp32 and fp16 are named by their size, 4 and 2) */
#define UGK_ELEM_BF16 0x102

/* ---- locations (cache_context.cu:2421-2422: GPUs are 0..G-1, the host is G; here G = 1) ---------- */
#define UGK_LOC_LOCAL 0u
#define UGK_LOC_HOST 1u
#define UGK_EMPTY_U32 0xffffffffu /* cache_hashtable.h:17 kEmptyPos */

/* One gather work item.  Takes the place of SrcKeyDstVal (cache_context.h:47-52); the location is not
 * stored because every group holds one location only.
 * Both fields are 32 bits, as in the reference: an index list addresses outputs of up to 2^32 rows and sources of up
 * to 2^32 rows.  ugk_classify_* therefore flags (UGK_ST_KEY_OUT_OF_RANGE) a key whose host row does not fit 32 bits
 * instead of listing it, so the factored extraction (ugk_classify_* + ugk_gather_group) serves host tables of up to
 * 2^32 rows; ugk_extract_mix_* and ugk_gather_direct_i64 carry 64-bit rows and have no such limit. */
typedef struct {
  uint32_t dst_off; /* output row */
  uint32_t src_off; /* row inside the group's source (cache slot, or host row) */
} ugk_idx_t;

/* Bucket of the open-addressing table.  Takes the place of BucketO2N (cache_hashtable.h:44-49) with a
 * 64-bit key and a 32-bit offset so sparse 2^40 ids and > 2^28 rows fit. */
typedef struct {
  uint64_t key;  /* UGK_HASH_EMPTY = never used, UGK_HASH_TOMB = evicted */
  uint32_t off;  /* row inside the location */
  uint32_t meta; /* bit 31 = valid, bits 0..3 = location */
} ugk_bucket_t;
#define UGK_HASH_EMPTY 0xffffffffffffffffull
#define UGK_HASH_TOMB 0xfffffffffffffffeull
#define UGK_META_VALID 0x80000000u

/* Lookup table handle passed by value to kernels.
 * kind 0: none (direct mapping, cache_context.h:309-317 IsDirectMapping)
 * kind 1: flat  — uint32 per key of the key space, (loc << 28) + off, 0xffffffff = absent
 *                 (DeviceFlatHashTable, cache_hashtable.cuh:224-251)
 * kind 2: hash  — ugk_bucket_t[size], linear probing (replaces DeviceSimpleHashTable, cuh:154-222)
 * kind 3: compact hash — uint64[size] (size a multiple of 16, 128-byte aligned), one word per entry: low half the ROW
 *                 of the host table the key stands for (the key itself when fb_mul == 0, else (key * fb_mul) & fb_mask:
 *                 a bijection, so 32 bits identify the key), high half (loc << 28) + off as in the flat table; all ones
 *                 = never used, low half 0xfffffffe = evicted.  Same 8-byte entry as BucketO2N (cache_hashtable.h:44-49)
 *                 with sixteen of them probed per 128-byte line; needs rows below 0xfffffffe and slots below 2^28.
 *                 Every ugk_* call that takes a table takes the caller's keys for it, whatever the kind. */
#define UGK_TABLE_FLAT 1
#define UGK_TABLE_HASH 2
#define UGK_TABLE_HASH32 3
typedef struct {
  int32_t kind;
  int32_t reserved;
  void *table;
  uint64_t size; /* flat: number of keys; hash: number of buckets (kind 3: of 8-byte entries) */
  /* host row of a key the table does not hold: key itself when fb_mul == 0 (the reference's CPUFallback,
   * cache_hashtable.cuh:388-395), else (key * fb_mul) & fb_mask — the inverse of an odd-multiplier bijection on
   * 2^k ids, which lets sparse hashed ids address a dense host table without a second table */
  uint64_t fb_mul;
  uint64_t fb_mask;
} ugk_table_t;

typedef struct {
  char name[256];
  char arch[64];
  int32_t compute_units;
  int32_t wavefront_size;
  uint64_t total_mem;
  uint64_t lds_per_block;
} ugk_device_info_t;

const char *ugk_last_error(void);
/* version of this ABI; bumped on any signature change.  ugk_abi_version() is what the loaded library was built with:
 * a caller compiled against another UGK_ABI_VERSION must not go on. */
#define UGK_ABI_VERSION 22
int ugk_abi_version(void);

/* ---- runtime plumbing: Device::{AllocDataSpace,FreeDataSpace,CopyDataFromTo,StreamSync,CreateStream}
 *      (device.h:35-65; cuda/cuda_device.cc:36-135) ---------------------------------------------- */
int ugk_device_count(int *count);
int ugk_set_device(int dev);
int ugk_get_device_info(int dev, ugk_device_info_t *info);
int ugk_mem_info(size_t *free_bytes, size_t *total_bytes);
int ugk_malloc(void **ptr, size_t nbytes);
int ugk_free(void *ptr);
/* pinned, GPU-mapped host memory (the reference page-locks the caller's table with cudaHostRegister,
 * facade.cc:476; this platform needs the table to be allocated pinned instead) */
int ugk_host_malloc(void **ptr, size_t nbytes);
int ugk_host_free(void *ptr);
/* kind: 0 = ordinary host memory (kernels cannot read it), 1 = pinned host, 2 = device */
int ugk_pointer_kind(const void *ptr, int *kind);
int ugk_stream_create(void **stream);
/* stream whose kernels run on `num_cus` compute units only (the counterpart of the reference's SM-masked contexts
 * for the host source, mps_util.h:36-49 / cache_context.cu:4208-4218); default priority */
int ugk_stream_create_cu_masked(void **stream, int num_cus);
int ugk_stream_destroy(void *stream);
int ugk_stream_sync(void *stream);
/* *capturing = 1 while work enqueued on `stream` is being recorded into a HIP graph instead of being run, 0 when it
 * runs, UGK_CAPTURE_QUERY_REFUSED when the runtime refuses the question (the legacy default stream while another
 * stream of the process records in global mode: work enqueued on `stream` would be refused as well) */
#define UGK_CAPTURE_QUERY_REFUSED 2
int ugk_stream_is_capturing(void *stream, int *capturing);
/* ugk_stream_sync for callers that wait for short launches: enqueues a one-lane kernel that writes `value` into
 * *ticket_host (pinned host word from ugk_host_malloc) behind everything already enqueued on `stream`, and polls that
 * word from the host for up to spin_us microseconds before it falls back to waiting for the stream.  The word changes a
 * few microseconds before a wait for the stream would return (262,144-row gather: 49.7 against 53.3 us per launch +
 * wait).  `value` must differ from what the word holds (a counter).  What kernels enqueued before the ticket wrote into
 * pinned host memory is visible once the ticket is. */
int ugk_stream_sync_ticket(void *stream, uint32_t *ticket_host, uint32_t value, unsigned spin_us);
/* The same wait with a few device words brought along: one launch behind everything enqueued on `stream` copies
 * a_dev[0 .. n_a) and b_dev[0 .. n_b) (either may be NULL with a count of 0; n_a + n_b <= 63) to dst_host[1 ...] and
 * then writes `value` to dst_host[0]; the host polls dst_host[0] as above.  dst_host: pinned host words from
 * ugk_host_malloc, 1 + n_a + n_b of them.  For status words at the end of a sequence of launches: one launch and no
 * copy call, where a copy into pageable memory and a wait for the stream take two calls into the runtime. */
int ugk_words_to_host_ticket(const uint32_t *a_dev, unsigned n_a, const uint32_t *b_dev, unsigned n_b,
                             uint32_t *dst_host, uint32_t value, unsigned spin_us, void *stream);
/* The first launch of a kernel of one of this library's source files loads that file's code object onto the current
 * device, which takes 5 - 11 ms each the first time (a first gather of 51 MB: 12.4 ms, the second 0.9 ms).  This call
 * launches an empty kernel of every file on a stream of its own and waits for them, so that no later call pays; a
 * host library can make it from a helper thread while it is busy on the CPU. */
int ugk_preload_kernels(void);
int ugk_device_sync(void);
int ugk_event_create(void **event);
int ugk_event_destroy(void *event);
int ugk_event_record(void *event, void *stream);
int ugk_event_sync(void *event);
/* *complete = 1 if the work in front of the event's last record has finished, else 0; never waits */
int ugk_event_query(void *event, int *complete);
int ugk_stream_wait_event(void *stream, void *event);
int ugk_event_elapsed_ms(void *start, void *stop, float *ms);
/* async copy, direction inferred from the pointers */
int ugk_memcpy_async(void *dst, const void *src, size_t nbytes, void *stream);
/* fill kernel (not a memset node, so it is safe to capture and replay) */
int ugk_fill_u32(uint32_t *dst_dev, uint32_t value, size_t nwords, void *stream);
/* iota: cuda_utils.cu:29-34 arrange_array */
int ugk_arange_u32(uint32_t *dst_dev, uint32_t start, size_t n, void *stream);
/* streaming device copy used to calibrate counters and to measure the attainable HBM rate */
int ugk_copy_rows(void *dst_dev, const void *src_dev, size_t nbytes, void *stream);

/* ---- gather: extract_data + Combine (cache_context.cu:214-231, 1076-1100) -----------------------
 * out[dst(i), :] = src[srcrow(i), :] for row_bytes bytes.  max_blocks = 0 lets the kernel fill the
 * chip; a non-zero value caps the grid (the reference's limit_block / per-source SM budget). */
/* Where the rows an extraction writes go next, for the launches the calling thread makes from now on (the gathers and
 * ugk_extract_mix_*).  UGK_OUTPUT_AUTO: decided by size — an output of up to 192 MB is written with ordinary stores and
 * stays in the 256 MB memory-side cache for its consumer, a larger one with non-temporal stores.  UGK_OUTPUT_STREAMS:
 * non-temporal stores whatever the size (a caller that rotates its outputs over more buffers than the cache holds: the
 * rows of one launch are evicted by the next anyway, and evicting them costs more than streaming them, 51.4 us against
 * 47.5 us for 262,144 rows of 512 bytes).  UGK_OUTPUT_STAYS: ordinary stores whatever the size.  Never a byte of the
 * result depends on it.  The environment variable UGK_GATHER_NT_STORE=0/1 overrides both. */
#define UGK_OUTPUT_AUTO 0
#define UGK_OUTPUT_STREAMS 1
#define UGK_OUTPUT_STAYS 2
int ugk_set_output_hint(int hint);
/* IdxStoreDirect (cache_context.h:341-354): srcrow = keys[i], dst = i */
int ugk_gather_direct_u32(const void *src_dev, uint64_t src_rows, const uint32_t *keys_dev, size_t n, void *out_dev,
                          size_t row_bytes, unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror,
                          void *stream);
int ugk_gather_direct_i64(const void *src_dev, uint64_t src_rows, const int64_t *keys_dev, size_t n, void *out_dev,
                          size_t row_bytes, unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror,
                          void *stream);
/* IdxStoreDst (cache_context.h:356-361): srcrow = keys[i], dst = dst_off[i] (cache fill / refresh insert) */
int ugk_gather_scatter_u32(const void *src_dev, uint64_t src_rows, const uint32_t *keys_dev,
                           const uint32_t *dst_off_dev, size_t n, void *out_dev, uint64_t out_rows, size_t row_bytes,
                           unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror, void *stream);
int ugk_gather_scatter_i64(const void *src_dev, uint64_t src_rows, const int64_t *keys_dev,
                           const uint32_t *dst_off_dev, size_t n, void *out_dev, uint64_t out_rows, size_t row_bytes,
                           unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror, void *stream);
/* re-expansion after a deduplicated extraction: for every i whose representative r = rep_dev[inverse_dev[i]] differs
 * from i, out[i, :] = out[r, :] (rows r were written by the gathers, rows i are their duplicates) */
int ugk_replicate_rows(void *out_dev, size_t row_bytes, const uint32_t *inverse_dev, const uint32_t *rep_dev, size_t n,
                       void *stream);
/* CombineOneGroup with DataIterPerLoc<IdxStoreCompact> (cache_context.cu:195-212, 855-859).
 * The group is idx[begin, begin+count) where, with c = counts_dev (written by ugk_classify_*):
 *   group UGK_LOC_LOCAL: begin = 0,            count = c[0]
 *   group UGK_LOC_HOST : begin = n - c[1],     count = c[1]
 * so no host round trip is needed between classify and gather.  n is the number of classified keys (grid upper
 * bound), out_rows the rows of the output (n, or more when classify ran with a destination map). */
int ugk_gather_group(const void *src_dev, uint64_t src_rows, const ugk_idx_t *idx_dev, const uint32_t *counts_dev,
                     uint32_t group, size_t n, void *out_dev, uint64_t out_rows, size_t row_bytes,
                     unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror, void *stream);
/* same with an explicit list (count known on the host) */
int ugk_gather_idx(const void *src_dev, uint64_t src_rows, const ugk_idx_t *idx_dev, size_t count, void *out_dev,
                   size_t row_bytes, unsigned max_blocks, uint32_t *status_dev, void *stream);

/* ---- lookup tables -------------------------------------------------------------------------------
 * flat: FlatHashTable ctor memset 0xFF (cache_hashtable.cu:588-607) is ugk_fill_u32(table, 0xffffffff, nkeys). */
/* number of buckets for n entries at the given load factor (replaces TableSize, cache_hashtable.cu:222-225) */
size_t ugk_hash_buckets_for(size_t n_entries, double load_factor);
int ugk_hash_init(ugk_bucket_t *table_dev, size_t nbuckets, void *stream);
/* the same for a table of any kind: entries of a compact table (kind 3) for n keys at the given load factor, a multiple
 * of 16; every entry of `t` set to "never used" / "absent"; the census of ugk_hash_census for kind 2 or 3 */
size_t ugk_hash32_entries_for(size_t n_entries, double load_factor);
int ugk_table_init(ugk_table_t t, void *stream);
int ugk_table_census(ugk_table_t t, uint64_t *census_dev, void *stream);
/* insert_hashmap_unique + InsertWithLoc / InsertSeqOffWithLoc (cache_hashtable.cu:249-268;
 * cache_hashtable.cuh:601-608): value = (loc, offs ? offs[i] : seq_base + i).  Keys must be unique and absent. */
int ugk_table_insert_u32(ugk_table_t t, const uint32_t *keys_dev, const uint32_t *offs_dev, uint32_t seq_base,
                         uint32_t loc, size_t n, uint32_t *status_dev, void *stream);
int ugk_table_insert_i64(ugk_table_t t, const int64_t *keys_dev, const uint32_t *offs_dev, uint32_t seq_base,
                         uint32_t loc, size_t n, uint32_t *status_dev, void *stream);
/* evict_hashmap_unique (cache_hashtable.cu:269-308) */
int ugk_table_evict_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint32_t *status_dev, void *stream);
int ugk_table_evict_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint32_t *status_dev, void *stream);
/* the same, and the bit of the cache slot every evicted key held is cleared in slot_bits_dev (one bit per slot, nslots
 * bits): what LookupOffset + ReturnOffset + Evict do to the free list (cache_context.cu:4005-4020), in the one kernel that
 * has the bucket in its hands anyway */
int ugk_table_evict_release_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint64_t *slot_bits_dev,
                                uint64_t nslots, uint32_t *status_dev, void *stream);
int ugk_table_evict_release_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint64_t *slot_bits_dev,
                                uint64_t nslots, uint32_t *status_dev, void *stream);
/* LookupValCustom with SepLocOffset (cache_hashtable.cuh:420-434): loc_out/off_out per key; a miss gives
 * (fallback_loc, (uint32)key).  Either output may be NULL (OffsetOnly, cuh:396-407). */
int ugk_table_lookup_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint32_t fallback_loc,
                         uint32_t *loc_out_dev, uint32_t *off_out_dev, void *stream);
int ugk_table_lookup_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint32_t fallback_loc,
                         uint32_t *loc_out_dev, uint32_t *off_out_dev, void *stream);
/* CountEntries (cache_hashtable.cu:742-777): census_dev[3] = occupied, tombstoned, never used */
int ugk_hash_census(const ugk_bucket_t *table_dev, size_t nbuckets, uint64_t *census_dev, void *stream);

/* ---- classify + partition by source ---------------------------------------------------------------
 * Replaces GetMissCacheIndex + CubSortDispatcher + SplitGroup/find_boundary
 * (cache_context.cu:702-761, 825-847; cub_sort_wrapper.cuh:472-486) with ONE kernel:
 * per key a table lookup (one probe per lane, wavefront-cooperative continuation on collisions), then a
 * wavefront-ballot prefix scan and LDS-staged compaction into idx_dev[0..n):
 *   local hits  fill idx[0, c[0])          as {dst_off = i, src_off = cache slot}
 *   host misses fill idx[n - c[1], n)      as {dst_off = i, src_off = host row = key}
 * counts_dev[0..1] (one 8-byte aligned word) must be zero on entry; the kernel also zeroes next_counts_dev[0..1] (may be NULL) so a
 * caller can rotate two counter pairs and never launch a memset.  host_rows bounds the miss offsets.
 * A key found with a location other than local/host sets UGK_ST_KEY_OUT_OF_RANGE (one GPU has two sources).
 * dst_map_dev (may be NULL): output row of key i is dst_map_dev[i] instead of i (deduplicated extraction: the keys
 * are the distinct ones, their output rows the first occurrences). */
int ugk_classify_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint64_t host_rows, const uint32_t *dst_map_dev,
                     ugk_idx_t *idx_dev, uint32_t *counts_dev, uint32_t *next_counts_dev, uint32_t *status_dev,
                     uint32_t *host_mirror, void *stream);
int ugk_classify_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint64_t host_rows, const uint32_t *dst_map_dev,
                     ugk_idx_t *idx_dev, uint32_t *counts_dev, uint32_t *next_counts_dev, uint32_t *status_dev,
                     uint32_t *host_mirror, void *stream);

/* ---- the keys the cache does not serve: the COLL_SKIP_LOCAL pre-filter of GetMissCacheIndex
 *      (cache_context.cu:728-741: CubSelectIndex with CubSelectOpLocIsNot, then SelectArrayByIdx) ---------------------
 * ugk_nonlocal_flags_*: bit i of flags_dev (ceil(n / 64) words, every word written) = key i is not found in the table
 * with the local location (it is found with the host's, or not at all).  The ascending positions of the set bits come
 * from ugk_bitmap_count + ugk_bitmap_emit (below), which is the reference's stable select; ugk_select_keys_*:
 * out_dev[j] = keys_dev[sel_dev[j]] for j < m. */
int ugk_nonlocal_flags_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint64_t *flags_dev, void *stream);
int ugk_nonlocal_flags_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint64_t *flags_dev, void *stream);
int ugk_select_keys_u32(const uint32_t *keys_dev, const uint32_t *sel_dev, size_t m, uint32_t *out_dev, void *stream);
int ugk_select_keys_i64(const int64_t *keys_dev, const uint32_t *sel_dev, size_t m, int64_t *out_dev, void *stream);

/* ---- single-kernel mixed-source extraction: kDirectNoGroup with DataIterMixLoc
 *      (cache_context.cu:137-159, 1295-1329): lookup and gather fused, source picked per row ----------
 * group_counts_host (may be NULL): pinned, GPU-mapped host memory (ugk_host_malloc) of ugk_extract_mix_max_groups()
 * 8-byte words.  Workgroup b leaves in word b, for the keys it handled, (rows not taken from the cache << 32) | rows
 * taken from the cache — a posted write nobody waits for.  *num_groups_host (ordinary host memory, written by the call
 * itself before it returns, may be NULL) = the number of workgroups launched: once the stream has been waited for,
 * the sum of that many words gives the group sizes ugk_gather_group reports on the factored path.  Rows skipped for
 * a key without a row (status_dev flagged) are counted with the host rows.  n must stay below 2^32.
 * others_hint: how many of the n rows will NOT come from the cache, where the caller knows (a batch of keys selected
 * for being non-local, say), UGK_HINT_UNKNOWN where it does not.  Only the launch shape depends on it (at half the rows
 * or more, and rows of 512 bytes or more, the grid is capped to 128 workgroups: the host link takes rows faster from a
 * few workgroups than from a chip full of them, and a batch that mostly hits would be three times slower on so few, so
 * a guess is worse than no hint), never a byte of the result. */
#define UGK_HINT_UNKNOWN 0xffffffffu
unsigned ugk_extract_mix_max_groups(void);
int ugk_extract_mix_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, const void *cache_dev, uint64_t cache_rows,
                        const void *host_dev, uint64_t host_rows, void *out_dev, size_t row_bytes,
                        uint32_t *status_dev, uint32_t *host_mirror, uint64_t *group_counts_host,
                        uint32_t *num_groups_host, uint32_t others_hint, void *stream);
int ugk_extract_mix_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, const void *cache_dev, uint64_t cache_rows,
                        const void *host_dev, uint64_t host_rows, void *out_dev, size_t row_bytes,
                        uint32_t *status_dev, uint32_t *host_mirror, uint64_t *group_counts_host,
                        uint32_t *num_groups_host, uint32_t others_hint, void *stream);

/* ---- pooled extraction: lookup + per-sample combination of a multi-hot feature in one kernel ---------------------
 * The reference's sparse layer looks the distinct ids up and hands the rows to embedding_lookup_sparse
 * (python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:196-265: unique -> lookup -> gather -> weighted
 * segment sum / mean / sqrtn).  Here the rows of segment r, ids_dev[seg_off_dev[r] .. seg_off_dev[r + 1]), are read
 * from where they live (table t, cache_dev, host_dev as for ugk_extract_mix_*; t.kind 0 = no table: row = id, read from
 * host_dev, which may be HBM) and combined on the way:
 *   out[r, :] = sum_j w_j x_j                                   combiner 0 (sum)
 *             = sum_j w_j x_j / sum_j w_j                       combiner 1 (mean)
 *             = sum_j w_j x_j / sqrt(sum_j w_j^2)               combiner 2 (sqrtn)
 * with w_j = weights_dev[j] (1 when weights_dev is NULL), a zero denominator giving a zero row (div_no_nan), an empty
 * segment a zero row.  Elements are fp32 (elem_bytes 4), fp16 (2) or bfloat16 (UGK_ELEM_BF16: two bytes as well) and
 * are added in fp32 in the order of the ids, one
 * fused multiply-add each; the output has the element type of the rows.  The nnz x row_bytes intermediate of a lookup
 * followed by a segment sum is never written.  seg_off_dev: n_rows + 1 ascending offsets into ids_dev, the last one
 * nnz.  row_bytes: a multiple of 16, at most 4096.  Status, host mirror and the per-workgroup count words are those of
 * ugk_extract_mix_* (the counts are of ids, not of output rows).  An id without a row sets UGK_ST_KEY_OUT_OF_RANGE and
 * adds nothing; a segment whose offsets leave [0, nnz] or run backwards sets UGK_ST_BAD_SEGMENT, reads no id and
 * gives a zero row; offsets that do not begin at 0 or do not end at nnz set the same bit (the rows are computed as the
 * offsets say, but the counts of ids per source then do not add up to nnz). */
/* The offsets ugk_extract_pool_* takes, from the row of every entry of a sparse feature in row-major order (the
 * indices[:, 0] of the SparseTensor of sparse_lookup_layer.py:196-265): seg_off_dev[r] = number of entries whose row is
 * below r, for r = 0 .. n_rows (n_rows + 1 words; rows without an entry get empty segments).  One launch, no
 * synchronisation.  Entries that are out of order or outside [0, n_rows) set UGK_ST_BAD_SEGMENT (status_dev and
 * host_mirror may be NULL) and leave words of seg_off_dev unwritten. */
int ugk_segment_offsets_i64(const int64_t *sorted_rows_dev, size_t nnz, size_t n_rows, int64_t *seg_off_dev,
                            uint32_t *status_dev, uint32_t *host_mirror, void *stream);
int ugk_extract_pool_u32(ugk_table_t t, const uint32_t *ids_dev, const int64_t *seg_off_dev, const float *weights_dev,
                         size_t n_rows, uint64_t nnz, int combiner, int elem_bytes, const void *cache_dev,
                         uint64_t cache_rows, const void *host_dev, uint64_t host_rows, void *out_dev, size_t row_bytes,
                         uint32_t *status_dev, uint32_t *host_mirror, uint64_t *group_counts_host,
                         uint32_t *num_groups_host, void *stream);
int ugk_extract_pool_i64(ugk_table_t t, const int64_t *ids_dev, const int64_t *seg_off_dev, const float *weights_dev,
                         size_t n_rows, uint64_t nnz, int combiner, int elem_bytes, const void *cache_dev,
                         uint64_t cache_rows, const void *host_dev, uint64_t host_rows, void *out_dev, size_t row_bytes,
                         uint32_t *status_dev, uint32_t *host_mirror, uint64_t *group_counts_host,
                         uint32_t *num_groups_host, void *stream);

/* The same with every looked-up row clipped to the l2 norm max_norm before it is weighted (the max_norm of the sparse
 * layer, sparse_lookup_layer.py:95-140: x * max_norm / max(||x||_2, max_norm), norms summed in fp32); max_norm = 0:
 * no clipping, exactly ugk_extract_pool_*. */
int ugk_extract_pool_clip_u32(ugk_table_t t, const uint32_t *ids_dev, const int64_t *seg_off_dev,
                              const float *weights_dev, size_t n_rows, uint64_t nnz, int combiner, int elem_bytes,
                              float max_norm, const void *cache_dev, uint64_t cache_rows, const void *host_dev,
                              uint64_t host_rows, void *out_dev, size_t row_bytes, uint32_t *status_dev,
                              uint32_t *host_mirror, uint64_t *group_counts_host, uint32_t *num_groups_host,
                              void *stream);
int ugk_extract_pool_clip_i64(ugk_table_t t, const int64_t *ids_dev, const int64_t *seg_off_dev,
                              const float *weights_dev, size_t n_rows, uint64_t nnz, int combiner, int elem_bytes,
                              float max_norm, const void *cache_dev, uint64_t cache_rows, const void *host_dev,
                              uint64_t host_rows, void *out_dev, size_t row_bytes, uint32_t *status_dev,
                              uint32_t *host_mirror, uint64_t *group_counts_host, uint32_t *num_groups_host,
                              void *stream);

/* ---- rows that crossed the host link once, kept where a refresh finds them ---------------------------------------
 * The rows a refresh inserts (RefreshSession::refresh_after_solve_new, cache_context.cu:4054-4090: rows copied host ->
 * HBM in throttled batches) are rows recent lookups missed, i.e. rows that have just crossed the host link into some
 * lookup's output.  A stage is a direct-mapped set of such rows in HBM: entry h = fmix64(row) & mask holds the bytes of
 * the host row named by the low 32 bits of owner[h] whenever the high 32 bits (the tag of the launch that wrote it) are
 * non-zero.  ugk_extract_mix_staged_* is ugk_extract_mix_* that also files every row it takes from the host table in the
 * stage (first writer of a launch wins an entry; `epoch` must be non-zero and differ from launch to launch);
 * ugk_gather_scatter_staged_u32 is ugk_gather_scatter_u32 out of the host table that takes a row from the stage when it
 * is there, and adds the number of such rows to *staged_dev (device word, may be NULL).  With rest_count_dev (device
 * word, zero on entry; NULL = off) the rows the stage does not hold are not copied but listed, in any order, as
 * rest_rows_dev[j] / rest_dst_off_dev[j] for j < *rest_count_dev (lists of n words each): a background refresh copies
 * those itself, throttled, over the host link.  With done_count_dev as well (device word, zero on entry; needs the
 * rest lists) the rows that were copied out of the stage are listed too, from the back of the same lists:
 * rest_rows_dev[n - 1 - j] / rest_dst_off_dev[n - 1 - j] for j < *done_count_dev, so that a caller can publish them
 * in its table before the rest has arrived.  Results are the same
 * bytes with and without a stage: the host table does not change under a cache.  An entry is only consistent at launch
 * boundaries, so the staged gather must not read a stage that an extraction in flight writes (a caller with lookups
 * running beside its refreshes keeps two stages and reads the one the lookups have been switched away from).  For the
 * same reason two staged extractions that may run at the same time (launches on different streams with nothing that
 * orders them) must not share a stage: both could claim one entry and interleave the 16-byte stores of two different
 * rows under an owner word that names one of them.  Launches on one stream are ordered and may share it.
 * rows_dev: (mask + 1) x row_bytes bytes; owner_dev: mask + 1 words, zero-filled once; host rows must fit 32 bits. */
typedef struct {
  void *rows_dev;
  uint64_t *owner_dev;
  uint64_t mask;  /* entries - 1, entries a power of two */
  uint32_t epoch; /* launch tag, non-zero (ignored by the gather) */
  uint32_t reserved;
} ugk_stage_t;
int ugk_extract_mix_staged_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, const void *cache_dev,
                               uint64_t cache_rows, const void *host_dev, uint64_t host_rows, void *out_dev,
                               size_t row_bytes, uint32_t *status_dev, uint32_t *host_mirror,
                               uint64_t *group_counts_host, uint32_t *num_groups_host, uint32_t others_hint,
                               ugk_stage_t stage, void *stream);
int ugk_extract_mix_staged_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, const void *cache_dev,
                               uint64_t cache_rows, const void *host_dev, uint64_t host_rows, void *out_dev,
                               size_t row_bytes, uint32_t *status_dev, uint32_t *host_mirror,
                               uint64_t *group_counts_host, uint32_t *num_groups_host, uint32_t others_hint,
                               ugk_stage_t stage, void *stream);
int ugk_gather_scatter_staged_u32(const void *host_dev, uint64_t host_rows, const uint32_t *rows_dev,
                                  const uint32_t *dst_off_dev, size_t n, void *out_dev, uint64_t out_rows,
                                  size_t row_bytes, ugk_stage_t stage, unsigned max_blocks, uint32_t *status_dev,
                                  uint32_t *staged_dev, uint32_t *rest_rows_dev, uint32_t *rest_dst_off_dev,
                                  uint32_t *rest_count_dev, uint32_t *done_count_dev, void *stream);

/* ---- key dedup (the caller-side array_ops.unique of
 *      python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:197) ------------------------
 * unique_out[0..*n_unique) = distinct keys (order unspecified), inverse_out[i] = position of keys[i] in it.
 * workspace_dev: workspace_bytes >= ugk_dedup_workspace_bytes(n) bytes, zero-filled once at allocation and then
 * reused as is by batches of any size up to the one it was sized for (slots are epoch-tagged, so no per-call
 * clearing; the layout inside depends on workspace_bytes only, which must therefore be the same on every call that
 * shares the workspace); epoch must be non-zero and different on every such call.  n_unique_dev must be zero on entry.
 * rep_out_dev (may be NULL): rep_out_dev[u] = index of the first occurrence that introduced unique key u.
 * n_unique_host (may be NULL): pinned host word that receives *n_unique_dev when the second kernel runs. */
size_t ugk_dedup_workspace_bytes(size_t n);
int ugk_dedup_u32(const uint32_t *keys_dev, size_t n, void *workspace_dev, size_t workspace_bytes, uint32_t epoch,
                  uint32_t *unique_out_dev, uint32_t *inverse_out_dev, uint32_t *rep_out_dev, uint32_t *n_unique_dev,
                  uint32_t *n_unique_host, void *stream);
int ugk_dedup_i64(const int64_t *keys_dev, size_t n, void *workspace_dev, size_t workspace_bytes, uint32_t epoch,
                  int64_t *unique_out_dev, uint32_t *inverse_out_dev, uint32_t *rep_out_dev, uint32_t *n_unique_dev,
                  uint32_t *n_unique_host, void *stream);

/* The same deduplication for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The slot set and the per-occurrence ids,
 * which ugk_dedup_* take from workspace_dev, live in a static device array of the library (20 MiB + 320 bytes on every
 * GPU the library runs on, held until the process ends), and so does the epoch tag, which the call advances itself on
 * the device: every launch of the call, also a replay of a captured one, sees a fresh tag.  The call makes no
 * hipMalloc / hipFree and no allocating library call; *n_unique_dev is cleared by the call (an output, not an in/out).
 * key_bytes: 4 (uint32 keys) or 8 (int64 keys).  n may not exceed UGK_DEDUP_STATIC_MAX_KEYS: larger batches are
 * refused with an error.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
 * streams, or threads) race and give wrong results; calls ordered one after the other, on any streams, are fine.
 * The first call on a device looks the array's address up (hipGetSymbolAddress): make that call outside a capture. */
#define UGK_DEDUP_STATIC_MAX_KEYS (1u << 20)
int ugk_dedup_static(const void *keys_dev, uint32_t key_bytes, size_t n, void *unique_out_dev,
                     uint32_t *inverse_out_dev, uint32_t *rep_out_dev, uint32_t *n_unique_dev, uint32_t *n_unique_host,
                     void *stream);

/* ---- hotness counters on the device: FreqRecorder::Record (freq_recorder.cc:227-253) without the copy of the keys
 *      to the host, the record thread of python_tf2/collcache_tf2/collcache_tf2/core/lookup_manager.cc:291-312 ----
 * counts_dev: one uint32 per row of the host table, zero-filled once.  ugk_record_*: counts_dev[row(key)] += 1 for
 * every key of the batch; row(key) = key for dense ids (key_inv = 0), else (key * key_inv) & key_mask, the inverse of
 * the sparse-id map (the fb_mul / fb_mask of ugk_table_t).  A key without a row sets UGK_ST_KEY_OUT_OF_RANGE and is
 * not counted. */
/* observed_dev (may be NULL): one bit per row, ceil(num_rows / 64) words, zero-filled once; the bit of a row is set
 * when its counter leaves zero, so the bitmap is "counter above zero" at every launch boundary.  ugk_record_drain
 * clears the bits of the counters it resets; ugk_rank_place reads it to skip its passes over the counters. */
int ugk_record_u32(const uint32_t *keys_dev, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts_dev,
                   uint64_t num_rows, uint64_t *observed_dev, uint32_t *status_dev, uint32_t *host_mirror,
                   void *stream);
int ugk_record_i64(const int64_t *keys_dev, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts_dev,
                   uint64_t num_rows, uint64_t *observed_dev, uint32_t *status_dev, uint32_t *host_mirror,
                   void *stream);
/* hands rows [first_row, first_row + num_rows) to the host: every non-zero counter becomes one word
 * (count << 32) | row in entries_dev (order unspecified; the layout of the reference's FreqEntry {key, cnt},
 * freq_recorder.h:32-40) and is reset to zero in the same atomic step, so a ugk_record_* running concurrently loses
 * nothing.  At most `capacity` entries are written; counters that did not fit stay as they are.
 * n_entries_dev: device word, zero on first use, left zero.  host_out: two pinned host words,
 * [0] = entries written, [1] = 1 when rows were left over (call again). */
int ugk_record_drain(uint32_t *counts_dev, uint64_t first_row, uint64_t num_rows, uint64_t *observed_dev,
                     uint64_t *entries_dev, uint32_t capacity, uint32_t *n_entries_dev, uint32_t *host_out,
                     void *stream);
/* the way back: counts_dev[row] += count for the n words (count << 32) | row of entries_dev (rows need not be distinct),
 * with the observed bit of every row whose counter leaves zero.  What a cache was built from (the ranking of a
 * presample, FreqRecorder::Sort's list, freq_recorder.cc:275-281) thereby becomes the device-side counters' starting
 * point.  A row outside [0, num_rows) sets UGK_ST_KEY_OUT_OF_RANGE and is skipped. */
int ugk_record_restore(const uint64_t *entries_dev, size_t n, uint32_t *counts_dev, uint64_t num_rows,
                       uint64_t *observed_dev, uint32_t *status_dev, void *stream);

/* ---- re-placement on the device, from the counters of ugk_record_* ---------------------------------------------
 * Stands, for hotness counted on the device, for the host passes of a refresh: FreqRecorder::Sort
 * (freq_recorder.cc:275-281), RepSolver::Solve (optimal_solver_class.cc:1869-1924) and the key-list scans
 * DetectKeysForAllSource / DetectKeysWithCond (cache_hashtable.cuh:693-835) behind
 * RefreshSession::refresh_after_solve_new (cache_context.cu:3944-4107).
 * Rank of row r with counter c: c > 0: (c << 32) | r;  c == 0: 0xffffffff - r  (never-counted rows rank behind all
 * counted ones, in ascending row order).  All ranks are distinct.
 * ugk_rank_place: bit r of in_new_dev (ceil(num_rows / 64) words, every word written) = row r is one of the k
 * best-ranked rows of [0, num_rows) (k == 0: no row; k >= num_rows: every row).  Two streaming passes over the
 * counters (five when the k-th best count is 2047 or more) and a few launches over bitmaps; no host round trip.
 * With reset_counts == 0 the first pass also splits the rows by the k-th best count of the placement that used ws_dev
 * last, and when that count still is the k-th best (counters that are kept only grow, it moves slowly) the second
 * pass is skipped: one pass over the counters, 0.47 against 0.87 ms at 500 M rows.  The result does not depend on
 * what ws_dev held; give the placements of one cache one workspace.
 * counts_dev must be 16-byte aligned; num_rows < 2^32 - 1; ws_dev: ugk_rank_workspace_bytes() bytes, 8-byte aligned;
 * scratch_bitmap_dev: as large as in_new_dev, overwritten.  With reset_counts != 0 the counters (and observed_dev)
 * are zeroed on the way.  observed_dev (may be NULL): the bitmap ugk_record_* keeps; when fewer rows were observed
 * than k asks for, the k-th best count is 0 without looking and no pass over the counters is made at all.
 * ugk_rank_place_keep: the same with keep_dev (may be NULL: then it is ugk_rank_place), a bitmap of rows that win
 * ties: among the rows whose counter equals the k-th best count, those with their bit in keep_dev come first, and
 * inside either group the order above holds.  With keep_dev = the rows cached now, a refresh moves no row whose
 * hotness does not tell it apart from the row it would replace (a cache filled from a ranking the counters do not know,
 * or wider than the set of rows observed so far, otherwise trades its never-counted rows for the lowest-numbered
 * ones).  keep_dev is read only and may not be one of the two output bitmaps; ugk_rank_threshold reports the last row
 * taken from the group that was cut.
 * ugk_rank_place_observed: the placement for a caller that knows that fewer than k rows were observed (say, the rows
 * observed at the last placement plus the keys counted since stay below k), 0 < k < num_rows: in_new = every observed
 * row and the lowest k - |observed| never-observed rows, what ugk_rank_place computes in that case, in four launches
 * over the bitmaps and none over the counters.  If k or more rows turn out to be observed, UGK_ST_PLACE_PROMISE is set
 * in *status_dev and in_new_dev is left as it was.  counts_dev may be NULL when reset_counts is 0 (only the bitmap is
 * read then: "observed" can be any set of rows that are in for sure).  cached_dev (may be NULL; then evict_ws_dev, insert_ws_dev and
 * totals_host may be NULL too): the rows cached now; the rows that leave (cached & ~in_new) and that come in
 * (in_new & ~cached) are counted in the same pass: evict_ws_dev / insert_ws_dev (ugk_bitmap_workspace_bytes() each)
 * are left as ugk_bitmap_count(cached, in_new) / ugk_bitmap_count(in_new, cached) would leave them, ready for
 * ugk_bitmap_emit, and totals_host (three pinned words) receives [0] rows leaving, [1] rows coming in, [2] rows
 * observed (before a reset).
 * ugk_rank_threshold: copies the rank of the k-th best row of the last ugk_rank_place to the host (blocking; for tests
 * and logs; all ones for k == 0, zero for k >= num_rows). */
size_t ugk_rank_workspace_bytes(void);
int ugk_rank_place(uint32_t *counts_dev, uint64_t num_rows, uint64_t k, void *ws_dev, uint64_t *in_new_dev,
                   uint64_t *scratch_bitmap_dev, uint64_t *observed_dev, int reset_counts, void *stream);
int ugk_rank_place_keep(uint32_t *counts_dev, uint64_t num_rows, uint64_t k, void *ws_dev, uint64_t *in_new_dev,
                        uint64_t *scratch_bitmap_dev, uint64_t *observed_dev, const uint64_t *keep_dev,
                        int reset_counts, void *stream);
int ugk_rank_place_observed(uint32_t *counts_dev, uint64_t num_rows, uint64_t k, void *ws_dev, uint64_t *in_new_dev,
                            uint64_t *observed_dev, int reset_counts, const uint64_t *cached_dev, void *evict_ws_dev,
                            void *insert_ws_dev, uint32_t *totals_host, uint32_t *status_dev, void *stream);
int ugk_rank_threshold(const void *ws_dev, uint64_t *threshold_host, void *stream);
/* Ordered compaction over bitmaps.  The set S = { p < nbits : bit p of m is set }, m = (invert_a ? ~a : a) & ~b
 * (b_dev may be NULL).  ugk_bitmap_count writes |S| to *total_host (pinned host word, may be NULL) and leaves the
 * per-chunk offsets in ws_dev (ugk_bitmap_workspace_bytes() bytes); ugk_bitmap_emit, called with the same a, b,
 * invert_a and nbits while the bitmaps are unchanged, writes the first max_out elements of S in ascending order.
 * With these, evict = cached & ~new, insert = new & ~cached and free slots = ~used are the same three launches
 * (the set algebra of cache_context.cu:3975-4003).  nbits <= 2^32 - 1. */
size_t ugk_bitmap_workspace_bytes(void);
int ugk_bitmap_count(const uint64_t *a_dev, const uint64_t *b_dev, int invert_a, uint64_t nbits, void *ws_dev,
                     uint32_t *total_host, void *stream);
int ugk_bitmap_emit(const uint64_t *a_dev, const uint64_t *b_dev, int invert_a, uint64_t nbits, const void *ws_dev,
                    uint32_t *out_dev, uint64_t max_out, void *stream);
/* ugk_bitmap_count(a, b, 0, ..., ws_ab) and ugk_bitmap_count(b, a, 0, ..., ws_ba) in one pass over the two bitmaps:
 * totals_host (two pinned words, may be NULL) receives [0] |a & ~b| and [1] |b & ~a| */
int ugk_bitmap_count_diff(const uint64_t *a_dev, const uint64_t *b_dev, uint64_t nbits, void *ws_ab_dev,
                          void *ws_ba_dev, uint32_t *totals_host, void *stream);
/* both differences of two bitmaps in one pass: a & ~b to out_ab_dev and b & ~a to out_ba_dev, each exactly what
 * ugk_bitmap_emit(a, b, 0, ...) / ugk_bitmap_emit(b, a, 0, ...) writes, from the workspaces ugk_bitmap_count(a, b) and
 * ugk_bitmap_count(b, a) (or ugk_rank_place_observed) left.  A list with a maximum of 0 is not written. */
int ugk_bitmap_emit_diff(const uint64_t *a_dev, const uint64_t *b_dev, uint64_t nbits, const void *ws_ab_dev,
                         const void *ws_ba_dev, uint32_t *out_ab_dev, uint64_t max_ab, uint32_t *out_ba_dev,
                         uint64_t max_ba, void *stream);
/* sets (set != 0) or clears the bits listed in idx_dev; a position >= nbits flags UGK_ST_KEY_OUT_OF_RANGE */
int ugk_bitmap_update(uint64_t *bitmap_dev, uint64_t nbits, const uint32_t *idx_dev, size_t n, int set,
                      uint32_t *status_dev, void *stream);
/* sets every bit up to and including position *last_pos_dev (device word): after the lowest free slots have been taken,
 * the last of them being *last_pos_dev, that is what ReserveOffsetFront (cache_hashtable.cuh:647-655) did to the slot
 * bitmap; a position >= nbits flags UGK_ST_KEY_OUT_OF_RANGE and changes nothing */
int ugk_bitmap_set_through(uint64_t *bitmap_dev, uint64_t nbits, const uint32_t *last_pos_dev, uint32_t *status_dev,
                           void *stream);
/* sparse-id mode: caller-side id of each listed host row, (row * mul) & mask (the inverse of the map ugk_table_t
 * carries in fb_mul / fb_mask) */
int ugk_rows_to_keys(const uint32_t *rows_dev, size_t n, uint64_t mul, uint64_t mask, int64_t *keys_out_dev,
                     void *stream);

#ifdef __cplusplus
}
#endif
#endif /* UGACHE_HIP_H_ */
