/*
 * TEST INFRASTRUCTURE ONLY — the CPU oracle of the embedding-extraction path.
 *
 * A plain-C restatement of what the reference (SJTU-IPADS/ugache, directory
 * coll_cache_lib/) computes on the path
 *     keys -> (source, offset) lookup -> group by source -> per-source gather
 * and of the placement / refresh bookkeeping that feeds it.  Nothing shipped may
 * link or call this library: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py do, and only as the checker.
 *
 * Every function names the reference file:line it follows.  The reference holds
 * no golden vectors or unit tests for this path, so each function is pinned by
 * tests/test_oracle_*.py against an independent definition:
 *   orc_murmur3_32_u32   – the published smhasher known answers for MurmurHash3_x86_32
 *   orc_table_size       – closed form 2^floor(1+log2(n/2)) << scale on hand-worked cases
 *   orc_simple_* / flat  – dict-model invariants (found-after-insert, miss-after-evict, bucket census)
 *   orc_lookup_src_dst   – Python dict restatement of the hit/miss rule
 *   orc_sort_idx         – numpy.sort on the packed 64-bit words
 *   orc_find_boundary    – numpy.bincount / cumsum
 *   orc_extract_* / orc_gather_*  – numpy.take and a brute-force loop
 *   orc_freq_rank        – numpy.unique + lexsort on (count desc, key desc)
 *   orc_rep_solve, orc_cache_capacity – closed forms on hand-worked cases
 *   orc_refresh_plan     – Python set algebra and free-list conservation
 *   orc_dedup            – numpy.unique(return_inverse=True)
 *   orc_pool_f64         – numpy.add.at over float64 rows, and hand-worked segments
 *   orc_pool_clip_f64    – hand-worked rows on either side of the norm (3-4-5 triangles), numpy.linalg.norm
 *   orc_extract_flat_i64_omp – numpy.where / numpy.take over a cache copy that differs from the host rows, a
 *                              brute-force modular inverse for the sparse ids
 * No function here is "parity unpinned".
 */
#ifndef UGACHE_ORACLE_H_
#define UGACHE_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_EMPTY_KEY 0xffffffffu /* constant.h:83 kEmptyKey */
#define ORC_EMPTY_POS 0xffffffffu /* cache_hashtable.h:17 kEmptyPos */

/* cache_hashtable.h:44-49 BucketO2N, 8 bytes */
typedef struct {
  uint32_t state_key;
  uint32_t val; /* EmbCacheOff: (loc << 28) + off, cache_hashtable.h:20-28 */
} orc_bucket_t;

/* cache_context.h:47-52 SrcKeyDstVal, 8 bytes, little endian word = (src << 32) | dst */
typedef struct {
  uint32_t dst_off;
  uint32_t src; /* EmbCacheOff */
} orc_idx_t;

/* cache_hashtable.cuh:56-135  MurmurHash3_32<IdType> for one 4-byte key */
uint32_t orc_murmur3_32_u32(uint32_t key, uint32_t seed);
/* same routine for an arbitrary byte string (used only to check the known answers) */
uint32_t orc_murmur3_32_bytes(const void *data, int len, uint32_t seed);

/* cache_hashtable.cu:222-225 TableSize */
size_t orc_table_size(size_t num, size_t scale);

/* cache_hashtable.h:20-28 EmbCacheOff */
uint32_t orc_pack(uint32_t loc, uint32_t off);
uint32_t orc_loc(uint32_t packed);
uint32_t orc_off(uint32_t packed);

/* ---- "simple" open-addressing table: cache_hashtable.cuh:154-222, cache_hashtable.cu:52-131 ---- */
/* table must hold orc_table_size(n, 2) buckets; init = memset 0xFF (cache_hashtable.cu:432-457) */
void orc_simple_init(orc_bucket_t *table, size_t nbuckets);
/* InsertO2N applied key by key; returns 0, or -1 when a key is already present (the reference asserts) */
int orc_simple_insert(orc_bucket_t *table, size_t nbuckets, const uint32_t *keys, const uint32_t *vals, size_t n);
/* SearchO2N: bucket position or ORC_EMPTY_POS */
uint32_t orc_simple_search(const orc_bucket_t *table, size_t nbuckets, uint32_t key);
/* evict_hashmap_unique (cache_hashtable.cu:269-288): state_key |= 0x80000000; -1 if a key is absent */
int orc_simple_evict(orc_bucket_t *table, size_t nbuckets, const uint32_t *keys, size_t n);
/* CountEntries (cache_hashtable.cu:742-777): occupied / tombstoned / never used */
void orc_simple_census(const orc_bucket_t *table, size_t nbuckets, size_t out[3]);

/* ---- "flat" direct-indexed table: cache_hashtable.cuh:224-251, cache_hashtable.cu:289-308 ---- */
void orc_flat_init(uint32_t *table, size_t nkeys);
void orc_flat_insert(uint32_t *table, const uint32_t *keys, const uint32_t *vals, size_t n);
void orc_flat_evict(uint32_t *table, const uint32_t *keys, size_t n);

/* LookupSrcDst + LookupHelper (cache_hashtable.cuh:480-503, 583-594):
 * idx[i] = { dst_off = i, src = hit ? bucket val : (fallback_loc, key) }.
 * Exactly one of simple / flat is non-NULL. */
void orc_lookup_src_dst(const orc_bucket_t *simple, size_t nbuckets, const uint32_t *flat,
                        const uint32_t *keys, size_t n, uint32_t fallback_loc, orc_idx_t *idx);

/* CubSortKeyInPlace<uint64_t> over all 64 bits (cub_sort_wrapper.cuh:222-249, cache_context.cu:743-749):
 * ascending order of (src << 32 | dst) == order (loc, src_off, dst_off). */
void orc_sort_idx(orc_idx_t *idx, size_t n);

/* SplitGroup + find_boundary (cache_context.cu:376-396, 825-847): group_offset[0..num_location] */
void orc_find_boundary(const orc_idx_t *idx, size_t n, int num_location, uint32_t *group_offset);

/* CombineOneGroup -> extract_data with DataIterPerLoc<IdxStoreCompact> (cache_context.cu:195-231, 855-859) */
void orc_extract_group(const orc_idx_t *idx, size_t n, const void *src, void *out, size_t row_bytes);
/* DataIterMixLoc (cache_context.cu:137-159): per-row source chosen from src_by_loc[loc] */
void orc_extract_mix(const orc_idx_t *idx, size_t n, const void *const *src_by_loc, void *out, size_t row_bytes);

/* direct mapping fast path, IdxStoreDirect (cache_context.h:341-354; cache_context.cu:1199-1231).
 * Single-threaded statement; returns -1 if any key >= num_rows. */
int orc_gather_u32(const void *table, size_t num_rows, const uint32_t *keys, size_t n, void *out, size_t row_bytes);
int orc_gather_i64(const void *table, size_t num_rows, const int64_t *keys, size_t n, void *out, size_t row_bytes);
/* scatter form used by the refresh insert, IdxStoreDst (cache_context.h:356-361) */
void orc_gather_scatter_u32(const void *table, const uint32_t *keys, const uint32_t *dst, size_t n, void *out,
                            size_t row_bytes);

/* whole ExtractFeat for one GPU + host (cache_context.cu:1330-1344, 1405-1465):
 * lookup -> sort -> boundary -> gather host group, gather local group.
 * local_loc = 0, cpu_loc = 1.  group_offset_out (3 words) may be NULL. */
void orc_extract_feat(const orc_bucket_t *simple, size_t nbuckets, const uint32_t *flat, const uint32_t *keys,
                      size_t n, const void *cache, const void *host_table, void *out, size_t row_bytes,
                      uint32_t *group_offset_out);

/* FreqRecorder::Record + GlobalCombine + Sort (freq_recorder.cc:227-293):
 * count every key of the stream, order entries by the 64-bit word (cnt << 32 | key), descending.
 * rank_keys / rank_cnts need room for n entries; returns the number of distinct keys. */
size_t orc_freq_rank(const uint32_t *stream, size_t n, uint32_t *rank_keys, uint32_t *rank_cnts);

/* RepSolver::Solve (optimal_solver_class.cc:1869-1924): the first
 * (IdType)(num_node * (pct100 / 100.0)) ranks go to block 0 (cached), the rest to block 1 (host).
 * rank_keys must list all num_node keys.  Returns the number of cached keys. */
uint32_t orc_rep_solve(const uint32_t *rank_keys, uint32_t num_node, double pct100, uint32_t *nid_to_block);

/* cache_context.cu:2473  _cache_space_capacity = (size_t)(num_total_nodes * (cache_percentage + 0.001)) */
size_t orc_cache_capacity(size_t num_total_nodes, double cache_percentage);

/* refresh_after_solve_new steps 1-3 and 6 (cache_context.cu:3944-4107) for one GPU, with key lists
 * taken in ascending key order:
 *   new_local = { k : new_block[k] == 0 },  insert = new_local \ old_local,  evict = old_cached \ new_local
 *   free list: evicted offsets appended at the back (ReturnOffset, cache_hashtable.cuh:635-640),
 *              inserted keys take offsets from the front (ReserveOffsetFront, :647-655).
 * slot_of[k] = current slot of cached key k (or ORC_EMPTY_POS); updated in place.
 * free_list has room for `capacity` entries, *n_free is updated.
 * evict_keys / insert_keys / insert_slots need room for num_node entries.
 * Returns 0, or -1 when an invariant of the reference's CHECKs fails. */
int orc_refresh_plan(const uint32_t *old_block, const uint32_t *new_block, uint32_t num_node, uint32_t *slot_of,
                     uint32_t *free_list, size_t *n_free, uint32_t *evict_keys, size_t *n_evict,
                     uint32_t *insert_keys, uint32_t *insert_slots, size_t *n_insert);

/* caller-side dedup (python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:197 array_ops.unique):
 * unique keys in first-occurrence order and inverse[i] = position of keys[i] in unique.  Returns #unique. */
size_t orc_dedup_i64(const int64_t *keys, size_t n, int64_t *unique, uint32_t *inverse);

/* The per-sample combination that follows a sparse lookup (embedding_lookup_sparse as called by
 * python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:196-265), in double precision:
 * out[r, :] = sum over j in [seg_off[r], seg_off[r + 1]) of w_j * table[ids[j], :] (w_j = 1 when weights is NULL),
 * divided by sum w_j (combiner 1, "mean") or sqrt(sum w_j^2) (combiner 2, "sqrtn"); a zero denominator gives a zero
 * row (div_no_nan).  table: [num_rows_table, dim] doubles.  Returns non-zero if an id is out of range. */
int orc_pool_f64(const double *table, size_t num_rows_table, size_t dim, const int64_t *ids, const int64_t *seg_off,
                 const double *weights, size_t n_rows, int combiner, double *out);

/* the same with every looked-up row clipped to the l2 norm max_norm before it is weighted (max_norm <= 0: no clipping):
 * x * max_norm / max(||x||_2, max_norm), the clip_by_norm that embedding_lookup_sparse applies when the layer is given
 * max_norm (sparse_lookup_layer.py:95-140, 264) */
int orc_pool_clip_f64(const double *table, size_t num_rows_table, size_t dim, const int64_t *ids,
                      const int64_t *seg_off, const double *weights, size_t n_rows, int combiner, double max_norm,
                      double *out);

/* ---- CPU baseline leg (bench.py only): the same gather as orc_gather_*, OpenMP over keys ---- */
int orc_omp_threads(void);
int orc_gather_u32_omp(const void *table, size_t num_rows, const uint32_t *keys, size_t n, void *out,
                       size_t row_bytes);
int orc_gather_i64_omp(const void *table, size_t num_rows, const int64_t *keys, size_t n, void *out,
                       size_t row_bytes);

/* the mixed-source step of the CPU baseline: per key, id -> row (row = key when key_inv == 0, else
 * (key * key_inv) & key_mask), lookup in the flat table of the whole row space (ORC_EMPTY_POS or a packed
 * (location, slot) with location 0 = the cache copy), then memcpy of the row from the cache copy or from the host
 * table; OpenMP over keys.  count_out (may be NULL): rows taken from the cache copy / from the host table.
 * Returns -1 if a key has no row or a slot lies outside the cache copy. */
int orc_extract_flat_i64_omp(const uint32_t *flat, size_t num_rows, uint64_t key_inv, uint64_t key_mask,
                             const int64_t *keys, size_t n, const void *cache, size_t cache_rows, const void *host_table,
                             void *out, size_t row_bytes, uint64_t count_out[2]);

#ifdef __cplusplus
}
#endif
#endif
