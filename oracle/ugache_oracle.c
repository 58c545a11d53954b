/*
 * TEST INFRASTRUCTURE ONLY — see ugache_oracle.h.  CPU restatement of the reference's
 * embedding-extraction path (coll_cache_lib/ of SJTU-IPADS/ugache); never part of the product.
 */
#include "ugache_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------
 * MurmurHash3_x86_32 as used by the reference (cache_hashtable.cuh:56-135): body over 4-byte
 * blocks, tail switch, "h1 ^= len", fmix32.
 * ------------------------------------------------------------------------------------------ */
static inline uint32_t rotl32(uint32_t x, int r) { return (x << r) | (x >> (32 - r)); }

static inline uint32_t fmix32(uint32_t h) {
  h ^= h >> 16;
  h *= 0x85ebca6bu;
  h ^= h >> 13;
  h *= 0xc2b2ae35u;
  h ^= h >> 16;
  return h;
}

uint32_t orc_murmur3_32_bytes(const void *data_, int len, uint32_t seed) {
  const uint8_t *data = (const uint8_t *)data_;
  const int nblocks = len / 4;
  uint32_t h1 = seed;
  const uint32_t c1 = 0xcc9e2d51u, c2 = 0x1b873593u;
  for (int i = 0; i < nblocks; i++) {
    uint32_t k1;
    memcpy(&k1, data + 4 * i, 4);
    k1 *= c1;
    k1 = rotl32(k1, 15);
    k1 *= c2;
    h1 ^= k1;
    h1 = rotl32(h1, 13);
    h1 = h1 * 5 + 0xe6546b64u;
  }
  const uint8_t *tail = data + nblocks * 4;
  uint32_t k1 = 0;
  switch (len & 3) {
    case 3: k1 ^= (uint32_t)tail[2] << 16; /* fallthrough */
    case 2: k1 ^= (uint32_t)tail[1] << 8;  /* fallthrough */
    case 1:
      k1 ^= tail[0];
      k1 *= c1;
      k1 = rotl32(k1, 15);
      k1 *= c2;
      h1 ^= k1;
  }
  h1 ^= (uint32_t)len;
  return fmix32(h1);
}

uint32_t orc_murmur3_32_u32(uint32_t key, uint32_t seed) { return orc_murmur3_32_bytes(&key, 4, seed); }

/* cache_hashtable.cu:222-225 */
size_t orc_table_size(size_t num, size_t scale) {
  const size_t next_pow2 = (size_t)1 << (size_t)(1 + log2((double)(num >> 1)));
  return next_pow2 << scale;
}

/* cache_hashtable.h:20-28 */
uint32_t orc_pack(uint32_t loc, uint32_t off) { return (loc << 28) + off; }
uint32_t orc_loc(uint32_t p) { return (p >> 28) & 0x0f; }
uint32_t orc_off(uint32_t p) { return p & 0x0fffffffu; }

/* ------------------------------------------------------------------------------------------
 * simple table
 * ------------------------------------------------------------------------------------------ */
void orc_simple_init(orc_bucket_t *table, size_t nbuckets) { memset(table, 0xFF, nbuckets * sizeof(orc_bucket_t)); }

/* HashO2N (cache_hashtable.cuh:211-217): murmur(id) % size, default seed 0 */
static inline uint32_t hash_o2n(uint32_t id, size_t nbuckets) {
  return (uint32_t)(orc_murmur3_32_u32(id, 0) % nbuckets);
}

/* InsertO2N + AttemptInsertAtO2N (cache_hashtable.cu:75-131): walk pos = H(pos + delta), delta = 1,2,..,
 * and take the first bucket whose top bit is set (never used, or tombstoned). */
int orc_simple_insert(orc_bucket_t *table, size_t nbuckets, const uint32_t *keys, const uint32_t *vals, size_t n) {
  for (size_t i = 0; i < n; i++) {
    const uint32_t id = keys[i];
    uint32_t pos = hash_o2n(id, nbuckets);
    uint32_t delta = 1;
    for (;;) {
      const uint32_t old = table[pos].state_key;
      if ((old & 0x80000000u) != 0) {
        table[pos].state_key = id;
        table[pos].val = vals[i];
        break;
      }
      if ((old & 0x7fffffffu) == id) return -1; /* the reference asserts on a duplicate key */
      pos = hash_o2n(pos + delta, nbuckets);
      delta += 1;
    }
  }
  return 0;
}

/* SearchO2N (cache_hashtable.cuh:175-190) */
uint32_t orc_simple_search(const orc_bucket_t *table, size_t nbuckets, uint32_t id) {
  uint32_t pos = hash_o2n(id, nbuckets);
  uint32_t delta = 1;
  while ((table[pos].state_key & 0x7fffffffu) != id) {
    if (table[pos].state_key == ORC_EMPTY_KEY) return ORC_EMPTY_POS;
    pos = hash_o2n(pos + delta, nbuckets);
    delta += 1;
  }
  if (table[pos].state_key & 0x80000000u) return ORC_EMPTY_POS;
  return pos;
}

int orc_simple_evict(orc_bucket_t *table, size_t nbuckets, const uint32_t *keys, size_t n) {
  for (size_t i = 0; i < n; i++) {
    const uint32_t pos = orc_simple_search(table, nbuckets, keys[i]);
    if (pos == ORC_EMPTY_POS) return -1;
    table[pos].state_key |= 0x80000000u;
  }
  return 0;
}

void orc_simple_census(const orc_bucket_t *table, size_t nbuckets, size_t out[3]) {
  out[0] = out[1] = out[2] = 0;
  for (size_t i = 0; i < nbuckets; i++) {
    const uint32_t s = table[i].state_key;
    if (s == ORC_EMPTY_KEY) out[2]++;
    else if (s & 0x80000000u) out[1]++;
    else out[0]++;
  }
}

/* ------------------------------------------------------------------------------------------
 * flat table: one 4-byte value per key of the key space, 0xffffffff = not cached
 * ------------------------------------------------------------------------------------------ */
void orc_flat_init(uint32_t *table, size_t nkeys) { memset(table, 0xFF, nkeys * sizeof(uint32_t)); }
void orc_flat_insert(uint32_t *table, const uint32_t *keys, const uint32_t *vals, size_t n) {
  for (size_t i = 0; i < n; i++) table[keys[i]] = vals[i];
}
void orc_flat_evict(uint32_t *table, const uint32_t *keys, size_t n) {
  for (size_t i = 0; i < n; i++) table[keys[i]] = ORC_EMPTY_POS;
}

/* ------------------------------------------------------------------------------------------
 * lookup -> idx entries
 * ------------------------------------------------------------------------------------------ */
void orc_lookup_src_dst(const orc_bucket_t *simple, size_t nbuckets, const uint32_t *flat, const uint32_t *keys,
                        size_t n, uint32_t fallback_loc, orc_idx_t *idx) {
  for (size_t i = 0; i < n; i++) {
    const uint32_t key = keys[i];
    idx[i].dst_off = (uint32_t)i;
    if (flat) {
      const uint32_t v = flat[key];
      idx[i].src = (v == ORC_EMPTY_POS) ? orc_pack(fallback_loc, key) : v;
    } else {
      const uint32_t pos = orc_simple_search(simple, nbuckets, key);
      idx[i].src = (pos == ORC_EMPTY_POS) ? orc_pack(fallback_loc, key) : simple[pos].val;
    }
  }
}

static int cmp_u64(const void *a, const void *b) {
  uint64_t x, y;
  memcpy(&x, a, 8);
  memcpy(&y, b, 8);
  return (x > y) - (x < y);
}

void orc_sort_idx(orc_idx_t *idx, size_t n) { qsort(idx, n, sizeof(orc_idx_t), cmp_u64); }

void orc_find_boundary(const orc_idx_t *idx, size_t n, int num_location, uint32_t *group_offset) {
  /* GetMissCacheIndex zeroes the array (cache_context.cu:752), SplitGroup sets the last entry (:834) */
  for (int i = 0; i <= num_location; i++) group_offset[i] = 0;
  group_offset[num_location] = (uint32_t)n;
  if (n == 0) return;
  for (size_t i = 0; i < n; i++) {
    const uint32_t loc = orc_loc(idx[i].src);
    if (i == n - 1 || loc != orc_loc(idx[i + 1].src)) group_offset[loc + 1] = (uint32_t)(i + 1);
  }
  for (int i = 1; i < num_location; i++) {
    if (group_offset[i + 1] == 0) group_offset[i + 1] = group_offset[i];
  }
}

void orc_extract_group(const orc_idx_t *idx, size_t n, const void *src, void *out, size_t row_bytes) {
  for (size_t i = 0; i < n; i++) {
    memcpy((char *)out + (size_t)idx[i].dst_off * row_bytes,
           (const char *)src + (size_t)orc_off(idx[i].src) * row_bytes, row_bytes);
  }
}

void orc_extract_mix(const orc_idx_t *idx, size_t n, const void *const *src_by_loc, void *out, size_t row_bytes) {
  for (size_t i = 0; i < n; i++) {
    const char *src = (const char *)src_by_loc[orc_loc(idx[i].src)];
    memcpy((char *)out + (size_t)idx[i].dst_off * row_bytes, src + (size_t)orc_off(idx[i].src) * row_bytes,
           row_bytes);
  }
}

int orc_gather_u32(const void *table, size_t num_rows, const uint32_t *keys, size_t n, void *out, size_t row_bytes) {
  for (size_t i = 0; i < n; i++) {
    if (keys[i] >= num_rows) return -1;
    memcpy((char *)out + i * row_bytes, (const char *)table + (size_t)keys[i] * row_bytes, row_bytes);
  }
  return 0;
}

int orc_gather_i64(const void *table, size_t num_rows, const int64_t *keys, size_t n, void *out, size_t row_bytes) {
  for (size_t i = 0; i < n; i++) {
    if (keys[i] < 0 || (uint64_t)keys[i] >= num_rows) return -1;
    memcpy((char *)out + i * row_bytes, (const char *)table + (size_t)keys[i] * row_bytes, row_bytes);
  }
  return 0;
}

void orc_gather_scatter_u32(const void *table, const uint32_t *keys, const uint32_t *dst, size_t n, void *out,
                            size_t row_bytes) {
  for (size_t i = 0; i < n; i++) {
    memcpy((char *)out + (size_t)dst[i] * row_bytes, (const char *)table + (size_t)keys[i] * row_bytes, row_bytes);
  }
}

void orc_extract_feat(const orc_bucket_t *simple, size_t nbuckets, const uint32_t *flat, const uint32_t *keys,
                      size_t n, const void *cache, const void *host_table, void *out, size_t row_bytes,
                      uint32_t *group_offset_out) {
  uint32_t group_offset[3] = {0, 0, 0};
  if (n > 0) {
    orc_idx_t *idx = (orc_idx_t *)malloc(n * sizeof(orc_idx_t));
    orc_lookup_src_dst(simple, nbuckets, flat, keys, n, /*cpu location*/ 1, idx);
    orc_sort_idx(idx, n);
    orc_find_boundary(idx, n, 2, group_offset);
    /* host group first, then the local group (cache_context.cu:1424-1447) */
    orc_extract_group(idx + group_offset[1], group_offset[2] - group_offset[1], host_table, out, row_bytes);
    orc_extract_group(idx + group_offset[0], group_offset[1] - group_offset[0], cache, out, row_bytes);
    free(idx);
  }
  if (group_offset_out) memcpy(group_offset_out, group_offset, sizeof(group_offset));
}

/* ------------------------------------------------------------------------------------------
 * hotness ranking and placement
 * ------------------------------------------------------------------------------------------ */
static int cmp_u32(const void *a, const void *b) {
  const uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
  return (x > y) - (x < y);
}
static int cmp_u64_desc(const void *a, const void *b) { return -cmp_u64(a, b); }

size_t orc_freq_rank(const uint32_t *stream, size_t n, uint32_t *rank_keys, uint32_t *rank_cnts) {
  if (n == 0) return 0;
  uint32_t *sorted = (uint32_t *)malloc(n * sizeof(uint32_t));
  memcpy(sorted, stream, n * sizeof(uint32_t));
  qsort(sorted, n, sizeof(uint32_t), cmp_u32);
  /* FreqEntry {key, cnt} read as one little-endian uint64 = (cnt << 32) | key (freq_recorder.h:32-35, .cc:275) */
  uint64_t *ent = (uint64_t *)malloc(n * sizeof(uint64_t));
  size_t m = 0;
  for (size_t i = 0; i < n;) {
    size_t j = i;
    while (j < n && sorted[j] == sorted[i]) j++;
    ent[m++] = ((uint64_t)(j - i) << 32) | sorted[i];
    i = j;
  }
  qsort(ent, m, sizeof(uint64_t), cmp_u64_desc);
  for (size_t r = 0; r < m; r++) {
    rank_keys[r] = (uint32_t)(ent[r] & 0xffffffffu);
    rank_cnts[r] = (uint32_t)(ent[r] >> 32);
  }
  free(ent);
  free(sorted);
  return m;
}

uint32_t orc_rep_solve(const uint32_t *rank_keys, uint32_t num_node, double pct100, uint32_t *nid_to_block) {
  const uint32_t num_cached = (uint32_t)(num_node * (pct100 / (double)100));
  for (uint32_t rank = 0; rank < num_node; rank++) nid_to_block[rank_keys[rank]] = (rank < num_cached) ? 0 : 1;
  return num_cached;
}

size_t orc_cache_capacity(size_t num_total_nodes, double cache_percentage) {
  return (size_t)(num_total_nodes * (cache_percentage + 0.001));
}

int orc_refresh_plan(const uint32_t *old_block, const uint32_t *new_block, uint32_t num_node, uint32_t *slot_of,
                     uint32_t *free_list, size_t *n_free, uint32_t *evict_keys, size_t *n_evict,
                     uint32_t *insert_keys, uint32_t *insert_slots, size_t *n_insert) {
  size_t ne = 0, ni = 0, n_old = 0, n_new = 0, n_preserved = 0;
  for (uint32_t k = 0; k < num_node; k++) {
    const int was = old_block[k] == 0, is = new_block[k] == 0;
    n_old += was;
    n_new += is;
    if (is && !was) insert_keys[ni++] = k;
    if (was && !is) evict_keys[ne++] = k;
    if (was && is) n_preserved++;
  }
  /* cache_context.cu:3992  evicted + preserved == old cached */
  if (ne + n_preserved != n_old) return -1;
  /* step 3: offsets of evicted keys go to the back of the free list, then the keys are evicted */
  for (size_t i = 0; i < ne; i++) {
    if (slot_of[evict_keys[i]] == ORC_EMPTY_POS) return -1;
    free_list[(*n_free)++] = slot_of[evict_keys[i]];
    slot_of[evict_keys[i]] = ORC_EMPTY_POS;
  }
  /* cache_context.cu:4010 and the CHECK in ReserveOffsetFront (cache_hashtable.cuh:648: strictly more free than taken) */
  if (ne > *n_free) return -1;
  if (ni > 0) {
    if (!(*n_free > ni)) return -1;
    for (size_t i = 0; i < ni; i++) {
      insert_slots[i] = free_list[i];
      slot_of[insert_keys[i]] = free_list[i];
    }
    memmove(free_list, free_list + ni, (*n_free - ni) * sizeof(uint32_t));
    *n_free -= ni;
  }
  *n_evict = ne;
  *n_insert = ni;
  return 0;
}

/* ------------------------------------------------------------------------------------------
 * dedup, first-occurrence order (a tiny open-addressing set; keys are arbitrary int64)
 * ------------------------------------------------------------------------------------------ */
static inline uint64_t mix64(uint64_t x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdull;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ull;
  x ^= x >> 33;
  return x;
}

int orc_pool_f64(const double *table, size_t num_rows_table, size_t dim, const int64_t *ids, const int64_t *seg_off,
                 const double *weights, size_t n_rows, int combiner, double *out) {
  return orc_pool_clip_f64(table, num_rows_table, dim, ids, seg_off, weights, n_rows, combiner, 0.0, out);
}

/* with max_norm > 0 every looked-up row is first clipped to that l2 norm (clip_by_norm over axis 1, applied to the
 * embeddings before they are weighted: sparse_lookup_layer.py:95-140 hands max_norm to embedding_lookup_sparse):
 * x * max_norm / max(||x||, max_norm) */
int orc_pool_clip_f64(const double *table, size_t num_rows_table, size_t dim, const int64_t *ids,
                      const int64_t *seg_off, const double *weights, size_t n_rows, int combiner, double max_norm,
                      double *out) {
  for (size_t r = 0; r < n_rows; ++r) {
    double *o = out + r * dim;
    double den = 0.0;
    for (size_t c = 0; c < dim; ++c) o[c] = 0.0;
    for (int64_t j = seg_off[r]; j < seg_off[r + 1]; ++j) {
      if (ids[j] < 0 || (uint64_t)ids[j] >= num_rows_table) return 1;
      double w = weights ? weights[j] : 1.0;
      const double *x = table + (size_t)ids[j] * dim;
      den += combiner == 2 ? w * w : w; /* the denominator is made of the weights alone */
      if (max_norm > 0.0) {
        double ss = 0.0;
        for (size_t c = 0; c < dim; ++c) ss += x[c] * x[c];
        const double norm = sqrt(ss);
        w *= max_norm / (norm > max_norm ? norm : max_norm);
      }
      for (size_t c = 0; c < dim; ++c) o[c] += w * x[c];
    }
    if (combiner == 0) continue;
    if (combiner == 2) den = sqrt(den);
    for (size_t c = 0; c < dim; ++c) o[c] = den != 0.0 ? o[c] / den : 0.0;
  }
  return 0;
}

size_t orc_dedup_i64(const int64_t *keys, size_t n, int64_t *unique, uint32_t *inverse) {
  size_t cap = 16;
  while (cap < 2 * n) cap <<= 1;
  uint32_t *slot = (uint32_t *)malloc(cap * sizeof(uint32_t)); /* index into unique, or EMPTY */
  memset(slot, 0xFF, cap * sizeof(uint32_t));
  size_t nu = 0;
  for (size_t i = 0; i < n; i++) {
    size_t p = mix64((uint64_t)keys[i]) & (cap - 1);
    for (;;) {
      if (slot[p] == 0xffffffffu) {
        slot[p] = (uint32_t)nu;
        unique[nu] = keys[i];
        inverse[i] = (uint32_t)nu;
        nu++;
        break;
      }
      if (unique[slot[p]] == keys[i]) {
        inverse[i] = slot[p];
        break;
      }
      p = (p + 1) & (cap - 1);
    }
  }
  free(slot);
  return nu;
}

/* ------------------------------------------------------------------------------------------
 * CPU baseline: the gather, parallel over keys
 * ------------------------------------------------------------------------------------------ */
int orc_omp_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

int orc_gather_u32_omp(const void *table, size_t num_rows, const uint32_t *keys, size_t n, void *out,
                       size_t row_bytes) {
  int bad = 0;
#pragma omp parallel for schedule(static) reduction(| : bad)
  for (size_t i = 0; i < n; i++) {
    if (keys[i] >= num_rows) {
      bad |= 1;
      continue;
    }
    memcpy((char *)out + i * row_bytes, (const char *)table + (size_t)keys[i] * row_bytes, row_bytes);
  }
  return bad ? -1 : 0;
}

int orc_gather_i64_omp(const void *table, size_t num_rows, const int64_t *keys, size_t n, void *out,
                       size_t row_bytes) {
  int bad = 0;
#pragma omp parallel for schedule(static) reduction(| : bad)
  for (size_t i = 0; i < n; i++) {
    if (keys[i] < 0 || (uint64_t)keys[i] >= num_rows) {
      bad |= 1;
      continue;
    }
    memcpy((char *)out + i * row_bytes, (const char *)table + (size_t)keys[i] * row_bytes, row_bytes);
  }
  return bad ? -1 : 0;
}

/* The CPU form of the whole mixed-source step, one pass per key: id -> row (identity, or the inverse of the sparse-id
 * map), flat-table lookup (LookupHelper over the flat table, cache_hashtable.cuh:233-237, 480-503), source chosen per
 * row and copied (DataIterMixLoc, cache_context.cu:137-159, 195-231).  count_out[0] / [1] = rows taken from the cache
 * copy / from the host table. */
int orc_extract_flat_i64_omp(const uint32_t *flat, size_t num_rows, uint64_t key_inv, uint64_t key_mask,
                             const int64_t *keys, size_t n, const void *cache, size_t cache_rows, const void *host_table,
                             void *out, size_t row_bytes, uint64_t count_out[2]) {
  int bad = 0;
  uint64_t n_local = 0, n_host = 0;
#pragma omp parallel for schedule(static) reduction(| : bad) reduction(+ : n_local, n_host)
  for (size_t i = 0; i < n; i++) {
    uint64_t row = (uint64_t)keys[i];
    if (key_inv != 0) row = row <= key_mask ? (row * key_inv) & key_mask : ~(uint64_t)0;
    if (row >= num_rows) {
      bad |= 1;
      continue;
    }
    const uint32_t v = flat[row];
    const char *src;
    if (v != ORC_EMPTY_POS && orc_loc(v) == 0) {
      if (orc_off(v) >= cache_rows) {
        bad |= 1;
        continue;
      }
      src = (const char *)cache + (size_t)orc_off(v) * row_bytes;
      n_local++;
    } else {
      src = (const char *)host_table + (size_t)row * row_bytes;
      n_host++;
    }
    memcpy((char *)out + i * row_bytes, src, row_bytes);
  }
  if (count_out) count_out[0] = n_local, count_out[1] = n_host;
  return bad ? -1 : 0;
}
