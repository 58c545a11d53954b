// TEST INFRASTRUCTURE ONLY: a plain CPU model of the ugk_* C-ABI of include/ugache_hip.h.
//
// It exists so that the host library (ugache_amd/coll_cache_lib/*.cc) can be linked into one executable without a GPU
// and run under AddressSanitizer / UBSan and, separately, ThreadSanitizer: the library's own threads (lookups, the
// record stream, foreground and background refreshes, the serving loop) then run against "device memory" that is
// ordinary host memory.  It is never built into the package, never loaded by it and is no fallback: the product's
// libcoll_cache.so links libugache_hip.so only.
//
// Model: every call runs to completion inside the calling thread (a stream is a token, waiting for one is a no-op), so
// the order the library enqueues work in is the order it runs in.  Words that kernels touch with atomics on the GPU
// (table entries, buckets, counters, bitmap words, status words) are touched with atomics here; rows are
// copied with memcpy.  A refresh that overwrote a cache slot a lookup on another thread might still read would
// therefore show up as a data race under ThreadSanitizer, which is what the hand-shake between the two is there to
// prevent.  Layouts follow the header where it fixes them (flat entries, ugk_bucket_t, index records, bitmaps); the
// probe sequence of the hash table and the order of lists the header calls unspecified are this model's own.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "ugache_hip.h"

namespace {

thread_local char g_err[512];
int fail(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}
#define REQUIRE(c, ...) \
  do {                  \
    if (!(c)) return fail(__VA_ARGS__); \
  } while (0)

std::mutex g_mem_mu;
std::map<uintptr_t, std::pair<size_t, int>> g_blocks;  // base -> (bytes, kind)

int alloc_block(void **ptr, size_t nbytes, int kind) {
  void *p = nullptr;
  const size_t bytes = (std::max<size_t>(nbytes, 1) + 255) / 256 * 256;
  if (posix_memalign(&p, 256, bytes) != 0) return fail("out of memory (%zu bytes)", nbytes);
  memset(p, 0xA5, bytes);  // fresh device memory holds no particular value
  std::lock_guard<std::mutex> g(g_mem_mu);
  g_blocks[(uintptr_t)p] = {bytes, kind};
  *ptr = p;
  return 0;
}
int free_block(void *ptr, int kind) {
  if (!ptr) return 0;
  {
    std::lock_guard<std::mutex> g(g_mem_mu);
    auto it = g_blocks.find((uintptr_t)ptr);
    if (it == g_blocks.end() || it->second.second != kind) return fail("free of a pointer that was not allocated here");
    g_blocks.erase(it);
  }
  free(ptr);
  return 0;
}

// Loads acquire and stores release: what a kernel wrote before it published a word (a row copied into a slot before
// its key went into the table, by an earlier launch on the GPU) is visible to whoever reads that word.
template <typename T>
T ld(const T *p) {
  return __atomic_load_n(p, __ATOMIC_ACQUIRE);
}
template <typename T>
void st(T *p, T v) {
  __atomic_store_n(p, v, __ATOMIC_RELEASE);
}
void or_status(uint32_t *status, uint32_t bits, uint32_t *mirror = nullptr) {
  __atomic_fetch_or(status, bits, __ATOMIC_RELAXED);
  if (mirror) st(mirror, bits);
}

uint64_t fmix64(uint64_t x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdull;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ull;
  x ^= x >> 33;
  return x;
}
uint64_t k64(uint32_t k) { return k; }
uint64_t k64(int64_t k) { return (uint64_t)k; }
uint64_t fallback_row(const ugk_table_t &t, uint64_t key) {
  if (t.fb_mul == 0) return key;
  return key <= t.fb_mask ? ((key * t.fb_mul) & t.fb_mask) : ~0ull;
}

constexpr uint32_t kH32Tomb = 0xfffffffeu;
constexpr uint64_t kH32EmptyWord = ~0ull, kH32TombWord = 0x00000000fffffffeull;
uint64_t h32_home(uint64_t row, uint64_t nentries) {
  return (uint64_t)(((unsigned __int128)fmix64(row) * (nentries >> 4)) >> 64) << 4;
}

struct Found {
  bool hit;
  uint32_t loc, off;
};
Found lookup(const ugk_table_t &t, uint64_t key) {
  Found f{false, 0, 0};
  if (t.kind == 1) {
    if (key < t.size) {
      const uint32_t v = ld(reinterpret_cast<const uint32_t *>(t.table) + key);
      if (v != UGK_EMPTY_U32) f = Found{true, (v >> 28) & 0xfu, v & 0x0fffffffu};
    }
  } else if (t.kind == 2) {
    const ugk_bucket_t *b = reinterpret_cast<const ugk_bucket_t *>(t.table);
    uint64_t pos = fmix64(key) % t.size;
    for (uint64_t step = 0; step < t.size; ++step) {
      const uint64_t cur = ld(&b[pos].key);
      if (cur == key) {
        const uint64_t om = ld(reinterpret_cast<const uint64_t *>(&b[pos].off));
        const uint32_t meta = (uint32_t)(om >> 32);
        if (meta & UGK_META_VALID) f = Found{true, meta & 0xfu, (uint32_t)om};
        return f;
      }
      if (cur == UGK_HASH_EMPTY) return f;
      if (++pos == t.size) pos = 0;
    }
  } else if (t.kind == 3) {
    // 8-byte entries {row, (loc << 28) + off}, keyed by the row the key stands for; probing starts at a 16-entry line
    const uint64_t row = fallback_row(t, key);
    if (row >= kH32Tomb) return f;
    const uint64_t *w = reinterpret_cast<const uint64_t *>(t.table);
    uint64_t pos = h32_home(row, t.size);
    for (uint64_t step = 0; step < t.size; ++step) {
      const uint64_t cur = ld(w + pos);
      if ((uint32_t)cur == (uint32_t)row) {
        const uint32_t v = (uint32_t)(cur >> 32);
        return Found{true, (v >> 28) & 0xfu, v & 0x0fffffffu};
      }
      if (cur == kH32EmptyWord) return f;
      if (++pos == t.size) pos = 0;
    }
  }
  return f;
}
int check_table(const ugk_table_t &t, const char *who) {
  REQUIRE(t.kind >= 1 && t.kind <= 3, "%s: table kind %d is not flat(1), hash(2) or compact hash(3)", who, t.kind);
  REQUIRE(t.table && t.size, "%s: empty table", who);
  if (t.kind == 2) REQUIRE(t.size % 8 == 0 && (uintptr_t)t.table % 128 == 0, "%s: hash table layout", who);
  if (t.kind == 3) REQUIRE(t.size % 16 == 0 && (uintptr_t)t.table % 128 == 0, "%s: compact hash table layout", who);
  return 0;
}

void copy_row(void *dst, const void *src, size_t bytes) { memcpy(dst, src, bytes); }

template <typename K>
int gather_direct(const void *src, uint64_t src_rows, const K *keys, const uint32_t *dst, size_t n, void *out,
                  uint64_t out_rows, size_t rb, uint32_t *status, uint32_t *mirror) {
  if (n == 0) return 0;
  REQUIRE(src && out && keys && status, "gather: null pointer");
  for (size_t i = 0; i < n; ++i) {
    const uint64_t s = k64(keys[i]), d = dst ? dst[i] : i;
    if (s >= src_rows || d >= out_rows) {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE, mirror);
      continue;
    }
    copy_row((char *)out + d * rb, (const char *)src + s * rb, rb);
  }
  return 0;
}

int gather_list(const void *src, uint64_t src_rows, const ugk_idx_t *idx, size_t count, void *out, uint64_t out_rows,
                size_t rb, uint32_t *status, uint32_t *mirror) {
  for (size_t i = 0; i < count; ++i) {
    if (idx[i].src_off >= src_rows || idx[i].dst_off >= out_rows) {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE, mirror);
      continue;
    }
    copy_row((char *)out + (size_t)idx[i].dst_off * rb, (const char *)src + (size_t)idx[i].src_off * rb, rb);
  }
  return 0;
}

template <typename K>
int table_insert(ugk_table_t t, const K *keys, const uint32_t *offs, uint32_t seq_base, uint32_t loc, size_t n,
                 uint32_t *status) {
  if (n == 0) return 0;
  if (check_table(t, "ugk_table_insert")) return 1;
  REQUIRE(keys && status && loc < 16, "ugk_table_insert: bad argument");
  for (size_t i = 0; i < n; ++i) {
    const uint64_t key = k64(keys[i]);
    const uint32_t off = offs ? offs[i] : seq_base + (uint32_t)i;
    if (t.kind == 1) {
      if (key >= t.size || off > 0x0fffffffu) {
        or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
        continue;
      }
      const uint32_t old = __atomic_exchange_n(reinterpret_cast<uint32_t *>(t.table) + key, (loc << 28) + off,
                                               __ATOMIC_ACQ_REL);
      if (old != UGK_EMPTY_U32) or_status(status, UGK_ST_DUP_KEY);
      continue;
    }
    if (t.kind == 3) {
      const uint64_t row = fallback_row(t, key);
      if (row >= kH32Tomb || off > 0x0fffffffu) {
        or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
        continue;
      }
      uint64_t *w = reinterpret_cast<uint64_t *>(t.table);
      uint64_t pos = h32_home(row, t.size), first_tomb = ~0ull;
      bool dup = false;
      for (uint64_t step = 0; step < t.size; ++step) {
        const uint64_t cur = ld(w + pos);
        if ((uint32_t)cur == (uint32_t)row) {
          dup = true;
          break;
        }
        if (cur == kH32EmptyWord) break;
        if (cur == kH32TombWord && first_tomb == ~0ull) first_tomb = pos;
        if (++pos == t.size) pos = 0;
      }
      if (dup) {
        or_status(status, UGK_ST_DUP_KEY);
        continue;
      }
      const uint64_t target = first_tomb != ~0ull ? first_tomb : pos;
      const uint64_t cur = ld(w + target);
      if (cur != kH32EmptyWord && cur != kH32TombWord) {
        or_status(status, UGK_ST_TABLE_FULL);
        continue;
      }
      st(w + target, ((uint64_t)(((loc & 0xfu) << 28) + off) << 32) | (uint32_t)row);  // row and value appear together
      continue;
    }
    if (key >= UGK_HASH_TOMB) {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
      continue;
    }
    ugk_bucket_t *b = reinterpret_cast<ugk_bucket_t *>(t.table);
    uint64_t pos = fmix64(key) % t.size, first_tomb = ~0ull;
    bool placed = false;
    for (uint64_t step = 0; step < t.size && !placed; ++step) {
      const uint64_t cur = ld(&b[pos].key);
      if (cur == key) {
        or_status(status, UGK_ST_DUP_KEY);
        placed = true;
      } else if (cur == UGK_HASH_EMPTY) {
        break;
      } else {
        if (cur == UGK_HASH_TOMB && first_tomb == ~0ull) first_tomb = pos;
        if (++pos == t.size) pos = 0;
      }
    }
    if (placed) continue;
    const uint64_t target = first_tomb != ~0ull ? first_tomb : pos;
    const uint64_t cur = ld(&b[target].key);
    if (cur != UGK_HASH_EMPTY && cur != UGK_HASH_TOMB) {
      or_status(status, UGK_ST_TABLE_FULL);
      continue;
    }
    st(&b[target].key, key);  // "present, not valid" until the next store: reads as a miss
    st(reinterpret_cast<uint64_t *>(&b[target].off), ((uint64_t)(UGK_META_VALID | loc) << 32) | off);
  }
  return 0;
}

template <typename K>
int table_evict(ugk_table_t t, const K *keys, size_t n, uint32_t *status, uint64_t *slot_bits = nullptr,
                uint64_t nslots = 0) {
  auto release = [&](uint32_t slot) {
    if (!slot_bits) return;
    if (slot >= nslots) or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
    else __atomic_fetch_and(slot_bits + (slot >> 6), ~(1ull << (slot & 63)), __ATOMIC_RELAXED);
  };
  if (n == 0) return 0;
  if (check_table(t, "ugk_table_evict")) return 1;
  REQUIRE(keys && status, "ugk_table_evict: null pointer");
  for (size_t i = 0; i < n; ++i) {
    const uint64_t key = k64(keys[i]);
    if (t.kind == 1) {
      if (key >= t.size) {
        or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
        continue;
      }
      const uint32_t old =
          __atomic_exchange_n(reinterpret_cast<uint32_t *>(t.table) + key, UGK_EMPTY_U32, __ATOMIC_ACQ_REL);
      if (old == UGK_EMPTY_U32) or_status(status, UGK_ST_EVICT_ABSENT);
      else release(old & 0x0fffffffu);
      continue;
    }
    if (t.kind == 3) {
      const uint64_t row = fallback_row(t, key);
      uint64_t *w = reinterpret_cast<uint64_t *>(t.table);
      uint64_t pos = row < kH32Tomb ? h32_home(row, t.size) : 0;
      bool gone = false;
      for (uint64_t step = 0; step < t.size && row < kH32Tomb; ++step) {
        const uint64_t cur = ld(w + pos);
        if ((uint32_t)cur == (uint32_t)row) {
          release((uint32_t)(cur >> 32) & 0x0fffffffu);
          st(w + pos, kH32TombWord);
          gone = true;
          break;
        }
        if (cur == kH32EmptyWord) break;
        if (++pos == t.size) pos = 0;
      }
      if (!gone) or_status(status, UGK_ST_EVICT_ABSENT);
      continue;
    }
    ugk_bucket_t *b = reinterpret_cast<ugk_bucket_t *>(t.table);
    uint64_t pos = fmix64(key) % t.size;
    bool done = false;
    for (uint64_t step = 0; step < t.size && !done && key < UGK_HASH_TOMB; ++step) {
      const uint64_t cur = ld(&b[pos].key);
      if (cur == key) {
        release((uint32_t)ld(reinterpret_cast<const uint64_t *>(&b[pos].off)));
        st(reinterpret_cast<uint64_t *>(&b[pos].off), (uint64_t)0);
        st(&b[pos].key, (uint64_t)UGK_HASH_TOMB);
        done = true;
      } else if (cur == UGK_HASH_EMPTY) {
        break;
      } else if (++pos == t.size) {
        pos = 0;
      }
    }
    if (!done) or_status(status, UGK_ST_EVICT_ABSENT);
  }
  return 0;
}

template <typename K>
int table_lookup(ugk_table_t t, const K *keys, size_t n, uint32_t fallback_loc, uint32_t *loc_out, uint32_t *off_out) {
  if (n == 0) return 0;
  if (check_table(t, "ugk_table_lookup")) return 1;
  for (size_t i = 0; i < n; ++i) {
    const uint64_t key = k64(keys[i]);
    const Found f = lookup(t, key);
    if (loc_out) loc_out[i] = f.hit ? f.loc : fallback_loc;
    if (off_out) off_out[i] = f.hit ? f.off : (uint32_t)fallback_row(t, key);
  }
  return 0;
}

template <typename K>
int classify(ugk_table_t t, const K *keys, size_t n, uint64_t host_rows, const uint32_t *dst_map, ugk_idx_t *idx,
             uint32_t *counts, uint32_t *next_counts, uint32_t *status, uint32_t *mirror) {
  REQUIRE(counts && status, "ugk_classify: null counters or status");
  if (check_table(t, "ugk_classify")) return 1;
  if (next_counts) next_counts[0] = next_counts[1] = 0;
  uint32_t h = counts[0], m = counts[1];
  for (size_t i = 0; i < n; ++i) {
    const uint64_t key = k64(keys[i]);
    const Found f = lookup(t, key);
    const uint32_t d = dst_map ? dst_map[i] : (uint32_t)i;
    if (f.hit && f.loc == UGK_LOC_LOCAL) idx[h++] = ugk_idx_t{d, f.off};
    else if (f.hit && f.loc == UGK_LOC_HOST && f.off < host_rows) idx[n - ++m] = ugk_idx_t{d, f.off};
    else if (!f.hit && fallback_row(t, key) < host_rows && fallback_row(t, key) <= 0xffffffffull)
      idx[n - ++m] = ugk_idx_t{d, (uint32_t)fallback_row(t, key)};
    else or_status(status, UGK_ST_KEY_OUT_OF_RANGE, mirror);
  }
  counts[0] = h;
  counts[1] = m;
  return 0;
}

template <typename K>
int nonlocal_flags(ugk_table_t t, const K *keys, size_t n, uint64_t *flags) {
  if (n == 0) return 0;
  if (check_table(t, "ugk_nonlocal_flags")) return 1;
  for (size_t w = 0; w < (n + 63) / 64; ++w) {
    uint64_t bits = 0;
    for (size_t i = w * 64; i < std::min(n, w * 64 + 64); ++i) {
      const Found f = lookup(t, k64(keys[i]));
      if (!(f.hit && f.loc == UGK_LOC_LOCAL)) bits |= 1ull << (i & 63);
    }
    flags[w] = bits;
  }
  return 0;
}

template <typename K>
int extract_mix(ugk_table_t t, const K *keys, size_t n, const void *cache, uint64_t cache_rows, const void *host,
                uint64_t host_rows, void *out, size_t rb, uint32_t *status, uint32_t *mirror, uint64_t *counts,
                uint32_t *num_groups, const ugk_stage_t *stage = nullptr) {
  if (num_groups) *num_groups = 0;
  if (n == 0) return 0;
  REQUIRE(keys && out && status, "ugk_extract_mix: null keys, output or status");
  if (check_table(t, "ugk_extract_mix")) return 1;
  REQUIRE(rb > 0 && rb % 16 == 0, "ugk_extract_mix: rows must be multiples of 16 bytes (row_bytes=%zu)", rb);
  uint64_t local = 0, others = 0;
  for (size_t i = 0; i < n; ++i) {
    const uint64_t key = k64(keys[i]);
    const Found f = lookup(t, key);
    const char *row = nullptr;
    bool from_cache = false;
    if (f.hit && f.loc == UGK_LOC_LOCAL && f.off < cache_rows) {
      row = (const char *)cache + (size_t)f.off * rb;
      from_cache = true;
    } else if (f.hit && f.loc == UGK_LOC_HOST && f.off < host_rows) {
      row = (const char *)host + (size_t)f.off * rb;
    } else if (!f.hit && fallback_row(t, key) < host_rows) {
      row = (const char *)host + fallback_row(t, key) * rb;
    } else {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE, mirror);
    }
    if (row) copy_row((char *)out + i * rb, row, rb);
    if (row && !from_cache && stage) {
      const uint64_t r = (uint64_t)(row - (const char *)host) / rb;
      const uint64_t h = fmix64(r) & stage->mask;
      const uint64_t cur = stage->owner_dev[h];
      const uint32_t tag = (uint32_t)(cur >> 32);
      if (r <= 0xffffffffull && tag != stage->epoch && !(tag != 0 && (uint32_t)cur == (uint32_t)r)) {
        stage->owner_dev[h] = ((uint64_t)stage->epoch << 32) | (uint32_t)r;
        copy_row((char *)stage->rows_dev + h * rb, row, rb);
      }
    }
    if (from_cache) ++local;
    else ++others;
  }
  if (counts) counts[0] = (others << 32) | local;
  if (num_groups) *num_groups = 1;
  return 0;
}

// fp16 <-> fp32 without compiler support for _Float16 in every build: the bit patterns by hand
inline float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 31u, man = h & 1023u;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) bits = sign;
    else {
      int e = -1;
      uint32_t m = man;
      do { ++e; m <<= 1; } while (!(m & 1024u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 1023u) << 13);
    }
  } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
  else bits = sign | ((exp + 112u) << 23) | (man << 13);
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
inline uint16_t float_to_half(float f) {  // round to nearest even
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to infinity
  if (x < 0x33000001u) return (uint16_t)sign;               // rounds to zero
  int e = (int)(x >> 23) - 127;
  uint32_t m = (x & 0x7fffffu) | 0x800000u;
  int shift = e < -14 ? 13 + (-14 - e) : 13;
  uint32_t half_m = m >> shift, rest = m & ((1u << shift) - 1), mid = 1u << (shift - 1);
  if (rest > mid || (rest == mid && (half_m & 1u))) ++half_m;
  const uint32_t half_e = e < -14 ? 0 : (uint32_t)(e + 15);
  return (uint16_t)(sign | ((half_e << 10) + (half_m - (e < -14 ? 0 : 1024u))));
}

template <typename K>
int extract_pool(ugk_table_t t, const K *ids, const int64_t *seg_off, const float *weights, size_t n_rows,
                 uint64_t nnz, int combiner, int elem_bytes, const void *cache, uint64_t cache_rows, const void *host,
                 uint64_t host_rows, void *out, size_t rb, uint32_t *status, uint32_t *mirror, uint64_t *counts,
                 uint32_t *num_groups, float max_norm = 0.f) {
  if (num_groups) *num_groups = 0;
  if (n_rows == 0) return 0;
  REQUIRE(seg_off && out && status && (nnz == 0 || ids), "ugk_extract_pool: null pointer");
  REQUIRE(max_norm >= 0.f, "ugk_extract_pool: negative max_norm");
  REQUIRE(combiner >= 0 && combiner <= 2 && (elem_bytes == 2 || elem_bytes == 4 || elem_bytes == UGK_ELEM_BF16),
          "ugk_extract_pool: bad argument");
  const bool bf16 = elem_bytes == UGK_ELEM_BF16;
  elem_bytes &= 0xf;
  REQUIRE(rb > 0 && rb % 16 == 0 && rb <= 4096, "ugk_extract_pool: rows of %zu bytes", rb);
  if (t.kind != 0 && check_table(t, "ugk_extract_pool")) return 1;
  const size_t dim = rb / elem_bytes;
  uint64_t local = 0, others = 0;
  std::vector<float> acc(dim);
  for (size_t r = 0; r < n_rows; ++r) {
    std::fill(acc.begin(), acc.end(), 0.f);
    float wsum = 0.f;
    int64_t beg = seg_off[r], end = seg_off[r + 1];
    if (beg < 0 || end > (int64_t)nnz || end < beg) {
      or_status(status, UGK_ST_BAD_SEGMENT, mirror);
      beg = end = 0;
    } else if ((r == 0 && beg != 0) || (r + 1 == n_rows && end != (int64_t)nnz)) {
      or_status(status, UGK_ST_BAD_SEGMENT, mirror);  // the ids are not covered from the first to the last
    }
    for (int64_t j = beg; j < end; ++j) {
      const uint64_t key = k64(ids[j]);
      const Found f = t.kind ? lookup(t, key) : Found{false, 0, 0};
      const char *row = nullptr;
      bool from_cache = false;
      if (f.hit && f.loc == UGK_LOC_LOCAL && f.off < cache_rows) {
        row = (const char *)cache + (size_t)f.off * rb;
        from_cache = true;
      } else if (f.hit && f.loc == UGK_LOC_HOST && f.off < host_rows) {
        row = (const char *)host + (size_t)f.off * rb;
      } else if (!f.hit && fallback_row(t, key) < host_rows) {
        row = (const char *)host + fallback_row(t, key) * rb;
      } else {
        or_status(status, UGK_ST_KEY_OUT_OF_RANGE, mirror);
      }
      if (from_cache) ++local;
      else ++others;
      if (!row) continue;
      float w = weights ? weights[j] : 1.f;
      wsum += combiner == 2 ? w * w : w;
      auto element = [&](size_t c) {
        float x;
        if (elem_bytes == 4) memcpy(&x, row + c * 4, 4);
        else {
          uint16_t h;
          memcpy(&h, row + c * 2, 2);
          if (bf16) {
            const uint32_t u = (uint32_t)h << 16;
            memcpy(&x, &u, 4);
          } else {
            x = half_to_float(h);
          }
        }
        return x;
      };
      if (max_norm > 0.f) {  // the row clipped to that l2 norm before it is weighted
        float ss = 0.f;
        for (size_t c = 0; c < dim; ++c) ss = std::fma(element(c), element(c), ss);
        w *= max_norm / std::max(std::sqrt(ss), max_norm);
      }
      for (size_t c = 0; c < dim; ++c) acc[c] = std::fma(w, element(c), acc[c]);
    }
    const float denom = combiner == 1 ? wsum : combiner == 2 ? std::sqrt(wsum) : 1.f;
    for (size_t c = 0; c < dim; ++c) {
      const float y = denom != 0.f ? acc[c] / denom : 0.f;
      if (elem_bytes == 4) memcpy((char *)out + (r * dim + c) * 4, &y, 4);
      else {
        uint16_t h;
        if (bf16) {
          uint32_t u;
          memcpy(&u, &y, 4);
          h = (u & 0x7fffffffu) > 0x7f800000u ? (uint16_t)((u >> 16) | 0x40u)
                                              : (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
        } else {
          h = float_to_half(y);
        }
        memcpy((char *)out + (r * dim + c) * 2, &h, 2);
      }
    }
  }
  if (counts) counts[0] = (others << 32) | local;
  if (num_groups) *num_groups = 1;
  return 0;
}

template <typename K>
int dedup(const K *keys, size_t n, K *unique_out, uint32_t *inverse, uint32_t *rep, uint32_t *n_unique,
          uint32_t *n_unique_host) {
  if (n == 0) return 0;
  REQUIRE(keys && unique_out && inverse && n_unique, "ugk_dedup: null pointer");
  std::unordered_map<uint64_t, uint32_t> seen;
  uint32_t nu = *n_unique;
  for (size_t i = 0; i < n; ++i) {
    auto it = seen.find(k64(keys[i]));
    if (it == seen.end()) {
      seen.emplace(k64(keys[i]), nu);
      unique_out[nu] = keys[i];
      if (rep) rep[nu] = (uint32_t)i;
      inverse[i] = nu++;
    } else {
      inverse[i] = it->second;
    }
  }
  *n_unique = nu;
  if (n_unique_host) *n_unique_host = nu;
  return 0;
}

template <typename K>
int record(const K *keys, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts, uint64_t num_rows,
           uint64_t *observed, uint32_t *status, uint32_t *mirror) {
  if (n == 0) return 0;
  REQUIRE(keys && counts && status, "ugk_record: null pointer");
  ugk_table_t map{};
  map.fb_mul = key_inv;
  map.fb_mask = key_mask;
  for (size_t i = 0; i < n; ++i) {
    const uint64_t row = fallback_row(map, k64(keys[i]));
    if (row >= num_rows) {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE, mirror);
      continue;
    }
    const uint32_t before = __atomic_fetch_add(counts + row, 1u, __ATOMIC_RELAXED);
    if (before == 0 && observed) __atomic_fetch_or(observed + (row >> 6), 1ull << (row & 63), __ATOMIC_RELAXED);
  }
  return 0;
}

uint64_t bm_word(const uint64_t *a, const uint64_t *b, int invert_a, uint64_t nbits, uint64_t w) {
  uint64_t m = ld(a + w);
  if (invert_a) m = ~m;
  if (b) m &= ~ld(b + w);
  if (nbits - w * 64 < 64) m &= (1ull << (nbits - w * 64)) - 1ull;
  return m;
}

// ---- streams, events and the rules of recording a stream into a graph -----------------------------------------------
// Work enqueued on a stream still runs at once (see the top of the file), also while the stream "captures": what the
// model adds is the bookkeeping the runtime keeps for a capture, so that a sequence of calls that the runtime refuses,
// or that leaves objects of the library tied to a graph the caller owns, is reported here, on the CPU:
//   - an event recorded on a capturing stream is a captured event; a stream that waits for one joins the capture;
//   - a captured event cannot be waited for, queried or timed on the host; a capturing stream cannot be waited for, nor
//     can the device while any stream captures; memory cannot be allocated or freed meanwhile (global capture mode);
//   - a capturing stream cannot wait for an event recorded outside the capture;
//   - a stream that joined has to be joined back before the capture ends;
//   - a stream or event that took part in a capture must not be destroyed while the recorded graph lives, and -- the
//     rule of the library itself -- only the caller's stream takes part in the caller's capture: an event recorded or a
//     second stream joined while capturing is reported even where the runtime would accept it.
struct Stream {
  int capture = 0;      // id of the capture this stream records into, 0: runs its work
  bool origin = false;  // the capture was begun on this stream
  void *join_event = nullptr;  // joined stream: the last event recorded on it
  bool joined_back = true;
};
struct Event {
  std::chrono::steady_clock::time_point at;
  int captured_in = 0;  // id of the capture its last record went into, 0: recorded on a running stream
  Stream *recorded_on = nullptr;
};
struct Graph {
  std::vector<Stream *> streams;
  std::vector<void *> events;
  bool alive = true;
};
std::mutex g_rt_mu;  // guards everything below and the fields of every Stream and Event
Stream g_null_stream;
int g_capture_active = 0, g_capture_next = 1;
std::map<int, Graph> g_graphs;
std::vector<std::string> g_violations;
// which stream last filed rows in a stage (keyed by its owner words) and whether the host has waited for it since
std::map<const void *, std::pair<Stream *, bool>> g_stage_writers;

Stream *as_stream(void *s) { return s ? static_cast<Stream *>(s) : &g_null_stream; }
void violation(const char *fmt, ...) {
  char buf[256];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_violations.emplace_back(buf);
}
// caller holds g_rt_mu: the host has waited for `s` (null: for every stream)
void note_stream_idle(Stream *s) {
  for (auto &kv : g_stage_writers)
    if (s == nullptr || kv.second.first == s) kv.second.second = false;
}
void note_staged_launch(const ugk_stage_t &stage, void *stream) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  auto &w = g_stage_writers[stage.owner_dev];
  if (w.second && w.first != as_stream(stream))
    violation("two extractions on different streams, with no wait between them, file rows in one stage");
  w = {as_stream(stream), true};
}
// caller holds g_rt_mu
void note_host_wait(const char *what) {
  if (g_capture_active) violation("%s while a stream records into a graph", what);
}
bool referenced_by_live_graph(const void *obj) {
  for (auto &kv : g_graphs) {
    if (!kv.second.alive) continue;
    for (auto *s : kv.second.streams)
      if (s == obj) return true;
    for (auto *e : kv.second.events)
      if (e == obj) return true;
  }
  return false;
}

}  // namespace

// hooks of the model itself (declared in ugk_cpu_model.h): the driver plays the caller that records a graph
extern "C" {
int ugk_model_capture_begin(void *stream) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  Stream *s = as_stream(stream);
  REQUIRE(g_capture_active == 0 && s->capture == 0, "ugk_model_capture_begin: a capture is active already");
  g_capture_active = s->capture = g_capture_next++;
  s->origin = true;
  g_graphs[g_capture_active].streams.push_back(s);
  return 0;
}
int ugk_model_capture_end(void *stream, int *graph_id) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  Stream *s = as_stream(stream);
  REQUIRE(s->origin && s->capture == g_capture_active && g_capture_active != 0,
          "ugk_model_capture_end: no capture was begun on this stream");
  Graph &graph = g_graphs[g_capture_active];
  for (Stream *m : graph.streams) {
    if (m != s && !m->joined_back) violation("a stream that joined the capture was not joined back before its end");
    m->capture = 0;
    m->origin = false;
    m->join_event = nullptr;
    m->joined_back = true;
  }
  if (graph_id) *graph_id = g_capture_active;
  g_capture_active = 0;
  return 0;
}
void ugk_model_graph_destroy(int graph_id) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  auto it = g_graphs.find(graph_id);
  if (it != g_graphs.end()) it->second.alive = false;
}
size_t ugk_model_violations(char *text, size_t capacity) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  if (text && capacity) {
    std::string all;
    for (auto &v : g_violations) all += v + "\n";
    snprintf(text, capacity, "%s", all.c_str());
  }
  return g_violations.size();
}
void ugk_model_reset(void) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  g_violations.clear();
  g_graphs.clear();
  g_stage_writers.clear();
}
}

extern "C" {

const char *ugk_last_error(void) { return g_err; }
int ugk_abi_version(void) { return UGK_ABI_VERSION; }

int ugk_device_count(int *count) {
  *count = 1;
  return 0;
}
int ugk_set_device(int dev) {
  REQUIRE(dev == 0, "no device %d", dev);
  return 0;
}
int ugk_get_device_info(int dev, ugk_device_info_t *info) {
  REQUIRE(dev == 0 && info, "no device %d", dev);
  memset(info, 0, sizeof(*info));
  snprintf(info->name, sizeof(info->name), "cpu model of the ugk C-ABI (tests only)");
  snprintf(info->arch, sizeof(info->arch), "none");
  info->compute_units = 256;
  info->wavefront_size = 64;
  info->total_mem = 64ull << 30;
  info->lds_per_block = 65536;
  return 0;
}
int ugk_mem_info(size_t *free_bytes, size_t *total_bytes) {
  if (free_bytes) *free_bytes = 32ull << 30;
  if (total_bytes) *total_bytes = 64ull << 30;
  return 0;
}
static void note_allocation(const char *what) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  if (g_capture_active) violation("%s while a stream records into a graph", what);
}
int ugk_malloc(void **ptr, size_t nbytes) {
  note_allocation("device memory allocated");
  return alloc_block(ptr, nbytes, 2);
}
int ugk_free(void *ptr) {
  if (ptr) note_allocation("device memory freed");
  return free_block(ptr, 2);
}
int ugk_host_malloc(void **ptr, size_t nbytes) {
  note_allocation("pinned memory allocated");
  return alloc_block(ptr, nbytes, 1);
}
int ugk_host_free(void *ptr) {
  if (ptr) note_allocation("pinned memory freed");
  return free_block(ptr, 1);
}
int ugk_pointer_kind(const void *ptr, int *kind) {
  std::lock_guard<std::mutex> g(g_mem_mu);
  *kind = 0;
  auto it = g_blocks.upper_bound((uintptr_t)ptr);
  if (it != g_blocks.begin()) {
    --it;
    if ((uintptr_t)ptr < it->first + it->second.first) *kind = it->second.second;
  }
  return 0;
}
int ugk_stream_create(void **stream) {
  *stream = new Stream;
  return 0;
}
int ugk_stream_create_cu_masked(void **stream, int num_cus) {
  REQUIRE(num_cus > 0, "ugk_stream_create_cu_masked: %d compute units", num_cus);
  return ugk_stream_create(stream);
}
int ugk_stream_destroy(void *stream) {
  if (!stream) return 0;
  {
    std::lock_guard<std::mutex> g(g_rt_mu);
    if (as_stream(stream)->capture) violation("a stream was destroyed while it records into a graph");
    if (referenced_by_live_graph(stream)) violation("a stream that took part in a capture was destroyed while the graph lives");
    for (auto &kv : g_graphs)
      for (auto &m : kv.second.streams)
        if (m == stream) m = nullptr;
  }
  delete static_cast<Stream *>(stream);
  return 0;
}
int ugk_stream_sync(void *stream) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  if (as_stream(stream)->capture) violation("the host waited for a stream that records into a graph");
  note_stream_idle(as_stream(stream));
  return 0;
}
int ugk_stream_is_capturing(void *stream, int *capturing) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  *capturing = as_stream(stream)->capture != 0;
  return 0;
}
int ugk_stream_sync_ticket(void *stream, uint32_t *ticket_host, uint32_t value, unsigned) {
  REQUIRE(ticket_host, "ugk_stream_sync_ticket: null ticket word");
  {
    std::lock_guard<std::mutex> g(g_rt_mu);
    if (as_stream(stream)->capture) violation("the host waited for a ticket on a stream that records into a graph");
    note_stream_idle(as_stream(stream));
  }
  *ticket_host = value;
  return 0;
}
int ugk_words_to_host_ticket(const uint32_t *a, unsigned n_a, const uint32_t *b, unsigned n_b, uint32_t *dst,
                             uint32_t value, unsigned, void *stream) {
  REQUIRE(dst && (a || n_a == 0) && (b || n_b == 0) && n_a + n_b <= 63u, "ugk_words_to_host_ticket: bad argument");
  {
    std::lock_guard<std::mutex> g(g_rt_mu);
    if (as_stream(stream)->capture) violation("the host waited for a ticket on a stream that records into a graph");
    note_stream_idle(as_stream(stream));
  }
  for (unsigned i = 0; i < n_a; ++i) dst[1 + i] = a[i];
  for (unsigned i = 0; i < n_b; ++i) dst[1 + n_a + i] = b[i];
  dst[0] = value;
  return 0;
}
int ugk_preload_kernels(void) { return 0; }
int ugk_device_sync(void) {
  std::lock_guard<std::mutex> g(g_rt_mu);
  note_host_wait("the host waited for the device");
  note_stream_idle(nullptr);
  return 0;
}
int ugk_event_create(void **event) {
  *event = new Event{std::chrono::steady_clock::now()};
  return 0;
}
int ugk_event_destroy(void *event) {
  if (!event) return 0;
  {
    std::lock_guard<std::mutex> g(g_rt_mu);
    if (referenced_by_live_graph(event)) violation("an event that was recorded into a capture was destroyed while the graph lives");
    for (auto &kv : g_graphs)
      for (auto &e : kv.second.events)
        if (e == event) e = nullptr;
  }
  delete static_cast<Event *>(event);
  return 0;
}
int ugk_event_record(void *event, void *stream) {
  REQUIRE(event, "null event");
  std::lock_guard<std::mutex> g(g_rt_mu);
  Event *e = static_cast<Event *>(event);
  Stream *s = as_stream(stream);
  e->at = std::chrono::steady_clock::now();
  e->captured_in = s->capture;
  e->recorded_on = s;
  if (s->capture) {
    violation("an event was recorded on a stream that records into a graph: it belongs to the caller's capture now");
    g_graphs[s->capture].events.push_back(event);
    if (!s->origin) s->join_event = event;
  }
  return 0;
}
int ugk_event_sync(void *event) {
  REQUIRE(event, "null event");
  std::lock_guard<std::mutex> g(g_rt_mu);
  if (static_cast<Event *>(event)->captured_in) violation("the host waited for a captured event");
  return 0;
}
int ugk_event_query(void *event, int *complete) {
  REQUIRE(event && complete, "null pointer");
  std::lock_guard<std::mutex> g(g_rt_mu);
  if (static_cast<Event *>(event)->captured_in) violation("the host queried a captured event");
  *complete = 1;
  return 0;
}
int ugk_stream_wait_event(void *stream, void *event) {
  REQUIRE(event, "null event");
  std::lock_guard<std::mutex> g(g_rt_mu);
  Event *e = static_cast<Event *>(event);
  Stream *s = as_stream(stream);
  const bool live_capture = e->captured_in != 0 && e->captured_in == g_capture_active;
  if (live_capture && s->capture == 0) {
    // the waiting stream joins the capture the event belongs to
    violation("a second stream joined the caller's capture by waiting for a captured event");
    s->capture = e->captured_in;
    s->joined_back = false;
    g_graphs[s->capture].streams.push_back(s);
  } else if (live_capture && s->capture == e->captured_in) {
    Stream *from = e->recorded_on;
    if (from && from != s && !from->origin && from->join_event == event) from->joined_back = true;
  } else if (s->capture != 0 && !live_capture) {
    violation("a stream that records into a graph waited for an event recorded outside the capture");
  } else if (e->captured_in != 0) {
    violation("a stream waited for a captured event of a capture that has ended");
  }
  return 0;
}
int ugk_event_elapsed_ms(void *start, void *stop, float *ms) {
  REQUIRE(start && stop && ms, "null event");
  std::lock_guard<std::mutex> g(g_rt_mu);
  if (static_cast<Event *>(start)->captured_in || static_cast<Event *>(stop)->captured_in)
    violation("the time between captured events was asked for");
  *ms = std::chrono::duration<float, std::milli>(static_cast<Event *>(stop)->at - static_cast<Event *>(start)->at)
            .count();
  return 0;
}
int ugk_memcpy_async(void *dst, const void *src, size_t nbytes, void *) {
  if (nbytes) memmove(dst, src, nbytes);
  return 0;
}
int ugk_fill_u32(uint32_t *dst, uint32_t value, size_t nwords, void *) {
  for (size_t i = 0; i < nwords; ++i) st(dst + i, value);
  return 0;
}
int ugk_arange_u32(uint32_t *dst, uint32_t start, size_t n, void *) {
  for (size_t i = 0; i < n; ++i) dst[i] = start + (uint32_t)i;
  return 0;
}
int ugk_copy_rows(void *dst, const void *src, size_t nbytes, void *) {
  memcpy(dst, src, nbytes);
  return 0;
}

int ugk_set_output_hint(int hint) {
  REQUIRE(hint >= 0 && hint <= 2, "ugk_set_output_hint: unknown hint %d", hint);
  return 0;
}
int ugk_gather_direct_u32(const void *src, uint64_t src_rows, const uint32_t *keys, size_t n, void *out, size_t rb,
                          unsigned, uint32_t *status, uint32_t *mirror, void *) {
  return gather_direct(src, src_rows, keys, nullptr, n, out, ~0ull, rb, status, mirror);
}
int ugk_gather_direct_i64(const void *src, uint64_t src_rows, const int64_t *keys, size_t n, void *out, size_t rb,
                          unsigned, uint32_t *status, uint32_t *mirror, void *) {
  return gather_direct(src, src_rows, keys, nullptr, n, out, ~0ull, rb, status, mirror);
}
int ugk_gather_scatter_u32(const void *src, uint64_t src_rows, const uint32_t *keys, const uint32_t *dst, size_t n,
                           void *out, uint64_t out_rows, size_t rb, unsigned, uint32_t *status, uint32_t *mirror,
                           void *) {
  REQUIRE(n == 0 || dst, "ugk_gather_scatter_u32: null destinations");
  return gather_direct(src, src_rows, keys, dst, n, out, out_rows, rb, status, mirror);
}
int ugk_gather_scatter_i64(const void *src, uint64_t src_rows, const int64_t *keys, const uint32_t *dst, size_t n,
                           void *out, uint64_t out_rows, size_t rb, unsigned, uint32_t *status, uint32_t *mirror,
                           void *) {
  REQUIRE(n == 0 || dst, "ugk_gather_scatter_i64: null destinations");
  return gather_direct(src, src_rows, keys, dst, n, out, out_rows, rb, status, mirror);
}
int ugk_replicate_rows(void *out, size_t rb, const uint32_t *inverse, const uint32_t *rep, size_t n, void *) {
  for (size_t i = 0; i < n; ++i) {
    const size_t r = rep[inverse[i]];
    if (r != i) memcpy((char *)out + i * rb, (char *)out + r * rb, rb);
  }
  return 0;
}
int ugk_gather_group(const void *src, uint64_t src_rows, const ugk_idx_t *idx, const uint32_t *counts, uint32_t group,
                     size_t n, void *out, uint64_t out_rows, size_t rb, unsigned, uint32_t *status, uint32_t *mirror,
                     void *) {
  if (n == 0) return 0;
  REQUIRE(idx && counts && (group == UGK_LOC_LOCAL || group == UGK_LOC_HOST), "ugk_gather_group: bad argument");
  const uint32_t c = counts[group];
  if (mirror) mirror[1 + group] = c;
  const size_t begin = group == UGK_LOC_LOCAL ? 0 : n - c;
  return gather_list(src, src_rows, idx + begin, c, out, out_rows, rb, status, mirror);
}
int ugk_gather_idx(const void *src, uint64_t src_rows, const ugk_idx_t *idx, size_t count, void *out, size_t rb,
                   unsigned, uint32_t *status, void *) {
  return gather_list(src, src_rows, idx, count, out, ~0ull, rb, status, nullptr);
}

size_t ugk_hash_buckets_for(size_t n_entries, double load_factor) {
  if (!(load_factor > 0.0) || load_factor > 0.95) load_factor = 0.7;
  size_t nb = (size_t)std::ceil((double)n_entries / load_factor) + 1;
  if (nb < 64) nb = 64;
  return (nb + 7) / 8 * 8;
}
int ugk_hash_init(ugk_bucket_t *table, size_t nbuckets, void *) {
  REQUIRE(table && nbuckets && nbuckets % 8 == 0, "ugk_hash_init: bad table");
  for (size_t i = 0; i < nbuckets; ++i) {
    st(&table[i].key, (uint64_t)UGK_HASH_EMPTY);
    st(reinterpret_cast<uint64_t *>(&table[i].off), (uint64_t)0);
  }
  return 0;
}
int ugk_table_insert_u32(ugk_table_t t, const uint32_t *keys, const uint32_t *offs, uint32_t seq_base, uint32_t loc,
                         size_t n, uint32_t *status, void *) {
  return table_insert(t, keys, offs, seq_base, loc, n, status);
}
int ugk_table_insert_i64(ugk_table_t t, const int64_t *keys, const uint32_t *offs, uint32_t seq_base, uint32_t loc,
                         size_t n, uint32_t *status, void *) {
  return table_insert(t, keys, offs, seq_base, loc, n, status);
}
int ugk_table_evict_u32(ugk_table_t t, const uint32_t *keys, size_t n, uint32_t *status, void *) {
  return table_evict(t, keys, n, status);
}
int ugk_table_evict_i64(ugk_table_t t, const int64_t *keys, size_t n, uint32_t *status, void *) {
  return table_evict(t, keys, n, status);
}
int ugk_table_evict_release_u32(ugk_table_t t, const uint32_t *keys, size_t n, uint64_t *slot_bits, uint64_t nslots,
                                uint32_t *status, void *) {
  REQUIRE(n == 0 || slot_bits, "ugk_table_evict_release_u32: null slot bitmap");
  return table_evict(t, keys, n, status, slot_bits, nslots);
}
int ugk_table_evict_release_i64(ugk_table_t t, const int64_t *keys, size_t n, uint64_t *slot_bits, uint64_t nslots,
                                uint32_t *status, void *) {
  REQUIRE(n == 0 || slot_bits, "ugk_table_evict_release_i64: null slot bitmap");
  return table_evict(t, keys, n, status, slot_bits, nslots);
}
int ugk_table_lookup_u32(ugk_table_t t, const uint32_t *keys, size_t n, uint32_t fallback_loc, uint32_t *loc_out,
                         uint32_t *off_out, void *) {
  return table_lookup(t, keys, n, fallback_loc, loc_out, off_out);
}
int ugk_table_lookup_i64(ugk_table_t t, const int64_t *keys, size_t n, uint32_t fallback_loc, uint32_t *loc_out,
                         uint32_t *off_out, void *) {
  return table_lookup(t, keys, n, fallback_loc, loc_out, off_out);
}
int ugk_hash_census(const ugk_bucket_t *table, size_t nbuckets, uint64_t *census, void *) {
  REQUIRE(table && census, "ugk_hash_census: null pointer");
  uint64_t occ = 0, tomb = 0, empty = 0;
  for (size_t i = 0; i < nbuckets; ++i) {
    const uint64_t k = ld(&table[i].key);
    if (k == UGK_HASH_EMPTY) ++empty;
    else if (k == UGK_HASH_TOMB) ++tomb;
    else ++occ;
  }
  census[0] = occ;
  census[1] = tomb;
  census[2] = empty;
  return 0;
}

size_t ugk_hash32_entries_for(size_t n_entries, double load_factor) {
  if (!(load_factor > 0.0) || load_factor > 0.95) load_factor = 0.7;
  size_t ne = (size_t)std::ceil((double)n_entries / load_factor) + 1;
  if (ne < 64) ne = 64;
  return (ne + 15) / 16 * 16;
}
int ugk_table_init(ugk_table_t t, void *stream) {
  if (check_table(t, "ugk_table_init")) return 1;
  if (t.kind == 1) return ugk_fill_u32(static_cast<uint32_t *>(t.table), UGK_EMPTY_U32, t.size, stream);
  if (t.kind == 2) return ugk_hash_init(static_cast<ugk_bucket_t *>(t.table), t.size, stream);
  uint64_t *w = static_cast<uint64_t *>(t.table);
  for (size_t i = 0; i < t.size; ++i) st(w + i, kH32EmptyWord);
  return 0;
}
int ugk_table_census(ugk_table_t t, uint64_t *census, void *stream) {
  if (check_table(t, "ugk_table_census")) return 1;
  REQUIRE(t.kind == 2 || t.kind == 3, "ugk_table_census: a flat table has no buckets to count");
  REQUIRE(census, "ugk_table_census: null output");
  if (t.kind == 2) return ugk_hash_census(static_cast<const ugk_bucket_t *>(t.table), t.size, census, stream);
  uint64_t occ = 0, tomb = 0, empty = 0;
  const uint64_t *w = static_cast<const uint64_t *>(t.table);
  for (size_t i = 0; i < t.size; ++i) {
    const uint32_t k = (uint32_t)ld(w + i);
    if (k == 0xffffffffu) ++empty;
    else if (k == kH32Tomb) ++tomb;
    else ++occ;
  }
  census[0] = occ;
  census[1] = tomb;
  census[2] = empty;
  return 0;
}

int ugk_classify_u32(ugk_table_t t, const uint32_t *keys, size_t n, uint64_t host_rows, const uint32_t *dst_map,
                     ugk_idx_t *idx, uint32_t *counts, uint32_t *next_counts, uint32_t *status, uint32_t *mirror,
                     void *) {
  return classify(t, keys, n, host_rows, dst_map, idx, counts, next_counts, status, mirror);
}
int ugk_classify_i64(ugk_table_t t, const int64_t *keys, size_t n, uint64_t host_rows, const uint32_t *dst_map,
                     ugk_idx_t *idx, uint32_t *counts, uint32_t *next_counts, uint32_t *status, uint32_t *mirror,
                     void *) {
  return classify(t, keys, n, host_rows, dst_map, idx, counts, next_counts, status, mirror);
}
int ugk_nonlocal_flags_u32(ugk_table_t t, const uint32_t *keys, size_t n, uint64_t *flags, void *) {
  return nonlocal_flags(t, keys, n, flags);
}
int ugk_nonlocal_flags_i64(ugk_table_t t, const int64_t *keys, size_t n, uint64_t *flags, void *) {
  return nonlocal_flags(t, keys, n, flags);
}
int ugk_select_keys_u32(const uint32_t *keys, const uint32_t *sel, size_t m, uint32_t *out, void *) {
  for (size_t j = 0; j < m; ++j) out[j] = keys[sel[j]];
  return 0;
}
int ugk_select_keys_i64(const int64_t *keys, const uint32_t *sel, size_t m, int64_t *out, void *) {
  for (size_t j = 0; j < m; ++j) out[j] = keys[sel[j]];
  return 0;
}

unsigned ugk_extract_mix_max_groups(void) { return 16; }
int ugk_extract_mix_u32(ugk_table_t t, const uint32_t *keys, size_t n, const void *cache, uint64_t cache_rows,
                        const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *status, uint32_t *mirror,
                        uint64_t *counts, uint32_t *num_groups, uint32_t, void *) {
  return extract_mix(t, keys, n, cache, cache_rows, host, host_rows, out, rb, status, mirror, counts, num_groups);
}
int ugk_extract_mix_i64(ugk_table_t t, const int64_t *keys, size_t n, const void *cache, uint64_t cache_rows,
                        const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *status, uint32_t *mirror,
                        uint64_t *counts, uint32_t *num_groups, uint32_t, void *) {
  return extract_mix(t, keys, n, cache, cache_rows, host, host_rows, out, rb, status, mirror, counts, num_groups);
}

int ugk_segment_offsets_i64(const int64_t *rows, size_t nnz, size_t n_rows, int64_t *seg_off, uint32_t *status,
                            uint32_t *mirror, void *) {
  REQUIRE(seg_off && (nnz == 0 || rows), "ugk_segment_offsets: null pointer");
  for (size_t i = 0; i <= nnz; ++i) {
    const int64_t prev = i == 0 ? -1 : rows[i - 1];
    const int64_t cur = i == nnz ? (int64_t)n_rows : rows[i];
    if (cur < prev || cur < 0 || (i > 0 && prev < 0) || (i < nnz && cur >= (int64_t)n_rows) || prev >= (int64_t)n_rows) {
      if (status) or_status(status, UGK_ST_BAD_SEGMENT, mirror);
      continue;
    }
    for (int64_t r = prev + 1; r <= cur; ++r) seg_off[r] = (int64_t)i;
  }
  return 0;
}

int ugk_extract_pool_u32(ugk_table_t t, const uint32_t *ids, const int64_t *seg_off, const float *weights, size_t n_rows,
                         uint64_t nnz, int combiner, int elem_bytes, const void *cache, uint64_t cache_rows,
                         const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *status, uint32_t *mirror,
                         uint64_t *counts, uint32_t *num_groups, void *) {
  return extract_pool(t, ids, seg_off, weights, n_rows, nnz, combiner, elem_bytes, cache, cache_rows, host, host_rows,
                      out, rb, status, mirror, counts, num_groups);
}
int ugk_extract_pool_i64(ugk_table_t t, const int64_t *ids, const int64_t *seg_off, const float *weights, size_t n_rows,
                         uint64_t nnz, int combiner, int elem_bytes, const void *cache, uint64_t cache_rows,
                         const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *status, uint32_t *mirror,
                         uint64_t *counts, uint32_t *num_groups, void *) {
  return extract_pool(t, ids, seg_off, weights, n_rows, nnz, combiner, elem_bytes, cache, cache_rows, host, host_rows,
                      out, rb, status, mirror, counts, num_groups);
}

int ugk_extract_pool_clip_u32(ugk_table_t t, const uint32_t *ids, const int64_t *seg_off, const float *weights,
                              size_t n_rows, uint64_t nnz, int combiner, int elem_bytes, float max_norm,
                              const void *cache, uint64_t cache_rows, const void *host, uint64_t host_rows, void *out,
                              size_t rb, uint32_t *status, uint32_t *mirror, uint64_t *counts, uint32_t *num_groups,
                              void *) {
  return extract_pool(t, ids, seg_off, weights, n_rows, nnz, combiner, elem_bytes, cache, cache_rows, host, host_rows,
                      out, rb, status, mirror, counts, num_groups, max_norm);
}
int ugk_extract_pool_clip_i64(ugk_table_t t, const int64_t *ids, const int64_t *seg_off, const float *weights,
                              size_t n_rows, uint64_t nnz, int combiner, int elem_bytes, float max_norm,
                              const void *cache, uint64_t cache_rows, const void *host, uint64_t host_rows, void *out,
                              size_t rb, uint32_t *status, uint32_t *mirror, uint64_t *counts, uint32_t *num_groups,
                              void *) {
  return extract_pool(t, ids, seg_off, weights, n_rows, nnz, combiner, elem_bytes, cache, cache_rows, host, host_rows,
                      out, rb, status, mirror, counts, num_groups, max_norm);
}

int ugk_extract_mix_staged_u32(ugk_table_t t, const uint32_t *keys, size_t n, const void *cache, uint64_t cache_rows,
                               const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *status,
                               uint32_t *mirror, uint64_t *counts, uint32_t *num_groups, uint32_t, ugk_stage_t stage,
                               void *stream) {
  REQUIRE(stage.rows_dev && stage.owner_dev && stage.epoch, "ugk_extract_mix_staged: bad stage");
  note_staged_launch(stage, stream);
  return extract_mix(t, keys, n, cache, cache_rows, host, host_rows, out, rb, status, mirror, counts, num_groups,
                     &stage);
}
int ugk_extract_mix_staged_i64(ugk_table_t t, const int64_t *keys, size_t n, const void *cache, uint64_t cache_rows,
                               const void *host, uint64_t host_rows, void *out, size_t rb, uint32_t *status,
                               uint32_t *mirror, uint64_t *counts, uint32_t *num_groups, uint32_t, ugk_stage_t stage,
                               void *stream) {
  REQUIRE(stage.rows_dev && stage.owner_dev && stage.epoch, "ugk_extract_mix_staged: bad stage");
  note_staged_launch(stage, stream);
  return extract_mix(t, keys, n, cache, cache_rows, host, host_rows, out, rb, status, mirror, counts, num_groups,
                     &stage);
}
int ugk_gather_scatter_staged_u32(const void *host, uint64_t host_rows, const uint32_t *rows, const uint32_t *dst,
                                  size_t n, void *out, uint64_t out_rows, size_t rb, ugk_stage_t stage, unsigned,
                                  uint32_t *status, uint32_t *staged, uint32_t *rest_rows, uint32_t *rest_dst,
                                  uint32_t *rest_count, uint32_t *done_count, void *) {
  if (n == 0) return 0;
  REQUIRE(host && rows && dst && out && status && stage.rows_dev && stage.owner_dev, "staged gather: null pointer");
  REQUIRE(done_count == nullptr || rest_count, "staged gather: a done count without rest lists");
  for (size_t i = 0; i < n; ++i) {
    const uint64_t r = rows[i];
    if (r >= host_rows || dst[i] >= out_rows) {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
      continue;
    }
    const uint64_t h = fmix64(r) & stage.mask;
    const uint64_t cur = stage.owner_dev[h];
    const bool filed = (cur >> 32) != 0 && (uint32_t)cur == (uint32_t)r;
    if (!filed && rest_count) {
      rest_rows[*rest_count] = (uint32_t)r;
      rest_dst[(*rest_count)++] = dst[i];
      continue;
    }
    copy_row((char *)out + (size_t)dst[i] * rb, filed ? (const char *)stage.rows_dev + h * rb : (const char *)host + r * rb,
             rb);
    if (filed && staged) ++*staged;
    if (filed && done_count) {
      const size_t at = n - 1 - (*done_count)++;
      rest_rows[at] = (uint32_t)r;
      rest_dst[at] = dst[i];
    }
  }
  return 0;
}

size_t ugk_dedup_workspace_bytes(size_t) { return 64; }
int ugk_dedup_u32(const uint32_t *keys, size_t n, void *, size_t, uint32_t epoch, uint32_t *unique_out,
                  uint32_t *inverse, uint32_t *rep, uint32_t *n_unique, uint32_t *n_unique_host, void *) {
  REQUIRE(epoch != 0, "ugk_dedup: epoch must be non-zero");
  return dedup(keys, n, unique_out, inverse, rep, n_unique, n_unique_host);
}
int ugk_dedup_i64(const int64_t *keys, size_t n, void *, size_t, uint32_t epoch, int64_t *unique_out,
                  uint32_t *inverse, uint32_t *rep, uint32_t *n_unique, uint32_t *n_unique_host, void *) {
  REQUIRE(epoch != 0, "ugk_dedup: epoch must be non-zero");
  return dedup(keys, n, unique_out, inverse, rep, n_unique, n_unique_host);
}
int ugk_dedup_static(const void *keys, uint32_t key_bytes, size_t n, void *unique_out, uint32_t *inverse,
                     uint32_t *rep, uint32_t *n_unique, uint32_t *n_unique_host, void *) {
  REQUIRE(key_bytes == 4 || key_bytes == 8, "ugk_dedup_static: keys of %u bytes", key_bytes);
  REQUIRE(n <= UGK_DEDUP_STATIC_MAX_KEYS, "ugk_dedup_static: batch too large");
  *n_unique = 0;
  if (key_bytes == 4)
    return dedup((const uint32_t *)keys, n, (uint32_t *)unique_out, inverse, rep, n_unique, n_unique_host);
  return dedup((const int64_t *)keys, n, (int64_t *)unique_out, inverse, rep, n_unique, n_unique_host);
}

int ugk_record_u32(const uint32_t *keys, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts,
                   uint64_t num_rows, uint64_t *observed, uint32_t *status, uint32_t *mirror, void *) {
  return record(keys, n, key_inv, key_mask, counts, num_rows, observed, status, mirror);
}
int ugk_record_i64(const int64_t *keys, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts,
                   uint64_t num_rows, uint64_t *observed, uint32_t *status, uint32_t *mirror, void *) {
  return record(keys, n, key_inv, key_mask, counts, num_rows, observed, status, mirror);
}
int ugk_record_restore(const uint64_t *entries, size_t n, uint32_t *counts, uint64_t num_rows, uint64_t *observed,
                       uint32_t *status, void *) {
  if (n == 0) return 0;
  REQUIRE(entries && counts && status, "ugk_record_restore: null pointer");
  for (size_t i = 0; i < n; ++i) {
    const uint32_t row = (uint32_t)entries[i], cnt = (uint32_t)(entries[i] >> 32);
    if (row >= num_rows) {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
      continue;
    }
    if (cnt == 0) continue;
    const uint32_t before = __atomic_fetch_add(counts + row, cnt, __ATOMIC_RELAXED);
    if (before == 0 && observed) __atomic_fetch_or(observed + (row >> 6), 1ull << (row & 63), __ATOMIC_RELAXED);
  }
  return 0;
}
int ugk_record_drain(uint32_t *counts, uint64_t first_row, uint64_t num_rows, uint64_t *observed, uint64_t *entries,
                     uint32_t capacity, uint32_t *n_entries, uint32_t *host_out, void *) {
  REQUIRE(counts && entries && n_entries && host_out && capacity, "ugk_record_drain: bad argument");
  uint32_t written = 0, more = 0;
  for (uint64_t r = first_row; r < first_row + num_rows; ++r) {
    if (ld(counts + r) == 0) continue;
    if (written == capacity) {
      more = 1;
      break;
    }
    if (observed) __atomic_fetch_and(observed + (r >> 6), ~(1ull << (r & 63)), __ATOMIC_RELAXED);
    const uint32_t got = __atomic_exchange_n(counts + r, 0u, __ATOMIC_RELAXED);
    entries[written++] = ((uint64_t)got << 32) | (uint32_t)r;
  }
  host_out[0] = written;
  host_out[1] = more;
  *n_entries = 0;
  return 0;
}

size_t ugk_rank_workspace_bytes(void) { return 64; }
int ugk_rank_place_keep(uint32_t *counts, uint64_t num_rows, uint64_t k, void *ws, uint64_t *in_new,
                        uint64_t *scratch, uint64_t *observed, const uint64_t *keep, int reset_counts, void *);
int ugk_rank_place(uint32_t *counts, uint64_t num_rows, uint64_t k, void *ws, uint64_t *in_new, uint64_t *scratch,
                   uint64_t *observed, int reset_counts, void *stream) {
  return ugk_rank_place_keep(counts, num_rows, k, ws, in_new, scratch, observed, nullptr, reset_counts, stream);
}
// rows ordered by (count, kept, tie) with tie = row for counted rows and 0xffffffff - row for the others: three
// 32-bit fields do not fit one word, so the kept bit goes between the count and the tie of a 128-bit key
int ugk_rank_place_keep(uint32_t *counts, uint64_t num_rows, uint64_t k, void *ws, uint64_t *in_new,
                        uint64_t *scratch, uint64_t *observed, const uint64_t *keep, int reset_counts, void *) {
  REQUIRE(counts && ws && in_new && scratch, "ugk_rank_place: null pointer");
  REQUIRE(keep != in_new && keep != scratch, "ugk_rank_place_keep: the keep bitmap is one of the output bitmaps");
  REQUIRE(num_rows > 0 && num_rows < 0xffffffffull, "ugk_rank_place: rows do not fit 32 bits");
  const uint64_t n_words = (num_rows + 63) / 64;
  typedef unsigned __int128 Rank;
  std::vector<Rank> rank(num_rows);
  for (uint64_t r = 0; r < num_rows; ++r) {
    const uint32_t c = ld(counts + r);
    const uint64_t kept = keep ? (ld(keep + r / 64) >> (r & 63)) & 1 : 0;
    rank[r] = ((Rank)c << 64) | ((Rank)kept << 32) | (c ? (uint32_t)r : 0xffffffffu - (uint32_t)r);
  }
  Rank threshold;
  if (k == 0) threshold = ~(Rank)0;
  else if (k >= num_rows) threshold = 0;
  else {
    std::vector<Rank> tmp(rank);
    std::nth_element(tmp.begin(), tmp.begin() + (k - 1), tmp.end(), std::greater<Rank>());
    threshold = tmp[k - 1];
  }
  for (uint64_t w = 0; w < n_words; ++w) {
    uint64_t m = 0;
    for (uint64_t r = w * 64; r < std::min(num_rows, w * 64 + 64); ++r)
      if (k != 0 && rank[r] >= threshold) m |= 1ull << (r & 63);
    in_new[w] = m;
    scratch[w] = 0;
  }
  if (reset_counts) {
    for (uint64_t r = 0; r < num_rows; ++r) st(counts + r, 0u);
    if (observed)
      for (uint64_t w = 0; w < n_words; ++w) st(observed + w, (uint64_t)0);
  }
  // reported without the kept bit: (count << 32) | row, or 0xffffffff - row
  const uint32_t th_count = (uint32_t)(threshold >> 64), th_tie = (uint32_t)threshold;
  *static_cast<uint64_t *>(ws) = k == 0 ? ~0ull : k >= num_rows ? 0ull : ((uint64_t)th_count << 32) | th_tie;
  return 0;
}
int ugk_rank_place_observed(uint32_t *counts, uint64_t num_rows, uint64_t k, void *ws, uint64_t *in_new,
                            uint64_t *observed, int reset_counts, const uint64_t *cached, void *evict_ws,
                            void *insert_ws, uint32_t *totals_host, uint32_t *status, void *) {
  REQUIRE(ws && in_new && observed && status, "ugk_rank_place_observed: null pointer");
  REQUIRE(counts || !reset_counts, "ugk_rank_place_observed: counters to reset, but no counters");
  REQUIRE(num_rows > 0 && num_rows < 0xffffffffull, "ugk_rank_place_observed: rows do not fit 32 bits");
  REQUIRE(k > 0 && k < num_rows, "ugk_rank_place_observed: k outside (0, rows)");
  REQUIRE(in_new != observed && cached != in_new, "ugk_rank_place_observed: output bitmap is an input bitmap");
  REQUIRE(!cached || (evict_ws && insert_ws && totals_host && evict_ws != insert_ws),
          "ugk_rank_place_observed: counting what changes needs two workspaces and the host words");
  const uint64_t n_words = (num_rows + 63) / 64;
  uint64_t seen = 0;
  for (uint64_t w = 0; w < n_words; ++w) seen += __builtin_popcountll(ld(observed + w));
  if (totals_host) totals_host[2] = (uint32_t)seen;
  if (seen >= k) {
    or_status(status, UGK_ST_PLACE_PROMISE);
    if (cached) totals_host[0] = totals_host[1] = 0;
    return 0;
  }
  uint64_t need = k - seen, last_row = 0;
  uint32_t leaving = 0, coming = 0;
  for (uint64_t w = 0; w < n_words; ++w) {
    const uint64_t obs = ld(observed + w);
    uint64_t m = obs;
    for (uint64_t r = w * 64; r < std::min(num_rows, w * 64 + 64) && need; ++r)
      if (!((obs >> (r & 63)) & 1)) {
        m |= 1ull << (r & 63);
        last_row = r;
        --need;
      }
    in_new[w] = m;
    if (cached) {
      leaving += __builtin_popcountll(ld(cached + w) & ~m);
      coming += __builtin_popcountll(m & ~ld(cached + w));
    }
  }
  if (cached) {
    *static_cast<uint32_t *>(evict_ws) = totals_host[0] = leaving;
    *static_cast<uint32_t *>(insert_ws) = totals_host[1] = coming;
  }
  if (reset_counts) {
    for (uint64_t r = 0; r < num_rows; ++r) st(counts + r, 0u);
    for (uint64_t w = 0; w < n_words; ++w) st(observed + w, (uint64_t)0);
  }
  *static_cast<uint64_t *>(ws) = 0xffffffffull - last_row;
  return 0;
}
int ugk_rank_threshold(const void *ws, uint64_t *threshold_host, void *) {
  *threshold_host = *static_cast<const uint64_t *>(ws);
  return 0;
}
size_t ugk_bitmap_workspace_bytes(void) { return 64; }
int ugk_bitmap_count(const uint64_t *a, const uint64_t *b, int invert_a, uint64_t nbits, void *ws,
                     uint32_t *total_host, void *) {
  REQUIRE(a && ws && nbits > 0 && nbits <= 0xffffffffull, "ugk_bitmap_count: bad argument");
  uint32_t total = 0;
  for (uint64_t w = 0; w < (nbits + 63) / 64; ++w) total += __builtin_popcountll(bm_word(a, b, invert_a, nbits, w));
  *static_cast<uint32_t *>(ws) = total;
  if (total_host) *total_host = total;
  return 0;
}
int ugk_bitmap_emit(const uint64_t *a, const uint64_t *b, int invert_a, uint64_t nbits, const void *ws, uint32_t *out,
                    uint64_t max_out, void *) {
  REQUIRE(a && ws && nbits > 0 && nbits <= 0xffffffffull, "ugk_bitmap_emit: bad argument");
  if (max_out == 0) return 0;
  REQUIRE(out, "ugk_bitmap_emit: null output list");
  uint64_t pos = 0;
  for (uint64_t w = 0; w < (nbits + 63) / 64 && pos < max_out; ++w) {
    uint64_t m = bm_word(a, b, invert_a, nbits, w);
    while (m && pos < max_out) {
      out[pos++] = (uint32_t)(w * 64 + __builtin_ctzll(m));
      m &= m - 1;
    }
  }
  return 0;
}
int ugk_bitmap_count_diff(const uint64_t *a, const uint64_t *b, uint64_t nbits, void *ws_ab, void *ws_ba,
                          uint32_t *totals_host, void *stream) {
  REQUIRE(a && b && ws_ab && ws_ba && ws_ab != ws_ba, "ugk_bitmap_count_diff: bad argument");
  if (int rc = ugk_bitmap_count(a, b, 0, nbits, ws_ab, totals_host, stream)) return rc;
  return ugk_bitmap_count(b, a, 0, nbits, ws_ba, totals_host ? totals_host + 1 : nullptr, stream);
}
int ugk_bitmap_emit_diff(const uint64_t *a, const uint64_t *b, uint64_t nbits, const void *ws_ab, const void *ws_ba,
                         uint32_t *out_ab, uint64_t max_ab, uint32_t *out_ba, uint64_t max_ba, void *stream) {
  REQUIRE(a && b && ws_ab && ws_ba, "ugk_bitmap_emit_diff: null pointer");
  if (int rc = ugk_bitmap_emit(a, b, 0, nbits, ws_ab, out_ab, max_ab, stream)) return rc;
  return ugk_bitmap_emit(b, a, 0, nbits, ws_ba, out_ba, max_ba, stream);
}
int ugk_bitmap_update(uint64_t *bitmap, uint64_t nbits, const uint32_t *idx, size_t n, int set, uint32_t *status,
                      void *) {
  if (n == 0) return 0;
  REQUIRE(bitmap && idx && status, "ugk_bitmap_update: null pointer");
  for (size_t i = 0; i < n; ++i) {
    const uint32_t p = idx[i];
    if (p >= nbits) {
      or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
      continue;
    }
    if (set) __atomic_fetch_or(bitmap + (p >> 6), 1ull << (p & 63), __ATOMIC_RELAXED);
    else __atomic_fetch_and(bitmap + (p >> 6), ~(1ull << (p & 63)), __ATOMIC_RELAXED);
  }
  return 0;
}
int ugk_bitmap_set_through(uint64_t *bitmap, uint64_t nbits, const uint32_t *last_pos, uint32_t *status, void *) {
  REQUIRE(bitmap && last_pos && status && nbits, "ugk_bitmap_set_through: bad argument");
  if (*last_pos >= nbits) {
    or_status(status, UGK_ST_KEY_OUT_OF_RANGE);
    return 0;
  }
  for (uint64_t p = 0; p <= *last_pos; ++p) __atomic_fetch_or(bitmap + (p >> 6), 1ull << (p & 63), __ATOMIC_RELAXED);
  return 0;
}
int ugk_rows_to_keys(const uint32_t *rows, size_t n, uint64_t mul, uint64_t mask, int64_t *keys_out, void *) {
  REQUIRE(n == 0 || (rows && keys_out && (mul & 1ull)), "ugk_rows_to_keys: bad argument");
  for (size_t i = 0; i < n; ++i) keys_out[i] = (int64_t)(((uint64_t)rows[i] * mul) & mask);
  return 0;
}

}  // extern "C"
