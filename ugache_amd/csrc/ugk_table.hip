// Table maintenance kernels: init, insert, evict, plain lookup, census.
// Insert and evict run at cache-fill / refresh time only, so they use a simple per-lane probe loop; the
// per-batch lookup is the wavefront-cooperative one in ugk_table.cuh.
#include <cmath>
#include <cstddef>

#include "ugk_internal.h"
#include "ugk_table.cuh"

namespace ugk {
namespace {

__global__ __launch_bounds__(kBlock) void hash_init_kernel(ugk_bucket_t *table, size_t nb) {
  const u32x4 empty = {0xffffffffu, 0xffffffffu, 0u, 0u};
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < nb; i += (size_t)gridDim.x * kBlock)
    *reinterpret_cast<u32x4 *>(table + i) = empty;
}

template <typename K>
__global__ __launch_bounds__(kBlock) void flat_insert_kernel(uint32_t *table, uint64_t nkeys, const K *keys,
                                                             const uint32_t *offs, uint32_t seq_base, uint32_t loc,
                                                             size_t n, uint32_t *status) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    const uint64_t key = key_to_u64<K>(keys[i]);
    const uint32_t off = offs ? offs[i] : seq_base + (uint32_t)i;
    if (key >= nkeys || off > 0x0fffffffu) {
      atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
      continue;
    }
    const uint32_t old = atomicExch(table + key, (loc << 28) + off);
    if (old != UGK_EMPTY_U32) atomicOr(status, UGK_ST_DUP_KEY);
  }
}

// slot_bits (may be null): one bit per cache slot; the bit of the slot an evicted key held is cleared on the way
__device__ __forceinline__ void release_slot(unsigned long long *slot_bits, uint64_t nslots, uint32_t slot,
                                             uint32_t *status) {
  if (slot_bits == nullptr) return;
  if (slot >= nslots) {
    atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
    return;
  }
  atomicAnd(slot_bits + (slot >> 6), ~(1ull << (slot & 63u)));
}

template <typename K>
__global__ __launch_bounds__(kBlock) void flat_evict_kernel(uint32_t *table, uint64_t nkeys, const K *keys, size_t n,
                                                            unsigned long long *slot_bits, uint64_t nslots,
                                                            uint32_t *status) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    const uint64_t key = key_to_u64<K>(keys[i]);
    if (key >= nkeys) {
      atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
      continue;
    }
    const uint32_t old = atomicExch(table + key, UGK_EMPTY_U32);
    if (old == UGK_EMPTY_U32) atomicOr(status, UGK_ST_EVICT_ABSENT);
    else release_slot(slot_bits, nslots, old & 0x0fffffffu, status);
  }
}

__device__ __forceinline__ uint64_t load_key_relaxed(const ugk_bucket_t *b) {
  return __atomic_load_n(&b->key, __ATOMIC_RELAXED);
}

// off and meta are the second 8 bytes of a bucket: one aligned 8-byte store changes both at once
__device__ __forceinline__ void store_off_meta(ugk_bucket_t *b, uint32_t off, uint32_t meta) {
  static_assert(offsetof(ugk_bucket_t, off) == 8 && offsetof(ugk_bucket_t, meta) == 12 && sizeof(ugk_bucket_t) == 16,
                "bucket layout");
  __atomic_store_n(reinterpret_cast<uint64_t *>(&b->off), ((uint64_t)meta << 32) | off, __ATOMIC_RELAXED);
}

// Insert, eight keys per wavefront: an 8-lane group walks one key's probe sequence a 128-byte line (eight buckets) at a
// time, as the lookup does.  The key goes into the first reusable bucket of its probe sequence (a tombstone, else the
// first never-used bucket), but only once the whole sequence up to that never-used bucket has been seen not to hold the
// key already: a tombstone in front of a live copy of the key must not hide it.  With tombstones piling up between
// rebuilds that walk is tens of buckets long, which one lane per key did as a chain of dependent 16-byte loads (462 k
// keys into a 71 M-bucket table with 13 % tombstones: 207 us; the groups: 87 us).  One lane per key reading a whole
// line per step (eight loads in flight) was measured too: 99 us for the insert, 75 instead of 88 us for the evict
// below — what is left is a device-scope atomic per key (the CAS here, the slot bitmap there): a kernel that does
// little else than one such atomic per key takes 44 us for the same 462 k keys, whatever walk comes in front of it.
// Keys of one launch are distinct,
// so the only contest is for buckets; a group that loses one starts its walk again.
template <typename K>
__global__ __launch_bounds__(kBlock) void hash_insert_kernel(ugk_bucket_t *table, uint64_t nb, const K *keys,
                                                             const uint32_t *offs, uint32_t seq_base, uint32_t loc,
                                                             size_t n, uint32_t *status) {
  constexpr uint64_t kNone = ~0ull;
  const int lane = (int)lane_id();
  const int grp = lane >> 3, sub = lane & 7;
  const size_t wave = ((size_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  const size_t n_waves = (size_t)gridDim.x * (kBlock / kWave);
  const uint64_t lines = nb >> 3;
  for (size_t i0 = wave * 8; i0 < n; i0 += n_waves * 8) {  // wavefront-uniform: every ballot below sees all 64 lanes
    const size_t i = i0 + grp;
    const bool active = i < n;
    const uint64_t key = active ? key_to_u64<K>(keys[i]) : 0;
    const uint32_t off = active ? (offs ? offs[i] : seq_base + (uint32_t)i) : 0;
    bool done = !active;
    if (active && key_is_reserved(key)) {
      if (sub == 0) atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
      done = true;
    }
    const uint64_t home = done ? 0 : hash_home(key, nb);
    uint64_t win = home, first_tomb = kNone, steps = 0;
    while (__ballot(!done)) {
      uint64_t cur = 0;  // reads as some other key
      if (!done) cur = load_key_relaxed(table + win + sub);
      const uint32_t mb = (uint32_t)((__ballot(!done && cur == key) >> (grp * 8)) & 0xffull);
      const uint32_t eb = (uint32_t)((__ballot(!done && cur == UGK_HASH_EMPTY) >> (grp * 8)) & 0xffull);
      const uint32_t tb = (uint32_t)((__ballot(!done && cur == UGK_HASH_TOMB) >> (grp * 8)) & 0xffull);
      // what the group does with this line: 0 walk on, 1 the key is there already, 2 claim `target`
      int action = 0;
      uint64_t target = 0, expect = 0;
      if (!done) {
        const int fe = eb ? (__ffs(eb) - 1) : 8;
        const uint32_t in_front = fe < 8 ? ((1u << fe) - 1u) : 0xffu;  // buckets in front of the first never-used one
        if (mb & in_front) {
          action = 1;
        } else {
          if (first_tomb == kNone && (tb & in_front)) first_tomb = win + (uint64_t)(__ffs(tb & in_front) - 1);
          const bool lap_done = steps >= lines && first_tomb != kNone;  // no never-used bucket at all: take the tombstone
          if (fe < 8 || lap_done) {
            action = 2;
            target = first_tomb != kNone ? first_tomb : win + (uint64_t)fe;
            expect = first_tomb != kNone ? UGK_HASH_TOMB : UGK_HASH_EMPTY;
          }
        }
      }
      uint64_t seen = 0;
      if (action == 2 && sub == 0)
        seen = atomicCAS(reinterpret_cast<unsigned long long *>(&table[target].key), (unsigned long long)expect,
                         (unsigned long long)key);
      seen = shfl64(seen, grp * 8);
      if (action == 1) {
        if (sub == 0) atomicOr(status, UGK_ST_DUP_KEY);
        done = true;
      } else if (action == 2) {
        if (seen == expect) {
          // the bucket is ours: slot and valid bit appear together, in one 8-byte store.  Until then the bucket reads
          // as "key present, not valid", i.e. as a miss.
          if (sub == 0) store_off_meta(table + target, off, UGK_META_VALID | (loc & 0xfu));
          done = true;
        } else {  // another key of this launch took it: walk again from the start (rare)
          win = home;
          first_tomb = kNone;
          steps = 0;
        }
      } else if (!done) {
        win += 8;
        if (win >= nb) win = 0;
        if (++steps > 2 * lines + 2) {
          if (sub == 0) atomicOr(status, UGK_ST_TABLE_FULL);
          done = true;
        }
      }
    }
  }
}

template <typename K>
__global__ __launch_bounds__(kBlock) void hash_evict_kernel(ugk_bucket_t *table, uint64_t nb, const K *keys,
                                                            size_t n, unsigned long long *slot_bits, uint64_t nslots,
                                                            uint32_t *status) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    const uint64_t key = key_to_u64<K>(keys[i]);
    uint64_t pos = key_is_reserved(key) ? 0 : hash_home(key, nb);
    bool done = key_is_reserved(key);
    if (done) atomicOr(status, UGK_ST_EVICT_ABSENT);
    for (uint64_t step = 0; step < nb && !done; ++step) {
      const uint64_t cur = load_key_relaxed(table + pos);
      if (cur == key) {
        if (slot_bits) release_slot(slot_bits, nslots, __atomic_load_n(&table[pos].off, __ATOMIC_RELAXED), status);
        // either order of these two stores is safe for a concurrent lookup: it sees the key still valid (its slot
        // keeps the row until a later lookup has passed), not valid, or gone
        store_off_meta(table + pos, 0u, 0u);
        __atomic_store_n(&table[pos].key, UGK_HASH_TOMB, __ATOMIC_RELAXED);
        done = true;
      } else if (cur == UGK_HASH_EMPTY) {
        atomicOr(status, UGK_ST_EVICT_ABSENT);
        done = true;
      } else if (++pos == nb) {
        pos = 0;
      }
    }
    if (!done) atomicOr(status, UGK_ST_EVICT_ABSENT);
  }
}

// ---- the compact table (kind 3): one 8-byte word per entry, sixteen to a line ------------------------------------
__global__ __launch_bounds__(kBlock) void h32_init_kernel(unsigned long long *table, size_t n) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
    table[i] = kH32EmptyWord;
}

// Insert, eight keys per wavefront, as hash_insert_kernel: an 8-lane group walks one key's probe sequence a line
// (sixteen entries, two per lane) at a time up to the first never-used entry, so that a tombstone in front of a live
// copy of the key cannot hide it, and claims the first reusable entry with one compare-and-swap on the whole word:
// row and value appear together.
// (Sixty-four keys per wavefront, the home lines of all of them requested before any is looked at, as the lookup does,
// was built for insert and evict and timed on 462,000 keys in a table of 71 M entries: 50 and 25 us either way.  What
// the kernels wait for is the line read and, for the insert, the compare-and-swap behind it, not the number of
// wavefronts.)
template <typename K>
__global__ __launch_bounds__(kBlock) void h32_insert_kernel(ugk_table_t t, const K *keys, const uint32_t *offs,
                                                            uint32_t seq_base, uint32_t loc, size_t n,
                                                            uint32_t *status) {
  constexpr uint64_t kNone = ~0ull;
  unsigned long long *table = reinterpret_cast<unsigned long long *>(t.table);
  const uint64_t ne = t.size;
  const int lane = (int)lane_id();
  const int grp = lane >> 3, sub = lane & 7;
  const size_t wave = ((size_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  const size_t n_waves = (size_t)gridDim.x * (kBlock / kWave);
  const uint64_t lines = ne >> 4;
  for (size_t i0 = wave * 8; i0 < n; i0 += n_waves * 8) {  // wavefront-uniform: every ballot below sees all 64 lanes
    const size_t i = i0 + grp;
    const bool active = i < n;
    const uint64_t row = active ? h32_row(t, key_to_u64<K>(keys[i])) : 0;
    const uint32_t off = active ? (offs ? offs[i] : seq_base + (uint32_t)i) : 0;
    bool done = !active;
    if (active && (row >= kH32Tomb || off > 0x0fffffffu)) {
      if (sub == 0) atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
      done = true;
    }
    const uint32_t r32 = (uint32_t)row;
    const uint64_t home = done ? 0 : h32_home(row, ne);
    uint64_t win = home, first_tomb = kNone, steps = 0;
    while (__ballot(!done)) {
      uint32_t k0 = 0, k1 = 0;  // read as some other key
      if (!done) {
        k0 = (uint32_t)__atomic_load_n(table + win + 2 * sub, __ATOMIC_RELAXED);
        k1 = (uint32_t)__atomic_load_n(table + win + 2 * sub + 1, __ATOMIC_RELAXED);
      }
      const int sh = grp * 8;
      const uint32_t mb = h32_interleave((uint32_t)(__ballot(!done && k0 == r32) >> sh),
                                         (uint32_t)(__ballot(!done && k1 == r32) >> sh));
      const uint32_t eb = h32_interleave((uint32_t)(__ballot(!done && k0 == kH32Empty) >> sh),
                                         (uint32_t)(__ballot(!done && k1 == kH32Empty) >> sh));
      const uint32_t tb = h32_interleave((uint32_t)(__ballot(!done && k0 == kH32Tomb) >> sh),
                                         (uint32_t)(__ballot(!done && k1 == kH32Tomb) >> sh));
      int action = 0;  // 0 walk on, 1 the key is there already, 2 claim `target`
      uint64_t target = 0, expect = 0;
      if (!done) {
        const int fe = eb ? (__ffs(eb) - 1) : 16;
        const uint32_t in_front = fe < 16 ? ((1u << fe) - 1u) : 0xffffu;  // entries in front of the first never-used one
        if (mb & in_front) {
          action = 1;
        } else {
          if (first_tomb == kNone && (tb & in_front)) first_tomb = win + (uint64_t)(__ffs(tb & in_front) - 1);
          const bool lap_done = steps >= lines && first_tomb != kNone;  // no never-used entry at all: take the tombstone
          if (fe < 16 || lap_done) {
            action = 2;
            target = first_tomb != kNone ? first_tomb : win + (uint64_t)fe;
            expect = first_tomb != kNone ? kH32TombWord : kH32EmptyWord;
          }
        }
      }
      uint64_t seen = 0;
      if (action == 2 && sub == 0)
        seen = atomicCAS(table + target, (unsigned long long)expect,
                         ((unsigned long long)(((loc & 0xfu) << 28) + off) << 32) | r32);
      seen = shfl64(seen, grp * 8);
      if (action == 1) {
        if (sub == 0) atomicOr(status, UGK_ST_DUP_KEY);
        done = true;
      } else if (action == 2) {
        if (seen == expect) {
          done = true;
        } else {  // another key of this launch took it: walk again from the start (rare)
          win = home;
          first_tomb = kNone;
          steps = 0;
        }
      } else if (!done) {
        win += 16;
        if (win >= ne) win = 0;
        if (++steps > 2 * lines + 2) {
          if (sub == 0) atomicOr(status, UGK_ST_TABLE_FULL);
          done = true;
        }
      }
    }
  }
}

// Evict, eight keys per wavefront: an 8-lane group reads its key's probe sequence a line at a time; the lane that holds
// the key's entry stores the tombstone word and releases the slot.  A live key sits in front of the first never-used
// entry of its sequence (inserts only ever take entries in front of it, evictions leave tombstones), so a line with
// the key in it settles the walk whatever else it holds, and one without the key but with a never-used entry ends it.
template <typename K>
__global__ __launch_bounds__(kBlock) void h32_evict_kernel(ugk_table_t t, const K *keys, size_t n,
                                                           unsigned long long *slot_bits, uint64_t nslots,
                                                           uint32_t *status) {
  unsigned long long *table = reinterpret_cast<unsigned long long *>(t.table);
  const uint64_t ne = t.size;
  const int lane = (int)lane_id();
  const int grp = lane >> 3, sub = lane & 7;
  const size_t wave = ((size_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  const size_t n_waves = (size_t)gridDim.x * (kBlock / kWave);
  const uint64_t lines = ne >> 4;
  for (size_t i0 = wave * 8; i0 < n; i0 += n_waves * 8) {  // wavefront-uniform: every ballot below sees all 64 lanes
    const size_t i = i0 + grp;
    const bool active = i < n;
    const uint64_t row = active ? h32_row(t, key_to_u64<K>(keys[i])) : 0;
    bool done = !active;
    if (active && row >= kH32Tomb) {  // no entry can hold it
      if (sub == 0) atomicOr(status, UGK_ST_EVICT_ABSENT);
      done = true;
    }
    const uint32_t r32 = (uint32_t)row;
    uint64_t win = done ? 0 : h32_home(row, ne), steps = 0;
    while (__ballot(!done)) {
      unsigned long long w0 = 0, w1 = 0;  // read as some other key
      if (!done) {
        w0 = __atomic_load_n(table + win + 2 * sub, __ATOMIC_RELAXED);
        w1 = __atomic_load_n(table + win + 2 * sub + 1, __ATOMIC_RELAXED);
      }
      const bool m0 = !done && (uint32_t)w0 == r32, m1 = !done && (uint32_t)w1 == r32;
      const int sh = grp * 8;
      const uint32_t hit = (uint32_t)(__ballot(m0 || m1) >> sh) & 0xffu;
      const uint32_t never = (uint32_t)(__ballot(!done && (w0 == kH32EmptyWord || w1 == kH32EmptyWord)) >> sh) & 0xffu;
      // The slots of the keys found in this step leave the slot bitmap.  Neighbouring keys of an evict list often hold
      // neighbouring slots (a refresh evicts runs of rows that went in together), whose bits share a word: the lanes
      // of the wavefront that hold a found entry merge their bits per word first, one atomic per word.
      const bool mine = !done && (m0 || m1);
      if (slot_bits) {
        const uint32_t slot = (uint32_t)((m0 ? w0 : w1) >> 32) & 0x0fffffffu;
        bool todo = mine;
        if (mine && slot >= nslots) {
          atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
          todo = false;
        }
        unsigned long long left = __ballot(todo);
        while (left) {  // wavefront-uniform: at most eight lanes hold an entry
          const int lead = __ffsll(left) - 1;
          const uint32_t word = __shfl(slot >> 6, lead);
          const bool same = todo && (slot >> 6) == word;
          const unsigned long long group = __ballot(same);
          unsigned long long bits = 0;
          for (unsigned long long g = group; g; g &= g - 1) {
            const int l = __ffsll(g) - 1;
            bits |= 1ull << (__shfl(slot, l) & 63u);
          }
          if (lane == lead) atomicAnd(slot_bits + word, ~bits);
          left &= ~group;
        }
      }
      if (!done) {
        if (hit) {
          if (mine) {
            // the entry leaves whole: a concurrent lookup sees the key there (its slot keeps the row until a later
            // lookup has passed) or gone
            __atomic_store_n(table + win + 2 * sub + (m0 ? 0 : 1), kH32TombWord, __ATOMIC_RELAXED);
          }
          done = true;
        } else if (never || ++steps > lines) {
          if (sub == 0) atomicOr(status, UGK_ST_EVICT_ABSENT);
          done = true;
        } else {
          win += 16;
          if (win >= ne) win = 0;
        }
      }
    }
  }
}

__global__ __launch_bounds__(kBlock) void h32_census_kernel(const unsigned long long *table, size_t n,
                                                            unsigned long long *census) {
  unsigned long long occ = 0, tomb = 0, empty = 0;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    const uint32_t k = (uint32_t)table[i];
    if (k == kH32Empty) ++empty;
    else if (k == kH32Tomb) ++tomb;
    else ++occ;
  }
  __shared__ unsigned long long red[3];
  if (threadIdx.x < 3) red[threadIdx.x] = 0;
  __syncthreads();
  atomicAdd(&red[0], occ);
  atomicAdd(&red[1], tomb);
  atomicAdd(&red[2], empty);
  __syncthreads();
  if (threadIdx.x < 3) atomicAdd(census + threadIdx.x, red[threadIdx.x]);
}

template <typename K, int KIND>
__global__ __launch_bounds__(kBlock) void lookup_kernel(ugk_table_t t, const K *keys, size_t n, uint32_t fallback_loc,
                                                        uint32_t *loc_out, uint32_t *off_out) {
  // whole wavefronts stay in the loop together: the hash lookup is cooperative
  const size_t n_round = (n + kWave - 1) / kWave * kWave;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n_round; i += (size_t)gridDim.x * kBlock) {
    const bool active = i < n;
    const uint64_t key = active ? key_to_u64<K>(keys[i]) : 0;
    const Found f = table_lookup<KIND>(t, key, active);
    if (active) {
      if (loc_out) loc_out[i] = f.hit ? f.loc : fallback_loc;
      if (off_out) off_out[i] = f.hit ? f.off : (uint32_t)fallback_row(t, key);
    }
  }
}

__global__ __launch_bounds__(kBlock) void census_kernel(const ugk_bucket_t *table, size_t nb,
                                                        unsigned long long *census) {
  unsigned long long occ = 0, tomb = 0, empty = 0;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < nb; i += (size_t)gridDim.x * kBlock) {
    const uint64_t k = table[i].key;
    if (k == UGK_HASH_EMPTY) ++empty;
    else if (k == UGK_HASH_TOMB) ++tomb;
    else ++occ;
  }
  __shared__ unsigned long long red[3];
  if (threadIdx.x < 3) red[threadIdx.x] = 0;
  __syncthreads();
  atomicAdd(&red[0], occ);
  atomicAdd(&red[1], tomb);
  atomicAdd(&red[2], empty);
  __syncthreads();
  if (threadIdx.x < 3) atomicAdd(census + threadIdx.x, red[threadIdx.x]);
}

int check_table(const ugk_table_t &t, const char *who) {
  UGK_REQUIRE(t.kind >= 1 && t.kind <= 3, "%s: table kind %d is not flat(1), hash(2) or compact hash(3)", who, t.kind);
  UGK_REQUIRE(t.table != nullptr && t.size > 0, "%s: empty table", who);
  if (t.kind == 2) {
    UGK_REQUIRE(t.size % 8 == 0, "%s: hash table needs a multiple of 8 buckets, got %llu", who,
                (unsigned long long)t.size);
    UGK_REQUIRE((uintptr_t)t.table % 128 == 0, "%s: hash table must be 128-byte aligned", who);
  }
  if (t.kind == 3) {
    UGK_REQUIRE(t.size % 16 == 0 && (t.size >> 4) <= 0xffffffffull,
                "%s: compact hash table needs a multiple of 16 entries and at most 2^32 lines, got %llu", who,
                (unsigned long long)t.size);
    UGK_REQUIRE((uintptr_t)t.table % 128 == 0, "%s: hash table must be 128-byte aligned", who);
  }
  return 0;
}

template <typename K>
int table_insert(ugk_table_t t, const K *keys, const uint32_t *offs, uint32_t seq_base, uint32_t loc, size_t n,
                 uint32_t *status, void *stream) {
  if (n == 0) return 0;
  if (check_table(t, "ugk_table_insert")) return 1;
  UGK_REQUIRE(keys && status, "ugk_table_insert: null keys or status");
  UGK_REQUIRE(loc < 16, "ugk_table_insert: location %u does not fit 4 bits", loc);
  const unsigned grid = clamp_grid((n + kBlock - 1) / kBlock, 0);
  if (t.kind == 1)
    hipLaunchKernelGGL(flat_insert_kernel<K>, dim3(grid), dim3(kBlock), 0, as_stream(stream), (uint32_t *)t.table,
                       t.size, keys, offs, seq_base, loc, n, status);
  else if (t.kind == 2)
    hipLaunchKernelGGL(hash_insert_kernel<K>, dim3(clamp_grid((n + 31) / 32, 0)), dim3(kBlock), 0, as_stream(stream),
                       (ugk_bucket_t *)t.table, t.size, keys, offs, seq_base, loc, n, status);
  else
    hipLaunchKernelGGL(h32_insert_kernel<K>, dim3(clamp_grid((n + 31) / 32, 0)), dim3(kBlock), 0, as_stream(stream),
                       t, keys, offs, seq_base, loc, n, status);
  UGK_HIP(hipGetLastError());
  return 0;
}

template <typename K>
int table_evict(ugk_table_t t, const K *keys, size_t n, uint64_t *slot_bits_dev, uint64_t nslots, uint32_t *status,
                void *stream) {
  if (n == 0) return 0;
  if (check_table(t, "ugk_table_evict")) return 1;
  UGK_REQUIRE(keys && status, "ugk_table_evict: null keys or status");
  unsigned long long *slot_bits = reinterpret_cast<unsigned long long *>(slot_bits_dev);
  const unsigned grid = clamp_grid((n + kBlock - 1) / kBlock, 0);
  if (t.kind == 1)
    hipLaunchKernelGGL(flat_evict_kernel<K>, dim3(grid), dim3(kBlock), 0, as_stream(stream), (uint32_t *)t.table,
                       t.size, keys, n, slot_bits, nslots, status);
  else if (t.kind == 2)
    hipLaunchKernelGGL(hash_evict_kernel<K>, dim3(grid), dim3(kBlock), 0, as_stream(stream), (ugk_bucket_t *)t.table,
                       t.size, keys, n, slot_bits, nslots, status);
  else
    hipLaunchKernelGGL(h32_evict_kernel<K>, dim3(clamp_grid((n + 31) / 32, 0)), dim3(kBlock), 0, as_stream(stream), t,
                       keys, n, slot_bits, nslots, status);
  UGK_HIP(hipGetLastError());
  return 0;
}

template <typename K>
int table_lookup_host(ugk_table_t t, const K *keys, size_t n, uint32_t fallback_loc, uint32_t *loc_out,
                      uint32_t *off_out, void *stream) {
  if (n == 0) return 0;
  if (check_table(t, "ugk_table_lookup")) return 1;
  UGK_REQUIRE(keys, "ugk_table_lookup: null keys");
  const unsigned grid = clamp_grid((n + kBlock - 1) / kBlock, 0);
  if (t.kind == 1)
    hipLaunchKernelGGL((lookup_kernel<K, 1>), dim3(grid), dim3(kBlock), 0, as_stream(stream), t, keys, n,
                       fallback_loc, loc_out, off_out);
  else if (t.kind == 2)
    hipLaunchKernelGGL((lookup_kernel<K, 2>), dim3(grid), dim3(kBlock), 0, as_stream(stream), t, keys, n,
                       fallback_loc, loc_out, off_out);
  else
    hipLaunchKernelGGL((lookup_kernel<K, 3>), dim3(grid), dim3(kBlock), 0, as_stream(stream), t, keys, n,
                       fallback_loc, loc_out, off_out);
  UGK_HIP(hipGetLastError());
  return 0;
}

}  // namespace
// an empty launch: what it costs is the load of this file's code object onto the device (see ugk_preload_kernels)
namespace {
__global__ void preload_table_kernel() {}
}  // namespace
void preload_table(hipStream_t stream) { hipLaunchKernelGGL(preload_table_kernel, dim3(1), dim3(1), 0, stream); }
}  // namespace ugk

using namespace ugk;

extern "C" {

size_t ugk_hash_buckets_for(size_t n_entries, double load_factor) {
  if (!(load_factor > 0.0) || load_factor > 0.95) load_factor = 0.7;
  size_t nb = (size_t)std::ceil((double)n_entries / load_factor) + 1;
  if (nb < 64) nb = 64;
  return (nb + 7) / 8 * 8;
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
  const unsigned grid = clamp_grid((t.size + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(h32_init_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream),
                     static_cast<unsigned long long *>(t.table), t.size);
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_table_census(ugk_table_t t, uint64_t *census_dev, void *stream) {
  if (check_table(t, "ugk_table_census")) return 1;
  UGK_REQUIRE(t.kind == 2 || t.kind == 3, "ugk_table_census: a flat table has no buckets to count");
  UGK_REQUIRE(census_dev, "ugk_table_census: null output");
  if (t.kind == 2) return ugk_hash_census(static_cast<const ugk_bucket_t *>(t.table), t.size, census_dev, stream);
  if (ugk_fill_u32(reinterpret_cast<uint32_t *>(census_dev), 0u, 6, stream)) return 1;
  const unsigned grid = clamp_grid((t.size + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(h32_census_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream),
                     static_cast<const unsigned long long *>(t.table), t.size,
                     reinterpret_cast<unsigned long long *>(census_dev));
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_hash_init(ugk_bucket_t *table_dev, size_t nbuckets, void *stream) {
  UGK_REQUIRE(table_dev && nbuckets > 0, "ugk_hash_init: empty table");
  UGK_REQUIRE(nbuckets % 8 == 0, "ugk_hash_init: bucket count must be a multiple of 8");
  const unsigned grid = clamp_grid((nbuckets + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(hash_init_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), table_dev, nbuckets);
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_table_insert_u32(ugk_table_t t, const uint32_t *keys_dev, const uint32_t *offs_dev, uint32_t seq_base,
                         uint32_t loc, size_t n, uint32_t *status_dev, void *stream) {
  return table_insert<uint32_t>(t, keys_dev, offs_dev, seq_base, loc, n, status_dev, stream);
}
int ugk_table_insert_i64(ugk_table_t t, const int64_t *keys_dev, const uint32_t *offs_dev, uint32_t seq_base,
                         uint32_t loc, size_t n, uint32_t *status_dev, void *stream) {
  return table_insert<int64_t>(t, keys_dev, offs_dev, seq_base, loc, n, status_dev, stream);
}
int ugk_table_evict_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint32_t *status_dev, void *stream) {
  return table_evict<uint32_t>(t, keys_dev, n, nullptr, 0, status_dev, stream);
}
int ugk_table_evict_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint32_t *status_dev, void *stream) {
  return table_evict<int64_t>(t, keys_dev, n, nullptr, 0, status_dev, stream);
}
int ugk_table_evict_release_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint64_t *slot_bits_dev,
                                uint64_t nslots, uint32_t *status_dev, void *stream) {
  UGK_REQUIRE(n == 0 || slot_bits_dev, "ugk_table_evict_release_u32: null slot bitmap");
  return table_evict<uint32_t>(t, keys_dev, n, slot_bits_dev, nslots, status_dev, stream);
}
int ugk_table_evict_release_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint64_t *slot_bits_dev,
                                uint64_t nslots, uint32_t *status_dev, void *stream) {
  UGK_REQUIRE(n == 0 || slot_bits_dev, "ugk_table_evict_release_i64: null slot bitmap");
  return table_evict<int64_t>(t, keys_dev, n, slot_bits_dev, nslots, status_dev, stream);
}
int ugk_table_lookup_u32(ugk_table_t t, const uint32_t *keys_dev, size_t n, uint32_t fallback_loc,
                         uint32_t *loc_out_dev, uint32_t *off_out_dev, void *stream) {
  return table_lookup_host<uint32_t>(t, keys_dev, n, fallback_loc, loc_out_dev, off_out_dev, stream);
}
int ugk_table_lookup_i64(ugk_table_t t, const int64_t *keys_dev, size_t n, uint32_t fallback_loc,
                         uint32_t *loc_out_dev, uint32_t *off_out_dev, void *stream) {
  return table_lookup_host<int64_t>(t, keys_dev, n, fallback_loc, loc_out_dev, off_out_dev, stream);
}

int ugk_hash_census(const ugk_bucket_t *table_dev, size_t nbuckets, uint64_t *census_dev, void *stream) {
  UGK_REQUIRE(table_dev && census_dev, "ugk_hash_census: null pointer");
  if (ugk_fill_u32(reinterpret_cast<uint32_t *>(census_dev), 0u, 6, stream)) return 1;
  const unsigned grid = clamp_grid((nbuckets + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(census_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), table_dev, nbuckets,
                     reinterpret_cast<unsigned long long *>(census_dev));
  UGK_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
