// Device-side lookup tables shared by the table, classify and fused-extraction kernels.
//
// flat table  : one uint32 per key of the key space, (loc << 28) + off, 0xffffffff = absent.
// hash table  : ugk_bucket_t[nbuckets] (16 bytes each, nbuckets a multiple of 8, base 128-byte aligned),
//               linear probing from home(key) = 8 * mulhi64(fmix64(key), nbuckets / 8): a probe sequence
//               starts at the first bucket of a 128-byte line, so at load 0.7 nine keys in ten are found
//               (or ruled out) inside the one line their lookup reads first.
//               A search stops at a never-used bucket, walks over tombstones and other keys.
//               A matching key only counts when its VALID bit is set; a key that is half-way through an
//               insert or an evict therefore reads as a miss, which is always correct because the host
//               table holds every row.
//
// compact hash table (kind 3): uint64[nentries] (nentries a multiple of 16, base 128-byte aligned), one word per entry:
//               low half = the ROW of the host table the key stands for (the key itself for dense ids, the inverse of
//               the sparse-id map otherwise: a bijection, so the 32-bit row identifies the key exactly), high half =
//               (loc << 28) + off as in the flat table.  Sixteen entries fill a 128-byte line, so at load 0.7 about
//               one key in a hundred is not settled by its home line (one in thirteen with the 16-byte buckets), and
//               the second, dependent round of a lookup all but disappears.  An entry appears and disappears whole
//               (one 8-byte word), so there is no "present, not yet valid" state.  0xffffffff_ffffffff = never used,
//               key half 0xfffffffe = tombstone; rows from 0xfffffffe on cannot be stored.
//
// Lookup is wavefront-cooperative: an 8-lane group reads one 128-byte line (eight adjacent buckets) of one key's
// probe sequence per step and a wavefront ballot decides match / never-used / continue.  Step 1 reads the
// home line of all 64 keys of the wavefront in eight rounds whose loads are independent of each other (all in
// flight together); step 2 follows the few keys whose home line was full without a match, eight at a time.
// A lookup therefore costs one line in the common case and never a chain of dependent 16-byte loads.
#pragma once

#include "ugk_internal.h"

namespace ugk {

__device__ __forceinline__ uint64_t fmix64(uint64_t x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdull;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ull;
  x ^= x >> 33;
  return x;
}

__device__ __forceinline__ uint64_t hash_home(uint64_t key, uint64_t nbuckets) {
  return __umul64hi(fmix64(key), nbuckets >> 3) << 3;
}

struct Found {
  bool hit;      // present and valid
  uint32_t loc;  // location of the row
  uint32_t off;  // row inside the location
};

__device__ __forceinline__ ugk_bucket_t load_bucket(const ugk_bucket_t *p) {
  const u32x4 v = *reinterpret_cast<const u32x4 *>(p);
  ugk_bucket_t b;
  b.key = ((uint64_t)v.y << 32) | v.x;
  b.off = v.z;
  b.meta = v.w;
  return b;
}

__device__ __forceinline__ uint64_t shfl64(uint64_t v, int src) {
  const uint32_t lo = __shfl((uint32_t)v, src);
  const uint32_t hi = __shfl((uint32_t)(v >> 32), src);
  return ((uint64_t)hi << 32) | lo;
}

// Flat lookup: one dependent 4-byte read.  Keys beyond the key space read as absent.
__device__ __forceinline__ Found flat_lookup(const uint32_t *table, uint64_t nkeys, uint64_t key, bool active) {
  Found f{false, 0, 0};
  if (active && key < nkeys) {
    const uint32_t v = table[key];
    if (v != UGK_EMPTY_U32) {
      f.hit = true;
      f.loc = (v >> 28) & 0xfu;
      f.off = v & 0x0fffffffu;
    }
  }
  return f;
}

// host row of a key that is not in the table
__device__ __forceinline__ uint64_t fallback_row(const ugk_table_t &t, uint64_t key) {
  if (t.fb_mul == 0) return key;
  return key <= t.fb_mask ? ((key * t.fb_mul) & t.fb_mask) : ~0ull;  // ids beyond the id space have no row
}
// the row a compact table (kind 3) stores a key under
__device__ __forceinline__ uint64_t h32_row(const ugk_table_t &t, uint64_t key) { return fallback_row(t, key); }

// Wavefront-cooperative hash lookup in two steps.  All 64 lanes of the wavefront must call both (inactive lanes pass
// active = false).
struct HashProbe {
  Found f;
  uint64_t next_win;  // first bucket of the line step 2 has to read next
  bool pending;       // the home line was full and did not hold the key
};

// step 1: the home line of every lane's key.  In round r the eight 8-lane groups serve lanes 8r .. 8r+7.
// PASSES = 2: two passes of four rounds, the four line loads of a pass in flight together; PASSES = 1: all eight
// rounds in flight at once, which saves a round trip to memory per wavefront and costs about 30 more vector
// registers (fewer wavefronts per SIMD: taken where the launch does not fill them all anyway).
// ROUNDS: a caller whose keys sit in lanes 0 .. 8 * ROUNDS - 1 only (a wavefront that resolves fewer than 64 keys at a
// time) runs that many rounds; the shuffles and ballots of a round cost the same whether its lanes hold keys or not.
template <int PASSES, int ROUNDS = 8>
__device__ __forceinline__ HashProbe hash_probe_home(const ugk_bucket_t *table, uint64_t nb, uint64_t key,
                                                     bool active) {
  static_assert(ROUNDS >= 1 && ROUNDS <= 8 && ROUNDS % PASSES == 0, "whole passes of rounds");
  constexpr int PER = ROUNDS / PASSES;  // rounds whose loads are in flight together
  HashProbe p{Found{false, 0, 0}, 0, false};
  const int lane = (int)lane_id();
  const int grp = lane >> 3, sub = lane & 7;
  const uint64_t home = active ? hash_home(key, nb) : 0;
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    u32x4 raw[PER];
    uint64_t kk[PER];
    bool act[PER];
#pragma unroll
    for (int q = 0; q < PER; ++q) {
      const int owner = (pass * PER + q) * 8 + grp;
      kk[q] = shfl64(key, owner);
      const uint64_t hb = shfl64(home, owner);
      act[q] = __shfl((int)active, owner) != 0;
      raw[q] = u32x4{0xffffffffu, 0xffffffffu, 0u, 0u};  // reads as a never-used bucket
      if (act[q]) raw[q] = *reinterpret_cast<const u32x4 *>(table + hb + sub);
    }
#pragma unroll
    for (int q = 0; q < PER; ++q) {
      const int r = pass * PER + q;
      const uint64_t bkey = ((uint64_t)raw[q].y << 32) | raw[q].x;
      const bool is_match = act[q] && bkey == kk[q];
      const bool is_empty = act[q] && bkey == UGK_HASH_EMPTY;
      const uint32_t mb = (uint32_t)((__ballot(is_match) >> (grp * 8)) & 0xffull);
      const uint32_t eb = (uint32_t)((__ballot(is_empty) >> (grp * 8)) & 0xffull);
      const int fm = mb ? (__ffs(mb) - 1) : 8;
      const int fe = eb ? (__ffs(eb) - 1) : 8;
      const bool g_found = fm < fe;  // a key sits in front of the first never-used bucket of its probe sequence
      const bool g_done = g_found || fe < 8;
      const int hit_lane = grp * 8 + (g_found ? fm : 0);
      const uint32_t h_off = __shfl(raw[q].z, hit_lane);
      const uint32_t h_meta = __shfl(raw[q].w, hit_lane);
      const uint32_t g_flags = (g_done ? 1u : 0u) | (g_found ? 2u : 0u);
      // the owner of this round's key served by group g is lane 8r + g: it reads its group's result
      const int from = (lane & 7) * 8;
      const uint32_t r_flags = __shfl(g_flags, from);
      const uint32_t r_off = __shfl(h_off, from);
      const uint32_t r_meta = __shfl(h_meta, from);
      if ((lane >> 3) == r && active) {
        if (r_flags & 1u) {
          if ((r_flags & 2u) && (r_meta & UGK_META_VALID)) {
            p.f.hit = true;
            p.f.loc = r_meta & 0xfu;
            p.f.off = r_off;
          }
        } else {
          p.pending = true;
        }
      }
    }
  }
  p.next_win = home + 8 >= nb ? 0 : home + 8;
  return p;
}

// step 2: the pending lanes are served eight at a time, one 128-byte line per 8-lane group and step
__device__ __forceinline__ Found hash_probe_rest(const ugk_bucket_t *table, uint64_t nb, uint64_t key, HashProbe p) {
  Found f = p.f;
  bool pending = p.pending;
  uint64_t pend = __ballot(pending);
  if (pend == 0) return f;

  const int lane = (int)lane_id();
  const int grp = lane >> 3, sub = lane & 7;
  uint64_t win = p.next_win;  // next 8-bucket window this lane's key has to examine
  uint64_t steps = 0;
  const uint64_t max_steps = nb / 8 + 1;    // a full lap: give up (table without a never-used bucket)

  while (pend) {
    // the g-th 8-lane group serves the g-th pending lane
    const int rank = __popcll(pend & ((1ull << lane) - 1ull));
    uint64_t m = pend;
    for (int i = 0; i < grp; ++i) m &= m - 1;
    const int src = m ? (__ffsll((unsigned long long)m) - 1) : -1;
    const bool gactive = src >= 0;
    const int from = gactive ? src : lane;
    const uint64_t k = shfl64(key, from);
    const uint64_t w = shfl64(win, from);

    bool is_match = false, is_empty = false;
    ugk_bucket_t bb{0, 0, 0};
    if (gactive) {
      bb = load_bucket(table + w + sub);
      is_match = bb.key == k;
      is_empty = bb.key == UGK_HASH_EMPTY;
    }
    const uint32_t mb = (uint32_t)((__ballot(is_match) >> (grp * 8)) & 0xffull);
    const uint32_t eb = (uint32_t)((__ballot(is_empty) >> (grp * 8)) & 0xffull);
    const int fm = mb ? (__ffs(mb) - 1) : 8;
    const int fe = eb ? (__ffs(eb) - 1) : 8;
    // linear probing keeps a key in front of the first never-used bucket of its probe sequence
    const bool g_found = fm < fe;
    const bool g_done = g_found || fe < 8;
    const int hit_lane = grp * 8 + (g_found ? fm : 0);
    const uint32_t h_off = __shfl(bb.off, hit_lane);
    const uint32_t h_meta = __shfl(bb.meta, hit_lane);
    // group-uniform result word: bit 0 done, bit 1 found
    const uint32_t g_flags = (g_done ? 1u : 0u) | (g_found ? 2u : 0u);

    // hand the result back to the lane that owns the key
    const bool served = pending && rank < 8;
    const int back = served ? rank * 8 : lane;
    const uint32_t r_flags = __shfl(g_flags, back);
    const uint32_t r_off = __shfl(h_off, back);
    const uint32_t r_meta = __shfl(h_meta, back);
    if (served) {
      if (r_flags & 1u) {
        pending = false;
        if ((r_flags & 2u) && (r_meta & UGK_META_VALID)) {
          f.hit = true;
          f.loc = r_meta & 0xfu;
          f.off = r_off;
        }
      } else {
        win += 8;
        if (win >= nb) win = 0;
        if (++steps > max_steps) pending = false;
      }
    }
    pend = __ballot(pending);
  }
  return f;
}

// ---- the compact table (kind 3) -----------------------------------------------------------------------------------
constexpr uint32_t kH32Empty = 0xffffffffu, kH32Tomb = 0xfffffffeu;
constexpr uint64_t kH32EmptyWord = ~0ull, kH32TombWord = 0x00000000fffffffeull;

__device__ __forceinline__ uint64_t h32_home(uint64_t row, uint64_t nentries) {
  return __umul64hi(fmix64(row), nentries >> 4) << 4;
}

// bit i of `even` to bit 2i, bit i of `odd` to bit 2i + 1: the sixteen entries of a line in their order, from the two
// per-lane predicates of an 8-lane group (what the insert orders tombstones and never-used entries by)
__device__ __forceinline__ uint32_t h32_interleave(uint32_t even, uint32_t odd) {
  auto spread = [](uint32_t b) {
    b = (b | (b << 4)) & 0x0f0fu;
    b = (b | (b << 2)) & 0x3333u;
    return (b | (b << 1)) & 0x5555u;
  };
  return spread(even & 0xffu) | (spread(odd & 0xffu) << 1);
}

struct H32Line {
  bool found, done;
  uint32_t val;  // group-uniform
};

// what one 128-byte line says about `row`: every lane of the 8-lane group passes the 16 bytes it read (entries
// 2 * sub and 2 * sub + 1); act is group-uniform.  All 64 lanes call it.  No order among the entries is needed:
// every probe sequence enters a line at its first entry, inserts take the first reusable entry and evictions leave
// tombstones, so the never-used entries of a line are its tail and a live key sits in front of them — a line that
// holds the key settles the lookup, one without it but with a never-used entry ends it.
// (Measured at 262,144 keys / 99 % hits: 51.6 us against 53.0 us with the entries' order worked out from four ballots;
// a probe that also sends the home line's number instead of its address and lets the key's lane fetch the value
// straight from the lane that holds the entry, three permutes per round instead of seven: 53.5 us.)
__device__ __forceinline__ H32Line h32_examine(const u32x4 &raw, uint32_t row, bool act, int grp) {
  const bool first = act && raw.x == row, second = act && raw.z == row;
  const uint32_t m = (uint32_t)(__ballot(first || second) >> (grp * 8)) & 0xffu;
  const uint32_t e = (uint32_t)(__ballot(act && (raw.x == kH32Empty || raw.z == kH32Empty)) >> (grp * 8)) & 0xffu;
  H32Line r;
  r.found = m != 0;
  r.done = r.found || e != 0;
  const uint32_t mine = first ? raw.y : raw.w;
  r.val = __shfl(mine, grp * 8 + (m ? __ffs(m) - 1 : 0));
  return r;
}

template <int PASSES, int ROUNDS = 8>
__device__ __forceinline__ HashProbe h32_probe_home(const uint64_t *table, uint64_t n, uint64_t row, bool active) {
  static_assert(ROUNDS >= 1 && ROUNDS <= 8 && ROUNDS % PASSES == 0, "whole passes of rounds");
  constexpr int PER = ROUNDS / PASSES;
  HashProbe p{Found{false, 0, 0}, 0, false};
  const int lane = (int)lane_id();
  const int grp = lane >> 3, sub = lane & 7;
  const uint64_t home = active ? h32_home(row, n) : 0;
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    u32x4 raw[PER];
    uint32_t kk[PER];
    bool act[PER];
#pragma unroll
    for (int q = 0; q < PER; ++q) {
      const int owner = (pass * PER + q) * 8 + grp;
      kk[q] = __shfl((uint32_t)row, owner);
      const uint64_t hb = shfl64(home, owner);
      act[q] = __shfl((int)active, owner) != 0;
      raw[q] = u32x4{kH32Empty, kH32Empty, kH32Empty, kH32Empty};  // reads as never-used entries
      if (act[q]) raw[q] = reinterpret_cast<const u32x4 *>(table + hb)[sub];
    }
#pragma unroll
    for (int q = 0; q < PER; ++q) {
      const int r = pass * PER + q;
      const H32Line line = h32_examine(raw[q], kk[q], act[q], grp);
      const uint32_t g_flags = (line.done ? 1u : 0u) | (line.found ? 2u : 0u);
      const int from = (lane & 7) * 8;  // the owner of this round's key served by group g is lane 8r + g
      const uint32_t r_flags = __shfl(g_flags, from);
      const uint32_t r_val = __shfl(line.val, from);
      if ((lane >> 3) == r && active) {
        if (r_flags & 1u) {
          if (r_flags & 2u) {
            p.f.hit = true;
            p.f.loc = (r_val >> 28) & 0xfu;
            p.f.off = r_val & 0x0fffffffu;
          }
        } else {
          p.pending = true;
        }
      }
    }
  }
  p.next_win = home + 16 >= n ? 0 : home + 16;
  return p;
}

__device__ __forceinline__ Found h32_probe_rest(const uint64_t *table, uint64_t n, uint64_t row, HashProbe p) {
  Found f = p.f;
  bool pending = p.pending;
  uint64_t pend = __ballot(pending);
  if (pend == 0) return f;
  const int lane = (int)lane_id();
  const int grp = lane >> 3, sub = lane & 7;
  uint64_t win = p.next_win;
  uint64_t steps = 0;
  const uint64_t max_steps = n / 16 + 1;  // a full lap: give up (table without a never-used entry)
  while (pend) {
    // the g-th 8-lane group serves the g-th pending lane
    const int rank = __popcll(pend & ((1ull << lane) - 1ull));
    uint64_t m = pend;
    for (int i = 0; i < grp; ++i) m &= m - 1;
    const int src = m ? (__ffsll((unsigned long long)m) - 1) : -1;
    const bool gactive = src >= 0;
    const int from = gactive ? src : lane;
    const uint32_t k = __shfl((uint32_t)row, from);
    const uint64_t w = shfl64(win, from);
    u32x4 raw{kH32Empty, kH32Empty, kH32Empty, kH32Empty};
    if (gactive) raw = reinterpret_cast<const u32x4 *>(table + w)[sub];
    const H32Line line = h32_examine(raw, k, gactive, grp);
    const uint32_t g_flags = (line.done ? 1u : 0u) | (line.found ? 2u : 0u);
    const bool served = pending && rank < 8;
    const int back = served ? rank * 8 : lane;
    const uint32_t r_flags = __shfl(g_flags, back);
    const uint32_t r_val = __shfl(line.val, back);
    if (served) {
      if (r_flags & 1u) {
        pending = false;
        if (r_flags & 2u) {
          f.hit = true;
          f.loc = (r_val >> 28) & 0xfu;
          f.off = r_val & 0x0fffffffu;
        }
      } else {
        win += 16;
        if (win >= n) win = 0;
        if (++steps > max_steps) pending = false;
      }
    }
    pend = __ballot(pending);
  }
  return f;
}

template <int PASSES = 2, int ROUNDS = 8>
__device__ __forceinline__ Found hash_lookup_wave(const ugk_bucket_t *table, uint64_t nb, uint64_t key, bool active) {
  return hash_probe_rest(table, nb, key, hash_probe_home<PASSES, ROUNDS>(table, nb, key, active));
}

// Table lookup dispatch.  KIND is ugk_table_t::kind.  All lanes of the wavefront must call it; with ROUNDS < 8 only
// lanes 0 .. 8 * ROUNDS - 1 may be active.
template <int KIND, int PASSES = 2, int ROUNDS = 8>
__device__ __forceinline__ Found table_lookup(const ugk_table_t &t, uint64_t key, bool active) {
  if (KIND == 1) return flat_lookup(reinterpret_cast<const uint32_t *>(t.table), t.size, key, active);
  if (KIND == 2)
    return hash_lookup_wave<PASSES, ROUNDS>(reinterpret_cast<const ugk_bucket_t *>(t.table), t.size, key, active);
  if (KIND == 3) {
    // keyed by the row the key stands for; a key without a storable row is in no table
    const uint64_t row = active ? h32_row(t, key) : 0;
    const bool probe = active && row < kH32Tomb;
    const uint64_t *table = reinterpret_cast<const uint64_t *>(t.table);
    return h32_probe_rest(table, t.size, row, h32_probe_home<PASSES, ROUNDS>(table, t.size, row, probe));
  }
  return Found{false, 0, 0};
}

template <typename K>
__device__ __forceinline__ uint64_t key_to_u64(K k);
template <>
__device__ __forceinline__ uint64_t key_to_u64<uint32_t>(uint32_t k) {
  return k;
}
template <>
__device__ __forceinline__ uint64_t key_to_u64<int64_t>(int64_t k) {
  return (uint64_t)k;
}


// keys that collide with the two reserved bucket states cannot live in the hash table
__device__ __forceinline__ bool key_is_reserved(uint64_t k) { return k >= UGK_HASH_TOMB; }

}  // namespace ugk
