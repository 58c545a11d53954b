// What the kernels that look a key up and read its row in one go have in common (the fused extraction and the pooled
// one): where a key's row lives, and how a launch hands its per-source row counts to the host.
#pragma once

#include "ugk_internal.h"
#include "ugk_table.cuh"

namespace ugk {
namespace {

constexpr int kWavesPerBlock = kBlock / kWave;

typedef const __attribute__((address_space(1))) u32x4 *grow_t;  // a row in global memory (HBM, or mapped host memory)
typedef __attribute__((address_space(1))) u32x4 *gout_t;

// where a key's row lives, as an integer address (the head of the output for a key without a row, see below)
struct MixRow {
  uint64_t bits;
  uint64_t host_row;  // the row of the host table it is, ~0 for a row of the cache or no row
  bool has_row, from_cache;
};

__device__ __forceinline__ MixRow mix_resolve(const ugk_table_t &t, uint64_t key, bool active, const Found &f,
                                              const u32x4 *cache, uint64_t cache_rows, const u32x4 *host,
                                              uint64_t host_rows, const u32x4 *out, uint32_t vpr, uint32_t *status,
                                              uint32_t *host_mirror) {
  const u32x4 *rowp = nullptr;
  uint64_t host_row = ~0ull;
  if (active) {
    if (f.hit && f.loc == UGK_LOC_LOCAL && f.off < cache_rows) rowp = cache + (uint64_t)f.off * vpr;
    else if (f.hit && f.loc == UGK_LOC_HOST && f.off < host_rows) host_row = f.off;
    else if (!f.hit && fallback_row(t, key) < host_rows) host_row = fallback_row(t, key);
    else {
      atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
      if (host_mirror) host_mirror[0] = UGK_ST_KEY_OUT_OF_RANGE;
    }
  }
  // A key without a row copies nothing; its lanes read the head of the output instead (mapped whatever the key), so
  // that the loads of the copy carry no branch: behind a branch each of them waits for the one before.
  if (host_row != ~0ull) rowp = host + host_row * vpr;
  MixRow r;
  r.host_row = host_row;
  r.has_row = rowp != nullptr;
  r.bits = r.has_row ? reinterpret_cast<uint64_t>(rowp) : reinterpret_cast<uint64_t>(out);
  r.from_cache = r.has_row && f.hit && f.loc == UGK_LOC_LOCAL;
  return r;
}

// Group sizes for the host: every workgroup leaves its two sums in a word of its own in pinned host memory, a posted
// write nobody waits for; the host adds the words up after it has waited for the stream.  Handing them over through
// device-side atomics cost more than it looks: a 64-bit add and a dependent ticket per workgroup 16 us of a 69 us
// launch at 99 % hits (same-address atomics are performed one after the other at the memory side), one add whose
// result tells the last workgroup still 5 us (every workgroup ends by waiting for the round trip), and a device-scope
// fence per workgroup 13-49 % of a whole step (each writes back and invalidates the L2 of its XCD).
__device__ __forceinline__ void mix_leave_counts(uint32_t *block_tot, uint32_t wave_local, uint32_t wave_host,
                                                 unsigned long long *counts) {
  if (lane_id() == 0) {
    if (wave_local) atomicAdd(&block_tot[0], wave_local);
    if (wave_host) atomicAdd(&block_tot[1], wave_host);
  }
  __syncthreads();
  if (threadIdx.x == 0) counts[blockIdx.x] = ((unsigned long long)block_tot[1] << 32) | block_tot[0];
}

}  // namespace
}  // namespace ugk
