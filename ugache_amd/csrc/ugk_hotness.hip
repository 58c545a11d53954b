// Hotness counters on the device: one uint32 per row of the host table, bumped by the keys of a batch, and
// handed to the host as a compact (row, count) list.
//
// record : counts[row(key)] += 1.  HBM-bound by the key read plus one 64-byte line touched per distinct row; runs
//          beside the gathers on the caller's stream.
// drain  : scans the counters, turns every non-zero one into a (count << 32 | row) word in a compact list and
//          resets it to zero.  Reading and resetting is one atomic exchange, so a record kernel that runs at
//          the same time loses nothing: its increment lands either before the exchange (drained now) or after
//          it (drained next time).
#include "ugk_internal.h"
#include "ugk_table.cuh"

namespace ugk {
namespace {

// Hot rows are hot: with a skewed key distribution a few counters would take most of the atomics of a batch and
// serialise them in the memory-side atomic units.  Each workgroup therefore first counts its tile of keys in a small
// LDS table (row -> count, open addressing, at most half full) and then adds every distinct row of the tile to the
// global counters once.
constexpr int kRecKeysPerThread = 8;        // 2048 keys per tile, 4096 slots, 32 KB of LDS
constexpr uint32_t kRecEmpty = 0xffffffffu;  // rows are below 2^32 - 1

template <typename K, int KPT>
__global__ __launch_bounds__(kBlock) void record_kernel(const K *__restrict__ keys, size_t n, ugk_table_t map,
                                                        uint32_t *counts, uint64_t num_rows,
                                                        unsigned long long *observed, uint32_t *status,
                                                        uint32_t *host_mirror) {
  constexpr int kRecTile = kBlock * KPT;
  constexpr int kRecSlots = 2 * kRecTile;
  __shared__ uint32_t slot_row[kRecSlots];
  __shared__ uint32_t slot_cnt[kRecSlots];
  const int tid = threadIdx.x;
  for (int s = tid; s < kRecSlots; s += kBlock) {
    slot_row[s] = kRecEmpty;
    slot_cnt[s] = 0;
  }
  __syncthreads();
  bool bad = false;
  const size_t n_tiles = (n + kRecTile - 1) / kRecTile;
  for (size_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const size_t base = tile * kRecTile;
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
      const size_t i = base + (size_t)j * kBlock + tid;
      if (i >= n) continue;
      const uint64_t row64 = fallback_row(map, key_to_u64<K>(keys[i]));
      if (row64 >= num_rows) {
        bad = true;
        continue;
      }
      const uint32_t row = (uint32_t)row64;
      uint32_t h = (uint32_t)(fmix64(row) >> 40) & (kRecSlots - 1);
      for (;;) {
        const uint32_t seen = atomicCAS(&slot_row[h], kRecEmpty, row);
        if (seen == kRecEmpty || seen == row) {
          atomicAdd(&slot_cnt[h], 1u);
          break;
        }
        h = (h + 1) & (kRecSlots - 1);
      }
    }
    __syncthreads();
    if (observed == nullptr) {
      for (int s = tid; s < kRecSlots; s += kBlock) {
        const uint32_t c = slot_cnt[s];
        if (c) {
          atomicAdd(counts + slot_row[s], c);
          slot_row[s] = kRecEmpty;
          slot_cnt[s] = 0;
        }
      }
    } else {
      // a counter that leaves zero sets its row's bit: all adds of the thread go out first, their returned values are
      // looked at afterwards, so the round trips overlap
      constexpr int kPer = kRecSlots / kBlock;
      uint32_t rows[kPer], before[kPer];
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const int s = j * kBlock + tid;
        const uint32_t c = slot_cnt[s];
        rows[j] = slot_row[s];
        before[j] = 1;
        if (c) {
          before[j] = atomicAdd(counts + rows[j], c);
          slot_row[s] = kRecEmpty;
          slot_cnt[s] = 0;
        }
      }
#pragma unroll
      for (int j = 0; j < kPer; ++j)
        if (before[j] == 0) atomicOr(observed + (rows[j] >> 6), 1ull << (rows[j] & 63));
    }
    __syncthreads();
  }
  if (__ballot(bad) && lane_id() == 0) {
    atomicOr(status, (uint32_t)UGK_ST_KEY_OUT_OF_RANGE);
    if (host_mirror) host_mirror[0] = 1;
  }
}

// A wavefront owns a contiguous run of counters and goes over it twice: first it counts the non-zero ones, reserves
// that many list slots with ONE atomic (a reservation per 256 counters would serialise on the list's single counter:
// with 1 % of the rows hot nearly every group of 256 holds one), then it reads the run again, exchanges the non-zero
// counters for zero and writes their entries.  Counters only grow between the two passes, so the second pass finds at
// least what the first one counted; what it finds beyond the reservation stays for the next drain.
struct DrainVec {
  u32x4 c;
  uint64_t row0;
};

// vector v of the run: 4 adjacent counters from a 16-byte load; two pseudo vectors behind the last one carry the
// (at most 3 + 3) counters in front of the first and behind the last aligned vector
__device__ __forceinline__ DrainVec drain_load(const uint32_t *counts, uint64_t num_rows, uint64_t head, uint64_t n_vec,
                                               uint64_t v) {
  DrainVec d{u32x4{0, 0, 0, 0}, 0};
  if (v < n_vec) {
    d.c = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(counts + head) + v);
    d.row0 = head + v * 4;
  } else if (v == n_vec) {
    if (head > 0) d.c.x = counts[0];
    if (head > 1) d.c.y = counts[1];
    if (head > 2) d.c.z = counts[2];
  } else if (v == n_vec + 1) {
    d.row0 = head + n_vec * 4;
    const uint64_t left = num_rows - d.row0;
    if (left > 0) d.c.x = counts[d.row0];
    if (left > 1) d.c.y = counts[d.row0 + 1];
    if (left > 2) d.c.z = counts[d.row0 + 2];
  }
  return d;
}

__device__ __forceinline__ uint32_t nonzeros(const u32x4 &c) {
  return (c.x != 0) + (c.y != 0) + (c.z != 0) + (c.w != 0);
}

// the way back of a drain: counts handed over as (count << 32 | row) words are added to the counters
__global__ __launch_bounds__(kBlock) void restore_kernel(const unsigned long long *__restrict__ entries, size_t n,
                                                         uint32_t *counts, uint64_t num_rows,
                                                         unsigned long long *observed, uint32_t *status) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    const unsigned long long e = entries[i];
    const uint32_t row = (uint32_t)e, cnt = (uint32_t)(e >> 32);
    if (row >= num_rows) {
      atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
      continue;
    }
    if (cnt == 0) continue;
    const uint32_t before = atomicAdd(counts + row, cnt);
    if (before == 0 && observed) atomicOr(observed + (row >> 6), 1ull << (row & 63));  // the counter leaves zero
  }
}

__global__ __launch_bounds__(kBlock) void drain_kernel(uint32_t *counts, uint64_t num_rows, uint64_t first_row,
                                                       unsigned long long *observed, unsigned long long *entries,
                                                       uint32_t capacity, uint32_t *n_entries) {
  const int lane = (int)lane_id();
  const uint64_t wave = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  const uint64_t n_waves = (uint64_t)gridDim.x * (kBlock / kWave);
  const uint64_t head = min((uint64_t)num_rows, (uint64_t)((4 - (((uintptr_t)counts / 4) & 3)) & 3));
  const uint64_t n_vec = (num_rows - head) / 4;
  const uint64_t n_all = n_vec + 2;
  const uint64_t per_wave = ((n_all + n_waves - 1) / n_waves + kWave - 1) / kWave * kWave;
  const uint64_t begin = wave * per_wave, end = min(n_all, begin + per_wave);
  if (begin >= end) return;

  uint32_t found = 0;
  for (uint64_t v0 = begin; v0 < end; v0 += kWave) {
    const uint64_t v = v0 + lane;
    if (v < end) found += nonzeros(drain_load(counts, num_rows, head, n_vec, v).c);
  }
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) found += __shfl_xor(found, d);
  if (found == 0) return;  // wavefront-uniform
  uint32_t base = 0;
  if (lane == 0) base = atomicAdd(n_entries, found);
  base = __shfl(base, 0);

  uint32_t used = 0;  // slots of the reservation handed out so far (wavefront-uniform)
  for (uint64_t v0 = begin; v0 < end && used < found; v0 += kWave) {
    const uint64_t v = v0 + lane;
    DrainVec d{u32x4{0, 0, 0, 0}, 0};
    if (v < end) d = drain_load(counts, num_rows, head, n_vec, v);
    const uint32_t mine = nonzeros(d.c);
    uint32_t incl = mine;
#pragma unroll
    for (int s = 1; s < kWave; s <<= 1) {
      const uint32_t up = __shfl_up(incl, s);
      if (lane >= s) incl += up;
    }
    uint32_t idx = used + incl - mine;
    const uint32_t cc[4] = {d.c.x, d.c.y, d.c.z, d.c.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (cc[k] != 0) {
        // beyond the reservation or beyond the list: the counter stays as it is for the next drain
        if (idx < found && base + idx < capacity) {
          // the bit first: an increment that lands between the two steps is part of `got`, one that lands after
          // them finds the counter at zero and sets the bit again
          const uint64_t row = first_row + d.row0 + k;
          if (observed) atomicAnd(observed + (row >> 6), ~(1ull << (row & 63)));
          const uint32_t got = atomicExch(counts + d.row0 + k, 0u);
          entries[base + idx] = ((unsigned long long)got << 32) | (uint32_t)row;
        }
        ++idx;
      }
    }
    used += __shfl(incl, kWave - 1);
  }
}

__global__ void drain_finish_kernel(uint32_t *n_entries, uint32_t capacity, uint32_t *host_out) {
  // entries claimed beyond the capacity were not written; report what the list holds and whether rows are left
  const uint32_t claimed = *n_entries;
  host_out[0] = claimed < capacity ? claimed : capacity;
  host_out[1] = claimed > capacity ? 1u : 0u;
  *n_entries = 0;
}

template <typename K>
int record(const K *keys, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts, uint64_t num_rows,
           uint64_t *observed, uint32_t *status, uint32_t *host_mirror, void *stream) {
  if (n == 0) return 0;
  UGK_REQUIRE(keys && counts && status, "ugk_record: null pointer");
  UGK_REQUIRE(key_inv == 0 || (key_inv & 1ull), "ugk_record: the inverse key multiplier must be odd");
  UGK_REQUIRE(num_rows < 0xffffffffull, "ugk_record: rows must fit 32 bits");
  ugk_table_t map{};
  map.fb_mul = key_inv;
  map.fb_mask = key_mask;
  // 512-key tiles for batches whose 2048-key tiles would leave most compute units without a workgroup (65,536 keys
  // alone on the chip: 12.4 -> 5.9 us; 262,144: 17.7 -> 13.2 us uniform, 14.5 -> 15.5 us Zipf 1.05; at 1 M keys the
  // large tile wins on skewed keys, 40.9 against 55.2 us, because more duplicates meet in LDS)
  const int kpt = n <= (size_t)cu_count() * 1024 ? 2 : kRecKeysPerThread;
  const size_t tile = (size_t)kBlock * kpt;
  const unsigned grid = clamp_grid((n + tile - 1) / tile, 0);
#define UGK_GO(KPT)                                                                                              \
  hipLaunchKernelGGL((record_kernel<K, KPT>), dim3(grid), dim3(kBlock), 0, as_stream(stream), keys, n, map, counts, \
                     num_rows, reinterpret_cast<unsigned long long *>(observed), status, host_mirror)
  if (kpt == 2) UGK_GO(2);
  else UGK_GO(kRecKeysPerThread);
#undef UGK_GO
  UGK_HIP(hipGetLastError());
  return 0;
}

}  // namespace
// an empty launch: what it costs is the load of this file's code object onto the device (see ugk_preload_kernels)
namespace {
__global__ void preload_hotness_kernel() {}
}  // namespace
void preload_hotness(hipStream_t stream) { hipLaunchKernelGGL(preload_hotness_kernel, dim3(1), dim3(1), 0, stream); }
}  // namespace ugk

using namespace ugk;

extern "C" {

int ugk_record_u32(const uint32_t *keys_dev, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts_dev,
                   uint64_t num_rows, uint64_t *observed_dev, uint32_t *status_dev, uint32_t *host_mirror,
                   void *stream) {
  return record<uint32_t>(keys_dev, n, key_inv, key_mask, counts_dev, num_rows, observed_dev, status_dev, host_mirror,
                          stream);
}

int ugk_record_i64(const int64_t *keys_dev, size_t n, uint64_t key_inv, uint64_t key_mask, uint32_t *counts_dev,
                   uint64_t num_rows, uint64_t *observed_dev, uint32_t *status_dev, uint32_t *host_mirror,
                   void *stream) {
  return record<int64_t>(keys_dev, n, key_inv, key_mask, counts_dev, num_rows, observed_dev, status_dev, host_mirror,
                         stream);
}

int ugk_record_restore(const uint64_t *entries_dev, size_t n, uint32_t *counts_dev, uint64_t num_rows,
                       uint64_t *observed_dev, uint32_t *status_dev, void *stream) {
  if (n == 0) return 0;
  UGK_REQUIRE(entries_dev && counts_dev && status_dev, "ugk_record_restore: null pointer");
  UGK_REQUIRE(num_rows <= 0xffffffffull, "ugk_record_restore: rows must fit 32 bits");
  const unsigned grid = clamp_grid((n + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(restore_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream),
                     reinterpret_cast<const unsigned long long *>(entries_dev), n, counts_dev, num_rows,
                     reinterpret_cast<unsigned long long *>(observed_dev), status_dev);
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_record_drain(uint32_t *counts_dev, uint64_t first_row, uint64_t num_rows, uint64_t *observed_dev,
                     uint64_t *entries_dev, uint32_t capacity, uint32_t *n_entries_dev, uint32_t *host_out,
                     void *stream) {
  UGK_REQUIRE(counts_dev && entries_dev && n_entries_dev && host_out, "ugk_record_drain: null pointer");
  UGK_REQUIRE(capacity > 0, "ugk_record_drain: empty entry list");
  UGK_REQUIRE(first_row + num_rows <= 0xffffffffull, "ugk_record_drain: rows must fit 32 bits");
  if (num_rows) {
    // few, long wavefronts: one reservation each (8 workgroups per CU)
    const unsigned grid = clamp_grid((num_rows / 4 + 2 + kBlock - 1) / kBlock, (unsigned)cu_count() * 8u);
    hipLaunchKernelGGL(drain_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), counts_dev + first_row, num_rows,
                       first_row, reinterpret_cast<unsigned long long *>(observed_dev),
                       reinterpret_cast<unsigned long long *>(entries_dev), capacity, n_entries_dev);
    UGK_HIP(hipGetLastError());
  }
  hipLaunchKernelGGL(drain_finish_kernel, dim3(1), dim3(1), 0, as_stream(stream), n_entries_dev, capacity, host_out);
  UGK_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
