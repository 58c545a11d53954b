// Pooled extraction: the lookup of a multi-hot feature and its per-sample combination in one kernel
// (ugk_extract_pool_*).
#include <hip/hip_fp16.h>

#include <cstdlib>

#include "ugk_internal.h"
#include "ugk_mix.cuh"
#include "ugk_table.cuh"

namespace ugk {
namespace {

// ---- pooled extraction -------------------------------------------------------------------------------------
// out[r, :] = combine_j( w_j * row(ids[j]) ) over the ids j of segment r = [seg_off[r], seg_off[r + 1]): the lookup of
// a multi-hot feature and the per-sample combination that follows it (embedding_lookup_sparse behind
// python_tf2/collcache_tf2/collcache_tf2/core/sparse_lookup_layer.py:196-265) in one pass, so that the nnz x row_bytes
// intermediate of a lookup followed by a segment sum is never written or read back.  A group of LPR lanes owns an
// output row: its lanes resolve LPR of the row's ids at a time (the table lookup is the fused extraction's), then
// every id's row is read once, 16 bytes per lane and chunk, and added in fp32 in the order of the ids.
// the elements of a 16-byte chunk as floats and back.  `bf16` picks between the two two-byte formats at run time (a
// wavefront-uniform branch), so that bfloat16 rows cost no kernels of their own.
template <typename E>
struct PoolElem;
template <>
struct PoolElem<float> {
  static constexpr int kPerChunk = 4;
  static __device__ __forceinline__ void unpack(const u32x4 &v, float *x, bool) {
    x[0] = __uint_as_float(v.x), x[1] = __uint_as_float(v.y), x[2] = __uint_as_float(v.z), x[3] = __uint_as_float(v.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float *x, bool) {
    return u32x4{__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3])};
  }
};
// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
template <>
struct PoolElem<__half> {
  static constexpr int kPerChunk = 8;
  static __device__ __forceinline__ void unpack(const u32x4 &v, float *x, bool bf16) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if (bf16) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        x[2 * k] = __uint_as_float(w[k] << 16);
        x[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        x[2 * k] = __half2float(__ushort_as_half((unsigned short)(w[k] & 0xffffu)));
        x[2 * k + 1] = __half2float(__ushort_as_half((unsigned short)(w[k] >> 16)));
      }
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float *x, bool bf16) {
    uint32_t w[4];
    if (bf16) {
#pragma unroll
      for (int k = 0; k < 4; ++k) w[k] = float_to_bf16_bits(x[2 * k]) | (float_to_bf16_bits(x[2 * k + 1]) << 16);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        w[k] = (uint32_t)__half_as_ushort(__float2half(x[2 * k])) |
               ((uint32_t)__half_as_ushort(__float2half(x[2 * k + 1])) << 16);
    }
    return u32x4{w[0], w[1], w[2], w[3]};
  }
};

constexpr int kPoolChunks = 4;  // 16-byte chunks of a row a lane may own: rows of up to LPR x 64 bytes

// CLIP: every looked-up row is clipped to the l2 norm max_norm before it is weighted (clip_by_norm over the row:
// x * max_norm / max(||x||, max_norm)).  The whole row has to be seen before any of it can be added, so the chunks of
// the U rows in flight are held in registers (up to 64 more than without), the squares summed per row over the lanes
// of the group, and the row's weight scaled; a kernel of its own, so that the plain combination keeps its registers.
template <typename K, int KIND, int LPR, typename E, bool CLIP>
__global__ __launch_bounds__(kBlock) void extract_pool_kernel(ugk_table_t t, const K *__restrict__ ids,
                                                              const long long *__restrict__ seg_off,
                                                              const float *__restrict__ weights, size_t n_rows,
                                                              long long nnz, const u32x4 *__restrict__ cache,
                                                              uint64_t cache_rows,
                                                              const u32x4 *__restrict__ host, uint64_t host_rows,
                                                              u32x4 *__restrict__ out, uint32_t vpr, int combiner, bool bf16,
                                                              float max_norm, uint32_t *status, uint32_t *host_mirror,
                                                              unsigned long long *counts) {
  constexpr int RPW = kWave / LPR;  // output rows per wavefront and pass
  constexpr int EPC = PoolElem<E>::kPerChunk;
  constexpr int U = 4;  // rows in flight per lane group
  static_assert(LPR % U == 0, "ids are taken in rounds of U");
  __shared__ uint32_t block_tot[2];
  if (threadIdx.x < 2) block_tot[threadIdx.x] = 0;
  __syncthreads();
  uint32_t wave_local = 0, wave_host = 0;
  const int lane = (int)lane_id();
  const int sub = lane % LPR, rg = lane / LPR;
  const size_t wave_global = (size_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
  const size_t n_waves = (size_t)gridDim.x * kWavesPerBlock;
  for (size_t row0 = wave_global * RPW; row0 < n_rows; row0 += n_waves * RPW) {  // wavefront-uniform
    const size_t r = row0 + rg;
    const bool row_ok = r < n_rows;
    long long beg = row_ok ? seg_off[r] : 0, end = row_ok ? seg_off[r + 1] : 0;
    if (beg < 0 || end > nnz || end < beg) {  // a segment outside the ids: nothing is read for it, its row is zeros
      if (sub == 0) {
        atomicOr(status, UGK_ST_BAD_SEGMENT);
        if (host_mirror) host_mirror[0] = UGK_ST_BAD_SEGMENT;
      }
      beg = end = 0;
    } else if (row_ok && sub == 0 && ((r == 0 && beg != 0) || (r + 1 == n_rows && end != nnz))) {
      // the offsets do not cover the ids from the first to the last (neighbouring segments share their boundary word,
      // so the two ends are all that can be wrong): the per-source id counts would not add up to nnz
      atomicOr(status, UGK_ST_BAD_SEGMENT);
      if (host_mirror) host_mirror[0] = UGK_ST_BAD_SEGMENT;
    }
    float acc[kPoolChunks][EPC];
#pragma unroll
    for (int c = 0; c < kPoolChunks; ++c)
#pragma unroll
      for (int e = 0; e < EPC; ++e) acc[c][e] = 0.f;
    float wsum = 0.f;  // this lane's share of the row's sum of weights (or of their squares)
    for (long long j0 = beg; __ballot(j0 < end) != 0ull; j0 += LPR) {  // until every group of the wavefront is through
      const long long j = j0 + sub;
      const bool active = j < end;
      const uint64_t key = active ? key_to_u64<K>(ids[j]) : 0;
      const Found f = table_lookup<KIND>(t, key, active);
      const MixRow row = mix_resolve(t, key, active, f, cache, cache_rows, host, host_rows, out, vpr, status, host_mirror);
      if (counts) {
        wave_local += __popcll(__ballot(row.from_cache));
        wave_host += __popcll(__ballot(active && !row.from_cache));
      }
      const bool use = active && row.has_row;  // a key without a row adds nothing (the launch is flagged)
      const float w = use ? (weights ? weights[j] : 1.f) : 0.f;
      wsum += combiner == 2 ? w * w : w;
      for (int s0 = 0; s0 < LPR; s0 += U) {
        if (__ballot(active && sub >= s0) == 0ull) break;  // no group has an id left in this round
        grow_t p[U];
        float wv[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int src = rg * LPR + s0 + u;
          p[u] = reinterpret_cast<grow_t>(shfl64(row.bits, src));
          wv[u] = __shfl(w, src);
          ok[u] = __shfl((int)use, src) != 0;
        }
        if constexpr (CLIP) {
          u32x4 v[kPoolChunks][U];
          float ss[U];
#pragma unroll
          for (int u = 0; u < U; ++u) ss[u] = 0.f;
#pragma unroll
          for (int c = 0; c < kPoolChunks; ++c) {
            const uint32_t col = (uint32_t)c * LPR + sub;
#pragma unroll
            for (int u = 0; u < U; ++u) v[c][u] = col < vpr ? __builtin_nontemporal_load(p[u] + col) : u32x4{0, 0, 0, 0};
          }
#pragma unroll
          for (int c = 0; c < kPoolChunks; ++c) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
              float x[EPC];
              PoolElem<E>::unpack(v[c][u], x, bf16);  // a chunk past the row's end is zeros in either two-byte format
#pragma unroll
              for (int e = 0; e < EPC; ++e) ss[u] = fmaf(x[e], x[e], ss[u]);
            }
          }
#pragma unroll
          for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int d = LPR / 2; d > 0; d >>= 1) ss[u] += __shfl_xor(ss[u], d);
            wv[u] *= max_norm / fmaxf(sqrtf(ss[u]), max_norm);
          }
#pragma unroll
          for (int c = 0; c < kPoolChunks; ++c) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
              float x[EPC];
              PoolElem<E>::unpack(v[c][u], x, bf16);
              if (ok[u]) {
#pragma unroll
                for (int e = 0; e < EPC; ++e) acc[c][e] = fmaf(wv[u], x[e], acc[c][e]);
              }
            }
          }
        } else {
#pragma unroll
          for (int c = 0; c < kPoolChunks; ++c) {
            const uint32_t col = (uint32_t)c * LPR + sub;
            if (col < vpr) {
              u32x4 v[U];
#pragma unroll
              for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p[u] + col);
#pragma unroll
              for (int u = 0; u < U; ++u) {
                float x[EPC];
                PoolElem<E>::unpack(v[u], x, bf16);
                if (ok[u]) {
#pragma unroll
                  for (int e = 0; e < EPC; ++e) acc[c][e] = fmaf(wv[u], x[e], acc[c][e]);
                }
              }
            }
          }
        }
      }
    }
    // the row's denominator: every lane of the group holds a share
#pragma unroll
    for (int d = LPR / 2; d > 0; d >>= 1) wsum += __shfl_xor(wsum, d);
    const float denom = combiner == 1 ? wsum : combiner == 2 ? sqrtf(wsum) : 1.f;
    if (row_ok) {
#pragma unroll
      for (int c = 0; c < kPoolChunks; ++c) {
        const uint32_t col = (uint32_t)c * LPR + sub;
        if (col < vpr) {
          float y[EPC];
#pragma unroll
          for (int e = 0; e < EPC; ++e) y[e] = denom != 0.f ? acc[c][e] / denom : 0.f;  // div_no_nan
          out[r * vpr + col] = PoolElem<E>::pack(y, bf16);
        }
      }
    }
  }
  if (counts) mix_leave_counts(block_tot, wave_local, wave_host, counts);
}

constexpr int kPoolMaxRows = 8;  // output rows a lane group may own per pass

// The same for short segments.  A lane group owns `rows_per_group` consecutive output rows per pass and walks their
// ids as one list: position f of the list is id seg_beg[k] + (f - seg_start[k]) of the group's row k, the last k whose
// seg_start is <= f.  The lanes resolve LPR positions at a time; the rows behind them are then read U at a time
// whatever segments they belong to and added in the order of the list, an output row being written when the list
// moves on to a later one.  What keeps memory busy is then the number of ids, not the shape of the segments: with one
// row per group a sample of one or two ids leaves most of the group's lookups and loads unused (262,144 samples of
// one id: 84 us per call with one row per group, 70 us with four).  The bookkeeping costs registers (three
// wavefronts per SIMD instead of four), which is why samples of more ids stay with the kernel above (65,536 samples
// of 16 ids: 121 us here, 114 us there).
template <typename K, int KIND, int LPR, typename E>
__global__ __launch_bounds__(kBlock) void extract_pool_rows_kernel(ugk_table_t t, const K *__restrict__ ids,
                                                              const long long *__restrict__ seg_off,
                                                              const float *__restrict__ weights, size_t n_rows,
                                                              long long nnz, int rows_per_group,
                                                              const u32x4 *__restrict__ cache, uint64_t cache_rows,
                                                              const u32x4 *__restrict__ host, uint64_t host_rows,
                                                              u32x4 *__restrict__ out, uint32_t vpr, int combiner, bool bf16,
                                                              uint32_t *status, uint32_t *host_mirror,
                                                              unsigned long long *counts) {
  constexpr int RPW = kWave / LPR;  // lane groups per wavefront
  constexpr int EPC = PoolElem<E>::kPerChunk;
  constexpr int U = 4;  // rows in flight per lane group
  static_assert(LPR % U == 0 && LPR >= kPoolMaxRows, "ids are taken in rounds of U; a lane per owned row");
  __shared__ uint32_t block_tot[2];
  __shared__ long long seg_beg[kWavesPerBlock][RPW][kPoolMaxRows];    // first id of the group's row k
  __shared__ uint32_t seg_start[kWavesPerBlock][RPW][kPoolMaxRows];   // its first position in the group's list
  if (threadIdx.x < 2) block_tot[threadIdx.x] = 0;
  __syncthreads();
  uint32_t wave_local = 0, wave_host = 0;
  const int lane = (int)lane_id();
  const int sub = lane % LPR, rg = lane / LPR, wv_in_block = (int)(threadIdx.x / kWave);
  const size_t wave_global = (size_t)blockIdx.x * kWavesPerBlock + wv_in_block;
  const size_t n_waves = (size_t)gridDim.x * kWavesPerBlock;
  const size_t rows_per_wave = (size_t)RPW * rows_per_group;
  long long *my_beg = seg_beg[wv_in_block][rg];
  uint32_t *my_start = seg_start[wv_in_block][rg];
  for (size_t row0 = wave_global * rows_per_wave; row0 < n_rows; row0 += n_waves * rows_per_wave) {  // wavefront-uniform
    const size_t g0 = row0 + (size_t)rg * rows_per_group;  // the group's first row
    const int n_own = g0 < n_rows ? (int)min((size_t)rows_per_group, n_rows - g0) : 0;
    long long beg = 0;
    uint32_t len = 0;
    if (sub < n_own) {
      const long long b = seg_off[g0 + sub], e = seg_off[g0 + sub + 1];
      // a segment outside the ids: nothing is read for it, its row is zeros.  (The list of a group is counted in 32
      // bits; the launcher keeps batches of 2^28 ids and more away from this kernel, so the last test never fires.)
      if (b < 0 || e > nnz || e < b || e - b >= (1ll << 28)) {
        atomicOr(status, UGK_ST_BAD_SEGMENT);
        if (host_mirror) host_mirror[0] = UGK_ST_BAD_SEGMENT;
      } else {
        beg = b, len = (uint32_t)(e - b);
        if ((g0 + sub == 0 && b != 0) || (g0 + sub + 1 == n_rows && e != nnz)) {  // the ids are not covered end to end
          atomicOr(status, UGK_ST_BAD_SEGMENT);
          if (host_mirror) host_mirror[0] = UGK_ST_BAD_SEGMENT;
        }
      }
    }
    uint32_t incl = len;  // inclusive prefix over the group's rows (lanes past the owned rows add nothing)
#pragma unroll
    for (int d = 1; d < kPoolMaxRows; d <<= 1) {
      const uint32_t up = (uint32_t)__shfl_up((int)incl, d, LPR);
      if (sub >= d) incl += up;
    }
    const uint32_t total = (uint32_t)__shfl((int)incl, rg * LPR + kPoolMaxRows - 1);  // ids of the group this pass
    if (sub < kPoolMaxRows) my_beg[sub] = beg, my_start[sub] = incl - len;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float acc[kPoolChunks][EPC];
#pragma unroll
    for (int c = 0; c < kPoolChunks; ++c)
#pragma unroll
      for (int e = 0; e < EPC; ++e) acc[c][e] = 0.f;
    int cur = 0;       // the owned row the accumulators belong to
    float wsum = 0.f;  // its sum of weights (or of their squares) so far
    // one chunk of an owned row is complete: divide (div_no_nan), write, start the next row
    auto flush = [&](int c, uint32_t col, int k, float ws) {
      const float denom = combiner == 1 ? ws : combiner == 2 ? sqrtf(ws) : 1.f;
      float y[EPC];
#pragma unroll
      for (int e = 0; e < EPC; ++e) y[e] = denom != 0.f ? acc[c][e] / denom : 0.f, acc[c][e] = 0.f;
      out[(g0 + k) * vpr + col] = PoolElem<E>::pack(y, bf16);
    };
    for (uint32_t f0 = 0; __ballot(f0 < total) != 0ull; f0 += LPR) {  // until every group of the wavefront is through
      const uint32_t f = f0 + sub;
      const bool active = f < total;
      int k = 0;
      if (rows_per_group > 1) {
#pragma unroll
        for (int q = 1; q < kPoolMaxRows; ++q) k += my_start[q] <= f ? 1 : 0;  // rows past the owned ones start at total
      }
      const long long j = active ? my_beg[k] + (long long)(f - my_start[k]) : 0;
      const uint64_t key = active ? key_to_u64<K>(ids[j]) : 0;
      const Found fd = table_lookup<KIND>(t, key, active);
      const MixRow row = mix_resolve(t, key, active, fd, cache, cache_rows, host, host_rows, out, vpr, status, host_mirror);
      if (counts) {
        wave_local += __popcll(__ballot(row.from_cache));
        wave_host += __popcll(__ballot(active && !row.from_cache));
      }
      const bool use = active && row.has_row;  // a key without a row adds nothing (the launch is flagged)
      const float w = use ? (weights ? weights[j] : 1.f) : 0.f;
      const int meta = active ? (k | (use ? 0x100 : 0) | 0x200) : 0;  // owned row, "adds something", "is an id"
      for (int s0 = 0; s0 < LPR; s0 += U) {
        if (__ballot(active && sub >= s0) == 0ull) break;  // no group has an id left in this round
        grow_t p[U];
        float wv[U];
        int m[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int src = rg * LPR + s0 + u;
          p[u] = reinterpret_cast<grow_t>(shfl64(row.bits, src));
          wv[u] = __shfl(w, src);
          m[u] = __shfl(meta, src);
        }
#pragma unroll
        for (int c = 0; c < kPoolChunks; ++c) {
          const uint32_t col = (uint32_t)c * LPR + sub;
          if (col < vpr) {
            u32x4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p[u] + col);
            int cc = cur;  // every chunk walks the same ids from the same state
            float ws = wsum;
#pragma unroll
            for (int u = 0; u < U; ++u) {
              float x[EPC];
              PoolElem<E>::unpack(v[u], x, bf16);
              if (m[u] & 0x200) {
                for (const int ku = m[u] & 0xff; cc < ku; ++cc, ws = 0.f) flush(c, col, cc, ws);
                if (m[u] & 0x100) {
#pragma unroll
                  for (int e = 0; e < EPC; ++e) acc[c][e] = fmaf(wv[u], x[e], acc[c][e]);
                  ws += combiner == 2 ? wv[u] * wv[u] : wv[u];
                }
              }
            }
          }
        }
        // the state after these ids, for the lanes of every chunk alike (a lane may own no chunk at all)
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (m[u] & 0x200) {
            if (cur < (m[u] & 0xff)) cur = m[u] & 0xff, wsum = 0.f;
            if (m[u] & 0x100) wsum += combiner == 2 ? wv[u] * wv[u] : wv[u];
          }
        }
      }
    }
    // the row the list ended in, and the empty ones behind it
#pragma unroll
    for (int c = 0; c < kPoolChunks; ++c) {
      const uint32_t col = (uint32_t)c * LPR + sub;
      if (col < vpr) {
        float ws = wsum;
        for (int cc = cur; cc < n_own; ++cc, ws = 0.f) flush(c, col, cc, ws);
      }
    }
    __builtin_amdgcn_wave_barrier();  // the next pass rewrites the group's list
  }
  if (counts) mix_leave_counts(block_tot, wave_local, wave_host, counts);
}

template <typename K, int KIND, typename E>
int extract_pool_lpr(ugk_table_t t, const K *ids, const long long *seg_off, const float *weights, size_t n_rows,
                     const void *cache, uint64_t cache_rows, const void *host, uint64_t host_rows, void *out,
                     uint32_t vpr, uint64_t nnz, int combiner, bool bf16, float max_norm, uint32_t *status,
                     uint32_t *host_mirror, uint64_t *counts, uint32_t *num_groups, hipStream_t st) {
  // Lanes per output row: rows of up to 512 bytes go to 8 lanes of up to four chunks each (eight lane groups per
  // wavefront; with 32 lanes and two groups 65,536 samples of 16 ids took 123 us instead of 112 us), rows of up to
  // 2 KB to 32 lanes, longer ones to 64.
  int lpr = vpr <= 8 * kPoolChunks ? 8 : vpr <= 32 * kPoolChunks ? 32 : 64;
  if (const char *forced = getenv("UGK_POOL_LPR")) {  // for sweeps; never a byte of the result depends on it
    const int v = atoi(forced);
    if ((v == 8 || v == 32 || v == 64) && vpr <= (uint32_t)v * kPoolChunks) lpr = v;
  }
  // Output rows per lane group and pass.  One row each (extract_pool_kernel) is the faster kernel from two ids per
  // sample on (it needs fewer registers: four wavefronts per SIMD instead of three; at two ids the two are level);
  // for samples of mostly one id a group takes four rows as one list (extract_pool_rows_kernel), as long as the
  // launch still has wavefronts for every CU.
  const int groups_per_wave = kWave / lpr;
  int rows = n_rows && nnz <= (uint64_t)n_rows + n_rows / 2 ? 4 : 1;
  const size_t enough_waves = (size_t)cu_count() * 8;
  while (rows > 1 && n_rows / ((size_t)rows * groups_per_wave) < enough_waves) rows /= 2;
  if (const char *forced = getenv("UGK_POOL_ROWS")) {  // for sweeps, like the one above
    const int v = atoi(forced);
    if (v >= 1 && v <= kPoolMaxRows) rows = v;
  }
  if (nnz >= ((uint64_t)1 << 28)) rows = 1;  // the list of a group is counted in 32 bits
  const bool clip = max_norm > 0.f;
  if (clip) rows = 1;  // clipping lives in the kernel of one output row per lane group
  const size_t rows_per_block = (size_t)rows * groups_per_wave * kWavesPerBlock;
  const unsigned grid = clamp_grid((n_rows + rows_per_block - 1) / rows_per_block, 0);
  if (num_groups) *num_groups = grid;
#define UGK_POOL(L)                                                                                                    \
  if (clip)                                                                                                            \
    hipLaunchKernelGGL((extract_pool_kernel<K, KIND, L, E, true>), dim3(grid), dim3(kBlock), 0, st, t, ids, seg_off,   \
                       weights, n_rows, (long long)nnz, (const u32x4 *)cache, cache_rows, (const u32x4 *)host,         \
                       host_rows, (u32x4 *)out, vpr, combiner, bf16, max_norm, status, host_mirror,                    \
                       reinterpret_cast<unsigned long long *>(counts));                                                \
  else if (rows == 1)                                                                                                  \
    hipLaunchKernelGGL((extract_pool_kernel<K, KIND, L, E, false>), dim3(grid), dim3(kBlock), 0, st, t, ids, seg_off,  \
                       weights, n_rows, (long long)nnz, (const u32x4 *)cache, cache_rows, (const u32x4 *)host,         \
                       host_rows, (u32x4 *)out, vpr, combiner, bf16, 0.f, status, host_mirror,                         \
                       reinterpret_cast<unsigned long long *>(counts));                                                \
  else                                                                                                                 \
    hipLaunchKernelGGL((extract_pool_rows_kernel<K, KIND, L, E>), dim3(grid), dim3(kBlock), 0, st, t, ids, seg_off,    \
                       weights, n_rows, (long long)nnz, rows, (const u32x4 *)cache, cache_rows, (const u32x4 *)host,   \
                       host_rows, (u32x4 *)out, vpr, combiner, bf16, status, host_mirror,                              \
                       reinterpret_cast<unsigned long long *>(counts))
  if (lpr == 8) {
    UGK_POOL(8);
  } else if (lpr == 32) {
    UGK_POOL(32);
  } else {
    UGK_POOL(64);
  }
#undef UGK_POOL
  UGK_HIP(hipGetLastError());
  return 0;
}

// seg_off[r] = the number of entries whose row is below r: lane i owns the offsets of the rows that begin between
// entry i - 1 and entry i.  That is one offset where every row has an entry, which the lane writes itself; a run of
// rows without entries is written by the whole wavefront, 64 offsets a step.
__global__ __launch_bounds__(kBlock) void segment_offsets_kernel(const long long *__restrict__ rows, size_t nnz,
                                                                 size_t n_rows, long long *__restrict__ seg_off,
                                                                 uint32_t *status, uint32_t *host_mirror) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const int lane = (int)lane_id();
  for (size_t base = (size_t)blockIdx.x * kBlock + threadIdx.x - lane; base <= nnz; base += stride) {  // wavefront-uniform
    const size_t i = base + lane;
    long long prev = 0, cur = -1;  // an empty run for the lanes past the end
    if (i <= nnz) {
      prev = i == 0 ? -1 : rows[i - 1];
      cur = i == nnz ? (long long)n_rows : rows[i];
      // entries out of order or outside [0, n_rows): flagged; what is written stays inside seg_off
      if (cur < prev || cur < 0 || (i > 0 && prev < 0) || (i < nnz && cur >= (long long)n_rows) ||
          prev >= (long long)n_rows) {
        if (status) atomicOr(status, UGK_ST_BAD_SEGMENT);
        if (host_mirror) host_mirror[0] = UGK_ST_BAD_SEGMENT;
        prev = 0, cur = -1;
      }
    }
    const long long first = prev + 1, count = cur - prev;  // rows first .. first + count - 1 begin at entry i
    if (count == 1) seg_off[first] = (long long)i;
    for (unsigned long long runs = __ballot(count > 1); runs != 0ull; runs &= runs - 1ull) {
      const int src = __ffsll((long long)runs) - 1;
      const long long f = (long long)shfl64((uint64_t)first, src), c = (long long)shfl64((uint64_t)count, src);
      const long long at = (long long)(base + src);
      for (long long r = lane; r < c; r += kWave) seg_off[f + r] = at;
    }
  }
}

template <typename K>
int extract_pool(ugk_table_t t, const K *ids, const int64_t *seg_off, const float *weights, size_t n_rows, uint64_t nnz,
                 int combiner, int elem_bytes, const void *cache, uint64_t cache_rows, const void *host,
                 uint64_t host_rows, void *out, size_t row_bytes, float max_norm, uint32_t *status,
                 uint32_t *host_mirror, uint64_t *counts, uint32_t *num_groups, void *stream) {
  if (num_groups) *num_groups = 0;
  if (n_rows == 0) return 0;
  UGK_REQUIRE(seg_off && out && status, "ugk_extract_pool: null offsets, output or status");
  UGK_REQUIRE(max_norm >= 0.f, "ugk_extract_pool: max_norm %g is not a norm (0 = no clipping)", (double)max_norm);
  UGK_REQUIRE(nnz == 0 || ids, "ugk_extract_pool: null ids");
  UGK_REQUIRE(nnz <= (uint64_t)INT64_MAX, "ugk_extract_pool: %llu ids", (unsigned long long)nnz);
  UGK_REQUIRE((uintptr_t)counts % 8 == 0, "ugk_extract_pool: the count words must be 8-byte aligned");
  UGK_REQUIRE(combiner >= 0 && combiner <= 2, "ugk_extract_pool: combiner %d is not sum(0), mean(1) or sqrtn(2)", combiner);
  UGK_REQUIRE(elem_bytes == 4 || elem_bytes == 2 || elem_bytes == UGK_ELEM_BF16,
              "ugk_extract_pool: element code %d is not fp32 (4), fp16 (2) or bfloat16 (UGK_ELEM_BF16)", elem_bytes);
  const bool bf16 = elem_bytes == UGK_ELEM_BF16;
  UGK_REQUIRE(t.kind >= 0 && t.kind <= 3, "ugk_extract_pool: table kind %d", t.kind);
  if (t.kind != 0) UGK_REQUIRE(t.table && t.size, "ugk_extract_pool: empty table");
  if (t.kind >= 2)
    UGK_REQUIRE(t.size % (t.kind == 2 ? 8 : 16) == 0 && (uintptr_t)t.table % 128 == 0,
                "ugk_extract_pool: hash table must be 128-byte aligned with whole 128-byte lines of buckets");
  UGK_REQUIRE(cache_rows == 0 || cache, "ugk_extract_pool: null cache with %llu rows", (unsigned long long)cache_rows);
  UGK_REQUIRE(host_rows == 0 || host, "ugk_extract_pool: null host table with %llu rows", (unsigned long long)host_rows);
  const uintptr_t align = (uintptr_t)cache | (uintptr_t)host | (uintptr_t)out | (uintptr_t)row_bytes;
  UGK_REQUIRE(row_bytes > 0 && align % 16 == 0,
              "ugk_extract_pool: rows and buffers must be multiples of 16 bytes (row_bytes=%zu)", row_bytes);
  const uint32_t vpr = (uint32_t)(row_bytes / 16);
  UGK_REQUIRE(vpr <= (uint32_t)kWave * kPoolChunks, "ugk_extract_pool: rows of %zu bytes exceed %d", row_bytes,
              kWave * kPoolChunks * 16);
  const long long *so = reinterpret_cast<const long long *>(seg_off);
  hipStream_t st = as_stream(stream);
#define UGK_POOL_KIND(KIND)                                                                                          \
  (elem_bytes == 4 ? extract_pool_lpr<K, KIND, float>(t, ids, so, weights, n_rows, cache, cache_rows, host, host_rows, \
                                                      out, vpr, nnz, combiner, false, max_norm, status, host_mirror,  \
                                                      counts, num_groups, st)                                         \
                   : extract_pool_lpr<K, KIND, __half>(t, ids, so, weights, n_rows, cache, cache_rows, host,          \
                                                       host_rows, out, vpr, nnz, combiner, bf16, max_norm, status,    \
                                                       host_mirror, counts, num_groups, st))
  if (t.kind == 0) return UGK_POOL_KIND(0);
  if (t.kind == 1) return UGK_POOL_KIND(1);
  if (t.kind == 2) return UGK_POOL_KIND(2);
  return UGK_POOL_KIND(3);
#undef UGK_POOL_KIND
}

}  // namespace
// an empty launch: what it costs is the load of this file's code object onto the device (see ugk_preload_kernels)
namespace {
__global__ void preload_pool_kernel() {}
}  // namespace
void preload_pool(hipStream_t stream) { hipLaunchKernelGGL(preload_pool_kernel, dim3(1), dim3(1), 0, stream); }
}  // namespace ugk

using namespace ugk;

extern "C" {

int ugk_segment_offsets_i64(const int64_t *sorted_rows_dev, size_t nnz, size_t n_rows, int64_t *seg_off_dev,
                            uint32_t *status_dev, uint32_t *host_mirror, void *stream) {
  UGK_REQUIRE(seg_off_dev, "ugk_segment_offsets: null output");
  UGK_REQUIRE(nnz == 0 || sorted_rows_dev, "ugk_segment_offsets: null rows");
  UGK_REQUIRE(nnz < ((uint64_t)1 << 62) && n_rows < ((uint64_t)1 << 62), "ugk_segment_offsets: sizes out of range");
  const unsigned grid = clamp_grid((nnz + 1 + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(segment_offsets_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream),
                     reinterpret_cast<const long long *>(sorted_rows_dev), nnz, n_rows,
                     reinterpret_cast<long long *>(seg_off_dev), status_dev, host_mirror);
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_extract_pool_u32(ugk_table_t t, const uint32_t *ids_dev, const int64_t *seg_off_dev, const float *weights_dev,
                         size_t n_rows, uint64_t nnz, int combiner, int elem_bytes, const void *cache_dev,
                         uint64_t cache_rows, const void *host_dev, uint64_t host_rows, void *out_dev, size_t row_bytes,
                         uint32_t *status_dev, uint32_t *host_mirror, uint64_t *group_counts_host,
                         uint32_t *num_groups_host, void *stream) {
  return extract_pool<uint32_t>(t, ids_dev, seg_off_dev, weights_dev, n_rows, nnz, combiner, elem_bytes, cache_dev,
                                cache_rows, host_dev, host_rows, out_dev, row_bytes, 0.f, status_dev, host_mirror,
                                group_counts_host, num_groups_host, stream);
}

int ugk_extract_pool_i64(ugk_table_t t, const int64_t *ids_dev, const int64_t *seg_off_dev, const float *weights_dev,
                         size_t n_rows, uint64_t nnz, int combiner, int elem_bytes, const void *cache_dev,
                         uint64_t cache_rows, const void *host_dev, uint64_t host_rows, void *out_dev, size_t row_bytes,
                         uint32_t *status_dev, uint32_t *host_mirror, uint64_t *group_counts_host,
                         uint32_t *num_groups_host, void *stream) {
  return extract_pool<int64_t>(t, ids_dev, seg_off_dev, weights_dev, n_rows, nnz, combiner, elem_bytes, cache_dev,
                               cache_rows, host_dev, host_rows, out_dev, row_bytes, 0.f, status_dev, host_mirror,
                               group_counts_host, num_groups_host, stream);
}

int ugk_extract_pool_clip_u32(ugk_table_t t, const uint32_t *ids_dev, const int64_t *seg_off_dev,
                              const float *weights_dev, size_t n_rows, uint64_t nnz, int combiner, int elem_bytes,
                              float max_norm, const void *cache_dev, uint64_t cache_rows, const void *host_dev,
                              uint64_t host_rows, void *out_dev, size_t row_bytes, uint32_t *status_dev,
                              uint32_t *host_mirror, uint64_t *group_counts_host, uint32_t *num_groups_host,
                              void *stream) {
  return extract_pool<uint32_t>(t, ids_dev, seg_off_dev, weights_dev, n_rows, nnz, combiner, elem_bytes, cache_dev,
                                cache_rows, host_dev, host_rows, out_dev, row_bytes, max_norm, status_dev, host_mirror,
                                group_counts_host, num_groups_host, stream);
}

int ugk_extract_pool_clip_i64(ugk_table_t t, const int64_t *ids_dev, const int64_t *seg_off_dev,
                              const float *weights_dev, size_t n_rows, uint64_t nnz, int combiner, int elem_bytes,
                              float max_norm, const void *cache_dev, uint64_t cache_rows, const void *host_dev,
                              uint64_t host_rows, void *out_dev, size_t row_bytes, uint32_t *status_dev,
                              uint32_t *host_mirror, uint64_t *group_counts_host, uint32_t *num_groups_host,
                              void *stream) {
  return extract_pool<int64_t>(t, ids_dev, seg_off_dev, weights_dev, n_rows, nnz, combiner, elem_bytes, cache_dev,
                               cache_rows, host_dev, host_rows, out_dev, row_bytes, max_norm, status_dev, host_mirror,
                               group_counts_host, num_groups_host, stream);
}

}  // extern "C"
