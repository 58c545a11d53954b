// Row gather kernels for gfx950: out[dst(i), :] = src[srcrow(i), :].
//
// This is pure HBM (or host-link) traffic, so the kernel is built around 16-byte lanes and many rows in
// flight rather than around arithmetic:
//   * a row of V 16-byte vectors is copied by LPR = min(64, pow2ceil(V)) adjacent lanes, so one wavefront
//     instruction moves 64/LPR whole rows as fully coalesced segments (512-B rows: 2 rows, 128-B rows: 8);
//   * every lane keeps UNROLL = 2 independent rows in flight (both loads issued before the first store) and the
//     launch uses many small workgroups of one pass each:
//     measured on MI355X this beats deeper unrolling with fewer, longer-lived workgroups by ~15 %;
//   * loads carry the non-temporal hint (table rows are touched once); stores are ordinary write-back stores
//     while the output fits the 256 MB memory-side cache, so the consumer finds it there, and non-temporal
//     beyond that or when the caller says its outputs do not stay there (ugk_set_output_hint);
//   * the grid has one workgroup per pass of rows, or is capped by the caller so a host-link gather occupies
//     only a few CUs while the HBM gather runs next to it (then the workgroups stride over the batch);
//   * keys / index records are range-checked against the source's row count: a bad key sets a status bit
//     and its row is skipped instead of faulting.
#include <cstdlib>

#include "ugk_internal.h"
#include "ugk_table.cuh"

namespace ugk {
namespace {

constexpr uint64_t kNoLimit = ~0ull;

// ---- index functors (what the reference calls IdxStore*) -------------------------------------------
struct DirectU32 {
  const uint32_t *keys;
  __device__ __forceinline__ void get(size_t i, uint64_t &s, uint64_t &d) const {
    s = keys[i];
    d = i;
  }
};
struct DirectI64 {
  const int64_t *keys;
  __device__ __forceinline__ void get(size_t i, uint64_t &s, uint64_t &d) const {
    s = (uint64_t)keys[i];  // negative keys become huge and fail the range check
    d = i;
  }
};
struct ScatterU32 {
  const uint32_t *keys;
  const uint32_t *dst;
  __device__ __forceinline__ void get(size_t i, uint64_t &s, uint64_t &d) const {
    s = keys[i];
    d = dst[i];
  }
};
struct ScatterI64 {
  const int64_t *keys;
  const uint32_t *dst;
  __device__ __forceinline__ void get(size_t i, uint64_t &s, uint64_t &d) const {
    s = (uint64_t)keys[i];
    d = dst[i];
  }
};
struct IdxList {
  const ugk_idx_t *idx;
  __device__ __forceinline__ void get(size_t i, uint64_t &s, uint64_t &d) const {
    const uint2 e = *reinterpret_cast<const uint2 *>(idx + i);  // one 8-byte load
    d = e.x;
    s = e.y;
  }
};

template <typename V>
__device__ __forceinline__ V ld_stream(const V *p) {
  return __builtin_nontemporal_load(p);
}
template <typename V>
__device__ __forceinline__ void st_stream(V *p, V v) {
  __builtin_nontemporal_store(v, p);
}

// NT_STORE is a template parameter, not a launch argument: with a run-time flag the optimiser merges the two stores
// of `if (nt) stream(p, v); else *p = v;` into one and the non-temporal hint is lost (seen with UNROLL = 1).
template <typename V, int LPR, int UNROLL, bool NT_STORE, typename Idx>
__global__ __launch_bounds__(kBlock) void gather_kernel(Idx ix, const V *__restrict__ src, uint64_t src_rows,
                                                        V *__restrict__ out, uint64_t out_rows, uint32_t vpr,
                                                        const uint32_t *__restrict__ counts, uint32_t group, size_t n,
                                                        uint32_t *status, uint32_t *host_mirror) {
  size_t begin = 0, count = n;
  if (counts) {
    const uint32_t c = counts[group];
    count = c;
    begin = (group == UGK_LOC_LOCAL) ? 0 : n - c;
    if (host_mirror && blockIdx.x == 0 && threadIdx.x == 0) host_mirror[1 + group] = c;
  }
  constexpr int RPB = kBlock / LPR;  // rows copied by one block instruction
  const uint32_t lane = threadIdx.x % LPR;
  const uint32_t rib = threadIdx.x / LPR;
  constexpr size_t kPerIter = (size_t)RPB * UNROLL;

  for (size_t base = (size_t)blockIdx.x * kPerIter; base < count; base += (size_t)gridDim.x * kPerIter) {
    // the index words of all rows of the pass first, in flight together (a row past the end takes the last one's),
    // then the checks: a check between two of them would make the second wait for the first
    uint64_t s[UNROLL], d[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t r = base + (size_t)u * RPB + rib;
      ok[u] = r < count;
      ix.get(begin + (ok[u] ? r : count - 1), s[u], d[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (ok[u] && (s[u] >= src_rows || d[u] >= out_rows)) {
        ok[u] = false;
        if (lane == 0) {
          atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
          if (host_mirror) host_mirror[0] = UGK_ST_KEY_OUT_OF_RANGE;
        }
      }
    }
    for (uint32_t c0 = 0; c0 < vpr; c0 += LPR) {
      const uint32_t col = c0 + lane;
      if (col < vpr) {
        V v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
          if (ok[u]) v[u] = ld_stream(src + s[u] * vpr + col);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
          if (ok[u]) {
            if constexpr (NT_STORE) st_stream(out + d[u] * vpr + col, v[u]);
            else out[d[u] * vpr + col] = v[u];
          }
      }
    }
  }
}

// Re-expansion of duplicates inside one buffer: row i takes the bytes of its representative row.  Source and
// destination are the same allocation but never the same row, so the pointers are deliberately not __restrict__.
template <typename V, int LPR>
__global__ __launch_bounds__(kBlock) void replicate_kernel(V *out, uint32_t vpr, const uint32_t *__restrict__ inverse,
                                                           const uint32_t *__restrict__ rep, size_t n) {
  constexpr int RPB = kBlock / LPR;
  const uint32_t lane = threadIdx.x % LPR, rib = threadIdx.x / LPR;
  for (size_t base = (size_t)blockIdx.x * RPB; base < n; base += (size_t)gridDim.x * RPB) {
    const size_t i = base + rib;
    if (i >= n) continue;
    const size_t r = rep[inverse[i]];
    if (r == i) continue;
    for (uint32_t col = lane; col < vpr; col += LPR) out[i * vpr + col] = out[r * vpr + col];
  }
}

constexpr int kStagedUnroll = 8;  // rows a lane group keeps in flight in gather_staged_kernel
// Rows out of the host table, or out of the stage where it holds them (refresh inserts: most of the rows a refresh
// brings in were missed by the last few lookups and are filed there).  Lanes per row chosen at run time: this runs at
// refresh time, on some hundred thousand rows.
__global__ __launch_bounds__(kBlock) void gather_staged_kernel(const u32x4 *__restrict__ host, uint64_t host_rows,
                                                               const uint32_t *__restrict__ rows,
                                                               const uint32_t *__restrict__ dst, size_t n,
                                                               u32x4 *__restrict__ out, uint64_t out_rows, uint32_t vpr,
                                                               uint32_t lpr, ugk_stage_t stage, uint32_t *status,
                                                               uint32_t *staged, uint32_t *rest_rows,
                                                               uint32_t *rest_dst, uint32_t *rest_count,
                                                               uint32_t *done_count) {
  constexpr int UNROLL = kStagedUnroll;
  __shared__ uint32_t block_staged;
  if (threadIdx.x == 0) block_staged = 0;
  __syncthreads();
  const uint32_t lane = threadIdx.x % lpr, rib = threadIdx.x / lpr, rpb = kBlock / lpr;
  const size_t per_iter = (size_t)rpb * UNROLL;
  const u32x4 *stage_rows = reinterpret_cast<const u32x4 *>(stage.rows_dev);
  uint32_t mine = 0;
  for (size_t base = (size_t)blockIdx.x * per_iter; base < n; base += (size_t)gridDim.x * per_iter) {
    const u32x4 *src[UNROLL];
    uint64_t d[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t r = base + (size_t)u * rpb + rib;
      ok[u] = r < n;
      const uint64_t s = rows[ok[u] ? r : n - 1];
      d[u] = dst[ok[u] ? r : n - 1];
      if (ok[u] && (s >= host_rows || d[u] >= out_rows)) {
        ok[u] = false;
        if (lane == 0) atomicOr(status, UGK_ST_KEY_OUT_OF_RANGE);
      }
      const uint64_t h = fmix64(s) & stage.mask;
      const unsigned long long cur = stage.owner_dev[h];
      const bool filed = ok[u] && (cur >> 32) != 0 && (uint32_t)cur == (uint32_t)s;
      if (rest_count) {
        // Rows the stage does not hold are left for the caller's own (throttled) copy over the host link: listed, not
        // copied.  With done_count the rows that are copied here are listed too, from the back of the same lists, for
        // a caller that publishes rows as they arrive.  One atomic per wavefront and list: the first lane of every
        // row that goes on a list takes its place from a ballot.
        const bool lead = lane == 0 && ok[u];
        const unsigned long long to_rest = __ballot(lead && !filed);
        const unsigned long long to_done = __ballot(lead && filed && done_count != nullptr);
        const unsigned long long below = (1ull << lane_id()) - 1ull;
        uint32_t rest_base = 0, done_base = 0;
        if (lane_id() == 0) {
          if (to_rest) rest_base = atomicAdd(rest_count, (uint32_t)__popcll(to_rest));
          if (to_done) done_base = atomicAdd(done_count, (uint32_t)__popcll(to_done));
        }
        rest_base = __shfl(rest_base, 0);
        done_base = __shfl(done_base, 0);
        if (lead && !filed) {
          const uint32_t at = rest_base + (uint32_t)__popcll(to_rest & below);
          rest_rows[at] = (uint32_t)s;
          rest_dst[at] = (uint32_t)d[u];
        } else if (lead && filed && done_count) {
          const uint32_t at = (uint32_t)n - 1u - (done_base + (uint32_t)__popcll(to_done & below));
          rest_rows[at] = (uint32_t)s;
          rest_dst[at] = (uint32_t)d[u];
        }
        if (!filed) ok[u] = false;
      }
      src[u] = !ok[u] ? reinterpret_cast<const u32x4 *>(out) : filed ? stage_rows + h * vpr : host + s * vpr;
      if (filed && lane == 0) ++mine;
    }
    for (uint32_t c0 = 0; c0 < vpr; c0 += lpr) {
      const uint32_t col = c0 + lane;
      if (col < vpr) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = ld_stream(src[u] + col);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
          if (ok[u]) out[d[u] * vpr + col] = v[u];
      }
    }
  }
  if (staged == nullptr) return;
  if (mine) atomicAdd(&block_staged, mine);
  __syncthreads();
  if (threadIdx.x == 0 && block_staged) atomicAdd(staged, block_staged);
}

// A launch that may fill the chip (max_blocks == 0) gets one workgroup per pass of rows, however many that makes:
// workgroups start in order, so the rows being written at any moment form one window that moves through the output,
// which the memory side turns into far better write bursts than the same workgroups striding over the whole output
// (2 M keys of 512 bytes: 360 us against 377 us with 16,384 grid-striding workgroups; 1 M keys: 181 against 187 us).
unsigned gather_grid(size_t passes, unsigned max_blocks) {
  if (max_blocks) return clamp_grid(passes, max_blocks);
  if (passes == 0) passes = 1;
  return (unsigned)(passes > 0x7fffffffull ? 0x7fffffffull : passes);
}

template <typename V, int LPR, int UNROLL, typename Idx>
int launch_unrolled(Idx ix, const void *src, uint64_t src_rows, void *out, uint64_t out_rows, uint32_t vpr,
                    const uint32_t *counts, uint32_t group, size_t n, unsigned max_blocks, uint32_t *status,
                    uint32_t *host_mirror, bool nt, hipStream_t stream) {
  constexpr size_t kPerIter = (size_t)(kBlock / LPR) * UNROLL;
  const unsigned grid = gather_grid((n + kPerIter - 1) / kPerIter, max_blocks);
  if (nt)
    hipLaunchKernelGGL((gather_kernel<V, LPR, UNROLL, true, Idx>), dim3(grid), dim3(kBlock), 0, stream, ix,
                       reinterpret_cast<const V *>(src), src_rows, reinterpret_cast<V *>(out), out_rows, vpr, counts,
                       group, n, status, host_mirror);
  else
    hipLaunchKernelGGL((gather_kernel<V, LPR, UNROLL, false, Idx>), dim3(grid), dim3(kBlock), 0, stream, ix,
                       reinterpret_cast<const V *>(src), src_rows, reinterpret_cast<V *>(out), out_rows, vpr, counts,
                       group, n, status, host_mirror);
  UGK_HIP(hipGetLastError());
  return 0;
}

template <typename V, int LPR, typename Idx>
int launch_one(Idx ix, const void *src, uint64_t src_rows, void *out, uint64_t out_rows, uint32_t vpr,
               const uint32_t *counts, uint32_t group, size_t n, unsigned max_blocks, uint32_t *status,
               uint32_t *host_mirror, hipStream_t stream) {
  // two rows in flight per lane; one was measured with streaming stores and is no better (262,144 keys of 512 bytes
  // into rotating outputs 49.3 us against 47.9 us, 1 M keys 184 against 180 us)
  return launch_unrolled<V, LPR, 2, Idx>(ix, src, src_rows, out, out_rows, vpr, counts, group, n, max_blocks, status,
                                         host_mirror, nt_store_for(n * (size_t)vpr * sizeof(V)), stream);
}

template <typename V, typename Idx, bool ALL_LPR>
int launch_vec(Idx ix, const void *src, uint64_t src_rows, void *out, uint64_t out_rows, size_t row_bytes,
               const uint32_t *counts, uint32_t group, size_t n, unsigned max_blocks, uint32_t *status,
               uint32_t *host_mirror, hipStream_t stream) {
  const uint32_t vpr = (uint32_t)(row_bytes / sizeof(V));
#define UGK_GO(L) \
  return launch_one<V, L, Idx>(ix, src, src_rows, out, out_rows, vpr, counts, group, n, max_blocks, status, host_mirror, \
                               stream)
  if (ALL_LPR) {
    if (vpr <= 1) UGK_GO(1);
    if (vpr <= 2) UGK_GO(2);
    if (vpr <= 4) UGK_GO(4);
    if (vpr <= 8) UGK_GO(8);
    if (vpr <= 16) UGK_GO(16);
    if (vpr <= 32) UGK_GO(32);
    UGK_GO(64);
  } else {
    if (vpr <= 1) UGK_GO(1);
    if (vpr <= 16) UGK_GO(16);
    UGK_GO(64);
  }
#undef UGK_GO
}

template <typename Idx>
int launch_gather(Idx ix, const void *src, uint64_t src_rows, void *out, uint64_t out_rows, size_t row_bytes,
                  const uint32_t *counts, uint32_t group, size_t n, unsigned max_blocks, uint32_t *status,
                  uint32_t *host_mirror, void *stream) {
  if (n == 0) return 0;
  UGK_REQUIRE(src && out, "gather: null source or output");
  UGK_REQUIRE(status, "gather: null status word");
  UGK_REQUIRE(row_bytes > 0 && row_bytes <= (1u << 30), "gather: row_bytes %zu out of range", row_bytes);
  UGK_REQUIRE(n <= 0xffffffffull, "gather: batch of %zu rows exceeds 2^32", n);
  const uintptr_t align = (uintptr_t)src | (uintptr_t)out | (uintptr_t)row_bytes;
  hipStream_t st = as_stream(stream);
  if (align % 16 == 0)
    return launch_vec<u32x4, Idx, true>(ix, src, src_rows, out, out_rows, row_bytes, counts, group, n, max_blocks,
                                            status, host_mirror, st);
  if (align % 8 == 0)
    return launch_vec<unsigned long long, Idx, false>(ix, src, src_rows, out, out_rows, row_bytes, counts, group, n,
                                                      max_blocks,
                                            status, host_mirror, st);
  if (align % 4 == 0)
    return launch_vec<uint32_t, Idx, false>(ix, src, src_rows, out, out_rows, row_bytes, counts, group, n,
                                            max_blocks,
                                            status, host_mirror, st);
  if (align % 2 == 0)
    return launch_vec<uint16_t, Idx, false>(ix, src, src_rows, out, out_rows, row_bytes, counts, group, n,
                                            max_blocks,
                                            status, host_mirror, st);
  return launch_vec<uint8_t, Idx, false>(ix, src, src_rows, out, out_rows, row_bytes, counts, group, n, max_blocks,
                                            status, host_mirror, st);
}

}  // namespace

namespace {
thread_local int g_output_hint = 0;
}
bool nt_store_for(size_t out_bytes) {
  static int forced = [] {
    const char *e = getenv("UGK_GATHER_NT_STORE");
    return e ? atoi(e) : -1;
  }();
  if (forced >= 0) return forced != 0;
  if (g_output_hint == UGK_OUTPUT_STREAMS) return true;
  if (g_output_hint == UGK_OUTPUT_STAYS) return false;
  return out_bytes > ((size_t)192 << 20);
}
// an empty launch: what it costs is the load of this file's code object onto the device (see ugk_preload_kernels)
namespace {
__global__ void preload_gather_kernel() {}
}  // namespace
void preload_gather(hipStream_t stream) { hipLaunchKernelGGL(preload_gather_kernel, dim3(1), dim3(1), 0, stream); }
}  // namespace ugk

using namespace ugk;

extern "C" {

int ugk_set_output_hint(int hint) {
  UGK_REQUIRE(hint == UGK_OUTPUT_AUTO || hint == UGK_OUTPUT_STREAMS || hint == UGK_OUTPUT_STAYS,
              "ugk_set_output_hint: unknown hint %d", hint);
  g_output_hint = hint;
  return 0;
}

int ugk_gather_direct_u32(const void *src_dev, uint64_t src_rows, const uint32_t *keys_dev, size_t n, void *out_dev,
                          size_t row_bytes, unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror,
                          void *stream) {
  UGK_REQUIRE(n == 0 || keys_dev, "ugk_gather_direct_u32: null keys");
  return launch_gather(DirectU32{keys_dev}, src_dev, src_rows, out_dev, kNoLimit, row_bytes, nullptr, 0, n,
                       max_blocks, status_dev, host_mirror, stream);
}

int ugk_gather_direct_i64(const void *src_dev, uint64_t src_rows, const int64_t *keys_dev, size_t n, void *out_dev,
                          size_t row_bytes, unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror,
                          void *stream) {
  UGK_REQUIRE(n == 0 || keys_dev, "ugk_gather_direct_i64: null keys");
  return launch_gather(DirectI64{keys_dev}, src_dev, src_rows, out_dev, kNoLimit, row_bytes, nullptr, 0, n,
                       max_blocks, status_dev, host_mirror, stream);
}

int ugk_gather_scatter_u32(const void *src_dev, uint64_t src_rows, const uint32_t *keys_dev,
                           const uint32_t *dst_off_dev, size_t n, void *out_dev, uint64_t out_rows, size_t row_bytes,
                           unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror, void *stream) {
  UGK_REQUIRE(n == 0 || (keys_dev && dst_off_dev), "ugk_gather_scatter_u32: null keys or destinations");
  return launch_gather(ScatterU32{keys_dev, dst_off_dev}, src_dev, src_rows, out_dev, out_rows, row_bytes, nullptr, 0,
                       n, max_blocks, status_dev, host_mirror, stream);
}

int ugk_gather_scatter_i64(const void *src_dev, uint64_t src_rows, const int64_t *keys_dev,
                           const uint32_t *dst_off_dev, size_t n, void *out_dev, uint64_t out_rows, size_t row_bytes,
                           unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror, void *stream) {
  UGK_REQUIRE(n == 0 || (keys_dev && dst_off_dev), "ugk_gather_scatter_i64: null keys or destinations");
  return launch_gather(ScatterI64{keys_dev, dst_off_dev}, src_dev, src_rows, out_dev, out_rows, row_bytes, nullptr, 0,
                       n, max_blocks, status_dev, host_mirror, stream);
}

int ugk_gather_scatter_staged_u32(const void *host_dev, uint64_t host_rows, const uint32_t *rows_dev,
                                  const uint32_t *dst_off_dev, size_t n, void *out_dev, uint64_t out_rows,
                                  size_t row_bytes, ugk_stage_t stage, unsigned max_blocks, uint32_t *status_dev,
                                  uint32_t *staged_dev, uint32_t *rest_rows_dev, uint32_t *rest_dst_dev,
                                  uint32_t *rest_count_dev, uint32_t *done_count_dev, void *stream) {
  if (n == 0) return 0;
  UGK_REQUIRE(rest_count_dev == nullptr || (rest_rows_dev && rest_dst_dev),
              "ugk_gather_scatter_staged_u32: a rest count without the two rest lists");
  UGK_REQUIRE(done_count_dev == nullptr || rest_count_dev, "ugk_gather_scatter_staged_u32: a done count without rest lists");
  UGK_REQUIRE(n <= 0xffffffffull, "ugk_gather_scatter_staged_u32: %zu rows do not fit 32-bit list positions", n);
  UGK_REQUIRE(host_dev && rows_dev && dst_off_dev && out_dev && status_dev, "ugk_gather_scatter_staged_u32: null pointer");
  UGK_REQUIRE(stage.rows_dev && stage.owner_dev && ((stage.mask + 1) & stage.mask) == 0,
              "ugk_gather_scatter_staged_u32: the stage needs buffers and a power of two of entries");
  const uintptr_t align = (uintptr_t)host_dev | (uintptr_t)out_dev | (uintptr_t)stage.rows_dev | (uintptr_t)row_bytes;
  UGK_REQUIRE(row_bytes > 0 && align % 16 == 0,
              "ugk_gather_scatter_staged_u32: rows and buffers must be multiples of 16 bytes (row_bytes=%zu)", row_bytes);
  UGK_REQUIRE(host_rows <= 0x100000000ull, "ugk_gather_scatter_staged_u32: host rows must fit 32 bits");
  const uint32_t vpr = (uint32_t)(row_bytes / 16);
  uint32_t lpr = 1;
  while (lpr < vpr && lpr < 64) lpr <<= 1;
  const size_t per_iter = (size_t)(kBlock / lpr) * kStagedUnroll;
  const unsigned grid = clamp_grid((n + per_iter - 1) / per_iter, max_blocks);
  hipLaunchKernelGGL(gather_staged_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream),
                     reinterpret_cast<const u32x4 *>(host_dev), host_rows, rows_dev, dst_off_dev, n,
                     reinterpret_cast<u32x4 *>(out_dev), out_rows, vpr, lpr, stage, status_dev, staged_dev,
                     rest_rows_dev, rest_dst_dev, rest_count_dev, done_count_dev);
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_gather_group(const void *src_dev, uint64_t src_rows, const ugk_idx_t *idx_dev, const uint32_t *counts_dev,
                     uint32_t group, size_t n, void *out_dev, uint64_t out_rows, size_t row_bytes,
                     unsigned max_blocks, uint32_t *status_dev, uint32_t *host_mirror, void *stream) {
  UGK_REQUIRE(n == 0 || (idx_dev && counts_dev), "ugk_gather_group: null index list or counts");
  UGK_REQUIRE(group == UGK_LOC_LOCAL || group == UGK_LOC_HOST, "ugk_gather_group: group %u is not local/host", group);
  return launch_gather(IdxList{idx_dev}, src_dev, src_rows, out_dev, out_rows, row_bytes, counts_dev, group, n, max_blocks,
                       status_dev, host_mirror, stream);
}

int ugk_replicate_rows(void *out_dev, size_t row_bytes, const uint32_t *inverse_dev, const uint32_t *rep_dev, size_t n,
                       void *stream) {
  if (n == 0) return 0;
  UGK_REQUIRE(out_dev && inverse_dev && rep_dev, "ugk_replicate_rows: null pointer");
  UGK_REQUIRE(row_bytes > 0, "ugk_replicate_rows: empty rows");
  hipStream_t st = as_stream(stream);
  if (((uintptr_t)out_dev | row_bytes) % 16 == 0) {
    const uint32_t vpr = (uint32_t)(row_bytes / 16);
    if (vpr <= 8) {
      const unsigned grid = clamp_grid((n + kBlock / 8 - 1) / (kBlock / 8), 0);
      hipLaunchKernelGGL((replicate_kernel<u32x4, 8>), dim3(grid), dim3(kBlock), 0, st, (u32x4 *)out_dev, vpr,
                         inverse_dev, rep_dev, n);
    } else {
      const unsigned grid = clamp_grid((n + kBlock / 32 - 1) / (kBlock / 32), 0);
      hipLaunchKernelGGL((replicate_kernel<u32x4, 32>), dim3(grid), dim3(kBlock), 0, st, (u32x4 *)out_dev, vpr,
                         inverse_dev, rep_dev, n);
    }
  } else {
    const unsigned grid = clamp_grid((n + kBlock / 32 - 1) / (kBlock / 32), 0);
    hipLaunchKernelGGL((replicate_kernel<uint8_t, 32>), dim3(grid), dim3(kBlock), 0, st, (uint8_t *)out_dev,
                       (uint32_t)row_bytes, inverse_dev, rep_dev, n);
  }
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_gather_idx(const void *src_dev, uint64_t src_rows, const ugk_idx_t *idx_dev, size_t count, void *out_dev,
                   size_t row_bytes, unsigned max_blocks, uint32_t *status_dev, void *stream) {
  UGK_REQUIRE(count == 0 || idx_dev, "ugk_gather_idx: null index list");
  return launch_gather(IdxList{idx_dev}, src_dev, src_rows, out_dev, kNoLimit, row_bytes, nullptr, 0, count,
                       max_blocks, status_dev, nullptr, stream);
}

}  // extern "C"
