// Measurement kernels of `bench.py --probe link_latency` (bench_probes.py); built into libbench_probes.so beside this
// file.  Not part of the package: nothing under ugache_amd/ loads it.
//
//   bp_chase          one lane follows a chain of 8-byte links through a buffer (pinned host memory or HBM): every load
//                     depends on the one before, so time / hops is the latency of one read as a kernel sees it
//   bp_rows_inflight  a grid of a chosen size reads listed rows of 128 or 512 bytes with a chosen number of independent
//                     16-byte loads in flight per lane; nothing is written but one word per lane at the end, so the
//                     rate is that of the reads alone and the bytes in flight are known: grid x 256 lanes x U x 16
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

thread_local char g_err[256] = "";

__global__ void chase_kernel(const unsigned char *base, unsigned long long line_bytes, unsigned long long start,
                             unsigned long long hops, unsigned long long *last) {
  unsigned long long cur = start;
  for (unsigned long long h = 0; h < hops; ++h)
    cur = __builtin_nontemporal_load(reinterpret_cast<const unsigned long long *>(base + cur * line_bytes));
  *last = cur;
}

// LPR lanes of 16 bytes read one row; a wavefront reads 64 / LPR rows per round and U rounds are in flight together
template <int LPR, int U>
__global__ __launch_bounds__(256) void rows_inflight_kernel(const u32x4 *__restrict__ src, uint32_t vpr,
                                                            const uint32_t *__restrict__ rows, size_t n_rows,
                                                            uint32_t *__restrict__ sink) {
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63, sub = lane % LPR, rg = lane / LPR;
  const size_t wave = ((size_t)blockIdx.x * 256 + threadIdx.x) / 64, n_waves = (size_t)gridDim.x * 4;
  u32x4 acc = {0, 0, 0, 0};
  for (size_t r0 = wave * RPW * U; r0 < n_rows; r0 += n_waves * RPW * U) {  // wavefront-uniform
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = r0 + (size_t)u * RPW + rg;
      const size_t row = i < n_rows ? rows[i] : rows[0];
      v[u] = __builtin_nontemporal_load(src + row * vpr + sub);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  sink[(size_t)blockIdx.x * 256 + threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}

int fail(const char *what, hipError_t e) {
  snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
  return 1;
}

template <int LPR>
int launch_rows(int unroll, unsigned grid, const void *src, uint32_t vpr, const uint32_t *rows, size_t n_rows,
                uint32_t *sink, hipStream_t st) {
#define BP_CASE(U)                                                                                                  \
  case U:                                                                                                           \
    hipLaunchKernelGGL((rows_inflight_kernel<LPR, U>), dim3(grid), dim3(256), 0, st, (const u32x4 *)src, vpr, rows, \
                       n_rows, sink);                                                                               \
    break
  switch (unroll) {
    BP_CASE(1);
    BP_CASE(2);
    BP_CASE(4);
    BP_CASE(8);
    BP_CASE(16);
    default: snprintf(g_err, sizeof(g_err), "bp_rows_inflight: %d loads in flight per lane (1, 2, 4, 8, 16)", unroll); return 1;
  }
#undef BP_CASE
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : fail("bp_rows_inflight", e);
}

}  // namespace

extern "C" {

const char *bp_last_error(void) { return g_err; }

// base: buffer of lines of `line_bytes` bytes whose first 8 bytes hold the number of the next line of the chain;
// last_dev: device word that receives the line the chain ends at (so the loads cannot be dropped)
int bp_chase(const void *base, uint64_t line_bytes, uint64_t start, uint64_t hops, uint64_t *last_dev, void *stream) {
  hipLaunchKernelGGL(chase_kernel, dim3(1), dim3(1), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<const unsigned char *>(base), (unsigned long long)line_bytes,
                     (unsigned long long)start, (unsigned long long)hops, reinterpret_cast<unsigned long long *>(last_dev));
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : fail("bp_chase", e);
}

// rows_dev: n_rows row numbers into src (rows of row_bytes = 128 or 512 bytes); sink_dev: grid x 256 words
int bp_rows_inflight(const void *src, uint32_t row_bytes, const uint32_t *rows_dev, size_t n_rows, int unroll,
                     unsigned grid, uint32_t *sink_dev, void *stream) {
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (grid == 0 || n_rows == 0) return 0;
  if (row_bytes == 128) return launch_rows<8>(unroll, grid, src, 8, rows_dev, n_rows, sink_dev, st);
  if (row_bytes == 512) return launch_rows<32>(unroll, grid, src, 32, rows_dev, n_rows, sink_dev, st);
  snprintf(g_err, sizeof(g_err), "bp_rows_inflight: rows of %u bytes (128 or 512)", row_bytes);
  return 1;
}

}  // extern "C"
