// Internal helpers shared by the gfx950 translation units behind include/ugache_hip.h.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "ugache_hip.h"

int ugk_set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define UGK_HIP(expr)                                                                                        \
  do {                                                                                                       \
    hipError_t ugk_e_ = (expr);                                                                              \
    if (ugk_e_ != hipSuccess)                                                                                \
      return ugk_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(ugk_e_), __FILE__, __LINE__);   \
  } while (0)

#define UGK_REQUIRE(cond, ...)                        \
  do {                                                \
    if (!(cond)) return ugk_set_error(__VA_ARGS__);   \
  } while (0)

namespace ugk {

constexpr int kBlock = 256;  // 4 wavefronts of 64 lanes
constexpr int kWave = 64;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Number of compute units of the current device (cached per device).
int cu_count();

// Upper bound, in workgroups per CU, of grid-stride launches that should fill the chip (default 64: many short
// workgroups balance better than few long ones on this part); UGK_BLOCKS_PER_CU overrides.
int blocks_per_cu();

static inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

static inline unsigned clamp_grid(size_t want, unsigned max_blocks) {
  if (want == 0) want = 1;
  size_t cap = max_blocks ? (size_t)max_blocks : (size_t)cu_count() * (size_t)blocks_per_cu();
  if (want > cap) want = cap;
  return (unsigned)want;
}

// Non-temporal stores for an extraction whose output of `out_bytes` will not stay in the 256 MB memory-side cache
// anyway; ordinary write-back stores otherwise, so that the consumer finds the rows there.  The caller's hint
// (ugk_set_output_hint) and UGK_GATHER_NT_STORE=0/1 override the size rule.
bool nt_store_for(size_t out_bytes);

__device__ __forceinline__ unsigned lane_id() { return __lane_id(); }

// one per source file with kernels: launches an empty kernel of that file on `stream`
void preload_gather(hipStream_t stream);
void preload_hotness(hipStream_t stream);
void preload_partition(hipStream_t stream);
void preload_pool(hipStream_t stream);
void preload_refresh(hipStream_t stream);
void preload_table(hipStream_t stream);

}  // namespace ugk
