// Runtime plumbing of the C-ABI: memory, streams, events, copies, fill/iota kernels.
#include <cstdlib>
#include <cstring>

#include <atomic>
#include <chrono>

#include "ugk_internal.h"

static thread_local char g_err[1024] = "";

int ugk_set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}

namespace ugk {

int cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

int blocks_per_cu() {
  static int v = 0;
  if (v == 0) {
    const char *e = getenv("UGK_BLOCKS_PER_CU");
    v = e ? atoi(e) : 0;
    if (v <= 0) v = 64;
  }
  return v;
}

namespace {

__global__ __launch_bounds__(kBlock) void fill_u32_kernel(uint32_t *dst, uint32_t v, size_t n) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) dst[i] = v;
}

__global__ __launch_bounds__(kBlock) void arange_u32_kernel(uint32_t *dst, uint32_t start, size_t n) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
    dst[i] = start + (uint32_t)i;
}

// plain streaming copy, 16 bytes per lane, 4 vectors in flight per lane
__global__ __launch_bounds__(kBlock) void copy_v16_kernel(u32x4 *__restrict__ dst, const u32x4 *__restrict__ src,
                                                          size_t nvec) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  for (; i + 3 * stride < nvec; i += 4 * stride) {
    u32x4 a = __builtin_nontemporal_load(src + i);
    u32x4 b = __builtin_nontemporal_load(src + i + stride);
    u32x4 c = __builtin_nontemporal_load(src + i + 2 * stride);
    u32x4 d = __builtin_nontemporal_load(src + i + 3 * stride);
    __builtin_nontemporal_store(a, dst + i);
    __builtin_nontemporal_store(b, dst + i + stride);
    __builtin_nontemporal_store(c, dst + i + 2 * stride);
    __builtin_nontemporal_store(d, dst + i + 3 * stride);
  }
  for (; i < nvec; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

__global__ void copy_tail_kernel(uint8_t *dst, const uint8_t *src, size_t n) {
  for (size_t i = threadIdx.x; i < n; i += blockDim.x) dst[i] = src[i];
}

}  // namespace
}  // namespace ugk

using namespace ugk;

extern "C" {

const char *ugk_last_error(void) { return g_err; }
int ugk_abi_version(void) { return UGK_ABI_VERSION; }

int ugk_device_count(int *count) {
  UGK_REQUIRE(count, "ugk_device_count: null output");
  UGK_HIP(hipGetDeviceCount(count));
  return 0;
}

int ugk_set_device(int dev) {
  UGK_HIP(hipSetDevice(dev));
  return 0;
}

int ugk_get_device_info(int dev, ugk_device_info_t *info) {
  UGK_REQUIRE(info, "ugk_get_device_info: null output");
  hipDeviceProp_t p;
  UGK_HIP(hipGetDeviceProperties(&p, dev));
  memset(info, 0, sizeof(*info));
  snprintf(info->name, sizeof(info->name), "%s", p.name);
  snprintf(info->arch, sizeof(info->arch), "%s", p.gcnArchName);
  info->compute_units = p.multiProcessorCount;
  info->wavefront_size = p.warpSize;
  info->total_mem = p.totalGlobalMem;
  info->lds_per_block = p.sharedMemPerBlock;
  return 0;
}

int ugk_mem_info(size_t *free_bytes, size_t *total_bytes) {
  size_t f = 0, t = 0;
  UGK_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return 0;
}

int ugk_malloc(void **ptr, size_t nbytes) {
  UGK_REQUIRE(ptr, "ugk_malloc: null output");
  *ptr = nullptr;
  if (nbytes == 0) return 0;
  UGK_HIP(hipMalloc(ptr, nbytes));
  return 0;
}

int ugk_free(void *ptr) {
  if (ptr) UGK_HIP(hipFree(ptr));
  return 0;
}

int ugk_host_malloc(void **ptr, size_t nbytes) {
  UGK_REQUIRE(ptr, "ugk_host_malloc: null output");
  *ptr = nullptr;
  if (nbytes == 0) return 0;
  UGK_HIP(hipHostMalloc(ptr, nbytes, hipHostMallocMapped | hipHostMallocPortable));
  return 0;
}

int ugk_host_free(void *ptr) {
  if (ptr) UGK_HIP(hipHostFree(ptr));
  return 0;
}

int ugk_pointer_kind(const void *ptr, int *kind) {
  UGK_REQUIRE(kind, "ugk_pointer_kind: null output");
  hipPointerAttribute_t a;
  hipError_t e = hipPointerGetAttributes(&a, ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // ordinary host memory is reported as an error; clear it
    *kind = 0;
    return 0;
  }
  if (a.type == hipMemoryTypeDevice || a.type == hipMemoryTypeManaged || a.type == hipMemoryTypeArray)
    *kind = 2;
  else if (a.type == hipMemoryTypeHost)
    *kind = 1;
  else
    *kind = 0;
  return 0;
}

int ugk_stream_create(void **stream) {
  UGK_REQUIRE(stream, "ugk_stream_create: null output");
  hipStream_t s;
  // default priority on purpose: mixed stream priorities are not used anywhere in this library
  UGK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  return 0;
}

int ugk_stream_create_cu_masked(void **stream, int num_cus) {
  UGK_REQUIRE(stream, "ugk_stream_create_cu_masked: null output");
  const int total = cu_count();
  UGK_REQUIRE(num_cus > 0 && num_cus <= total, "ugk_stream_create_cu_masked: %d CUs requested, device has %d", num_cus,
              total);
  uint32_t mask[32] = {0};
  UGK_REQUIRE(total <= 32 * 32, "ugk_stream_create_cu_masked: device reports %d CUs", total);
  for (int i = 0; i < num_cus; ++i) mask[i / 32] |= 1u << (i % 32);
  hipStream_t s;
  UGK_HIP(hipExtStreamCreateWithCUMask(&s, (uint32_t)((total + 31) / 32), mask));
  *stream = s;
  return 0;
}

int ugk_stream_destroy(void *stream) {
  if (stream) UGK_HIP(hipStreamDestroy(as_stream(stream)));
  return 0;
}

int ugk_stream_sync(void *stream) {
  UGK_HIP(hipStreamSynchronize(as_stream(stream)));
  return 0;
}

int ugk_stream_is_capturing(void *stream, int *capturing) {
  UGK_REQUIRE(capturing, "ugk_stream_is_capturing: null output");
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(as_stream(stream), &st) != hipSuccess) {
    // the query itself is refused where it would touch a capture (the default stream while another stream of the
    // process records in global mode): work enqueued here would be refused too, and the caller is told so
    (void)hipGetLastError();
    *capturing = UGK_CAPTURE_QUERY_REFUSED;
    return 0;
  }
  *capturing = st != hipStreamCaptureStatusNone ? 1 : 0;
  return 0;
}

namespace {
__global__ void ticket_kernel(volatile uint32_t *word, uint32_t value) { *word = value; }
__global__ void preload_runtime_kernel() {}

// one wavefront: n_a + n_b device words to dst[1 ...], then the ticket to dst[0]
__global__ void words_ticket_kernel(const uint32_t *a, unsigned n_a, const uint32_t *b, unsigned n_b,
                                    volatile uint32_t *dst, uint32_t value) {
  const unsigned lane = threadIdx.x;
  if (lane < n_a) dst[1 + lane] = a[lane];
  else if (lane < n_a + n_b) dst[1 + lane] = b[lane - n_a];
  __threadfence_system();
  __syncthreads();
  if (lane == 0) {
    __threadfence_system();
    dst[0] = value;
  }
}
}  // namespace

int ugk_stream_sync_ticket(void *stream, uint32_t *ticket_host, uint32_t value, unsigned spin_us) {
  UGK_REQUIRE(ticket_host, "ugk_stream_sync_ticket: null ticket word");
  hipLaunchKernelGGL(ticket_kernel, dim3(1), dim3(1), 0, as_stream(stream), ticket_host, value);
  UGK_HIP(hipGetLastError());
  volatile uint32_t *word = ticket_host;
  const auto t0 = std::chrono::steady_clock::now();
  unsigned polls = 0;
  while (*word != value) {
    // the clock is read every 64 polls: a poll is a load of a line the device writes into, the clock a system call away
    if ((++polls & 63u) == 0 &&
        std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count() >=
            (long long)spin_us)
      break;
  }
  // the ticket says that everything enqueued in front of it has run: asking the runtime as well would give back the
  // microseconds the poll saved
  if (*word == value) return 0;
  UGK_HIP(hipStreamSynchronize(as_stream(stream)));
  return 0;
}

int ugk_words_to_host_ticket(const uint32_t *a_dev, unsigned n_a, const uint32_t *b_dev, unsigned n_b,
                             uint32_t *dst_host, uint32_t value, unsigned spin_us, void *stream) {
  UGK_REQUIRE(dst_host, "ugk_words_to_host_ticket: null destination");
  UGK_REQUIRE((a_dev || n_a == 0) && (b_dev || n_b == 0), "ugk_words_to_host_ticket: null source");
  UGK_REQUIRE(n_a + n_b <= 63u, "ugk_words_to_host_ticket: %u words, at most 63 fit one launch", n_a + n_b);
  hipLaunchKernelGGL(words_ticket_kernel, dim3(1), dim3(64), 0, as_stream(stream), a_dev, n_a, b_dev, n_b, dst_host,
                     value);
  UGK_HIP(hipGetLastError());
  volatile uint32_t *word = dst_host;
  const auto t0 = std::chrono::steady_clock::now();
  unsigned polls = 0;
  while (*word != value) {
    if ((++polls & 63u) == 0 &&
        std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count() >=
            (long long)spin_us)
      break;
  }
  if (*word != value) UGK_HIP(hipStreamSynchronize(as_stream(stream)));
  std::atomic_thread_fence(std::memory_order_acquire);
  return 0;
}

int ugk_preload_kernels(void) {
  hipStream_t st;
  UGK_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  hipLaunchKernelGGL(preload_runtime_kernel, dim3(1), dim3(1), 0, st);  // this file's own
  ugk::preload_gather(st);
  ugk::preload_hotness(st);
  ugk::preload_partition(st);
  ugk::preload_pool(st);
  ugk::preload_refresh(st);
  ugk::preload_table(st);
  const hipError_t launched = hipGetLastError();
  const hipError_t waited = hipStreamSynchronize(st);
  (void)hipStreamDestroy(st);
  UGK_HIP(launched);
  UGK_HIP(waited);
  return 0;
}

int ugk_device_sync(void) {
  UGK_HIP(hipDeviceSynchronize());
  return 0;
}

int ugk_event_create(void **event) {
  UGK_REQUIRE(event, "ugk_event_create: null output");
  hipEvent_t e;
  UGK_HIP(hipEventCreate(&e));
  *event = e;
  return 0;
}

int ugk_event_destroy(void *event) {
  if (event) UGK_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
  return 0;
}

int ugk_event_record(void *event, void *stream) {
  UGK_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
  return 0;
}

int ugk_event_sync(void *event) {
  UGK_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
  return 0;
}

int ugk_event_query(void *event, int *complete) {
  UGK_REQUIRE(event && complete, "ugk_event_query: null pointer");
  const hipError_t e = hipEventQuery(reinterpret_cast<hipEvent_t>(event));
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    *complete = 0;
    return 0;
  }
  UGK_HIP(e);
  *complete = 1;
  return 0;
}

int ugk_stream_wait_event(void *stream, void *event) {
  UGK_HIP(hipStreamWaitEvent(as_stream(stream), reinterpret_cast<hipEvent_t>(event), 0));
  return 0;
}

int ugk_event_elapsed_ms(void *start, void *stop, float *ms) {
  UGK_REQUIRE(ms, "ugk_event_elapsed_ms: null output");
  UGK_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
  return 0;
}

int ugk_memcpy_async(void *dst, const void *src, size_t nbytes, void *stream) {
  if (nbytes == 0) return 0;
  UGK_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDefault, as_stream(stream)));
  return 0;
}

int ugk_fill_u32(uint32_t *dst_dev, uint32_t value, size_t nwords, void *stream) {
  if (nwords == 0) return 0;
  UGK_REQUIRE(dst_dev, "ugk_fill_u32: null destination");
  const unsigned grid = clamp_grid((nwords + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), dst_dev, value, nwords);
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_arange_u32(uint32_t *dst_dev, uint32_t start, size_t n, void *stream) {
  if (n == 0) return 0;
  UGK_REQUIRE(dst_dev, "ugk_arange_u32: null destination");
  const unsigned grid = clamp_grid((n + kBlock - 1) / kBlock, 0);
  hipLaunchKernelGGL(arange_u32_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), dst_dev, start, n);
  UGK_HIP(hipGetLastError());
  return 0;
}

int ugk_copy_rows(void *dst_dev, const void *src_dev, size_t nbytes, void *stream) {
  if (nbytes == 0) return 0;
  UGK_REQUIRE(dst_dev && src_dev, "ugk_copy_rows: null pointer");
  UGK_REQUIRE(((uintptr_t)dst_dev % 16 == 0) && ((uintptr_t)src_dev % 16 == 0), "ugk_copy_rows: pointers must be 16-byte aligned");
  const size_t nvec = nbytes / 16;
  if (nvec) {
    const unsigned grid = clamp_grid((nvec + kBlock * 4 - 1) / (kBlock * 4), 0);
    hipLaunchKernelGGL(copy_v16_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), (u32x4 *)dst_dev,
                       (const u32x4 *)src_dev, nvec);
    UGK_HIP(hipGetLastError());
  }
  const size_t tail = nbytes - nvec * 16;
  if (tail) {
    hipLaunchKernelGGL(copy_tail_kernel, dim3(1), dim3(64), 0, as_stream(stream), (uint8_t *)dst_dev + nvec * 16,
                       (const uint8_t *)src_dev + nvec * 16, tail);
    UGK_HIP(hipGetLastError());
  }
  return 0;
}

}  // extern "C"
