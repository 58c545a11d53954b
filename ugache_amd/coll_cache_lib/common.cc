#include "common.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>

#include "logging.h"
#include "ugache_hip.h"

namespace coll_cache_lib {
namespace common {

std::ostream &operator<<(std::ostream &os, const Context &ctx) {
  switch (ctx.device_type) {
    case kMMAP: return os << "mmap:" << ctx.device_id;
    case kCPU: return os << "cpu:" << ctx.device_id;
    case kGPU: return os << "gpu:" << ctx.device_id;
    case kGPU_UM: return os << "gpu_um:" << ctx.device_id;
  }
  return os;
}

EagerGPUMemoryHandler::~EagerGPUMemoryHandler() {
  if (ptr_) {
    if (ugk_set_device(dev_id_) == 0) ugk_free(ptr_);
    ptr_ = nullptr;
  }
}

MemHandle EagerGPUAlloc(int dev_id, size_t nbytes) {
  auto ret = std::make_shared<EagerGPUMemoryHandler>();
  ret->dev_id_ = dev_id;
  ret->nbytes_ = nbytes;
  UGK_CALL(ugk_set_device(dev_id));
  size_t alloc = nbytes > ((size_t)1 << 21) ? RoundUp(nbytes, (size_t)1 << 21) : (nbytes ? nbytes : 256);
  UGK_CALL(ugk_malloc(&ret->ptr_, alloc));
  return ret;
}

PinnedHostMemoryHandler::~PinnedHostMemoryHandler() {
  if (ptr_) ugk_host_free(ptr_);
  ptr_ = nullptr;
}

MemHandle PinnedHostAlloc(size_t nbytes) {
  auto ret = std::make_shared<PinnedHostMemoryHandler>();
  ret->nbytes_ = nbytes;
  UGK_CALL(ugk_host_malloc(&ret->ptr_, nbytes ? nbytes : 64));
  return ret;
}

// ---- barrier -------------------------------------------------------------------------------------------
namespace {
struct BarrierState {
  std::atomic<int> count{0};
  std::atomic<int> generation{0};
};
}  // namespace

std::shared_ptr<AnonymousBarrier> AnonymousBarrier::_global_instance = std::make_shared<AnonymousBarrier>();
std::shared_ptr<AnonymousBarrier> AnonymousBarrier::_refresh_instance = std::make_shared<AnonymousBarrier>();

AnonymousBarrier::AnonymousBarrier() : _state(new BarrierState) {}
AnonymousBarrier::~AnonymousBarrier() { delete static_cast<BarrierState *>(_state); }
void AnonymousBarrier::SetWorker(int w) {
  CHECK_GE(w, 1);
  worker = w;
}
void AnonymousBarrier::Wait() {
  if (worker <= 1) return;
  auto *st = static_cast<BarrierState *>(_state);
  const int gen = st->generation.load(std::memory_order_acquire);
  if (st->count.fetch_add(1, std::memory_order_acq_rel) + 1 == worker) {
    st->count.store(0, std::memory_order_relaxed);
    st->generation.fetch_add(1, std::memory_order_release);
  } else {
    while (st->generation.load(std::memory_order_acquire) == gen) std::this_thread::yield();
  }
}

// ---- dtype helpers -------------------------------------------------------------------------------------
size_t GetDataTypeBytes(DataType dtype) {
  switch (dtype) {
    case kI8:
    case kU8: return 1;
    case kF16: return 2;
    case kF32:
    case kI32: return 4;
    case kI64:
    case kF64: return 8;
    case kF64_2: return 16;
    case kF64_4: return 32;
  }
  LOG(FATAL) << "unknown data type " << (int)dtype;
  return 0;
}

size_t GetTensorBytes(DataType dtype, const std::vector<size_t> &shape) {
  size_t n = 1;
  for (size_t s : shape) n *= s;
  return n * GetDataTypeBytes(dtype);
}

DataType nb_to_dt(size_t nbytes) {
  switch (nbytes) {
    case 1: return kU8;
    case 2: return kF16;
    case 4: return kF32;
    case 8: return kF64;
    case 16: return kF64_2;
    case 32: return kF64_4;
  }
  LOG(FATAL) << "no data type of " << nbytes << " bytes";
  return kU8;
}

Context CPU(int device_id) { return {kCPU, device_id}; }
Context CPU_CLIB(int device_id) { return {kCPU, device_id}; }
Context GPU(int device_id) { return {kGPU, device_id}; }

// ---- tensor --------------------------------------------------------------------------------------------
Tensor::~Tensor() {
  if (_owns_malloc && _data) free(_data);
  _data = nullptr;
}

bool Tensor::CanForceScale(DataType dt, const std::vector<size_t> &shape) const {
  return GetTensorBytes(dt, shape) <= _capacity;
}

void Tensor::ForceScale(DataType dt, const std::vector<size_t> &shape, Context ctx, const std::string &name) {
  CHECK(CanForceScale(dt, shape)) << "tensor " << _name << " of " << _capacity << " bytes cannot hold "
                                  << GetTensorBytes(dt, shape);
  _dtype = dt;
  _shape = shape;
  _nbytes = GetTensorBytes(dt, shape);
  (void)ctx;
  if (!name.empty()) _name = name;
}

TensorPtr Tensor::Empty(DataType dtype, const std::vector<size_t> &shape, Context ctx, const std::string &name) {
  CHECK(ctx.device_type == kCPU) << "Tensor::Empty only hands out host memory; GPU memory comes from an allocator";
  auto t = std::make_shared<Tensor>();
  t->_dtype = dtype;
  t->_shape = shape;
  t->_ctx = ctx;
  t->_name = name;
  t->_nbytes = GetTensorBytes(dtype, shape);
  t->_capacity = t->_nbytes;
  if (ctx.device_id == CPU_CUDA_HOST_MALLOC_DEVICE) {
    t->_external = PinnedHostAlloc(t->_nbytes);
    t->_data = t->_external->ptr();
  } else {
    t->_data = malloc(t->_nbytes ? t->_nbytes : 1);
    CHECK_NOTNULL(t->_data);
    t->_owns_malloc = true;
  }
  return t;
}

TensorPtr Tensor::EmptyExternal(DataType dtype, const std::vector<size_t> &shape,
                                const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                const std::string &name) {
  auto t = std::make_shared<Tensor>();
  t->_dtype = dtype;
  t->_shape = shape;
  t->_ctx = ctx;
  t->_name = name;
  t->_nbytes = GetTensorBytes(dtype, shape);
  t->_external = allocator(t->_nbytes);
  CHECK_NOTNULL(t->_external);
  t->_capacity = t->_external->nbytes() ? t->_external->nbytes() : t->_nbytes;
  t->_data = t->_external->ptr();
  return t;
}

TensorPtr Tensor::FromBlob(void *data, DataType dtype, const std::vector<size_t> &shape, Context ctx,
                           const std::string &name) {
  auto t = std::make_shared<Tensor>();
  t->_dtype = dtype;
  t->_shape = shape;
  t->_ctx = ctx;
  t->_name = name;
  t->_nbytes = GetTensorBytes(dtype, shape);
  t->_capacity = t->_nbytes;
  t->_data = data;
  return t;
}

TensorPtr Tensor::CopyToExternal(TensorPtr source, const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                 StreamHandle stream) {
  CHECK_NOTNULL(source);
  auto t = EmptyExternal(source->Type(), source->Shape(), allocator, ctx, source->Name());
  if (source->NumBytes() > 0) {
    UGK_CALL(ugk_memcpy_async(t->MutableData(), source->Data(), source->NumBytes(), stream));
    UGK_CALL(ugk_stream_sync(stream));  // the source may be pageable host memory that dies right after
  }
  return t;
}

TensorPtr Tensor::CopyBlob(const void *data, DataType dtype, const std::vector<size_t> &shape, Context from_ctx,
                           Context to_ctx, const std::string &name, StreamHandle stream) {
  CHECK(from_ctx.device_type == kCPU && to_ctx.device_type == kCPU) << "CopyBlob is host to host";
  (void)stream;
  auto t = Empty(dtype, shape, to_ctx, name);
  memcpy(t->MutableData(), data, t->NumBytes());
  return t;
}

// ---- misc ----------------------------------------------------------------------------------------------
std::string ToReadableSize(size_t nbytes) {
  char buf[64];
  const double kb = 1024.0, mb = kb * 1024, gb = mb * 1024;
  if (nbytes > gb) snprintf(buf, sizeof(buf), "%.2f GB", nbytes / gb);
  else if (nbytes > mb) snprintf(buf, sizeof(buf), "%.2f MB", nbytes / mb);
  else if (nbytes > kb) snprintf(buf, sizeof(buf), "%.2f KB", nbytes / kb);
  else snprintf(buf, sizeof(buf), "%.2f Bytes", (double)nbytes);
  return buf;
}

std::string ToPercentage(double p) {
  char buf[32];
  snprintf(buf, sizeof(buf), "%.2f %%", p * 100);
  return buf;
}

std::string GetEnv(const std::string &key) {
  const char *v = getenv(key.c_str());
  return v ? std::string(v) : std::string();
}

bool IsEnvSet(const std::string &key) {
  const std::string v = GetEnv(key);
  return v == "1" || v == "ON" || v == "TRUE" || v == "true" || v == "on";
}

}  // namespace common
}  // namespace coll_cache_lib
