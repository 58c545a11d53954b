// Core types of the facade, kept source-compatible with coll_cache_lib/common.h of the reference
// (IdType constant.h:28; DataType/Context/MemHandle/BarHandle/Tensor common.h:39-49, 110-168, 191-288) so that
// callers of CollCache / CacheContext compile unchanged.  Host C++ only: the GPU is reached through the
// C-ABI in ugache_hip.h.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <numeric>
#include <ostream>
#include <string>
#include <vector>

namespace coll_cache_lib {
namespace common {

using IdType = unsigned int;   // constant.h:28
using Id64Type = int64_t;      // wide keys: an extension over the reference, which is uint32 end to end

enum DataType {
  kF32 = 0,
  kF64 = 1,
  kF16 = 2,
  kU8 = 3,
  kI32 = 4,
  kI8 = 5,
  kI64 = 6,
  kF64_2 = 7,  // 16-byte unit
  kF64_4 = 8,  // 32-byte unit
};

enum DeviceType { kMMAP = 0, kCPU = 1, kGPU = 2, kGPU_UM = 3 };

enum CachePolicy {
  kCacheByDegree = 0,
  kCacheByHeuristic,
  kCacheByPreSample,
  kCacheByDegreeHop,
  kCacheByPreSampleStatic,
  kCacheByFakeOptimal,
  kDynamicCache,
  kCacheByRandom,
  kCollCache,
  kCollCacheIntuitive,
  kPartitionCache,
  kPartRepCache,
  kRepCache,
  kCollCacheAsymmLink,
  kCliquePart,
  kCliquePartByDegree,
  kSOK,
  kHPS,
  kCollFineGrain,
};

struct Context {
  DeviceType device_type;
  int device_id;
  Context() : device_type(kCPU), device_id(0) {}
  Context(DeviceType type, int id) : device_type(type), device_id(id) {}
  int GetCudaDeviceId() const { return (device_type == kCPU || device_type == kMMAP) ? -1 : device_id; }
  bool operator==(const Context &rhs) const { return device_type == rhs.device_type && device_id == rhs.device_id; }
};
std::ostream &operator<<(std::ostream &os, const Context &ctx);

using StreamHandle = void *;

class Tensor;
using TensorPtr = std::shared_ptr<Tensor>;

// All GPU memory of the cache is requested through a caller-supplied allocator returning one of these
// (common.h:140-149); the memory is released when the handle dies.
class ExternelGPUMemoryHandler {
 public:
  ExternelGPUMemoryHandler() {}
  virtual ~ExternelGPUMemoryHandler() {}
  virtual void *ptr() = 0;
  virtual size_t nbytes() { return 0; }
  template <typename T>
  T *ptr() {
    return static_cast<T *>(ptr());
  }
};
using MemHandle = std::shared_ptr<ExternelGPUMemoryHandler>;

// Device memory owned by the library itself (long-lived structures), rounded to 2 MiB like the reference's
// eager allocator (cache_context.cu:2612-2622).
class EagerGPUMemoryHandler : public ExternelGPUMemoryHandler {
 public:
  void *ptr_ = nullptr;
  int dev_id_ = 0;
  size_t nbytes_ = 0;
  EagerGPUMemoryHandler() {}
  ~EagerGPUMemoryHandler() override;
  void *ptr() override { return ptr_; }
  size_t nbytes() override { return nbytes_; }
};
MemHandle EagerGPUAlloc(int dev_id, size_t nbytes);

// Pinned, GPU-mapped host memory owned by the library.
class PinnedHostMemoryHandler : public ExternelGPUMemoryHandler {
 public:
  void *ptr_ = nullptr;
  size_t nbytes_ = 0;
  ~PinnedHostMemoryHandler() override;
  void *ptr() override { return ptr_; }
  size_t nbytes() override { return nbytes_; }
};
MemHandle PinnedHostAlloc(size_t nbytes);

class ExternalBarrierHandler {
 public:
  ExternalBarrierHandler() {}
  virtual ~ExternalBarrierHandler() {}
  virtual void Wait() = 0;
};
using BarHandle = std::shared_ptr<ExternalBarrierHandler>;

// Sense-reversing spin barrier for the replicas (threads) of one process.  The reference keeps the counter in
// an anonymous shared mapping so forked replicas can share it (common.cc:677-689, atomic_barrier.h:9-43); with
// one GPU there is one replica and Wait() returns at once.
class AnonymousBarrier : public ExternalBarrierHandler {
 public:
  AnonymousBarrier();
  ~AnonymousBarrier() override;
  void SetWorker(int worker);
  void Wait() override;
  int worker = 1;
  static std::shared_ptr<AnonymousBarrier> _global_instance;
  static std::shared_ptr<AnonymousBarrier> _refresh_instance;

 private:
  void *_state;
};

size_t GetDataTypeBytes(DataType dtype);
size_t GetTensorBytes(DataType dtype, const std::vector<size_t> &shape);
DataType nb_to_dt(size_t nbytes);

constexpr int CPU_CUDA_HOST_MALLOC_DEVICE = 0;
constexpr int CPU_CLIB_MALLOC_DEVICE = 1;
constexpr int CPU_FOREIGN = 2;
Context CPU(int device_id = CPU_CUDA_HOST_MALLOC_DEVICE);
Context CPU_CLIB(int device_id = CPU_CLIB_MALLOC_DEVICE);
Context GPU(int device_id = 0);

// Minimal n-d array descriptor with the accessors the path uses (common.h:191-288).
class Tensor : public std::enable_shared_from_this<Tensor> {
 public:
  Tensor() {}
  ~Tensor();
  bool Defined() const { return _data != nullptr; }
  DataType Type() const { return _dtype; }
  const std::vector<size_t> &Shape() const { return _shape; }
  const void *Data() const { return _data; }
  void *MutableData() { return _data; }
  template <typename T>
  T *Ptr() {
    return static_cast<T *>(_data);
  }
  template <typename T>
  const T *CPtr() const {
    return static_cast<const T *>(_data);
  }
  size_t NumBytes() const { return _nbytes; }
  Context Ctx() const { return _ctx; }
  size_t NumItem() const { return std::accumulate(_shape.begin(), _shape.end(), (size_t)1, std::multiplies<size_t>()); }
  std::string Name() const { return _name; }
  // shrink or regrow inside the existing allocation
  bool CanForceScale(DataType dt, const std::vector<size_t> &shape) const;
  void ForceScale(DataType dt, const std::vector<size_t> &shape, Context ctx, const std::string &name);

  // host memory from malloc (CPU_CLIB) or pinned memory (CPU()), owned by the tensor
  static TensorPtr Empty(DataType dtype, const std::vector<size_t> &shape, Context ctx, const std::string &name);
  static TensorPtr EmptyExternal(DataType dtype, const std::vector<size_t> &shape,
                                 const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                 const std::string &name);
  static TensorPtr FromBlob(void *data, DataType dtype, const std::vector<size_t> &shape, Context ctx,
                            const std::string &name);
  // copy a host or device tensor into memory from `allocator` (async on stream)
  static TensorPtr CopyToExternal(TensorPtr source, const std::function<MemHandle(size_t)> &allocator, Context ctx,
                                  StreamHandle stream = nullptr);
  static TensorPtr CopyBlob(const void *data, DataType dtype, const std::vector<size_t> &shape, Context from_ctx,
                            Context to_ctx, const std::string &name, StreamHandle stream = nullptr);

 private:
  void *_data = nullptr;
  DataType _dtype = kI32;
  Context _ctx;
  size_t _nbytes = 0;
  size_t _capacity = 0;
  std::vector<size_t> _shape;
  std::string _name;
  MemHandle _external;
  bool _owns_malloc = false;
};

std::string ToReadableSize(size_t nbytes);
std::string ToPercentage(double percentage);
std::string GetEnv(const std::string &key);
bool IsEnvSet(const std::string &key);

template <typename T>
inline T RoundUpDiv(T target, T unit) {
  return (target + unit - 1) / unit;
}
template <typename T>
inline T RoundUp(T target, T unit) {
  return RoundUpDiv(target, unit) * unit;
}

}  // namespace common
}  // namespace coll_cache_lib
