// The extern "C" shim over the facade: the counterpart of python/collcache/common/operation.cc.
#include "operation.h"

#include <sys/wait.h>

#include <cstring>
#include <iostream>
#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <mutex>
#include <string>
#include <thread>
#include <vector>
#include <unordered_map>

#include "facade.h"
#include "freq_recorder.h"
#include "logging.h"
#include "placement.h"
#include "profiler.h"
#include "run_config.h"
#include "timer.h"
#include "ugache_hip.h"

namespace coll_cache_lib {
namespace common {

namespace {
std::shared_ptr<CollCache> _coll_cache = nullptr;
std::shared_ptr<Profiler> _profiler = nullptr;
std::vector<std::shared_ptr<FreqRecorder>> _freq_recorder;
size_t steps[9] = {0};
size_t internal_feat_dim = 0;
size_t outside_feat_dim = 0;

class CallbackMemHandle : public ExternelGPUMemoryHandler {
 public:
  void *ptr_ = nullptr;
  size_t nbytes_ = 0;
  coll_cache_release_fn release_ = nullptr;
  void *user_ = nullptr;
  ~CallbackMemHandle() override {
    if (release_ && ptr_) release_(ptr_, user_);
  }
  void *ptr() override { return ptr_; }
  size_t nbytes() override { return nbytes_; }
};

std::function<MemHandle(size_t)> MakeAllocator(coll_cache_alloc_fn alloc, coll_cache_release_fn release, void *user,
                                               int replica_id) {
  if (alloc == nullptr) {
    const int dev = RunConfig::device_id_list.empty() ? 0 : RunConfig::device_id_list[replica_id];
    return [dev](size_t nbytes) -> MemHandle { return EagerGPUAlloc(dev, nbytes); };
  }
  return [alloc, release, user](size_t nbytes) -> MemHandle {
    auto h = std::make_shared<CallbackMemHandle>();
    h->ptr_ = alloc(nbytes, user);
    CHECK(h->ptr_ != nullptr || nbytes == 0) << "allocator callback returned NULL for " << nbytes << " bytes";
    h->nbytes_ = nbytes;
    h->release_ = release;
    h->user_ = user;
    return h;
  };
}

// The first launch out of each source file of the kernel library loads that file's code object onto the device, 5 to
// 11 ms apiece and some 40 ms in all, which the first build, lookup and refresh would pay where they stand.  A helper
// thread pays it from the moment the library is configured, while the caller records its presample and the host ranks
// it; every build waits for the thread before it touches the device (the build of a 1 M-row table with 100,000 rows
// cached: 25 -> 7 ms; of 100 M rows with 25 M cached: 0.285 -> 0.260 s).
struct KernelPreloader {
  std::thread thread;
  void Start(int device) {
    const char *knob = getenv("COLL_PRELOAD_KERNELS");  // the other knobs are read when a build starts: too late here
    if ((knob && knob[0] == '0') || thread.joinable()) return;
    thread = std::thread([device] {
      if (ugk_set_device(device) == 0) (void)ugk_preload_kernels();  // a failure here shows up at the first real launch
    });
  }
  void Join() {
    if (thread.joinable()) thread.join();
  }
  ~KernelPreloader() { Join(); }  // a process that configures and exits
};
KernelPreloader _preloader;

void coll_cache_config_from_map(std::unordered_map<std::string, std::string> &configs) {
  using CRC = RunConfig;
  CHECK(!CRC::is_configured);
  CHECK_EQ(ugk_abi_version(), UGK_ABI_VERSION) << "libugache_hip.so and libcoll_cache.so come from different builds";
  CHECK(configs.count("cache_percentage"));
  CHECK(configs.count("_cache_policy"));
  CHECK(configs.count("num_device"));
  CHECK(configs.count("num_global_step_per_epoch"));
  CHECK(configs.count("num_epoch"));
  CHECK(configs.count("num_total_item"));
  CHECK(configs.count("omp_thread_num"));

  CRC::cache_percentage = std::stod(configs["cache_percentage"]);
  CRC::cache_policy = static_cast<CachePolicy>(std::stoi(configs["_cache_policy"]));
  CRC::cross_process = true;
  CRC::num_device = std::stoull(configs["num_device"]);
  CHECK_EQ(CRC::num_device, (size_t)1) << "this build serves one GPU: num_device must be 1";
  CRC::device_id_list.resize(CRC::num_device);
  for (size_t i = 0; i < CRC::num_device; i++) CRC::device_id_list[i] = (int)i;
  CRC::num_global_step_per_epoch = std::stoull(configs["num_global_step_per_epoch"]);
  CRC::num_epoch = std::stoull(configs["num_epoch"]);
  CRC::num_total_item = std::stoull(configs["num_total_item"]);
  CRC::omp_thread_num = std::stoi(configs["omp_thread_num"]);
  CHECK_GT(CRC::omp_thread_num, 0);
  CRC::solver_omp_thread_num = CRC::omp_thread_num;
  CRC::solver_omp_thread_num_per_gpu = std::max<int>(1, CRC::omp_thread_num / (int)CRC::num_device);
  CRC::is_configured = true;

  _profiler = std::make_shared<Profiler>();
  AnonymousBarrier::_global_instance->SetWorker((int)CRC::num_device);
  AnonymousBarrier::_refresh_instance->SetWorker((int)CRC::num_device);
  _coll_cache = std::make_shared<CollCache>(nullptr, AnonymousBarrier::_global_instance);
  _coll_cache->_profiler = _profiler;
  _preloader.Start(CRC::device_id_list[0]);
}

// prefixes that stream-ordered serving steps have copied out and not counted yet (defined with the serving loop)
void CountPendingPrefixes(bool all);

// top_k: SIZE_MAX for the full rank order; else the placement that follows caches top_k keys and needs only to know
// which entries are the top_k best (FreqRankSolver reads the list as "the first top_k entries are cached")
ContFreqBuf *CombineAndRank(int replica_id, size_t top_k = SIZE_MAX) {
  CHECK_LT((size_t)replica_id, _freq_recorder.size()) << "coll_cache_record_init was not called";
  CHECK_NOTNULL(_freq_recorder[replica_id]);
  CountPendingPrefixes(/*all=*/true);
  // what the lookups counted on the device joins what coll_cache_record counted on the host
  if (_coll_cache && _coll_cache->num_replicas_built() > (size_t)replica_id && _coll_cache->session(replica_id)) {
    const size_t rows = _coll_cache->session(replica_id)->DrainHotness(_freq_recorder[replica_id].get());
    if (rows) LOG(INFO) << "hotness of " << rows << " rows taken from the device counters";
  }
  _freq_recorder[replica_id]->LocalCombineToShared();
  AnonymousBarrier::_global_instance->Wait();
  ContFreqBuf *freq_rank = nullptr;
  if (replica_id == 0) {
    _freq_recorder[0]->GlobalCombine();
    if (top_k == SIZE_MAX) _freq_recorder[0]->Sort();
    else _freq_recorder[0]->SelectTop(top_k);
    freq_rank = _freq_recorder[0]->global_cont_freq_buf;
  }
  return freq_rank;
}

void NormalizeHalf(DataType &dtype, size_t &dim) {
  outside_feat_dim = dim;
  if (dtype == kF16) {  // operation.cc:132-136: the library moves bytes, fp16 rows travel as dim/2 fp32 words
    CHECK(dim % 2 == 0);
    dtype = kF32;
    dim /= 2;
  }
  internal_feat_dim = dim;
}

}  // namespace

size_t max_num_keys = 0;

void coll_cache_init(int replica_id, size_t key_space_size, std::function<MemHandle(size_t)> allocator,
                     void *cpu_data, DataType dtype, size_t dim, double cache_percentage, StreamHandle stream) {
  CHECK(RunConfig::is_configured);
  NormalizeHalf(dtype, dim);
  ContFreqBuf *freq_rank = nullptr;
  const bool need_rank = cache_percentage != 0 && cache_percentage != 1;
  Timer t_rank;
  if (need_rank)
    freq_rank = CombineAndRank(
        replica_id, coll_cache::FreqRankSolver::NumCachedNodes((IdType)key_space_size, cache_percentage * 100));
  LOG(INFO) << "build: ranking " << t_rank.Passed() << " s";
  _preloader.Join();
  Timer t_build;
  _coll_cache->build_v2(replica_id, freq_rank, (IdType)key_space_size, allocator, cpu_data, dtype, dim,
                        cache_percentage, stream);
  // COLL_GPU_RECORD_SEED: the counters the lookups bump start from what this cache was ranked by
  auto session = _coll_cache->session(replica_id);
  if (RunConfig::gpu_record_seed && freq_rank && session && session->CountsOnDevice())
    session->SeedHotness(freq_rank->buf, freq_rank->entries.size());
  LOG(INFO) << "coll cache has been initialized successfully: build_v2 " << t_build.Passed() << " s";
}

extern "C" {

void coll_cache_config(const char **config_keys, const char **config_values, const size_t num_config_items) {
  CHECK(!RunConfig::is_configured);
  std::unordered_map<std::string, std::string> configs;
  for (size_t i = 0; i < num_config_items; i++) configs[std::string(config_keys[i])] = std::string(config_values[i]);
  coll_cache_config_from_map(configs);
}

void coll_cache_log_step_by_key(uint64_t key, int item, double val) {
  CHECK_NOTNULL(_profiler);
  CHECK_LT(item, (int)kNumLogStepItems);
  CHECK_GE(item, 0);
  _profiler->LogStep(key, static_cast<LogStepItem>(item), val);
}

void coll_cache_report_step_by_key(uint64_t key) {
  CHECK_NOTNULL(_profiler);
  _profiler->ReportStep(RunConfig::GetEpochFromKey(key), RunConfig::GetStepFromKey(key));
  std::cout.flush();
}

void coll_cache_report_step_average_by_key(uint64_t key) {
  CHECK_NOTNULL(_profiler);
  _profiler->ReportStepAverage(RunConfig::num_epoch - 1, RunConfig::num_global_step_per_epoch - 1);
  _profiler->ReportStepItemPercentiles(RunConfig::num_epoch - 1, RunConfig::num_global_step_per_epoch - 1,
                                       kLogL2CacheCopyTime, {50, 90, 95, 99, 99.9}, "tail_logl2featcopy");
  std::cout.flush();
}

void coll_cache_record_init(int replica_id) {
  CHECK(RunConfig::is_configured);
  _freq_recorder.resize(RunConfig::num_device);
  CHECK_LT((size_t)replica_id, _freq_recorder.size());
  _freq_recorder[replica_id] = std::make_shared<FreqRecorder>(RunConfig::num_total_item, replica_id);
}

void coll_cache_train_barrier(void) { AnonymousBarrier::_global_instance->Wait(); }

int coll_cache_wait_one_child(void) {
  int child_stat = 0;
  pid_t pid = waitpid(-1, &child_stat, 0);
  if (pid < 0) return 0;
  if (WIFSIGNALED(child_stat)) {
    LOG(ERROR) << "detect an abnormal terminated child, signal is " << strsignal(WTERMSIG(child_stat));
    return 1;
  }
  if (WEXITSTATUS(child_stat) != 0) {
    LOG(ERROR) << "detect a terminated child " << pid << ", status is " << WEXITSTATUS(child_stat);
    return 1;
  }
  return 0;
}

void coll_cache_print_memory_usage(void) {
  size_t free_b = 0, total_b = 0;
  UGK_CALL(ugk_mem_info(&free_b, &total_b));
  std::cout << "[HIP] gpu: usage: " << ToReadableSize(total_b - free_b) << "\n";
  std::cout.flush();
}

void coll_cache_lookup(int replica_id, uint32_t *key, size_t num_keys, void *output, StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  const uint64_t step_key = steps[replica_id] * RunConfig::num_device + replica_id;
  steps[replica_id]++;
  _coll_cache->lookup(replica_id, key, num_keys, output, stream, step_key);
}

void coll_cache_lookup_i64(int replica_id, const int64_t *key, size_t num_keys, void *output, StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  const uint64_t step_key = steps[replica_id] * RunConfig::num_device + replica_id;
  steps[replica_id]++;
  _coll_cache->lookup64(replica_id, key, num_keys, output, stream, step_key);
}

void coll_cache_lookup_pooled(int replica_id, const uint32_t *key, const int64_t *seg_off, const float *weights,
                              size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                              StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  const uint64_t step_key = steps[replica_id] * RunConfig::num_device + replica_id;
  steps[replica_id]++;
  _coll_cache->lookup_pooled(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes, output, stream,
                             step_key);
}

void coll_cache_lookup_pooled_i64(int replica_id, const int64_t *key, const int64_t *seg_off, const float *weights,
                                  size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                                  StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  const uint64_t step_key = steps[replica_id] * RunConfig::num_device + replica_id;
  steps[replica_id]++;
  _coll_cache->lookup_pooled64(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes, output,
                               stream, step_key);
}

size_t coll_cache_lookup_unique(int replica_id, const uint32_t *key, size_t num_keys, void *output,
                                uint32_t *inverse_out, StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  const uint64_t step_key = steps[replica_id] * RunConfig::num_device + replica_id;
  steps[replica_id]++;
  return _coll_cache->lookup_unique(replica_id, key, num_keys, output, inverse_out, stream, step_key);
}

size_t coll_cache_lookup_unique_i64(int replica_id, const int64_t *key, size_t num_keys, void *output,
                                    uint32_t *inverse_out, StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  const uint64_t step_key = steps[replica_id] * RunConfig::num_device + replica_id;
  steps[replica_id]++;
  return _coll_cache->lookup_unique64(replica_id, key, num_keys, output, inverse_out, stream, step_key);
}

void coll_cache_lookup_async(int replica_id, const uint32_t *key, size_t num_keys, void *output,
                             StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  steps[replica_id]++;
  _coll_cache->lookup_async(replica_id, key, num_keys, output, stream);
}

void coll_cache_lookup_async_i64(int replica_id, const int64_t *key, size_t num_keys, void *output,
                                 StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  steps[replica_id]++;
  _coll_cache->lookup_async64(replica_id, key, num_keys, output, stream);
}

void coll_cache_lookup_pooled_async(int replica_id, const uint32_t *key, const int64_t *seg_off, const float *weights,
                                    size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                                    StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  steps[replica_id]++;
  _coll_cache->lookup_pooled_async(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes, output,
                                   stream);
}

void coll_cache_lookup_pooled_async_i64(int replica_id, const int64_t *key, const int64_t *seg_off,
                                        const float *weights, size_t num_rows, size_t num_keys, int combiner,
                                        int elem_bytes, void *output, StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  steps[replica_id]++;
  _coll_cache->lookup_pooled_async64(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes,
                                     output, stream);
}

void coll_cache_set_pooled_max_norm(int replica_id, float max_norm) {
  CHECK_NOTNULL(_coll_cache);
  CHECK(max_norm >= 0.f) << "max_norm is an l2 norm (0 turns the clipping off), not " << max_norm;
  _coll_cache->session(replica_id)->SetPooledMaxNorm(max_norm);
}

void coll_cache_segment_offsets(int replica_id, const int64_t *sorted_rows, size_t num_entries, size_t num_rows,
                                int64_t *seg_off, StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  _coll_cache->segment_offsets(replica_id, sorted_rows, num_entries, num_rows, seg_off, stream);
}

void coll_cache_lookup_wait(int replica_id, StreamHandle stream) {
  CHECK_NOTNULL(_coll_cache);
  _coll_cache->lookup_wait(replica_id, stream);
  CountPendingPrefixes(/*all=*/true);
}

void coll_cache_record(int replica_id, uint32_t *key, size_t num_keys) {
  CHECK_LT((size_t)replica_id, _freq_recorder.size()) << "coll_cache_record_init was not called";
  _freq_recorder[replica_id]->Record(key, num_keys);
  max_num_keys = std::max(max_num_keys, num_keys);
}

void coll_cache_record_i64(int replica_id, const int64_t *key, size_t num_keys) {
  CHECK_LT((size_t)replica_id, _freq_recorder.size()) << "coll_cache_record_init was not called";
  _freq_recorder[replica_id]->Record(key, num_keys);
  max_num_keys = std::max(max_num_keys, num_keys);
}

void coll_cache_init_c(int replica_id, size_t key_space_size, coll_cache_alloc_fn alloc, coll_cache_release_fn release,
                       void *user, void *cpu_data, int dtype, size_t dim, double cache_percentage,
                       StreamHandle stream) {
  CHECK(RunConfig::is_configured);
  coll_cache_init(replica_id, key_space_size, MakeAllocator(alloc, release, user, replica_id), cpu_data,
                  static_cast<DataType>(dtype), dim, cache_percentage, stream);
}

void coll_cache_init_ranked_c(int replica_id, size_t key_space_size, const uint32_t *rank_keys,
                              const uint32_t *rank_freq, coll_cache_alloc_fn alloc, coll_cache_release_fn release,
                              void *user, void *cpu_data, int dtype, size_t dim, double cache_percentage,
                              StreamHandle stream) {
  CHECK(RunConfig::is_configured);
  DataType dt = static_cast<DataType>(dtype);
  NormalizeHalf(dt, dim);
  _preloader.Join();
  _coll_cache->build_v2(replica_id, const_cast<IdType *>(rank_keys), const_cast<IdType *>(rank_freq),
                        (IdType)key_space_size, MakeAllocator(alloc, release, user, replica_id), cpu_data, dt, dim,
                        cache_percentage, stream);
}

void coll_cache_build_all_c(coll_cache_alloc_fn alloc, coll_cache_release_fn release, void *user, void *cpu_data,
                            int dtype, size_t dim, double cache_percentage, StreamHandle stream) {
  CHECK(RunConfig::is_configured);
  CHECK_NOTNULL(_coll_cache);
  DataType dt = static_cast<DataType>(dtype);
  NormalizeHalf(dt, dim);
  _preloader.Join();
  _coll_cache->build([=](int replica_id) { return MakeAllocator(alloc, release, user, replica_id); }, cpu_data, dt, dim,
                     cache_percentage, stream);
}

void coll_cache_set_key_map(uint64_t mul, int bits) {
  CHECK(RunConfig::is_configured) << "coll_cache_config comes first";
  CHECK(_coll_cache == nullptr || _coll_cache->num_replicas_built() == 0) << "the key map cannot change after the build";
  RunConfig::SetKeyMap(mul, bits);
}

void coll_cache_refresh(int replica_id, StreamHandle stream, int foreground) {
  CHECK_NOTNULL(_coll_cache);
  Timer t_rank;
  // hotness counted on the device only, and asked to stay there: rank, place and diff on the device
  if (RunConfig::gpu_refresh && RunConfig::gpu_record && (size_t)replica_id < _freq_recorder.size() &&
      _freq_recorder[replica_id] && !_freq_recorder[replica_id]->HasCounts() && _coll_cache->session(replica_id) &&
      _coll_cache->session(replica_id)->CountsOnDevice()) {
    _coll_cache->refresh_on_device(replica_id, stream, foreground != 0);
    if (_profiler) _profiler->SetRefreshDuration(t_rank.Passed());
    return;
  }
  ContFreqBuf *freq_rank = CombineAndRank(
      replica_id, coll_cache::FreqRankSolver::NumCachedNodes((IdType)RunConfig::num_total_item,
                                                             RunConfig::cache_percentage * 100));
  LOG(INFO) << "refresh: ranking " << t_rank.Passed() << " s";
  _coll_cache->refresh(replica_id, freq_rank, stream, foreground != 0);
  if (_profiler) _profiler->SetRefreshDuration(t_rank.Passed());
}

}  // extern "C"

// ---- serving loop ------------------------------------------------------------------------------------------
namespace {
/** The thread that counts the recorded prefix of a batch on the host while the lookup of the same batch runs
 *  (lookup_manager.cc:291-312 with the record thread of lookup_manager.cc:158-178: posted before the lookup, waited
 *  for after it).  The prefix crosses into pinned memory on a stream of the recorder's own, behind an event on the
 *  caller's stream, so keys that earlier work on that stream produces are complete when they are copied. */
class RecordWorker {
 public:
  // at process exit without coll_cache_shutdown: the thread ends, the stream, event and staging memory are left to
  // the runtime, which may be half gone by then
  ~RecordWorker() { Stop(/*release=*/false); }
  /// hands the first `num` keys of `key` (device memory, `key_bytes` bytes each) to the thread
  void Post(int replica_id, int device, const void *key, size_t num, int key_bytes, StreamHandle stream) {
    Start(device);
    UGK_CALL(ugk_event_record(_keys_ready, stream));
    std::lock_guard<std::mutex> g(_mu);
    _replica = replica_id, _key = key, _num = num, _key_bytes = key_bytes;
    _pending = true, _done = false;
    _cv.notify_all();
  }
  /// returns when the posted prefix has been counted
  void Wait() {
    Timer t;
    std::unique_lock<std::mutex> g(_mu);
    _cv.wait(g, [this] { return _done; });
    Sample(_waited_s, t.Passed());
  }
  void Stop(bool release = true) {
    if (!_thread.joinable()) return;
    {
      std::lock_guard<std::mutex> g(_mu);
      _exit = true;
      _cv.notify_all();
    }
    _thread.join();
    _exit = false;
    if (!_copy_s.empty())
      LOG(INFO) << "record thread: " << _copy_s.size() << " batches; median copy " << Median(_copy_s) * 1e3
                << " ms, count " << Median(_count_s) * 1e3 << " ms, waited for after the lookup "
                << Median(_waited_s) * 1e3 << " ms";
    _copy_s.clear(), _count_s.clear(), _waited_s.clear();
    if (!release) return;
    if (_staging) UGK_CALL(ugk_host_free(_staging));
    UGK_CALL(ugk_event_destroy(_keys_ready));
    UGK_CALL(ugk_stream_destroy(_stream));
    _staging = nullptr, _staging_bytes = 0, _keys_ready = nullptr, _stream = nullptr;
  }

 private:
  void Start(int device) {
    if (_thread.joinable()) return;
    UGK_CALL(ugk_stream_create(&_stream));
    UGK_CALL(ugk_event_create(&_keys_ready));
    _thread = std::thread([this, device] {
      UGK_CALL(ugk_set_device(device));
      std::unique_lock<std::mutex> g(_mu);
      for (;;) {
        _cv.wait(g, [this] { return _pending || _exit; });
        if (_exit) return;
        _pending = false;
        g.unlock();
        const size_t bytes = _num * _key_bytes;
        if (bytes > _staging_bytes) {
          if (_staging) UGK_CALL(ugk_host_free(_staging));
          _staging_bytes = std::max<size_t>(bytes, 2 * _staging_bytes);
          UGK_CALL(ugk_host_malloc(&_staging, _staging_bytes));
        }
        Timer t_copy;
        UGK_CALL(ugk_stream_wait_event(_stream, _keys_ready));
        UGK_CALL(ugk_memcpy_async(_staging, _key, bytes, _stream));
        UGK_CALL(ugk_stream_sync(_stream));
        Sample(_copy_s, t_copy.Passed());
        Timer t_count;
        if (_key_bytes == 8)
          _freq_recorder[_replica]->Record(static_cast<const Id64Type *>(_staging), _num);
        else
          _freq_recorder[_replica]->Record(static_cast<const IdType *>(_staging), _num);
        Sample(_count_s, t_count.Passed());
        g.lock();
        _done = true;
        _cv.notify_all();
      }
    });
  }
  std::thread _thread;
  std::mutex _mu;
  std::condition_variable _cv;
  bool _pending = false, _done = true, _exit = false;
  int _replica = 0, _key_bytes = 4;
  const void *_key = nullptr;
  size_t _num = 0;
  StreamHandle _stream = nullptr;
  void *_keys_ready = nullptr;
  void *_staging = nullptr;  // pinned
  // durations of the first 4096 batches, for the log line at the end
  static void Sample(std::vector<double> &v, double s) {
    if (v.size() < 4096) v.push_back(s);
  }
  static double Median(std::vector<double> &v) {
    std::nth_element(v.begin(), v.begin() + v.size() / 2, v.end());
    return v[v.size() / 2];
  }
  std::vector<double> _copy_s, _count_s, _waited_s;
  size_t _staging_bytes = 0;
};

struct ForwardState {
  bool enable_refresh = false;
  bool periodic = false;
  uint64_t refresh_iter = 0;
  double record_fraction = 0.05;
  uint64_t step = 0;
  std::thread refresh_thread;
  std::atomic<bool> refresh_ongoing{false};
  std::atomic<uint64_t> refreshes_done{0};
  RecordWorker recorder;  // the host-record path
  // A small recorded prefix does not go through the recorder's thread: a copy kernel in front of the lookup, on the
  // lookup's stream, leaves it in this pinned buffer, and the step counts it itself once the blocking lookup has
  // returned.  Waking the thread and waiting for it cost a serving-sized batch more than its whole lookup
  // (1,024 keys: 55 us per step against 12 us for the lookup alone).
  void *inline_prefix = nullptr;
  size_t inline_prefix_bytes = 0;
  // A step that is enqueued and left cannot count its prefix when it returns: the copy kernel has not run yet.  Its
  // prefix waits in one of a few pinned buffers, behind an event, until a later step (or whoever needs the counts: a
  // ranking, coll_cache_lookup_wait, the shutdown) finds the event complete, or waits for it, and counts it.
  struct PendingPrefix {
    void *staging = nullptr;
    void *copied = nullptr;  // event behind the copy kernel
    size_t bytes = 0, num = 0;
    int replica = 0, key_bytes = 4;
  };
  static constexpr size_t kPendingSlots = 8;
  PendingPrefix pending[kPendingSlots];
  size_t pending_head = 0, pending_tail = 0;  // [tail, head) wait to be counted
  std::mutex pending_mu;                      // the steps' thread and a refresh thread that ranks
  ~ForwardState() {
    if (refresh_thread.joinable()) refresh_thread.join();  // a process that exits without coll_cache_shutdown
  }
};
ForwardState _forward;

void ForwardJoin() {
  if (_forward.refresh_thread.joinable()) _forward.refresh_thread.join();
}

// caller holds pending_mu
void CountPendingLocked(bool all) {
  ForwardState &fw = _forward;
  while (fw.pending_tail != fw.pending_head) {
    ForwardState::PendingPrefix &p = fw.pending[fw.pending_tail % ForwardState::kPendingSlots];
    if (all) {
      UGK_CALL(ugk_event_sync(p.copied));
    } else {
      int complete = 0;
      UGK_CALL(ugk_event_query(p.copied, &complete));
      if (!complete) break;
    }
    if ((size_t)p.replica < _freq_recorder.size() && _freq_recorder[p.replica]) {
      if (p.key_bytes == 8)
        _freq_recorder[p.replica]->Record(static_cast<const Id64Type *>(p.staging), p.num);
      else
        _freq_recorder[p.replica]->Record(static_cast<const IdType *>(p.staging), p.num);
    }
    fw.pending_tail++;
  }
}

void CountPendingPrefixes(bool all) {
  std::lock_guard<std::mutex> g(_forward.pending_mu);
  CountPendingLocked(all);
}

// the prefix of a stream-ordered step: a copy kernel on the caller's stream into the next pinned buffer, an event behind
// it; counted later (CountPendingPrefixes)
void PostPendingPrefix(int replica_id, const void *key, size_t num, int key_bytes, StreamHandle stream) {
  ForwardState &fw = _forward;
  std::lock_guard<std::mutex> g(fw.pending_mu);
  CountPendingLocked(/*all=*/false);
  if (fw.pending_head - fw.pending_tail == ForwardState::kPendingSlots) {  // every buffer waits: take the oldest
    ForwardState::PendingPrefix &oldest = fw.pending[fw.pending_tail % ForwardState::kPendingSlots];
    UGK_CALL(ugk_event_sync(oldest.copied));
    CountPendingLocked(/*all=*/false);
  }
  ForwardState::PendingPrefix &p = fw.pending[fw.pending_head % ForwardState::kPendingSlots];
  const size_t bytes = num * key_bytes;
  if (p.bytes < bytes) {
    if (p.staging) UGK_CALL(ugk_host_free(p.staging));
    p.bytes = std::max(bytes, RunConfig::record_inline_bytes);
    UGK_CALL(ugk_host_malloc(&p.staging, p.bytes));
  }
  if (p.copied == nullptr) UGK_CALL(ugk_event_create(&p.copied));
  p.replica = replica_id, p.num = num, p.key_bytes = key_bytes;
  UGK_CALL(ugk_copy_rows(p.staging, key, bytes, stream));
  UGK_CALL(ugk_event_record(p.copied, stream));
  fw.pending_head++;
}

void ReleasePendingPrefixes() {
  ForwardState &fw = _forward;
  std::lock_guard<std::mutex> g(fw.pending_mu);
  CountPendingLocked(/*all=*/true);
  for (auto &p : fw.pending) {
    if (p.staging) UGK_CALL(ugk_host_free(p.staging));
    if (p.copied) UGK_CALL(ugk_event_destroy(p.copied));
    p = ForwardState::PendingPrefix();
  }
  fw.pending_head = fw.pending_tail = 0;
}

// lookup(step_key, ordered): the extraction of the step — the plain lookup, or the pooled one; blocking, or
// (ordered) enqueued on the caller's stream and left.  A step whose recorded prefix this thread or the record thread
// counts blocks whatever the caller asked for: the record thread copies the prefix out of the caller's buffer while
// the step knows it to be alive.
template <typename KeyT, typename LookupFn>
void ForwardStep(int replica_id, const KeyT *key, size_t num_keys, StreamHandle stream, bool stream_ordered,
                 const LookupFn &lookup) {
  CHECK_NOTNULL(_coll_cache);
  CHECK_EQ(replica_id, 0);
  ForwardState &fw = _forward;
  auto session = _coll_cache->session(replica_id);
  const size_t num_record = fw.enable_refresh ? (size_t)(num_keys * fw.record_fraction) : 0;
  const size_t record_bytes = num_record * sizeof(KeyT);
  // who counts the prefix
  enum class Prefix {
    kNone,      // nothing to record
    kDevice,    // the lookup itself, into the device-side counters
    kThread,    // the record thread, from a copy it makes beside the lookup; the step waits for it
    kInline,    // this thread after the blocking lookup, from a copy a kernel in front of the lookup makes
    kDeferred,  // a later step (or the wait, or the ranking), from such a copy: the step is enqueued and left
  } prefix = Prefix::kNone;
  // A step that the caller is recording into a HIP graph is not a step of the loop: it runs when the caller replays
  // it.  Its prefix is counted where the device counts (the counting is part of the recorded lookup); the host cannot
  // count what a replay copies.  It starts no refresh either: the refresh thread would wait for a stream that records.
  int capturing = 0;
  if (stream_ordered) UGK_CALL(ugk_stream_is_capturing(stream, &capturing));
  if (num_record > 0) {
    const bool small = record_bytes <= RunConfig::record_inline_bytes && reinterpret_cast<uintptr_t>(key) % 16 == 0;
    if (RunConfig::gpu_record) {
      prefix = Prefix::kDevice;
    } else if (capturing) {
      prefix = Prefix::kNone;
    } else if (small && stream_ordered) {
      prefix = Prefix::kDeferred;
    } else {
      prefix = small ? Prefix::kInline : Prefix::kThread;
    }
  }
  switch (prefix) {
    case Prefix::kDevice: session->SetRecordLimit(num_record); break;
    case Prefix::kDeferred: PostPendingPrefix(replica_id, key, num_record, (int)sizeof(KeyT), stream); break;
    case Prefix::kInline:
      if (fw.inline_prefix_bytes < RunConfig::record_inline_bytes) {
        if (fw.inline_prefix) UGK_CALL(ugk_host_free(fw.inline_prefix));
        UGK_CALL(ugk_host_malloc(&fw.inline_prefix, RunConfig::record_inline_bytes));
        fw.inline_prefix_bytes = RunConfig::record_inline_bytes;
      }
      UGK_CALL(ugk_copy_rows(fw.inline_prefix, key, record_bytes, stream));  // complete when the lookup behind it is
      break;
    case Prefix::kThread:
      fw.recorder.Post(replica_id, session->DeviceId(), key, num_record, sizeof(KeyT), stream);
      break;
    case Prefix::kNone: break;
  }
  const uint64_t step_key = steps[replica_id] * RunConfig::num_device + replica_id;
  steps[replica_id]++;
  // the host's own counting (kInline, kThread) needs the lookup to have returned
  lookup(step_key, stream_ordered && prefix != Prefix::kInline && prefix != Prefix::kThread);
  switch (prefix) {
    case Prefix::kDevice: session->SetRecordLimit(SIZE_MAX); break;
    case Prefix::kInline:
      _freq_recorder[replica_id]->Record(static_cast<const KeyT *>(fw.inline_prefix), num_record);
      break;
    case Prefix::kThread: fw.recorder.Wait(); break;
    case Prefix::kDeferred:
    case Prefix::kNone: break;
  }
  if (capturing) return;
  const bool due = fw.enable_refresh && fw.refresh_iter > 0 &&
                   (fw.periodic ? (fw.step > 0 && fw.step % fw.refresh_iter == 0) : fw.step == fw.refresh_iter);
  if (due) {
    if (!fw.refresh_ongoing.load()) {
      fw.refresh_ongoing.store(true);
      ForwardJoin();
      CountPendingPrefixes(/*all=*/true);  // the refresh ranks what every step up to this one recorded
      fw.refresh_thread = std::thread([replica_id, stream]() {
        coll_cache_refresh(replica_id, stream, /*foreground=*/0);
        _forward.refreshes_done.fetch_add(1);
        _forward.refresh_ongoing.store(false);
      });
    } else {
      LOG(ERROR) << "skip refresh due to refresh already ongoing";
    }
  }
  fw.step++;
}
}  // namespace

extern "C" {

void coll_cache_forward_config(int enable_refresh, uint64_t refresh_iter, double record_fraction, int periodic) {
  CHECK(record_fraction >= 0 && record_fraction <= 1) << "record_fraction is a share of the batch";
  ForwardJoin();
  _forward.enable_refresh = enable_refresh != 0;
  _forward.refresh_iter = refresh_iter;
  _forward.record_fraction = record_fraction;
  _forward.periodic = periodic != 0;
  _forward.step = 0;
}

void coll_cache_forward(int replica_id, uint32_t *key, size_t num_keys, void *output, StreamHandle stream) {
  ForwardStep<IdType>(replica_id, key, num_keys, stream, false, [&](uint64_t step_key, bool) {
    _coll_cache->lookup(replica_id, key, num_keys, output, stream, step_key);
  });
}

void coll_cache_forward_i64(int replica_id, const int64_t *key, size_t num_keys, void *output, StreamHandle stream) {
  ForwardStep<Id64Type>(replica_id, key, num_keys, stream, false, [&](uint64_t step_key, bool) {
    _coll_cache->lookup64(replica_id, key, num_keys, output, stream, step_key);
  });
}

void coll_cache_forward_async(int replica_id, const uint32_t *key, size_t num_keys, void *output,
                              StreamHandle stream) {
  ForwardStep<IdType>(replica_id, key, num_keys, stream, true, [&](uint64_t step_key, bool ordered) {
    if (ordered)
      _coll_cache->lookup_async(replica_id, key, num_keys, output, stream);
    else
      _coll_cache->lookup(replica_id, key, num_keys, output, stream, step_key);
  });
}

void coll_cache_forward_async_i64(int replica_id, const int64_t *key, size_t num_keys, void *output,
                                  StreamHandle stream) {
  ForwardStep<Id64Type>(replica_id, key, num_keys, stream, true, [&](uint64_t step_key, bool ordered) {
    if (ordered)
      _coll_cache->lookup_async64(replica_id, key, num_keys, output, stream);
    else
      _coll_cache->lookup64(replica_id, key, num_keys, output, stream, step_key);
  });
}

void coll_cache_forward_pooled(int replica_id, const uint32_t *key, const int64_t *seg_off, const float *weights,
                               size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                               StreamHandle stream) {
  ForwardStep<IdType>(replica_id, key, num_keys, stream, false, [&](uint64_t step_key, bool) {
    _coll_cache->lookup_pooled(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes, output,
                               stream, step_key);
  });
}

void coll_cache_forward_pooled_i64(int replica_id, const int64_t *key, const int64_t *seg_off, const float *weights,
                                   size_t num_rows, size_t num_keys, int combiner, int elem_bytes, void *output,
                                   StreamHandle stream) {
  ForwardStep<Id64Type>(replica_id, key, num_keys, stream, false, [&](uint64_t step_key, bool) {
    _coll_cache->lookup_pooled64(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes, output,
                                 stream, step_key);
  });
}

void coll_cache_forward_pooled_async(int replica_id, const uint32_t *key, const int64_t *seg_off,
                                     const float *weights, size_t num_rows, size_t num_keys, int combiner,
                                     int elem_bytes, void *output, StreamHandle stream) {
  ForwardStep<IdType>(replica_id, key, num_keys, stream, true, [&](uint64_t step_key, bool ordered) {
    if (ordered)
      _coll_cache->lookup_pooled_async(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes,
                                       output, stream);
    else
      _coll_cache->lookup_pooled(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes, output,
                                 stream, step_key);
  });
}

void coll_cache_forward_pooled_async_i64(int replica_id, const int64_t *key, const int64_t *seg_off,
                                         const float *weights, size_t num_rows, size_t num_keys, int combiner,
                                         int elem_bytes, void *output, StreamHandle stream) {
  ForwardStep<Id64Type>(replica_id, key, num_keys, stream, true, [&](uint64_t step_key, bool ordered) {
    if (ordered)
      _coll_cache->lookup_pooled_async64(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes,
                                         output, stream);
    else
      _coll_cache->lookup_pooled64(replica_id, key, seg_off, weights, num_rows, num_keys, combiner, elem_bytes,
                                   output, stream, step_key);
  });
}

int coll_cache_forward_refresh_ongoing(void) { return _forward.refresh_ongoing.load() ? 1 : 0; }

uint64_t coll_cache_forward_join(void) {
  ForwardJoin();
  return _forward.refreshes_done.load();
}

void *coll_cache_alloc_host_table(size_t nbytes) {
  void *p = nullptr;
  UGK_CALL(ugk_host_malloc(&p, nbytes));
  return p;
}

void coll_cache_free_host_table(void *ptr) { UGK_CALL(ugk_host_free(ptr)); }

size_t coll_cache_max_num_keys(void) { return max_num_keys; }
void coll_cache_set_max_num_keys(size_t n) { max_num_keys = n; }

void coll_cache_last_group_offset(int replica_id, uint32_t out[3]) {
  CHECK_NOTNULL(_coll_cache);
  const uint32_t *g = _coll_cache->session(replica_id)->LastGroupOffset();
  out[0] = g[0];
  out[1] = g[1];
  out[2] = g[2];
}

void coll_cache_get_info(int replica_id, uint64_t out[8]) {
  CHECK_NOTNULL(_coll_cache);
  auto ctx = _coll_cache->cache_ctx(replica_id);
  memset(out, 0, 8 * sizeof(uint64_t));
  out[0] = ctx->CacheCapacityRows();
  out[1] = ctx->CachedRows();
  out[2] = (uint64_t)ctx->TableKind();
  out[3] = ctx->RowBytes();
  out[4] = RunConfig::num_total_item;
  out[5] = ctx->progress.load();
  out[6] = ctx->EntryManager() ? ctx->EntryManager()->NumFree() : 0;
  out[7] = ctx->EntryManager() ? ctx->EntryManager()->_num_rebuilds : 0;
}

uint64_t coll_cache_rows_from_stage(int replica_id) {
  CHECK_NOTNULL(_coll_cache);
  return _coll_cache->rows_from_stage(replica_id);
}

size_t coll_cache_get_cached_keys(int replica_id, uint32_t *out, size_t capacity) {
  CHECK_NOTNULL(_coll_cache);
  _coll_cache->cache_ctx(replica_id)->SyncHostLists();
  auto mgr = _coll_cache->cache_ctx(replica_id)->EntryManager();
  if (!mgr || !mgr->_cached_keys) return 0;  // (SyncHostLists has fetched a list the build left on the device)
  const size_t n = mgr->_cached_keys->NumItem();
  if (out) memcpy(out, mgr->_cached_keys->Data(), std::min(n, capacity) * sizeof(uint32_t));
  return n;
}

double coll_cache_get_step_value(uint64_t key, int item) {
  CHECK_NOTNULL(_profiler);
  CHECK(item >= 0 && item < (int)kNumLogStepItems);
  return _profiler->GetStep(key, static_cast<LogStepItem>(item));
}

size_t coll_cache_rank_hotness(int replica_id, uint32_t *keys_out, uint32_t *cnts_out, size_t capacity) {
  CHECK(RunConfig::is_configured);
  ContFreqBuf *rank = CombineAndRank(replica_id);
  CHECK_NOTNULL(rank);
  const size_t n = rank->size();
  for (size_t i = 0; i < std::min(n, capacity); i++) {
    if (keys_out) keys_out[i] = rank->buf[i].key;
    if (cnts_out) cnts_out[i] = rank->buf[i].cnt;
  }
  return n;
}

uint32_t coll_cache_place_ranked(const uint32_t *rank_keys, const uint32_t *rank_freq, uint32_t num_node,
                                 double cache_percentage, uint32_t *nid_to_block_out) {
  CHECK_NOTNULL(rank_keys);
  CHECK_NOTNULL(rank_freq);
  CHECK_NOTNULL(nid_to_block_out);
  coll_cache::FreqRankSolver solver;
  auto keys = Tensor::FromBlob(const_cast<uint32_t *>(rank_keys), kI32, {1, (size_t)num_node}, CPU(CPU_FOREIGN), "");
  auto freq = Tensor::FromBlob(const_cast<uint32_t *>(rank_freq), kI32, {1, (size_t)num_node}, CPU(CPU_FOREIGN), "");
  auto n2b = Tensor::FromBlob(nid_to_block_out, kI32, {(size_t)num_node}, CPU(CPU_FOREIGN), "");
  solver.Build(keys, freq, {0}, num_node, n2b);
  solver.Solve({0}, {cache_percentage * 100}, "BIN", RunConfig::coll_cache_hyperparam_T_local,
               RunConfig::coll_cache_hyperparam_T_cpu);
  uint32_t cached = 0;
  for (uint32_t k = 0; k < num_node; k++) cached += nid_to_block_out[k] == 0;
  return cached;
}

uint32_t coll_cache_place_recorded(int replica_id, uint32_t num_node, double cache_percentage,
                                   uint32_t *nid_to_block_out) {
  CHECK(RunConfig::is_configured);
  CHECK_NOTNULL(nid_to_block_out);
  CHECK_EQ((size_t)num_node, RunConfig::num_total_item);
  ContFreqBuf *rank = CombineAndRank(replica_id);
  CHECK_NOTNULL(rank);
  coll_cache::FreqRankSolver solver;
  auto n2b = Tensor::FromBlob(nid_to_block_out, kI32, {(size_t)num_node}, CPU(CPU_FOREIGN), "");
  solver.BuildSingleStream(rank, {0}, num_node, n2b);
  solver.Solve({0}, {cache_percentage * 100}, "BIN", RunConfig::coll_cache_hyperparam_T_local,
               RunConfig::coll_cache_hyperparam_T_cpu);
  uint32_t cached = 0;
  for (uint32_t k = 0; k < num_node; k++) cached += nid_to_block_out[k] == 0;
  return cached;
}

void coll_cache_shutdown(void) {
  _preloader.Join();
  ForwardJoin();
  _forward.recorder.Stop();
  ReleasePendingPrefixes();
  if (_forward.inline_prefix) {
    UGK_CALL(ugk_host_free(_forward.inline_prefix));
    _forward.inline_prefix = nullptr;
    _forward.inline_prefix_bytes = 0;
  }
  _forward.enable_refresh = false;
  _forward.step = 0;
  _forward.refreshes_done.store(0);
  if (_coll_cache && _coll_cache->num_replicas_built() > 0) {
    // stream-ordered lookups may still be in flight; their buffers and streams go away below
    UGK_CALL(ugk_device_sync());
    _coll_cache->release_replicas();
  }
  _coll_cache = nullptr;
  _profiler = nullptr;
  _freq_recorder.clear();
  memset(steps, 0, sizeof(steps));
  max_num_keys = 0;
  RunConfig::is_configured = false;
  RunConfig::SetKeyMap(0, 0);
}

}  // extern "C"

}  // namespace common
}  // namespace coll_cache_lib
