#include "facade.h"

#include <iostream>

#include "logging.h"
#include "placement.h"
#include "run_config.h"
#include "timer.h"

namespace coll_cache_lib {

// facade.cc:74-88
void CollCache::lookup(int replica_id, const IdType *nodes, const size_t num_nodes, void *output,
                       StreamHandle stream, uint64_t step_key) {
  Timer t;
  CHECK_LT((size_t)replica_id, _session_list.size());
  _session_list[replica_id]->ExtractFeat(nodes, num_nodes, output, stream, step_key);
  _profiler->LogStep(step_key, common::kLogL2CacheCopyTime, t.Passed());
}

void CollCache::lookup64(int replica_id, const Id64Type *nodes, const size_t num_nodes, void *output,
                         StreamHandle stream, uint64_t step_key) {
  Timer t;
  CHECK_LT((size_t)replica_id, _session_list.size());
  _session_list[replica_id]->ExtractFeat64(nodes, num_nodes, output, stream, step_key);
  _profiler->LogStep(step_key, common::kLogL2CacheCopyTime, t.Passed());
}

void CollCache::lookup_pooled(int replica_id, const IdType *nodes, const int64_t *seg_off, const float *weights,
                              size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                              StreamHandle stream, uint64_t step_key) {
  Timer t;
  CHECK_LT((size_t)replica_id, _session_list.size());
  _session_list[replica_id]->ExtractPooled(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes, output,
                                           stream, step_key);
  _profiler->LogStep(step_key, common::kLogL2CacheCopyTime, t.Passed());
}

void CollCache::lookup_pooled64(int replica_id, const Id64Type *nodes, const int64_t *seg_off, const float *weights,
                                size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                                StreamHandle stream, uint64_t step_key) {
  Timer t;
  CHECK_LT((size_t)replica_id, _session_list.size());
  _session_list[replica_id]->ExtractPooled64(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes,
                                             output, stream, step_key);
  _profiler->LogStep(step_key, common::kLogL2CacheCopyTime, t.Passed());
}

size_t CollCache::lookup_unique(int replica_id, const IdType *nodes, size_t num_nodes, void *output,
                                uint32_t *inverse_out, StreamHandle stream, uint64_t step_key) {
  Timer t;
  CHECK_LT((size_t)replica_id, _session_list.size());
  const size_t nu = _session_list[replica_id]->ExtractUnique(nodes, num_nodes, output, inverse_out, stream, step_key);
  _profiler->LogStep(step_key, common::kLogL2CacheCopyTime, t.Passed());
  return nu;
}

size_t CollCache::lookup_unique64(int replica_id, const Id64Type *nodes, size_t num_nodes, void *output,
                                  uint32_t *inverse_out, StreamHandle stream, uint64_t step_key) {
  Timer t;
  CHECK_LT((size_t)replica_id, _session_list.size());
  const size_t nu =
      _session_list[replica_id]->ExtractUnique64(nodes, num_nodes, output, inverse_out, stream, step_key);
  _profiler->LogStep(step_key, common::kLogL2CacheCopyTime, t.Passed());
  return nu;
}

namespace {
// every policy of the reference that runs a solver (facade.cc:110-152) reduces to the frequency-ranked
// placement when there is one GPU
void CheckPolicy() {
  switch (RunConfig::cache_policy) {
    case kRepCache:
    case kPartRepCache:
    case kPartitionCache:
    case kCollCacheIntuitive:
    case kCollCache:
    case kCollCacheAsymmLink:
    case kCollFineGrain:
    case kCliquePart:
      return;
    default:
      LOG(FATAL) << "cache policy " << (int)RunConfig::cache_policy << " has no solver";
  }
}
}  // namespace

void CollCache::take_solution(coll_cache::FreqRankSolver &solver, IdType num_node) {
  _block_placement = solver.block_placement;
  _block_access_advise = solver.block_access_from;
  _block_density = solver.block_density_tensor;
  _placed_top_rows = solver.defer_nid_to_block ? solver.top_rows : nullptr;
  _placed_extra = solver.defer_nid_to_block ? solver.num_extra : 0;
  _placed_num_node = num_node;
}

TensorPtr CollCache::EnsureNidToBlock() {
  if (_nid_to_block == nullptr && _placed_top_rows != nullptr) {
    _nid_to_block = Tensor::Empty(kI32, {(size_t)_placed_num_node}, CPU_CLIB(), "nid_to_block");
    coll_cache::FreqRankSolver::Materialize(_placed_top_rows->CPtr<IdType>(), _placed_top_rows->NumItem(),
                                            _placed_extra, _placed_num_node, _nid_to_block->Ptr<IdType>());
    _placed_top_rows = nullptr;
  }
  return _nid_to_block;
}

// facade.cc:93-160
void CollCache::solve_impl_master(IdType *ranking_nodes_list_ptr, IdType *ranking_nodes_freq_list_ptr,
                                  IdType num_node, bool defer) {
  CheckPolicy();
  std::vector<int> trainer_to_stream(RunConfig::num_device, 0);
  std::vector<coll_cache::PerT> trainer_cache_percent(RunConfig::num_device, RunConfig::cache_percentage * 100);
  auto ranking_nodes_list =
      Tensor::FromBlob(ranking_nodes_list_ptr, kI32, {1, (size_t)num_node}, CPU(CPU_FOREIGN), "ranking_nodes_list");
  auto ranking_nodes_freq_list = Tensor::FromBlob(ranking_nodes_freq_list_ptr, kI32, {1, (size_t)num_node},
                                                  CPU(CPU_FOREIGN), "ranking_nodes_freq_list");
  coll_cache::FreqRankSolver solver;
  solver.defer_nid_to_block = defer;
  _nid_to_block = defer ? nullptr : Tensor::Empty(kI32, {(size_t)num_node}, CPU_CLIB(), "nid_to_block");
  solver.Build(ranking_nodes_list, ranking_nodes_freq_list, trainer_to_stream, num_node, _nid_to_block);
  solver.Solve(trainer_to_stream, trainer_cache_percent, "BIN", RunConfig::coll_cache_hyperparam_T_local,
               RunConfig::coll_cache_hyperparam_T_cpu);
  take_solution(solver, num_node);
}

// facade.cc:161-236
void CollCache::solve_impl_master(ContFreqBuf *freq_rank, IdType num_node, bool defer) {
  CheckPolicy();
  std::vector<int> trainer_to_stream(RunConfig::num_device, 0);
  std::vector<coll_cache::PerT> trainer_cache_percent(RunConfig::num_device, RunConfig::cache_percentage * 100);
  coll_cache::FreqRankSolver solver;
  solver.defer_nid_to_block = defer;
  _nid_to_block = defer ? nullptr : Tensor::Empty(kI32, {(size_t)num_node}, CPU_CLIB(), "nid_to_block");
  solver.BuildSingleStream(freq_rank, trainer_to_stream, num_node, _nid_to_block);
  solver.Solve(trainer_to_stream, trainer_cache_percent, "BIN", RunConfig::coll_cache_hyperparam_T_local,
               RunConfig::coll_cache_hyperparam_T_cpu);
  take_solution(solver, num_node);
}

void CollCache::build_common(int replica_id, std::function<void()> solve, IdType num_node,
                             std::function<MemHandle(size_t)> gpu_mem_allocator, void *cpu_data, DataType dtype,
                             size_t dim, double cache_percentage, StreamHandle stream) {
  CHECK_EQ(replica_id, 0) << "this build serves one replica on one GPU";
  CHECK_EQ(RunConfig::num_device, (size_t)1) << "num_device must be 1";
  if (RunConfig::device_id_list.empty()) RunConfig::device_id_list = {0};
  const int device_id = RunConfig::device_id_list[replica_id];
  RunConfig::LoadConfigFromEnv();
  RunConfig::num_total_item = num_node;
  RunConfig::cache_percentage = cache_percentage;
  // rows are handled as opaque bytes; keep the reference's re-expression in 16-byte units for its logs
  // (facade.cc:457-465)
  if (RunConfig::coll_cache_scale_nb != 0) {
    const size_t emb_vec_nb = GetDataTypeBytes(dtype) * dim;
    if (emb_vec_nb >= RunConfig::coll_cache_scale_nb && emb_vec_nb % RunConfig::coll_cache_scale_nb == 0) {
      dim = emb_vec_nb / RunConfig::coll_cache_scale_nb;
      dtype = nb_to_dt(RunConfig::coll_cache_scale_nb);
    }
  }
  RunConfig::coll_cache_link_desc = coll_cache::AsymmLinkDesc::AutoBuild(GPU(device_id));
  this->_cache_ctx_list.resize(RunConfig::num_device);
  this->_session_list.resize(RunConfig::num_device);
  this->_refresh_session_list.resize(RunConfig::num_device);
  RunConfig::solver_omp_thread_num = RunConfig::omp_thread_num;
  RunConfig::solver_omp_thread_num_per_gpu = std::max<int>(1, RunConfig::omp_thread_num / (int)RunConfig::num_device);

  const bool need_solver = (cache_percentage != 0 && cache_percentage != 1);
  Timer t_solve;
  if (need_solver) solve();
  LOG(INFO) << "build: placement " << t_solve.Passed() << " s";
  this->_replica_barrier->Wait();

  auto cache_ctx = std::make_shared<CacheContext>(_replica_barrier);
  Context gpu_ctx = GPU(device_id);
  cache_ctx->build(gpu_mem_allocator, replica_id, this->shared_from_this(), cpu_data, dtype, dim, gpu_ctx,
                   cache_percentage, stream);
  UGK_CALL(ugk_stream_sync(stream));
  this->_cache_ctx_list[replica_id] = cache_ctx;
  this->_session_list[replica_id] = std::make_shared<ExtractSession>(cache_ctx);
  this->_refresh_session_list[replica_id] = std::make_shared<RefreshSession>();
  this->_refresh_session_list[replica_id]->_cache_ctx = cache_ctx;
  this->_refresh_session_list[replica_id]->stream = stream;
  this->_replica_barrier->Wait();
  // after the build the host scans belong to the refresher.  The reference's defaults (8 threads, 1 per GPU of an
  // 8-GPU node: run_config.cc:53-54) give the one GPU here all of them.
  RunConfig::solver_omp_thread_num = RunConfig::refresher_omp_thread_num;
  RunConfig::solver_omp_thread_num_per_gpu =
      std::max<int>(RunConfig::refresher_omp_thread_num_per_gpu,
                    RunConfig::refresher_omp_thread_num / (int)RunConfig::num_device);
}

// facade.cc:38-72
void CollCache::build(std::function<std::function<MemHandle(size_t)>(int)> allocator_builder, void *cpu_data,
                      DataType dtype, size_t dim, double cache_percentage, StreamHandle stream) {
  const bool partial = cache_percentage != 0 && cache_percentage != 1;
  CHECK(!partial || (HasPartialPlacement() && _block_access_advise != nullptr))
      << "CollCache::build places nothing itself: a partial cache needs the placement of an earlier build_v2 / refresh";
  if (partial) EnsureNidToBlock();
  const IdType num_node = partial ? (IdType)_nid_to_block->Shape()[0] : (IdType)RunConfig::num_total_item;
  for (size_t replica_id = 0; replica_id < RunConfig::num_device; replica_id++)
    build_common((int)replica_id, []() {}, num_node, allocator_builder((int)replica_id), cpu_data, dtype, dim,
                 cache_percentage, stream);
}

// facade.cc:283-381
void CollCache::build_v2(int replica_id, IdType *ranking_nodes_list_ptr, IdType *ranking_nodes_freq_list_ptr,
                         IdType num_node, std::function<MemHandle(size_t)> gpu_mem_allocator, void *cpu_data,
                         DataType dtype, size_t dim, double cache_percentage, StreamHandle stream) {
  build_common(
      replica_id,
      [&]() { solve_impl_master(ranking_nodes_list_ptr, ranking_nodes_freq_list_ptr, num_node, RunConfig::device_key_list); },
      num_node,
      gpu_mem_allocator, cpu_data, dtype, dim, cache_percentage, stream);
}

// facade.cc:430-511
void CollCache::build_v2(int replica_id, ContFreqBuf *freq_rank, IdType num_node,
                         std::function<MemHandle(size_t)> gpu_mem_allocator, void *cpu_data, DataType dtype,
                         size_t dim, double cache_percentage, StreamHandle stream) {
  build_common(
      replica_id, [&]() { solve_impl_master(freq_rank, num_node, RunConfig::device_key_list); }, num_node,
      gpu_mem_allocator, cpu_data, dtype, dim, cache_percentage, stream);
}

void CollCache::preserve_old_solution() {
  this->_old_block_access_advise = this->_block_access_advise;
  this->_old_block_density = this->_block_density;
  this->_old_block_placement = this->_block_placement;
  this->_old_nid_to_block = this->_nid_to_block;
  this->_block_access_advise = nullptr;
  this->_block_density = nullptr;
  this->_block_placement = nullptr;
  this->_nid_to_block = nullptr;
  this->_placed_top_rows = nullptr;
}

// facade.cc:383-428
void CollCache::refresh(int replica_id, IdType *ranking_nodes_list_ptr, IdType *ranking_nodes_freq_list_ptr,
                        StreamHandle stream, bool foreground) {
  CHECK_EQ(replica_id, 0);
  CHECK(HasPartialPlacement()) << "refresh needs a cache built with 0 < cache_percentage < 1";
  AnonymousBarrier::_refresh_instance->Wait();
  preserve_old_solution();
  solve_impl_master(ranking_nodes_list_ptr, ranking_nodes_freq_list_ptr, (IdType)RunConfig::num_total_item,
                    RunConfig::device_key_list);
  AnonymousBarrier::_refresh_instance->Wait();
  apply_solution(replica_id, stream, foreground);
  AnonymousBarrier::_refresh_instance->Wait();
}

// The new placement replaces the old one in the cache.  By default (COLL_DEVICE_KEY_LIST) the solver has left the
// key -> block array unwritten and the placement goes to the device as the rows it was computed from.
void CollCache::apply_solution(int replica_id, StreamHandle stream, bool foreground) {
  auto &refresher = this->_refresh_session_list[replica_id];
  refresher->stream = stream;
  if (_placed_top_rows != nullptr)
    refresher->refresh_from_ranked_rows(_session_list[replica_id].get(), _placed_top_rows, _placed_extra, foreground);
  else
    refresher->refresh_after_solve_main(foreground);
}

// facade.cc:513-557
void CollCache::refresh(int replica_id, ContFreqBuf *freq_rank, StreamHandle stream, bool foreground) {
  CHECK_EQ(replica_id, 0);
  CHECK(HasPartialPlacement()) << "refresh needs a cache built with 0 < cache_percentage < 1";
  AnonymousBarrier::_refresh_instance->Wait();
  Timer t_solve;
  preserve_old_solution();
  solve_impl_master(freq_rank, (IdType)RunConfig::num_total_item, RunConfig::device_key_list);
  const double solve_s = t_solve.Passed();
  AnonymousBarrier::_refresh_instance->Wait();
  Timer t_apply;
  apply_solution(replica_id, stream, foreground);
  AnonymousBarrier::_refresh_instance->Wait();
  LOG(INFO) << "refresh: placement " << solve_s << " s, evict + insert " << t_apply.Passed() << " s";
}

void CollCache::refresh_on_device(int replica_id, StreamHandle stream, bool foreground) {
  CHECK_EQ(replica_id, 0);
  CHECK(HasPartialPlacement()) << "refresh needs a cache built with 0 < cache_percentage < 1";
  CheckPolicy();
  AnonymousBarrier::_refresh_instance->Wait();
  Timer t_apply;
  const size_t num_cached = coll_cache::FreqRankSolver::NumCachedNodes((IdType)RunConfig::num_total_item,
                                                                       RunConfig::cache_percentage * 100);
  this->_refresh_session_list[replica_id]->stream = stream;
  this->_refresh_session_list[replica_id]->refresh_on_device(_session_list[replica_id].get(), num_cached, foreground);
  AnonymousBarrier::_refresh_instance->Wait();
  LOG(INFO) << "refresh on the device: " << t_apply.Passed() << " s";
}

void CollCache::report_last_epoch(uint64_t epoch) { _profiler->ReportStepAverageLastEpoch(epoch + 1, 0); }

void CollCache::report_avg() {
  _profiler->ReportStepAverage(RunConfig::num_epoch - 1, RunConfig::num_global_step_per_epoch - 1);
  std::cout.flush();
}

void CollCache::report(uint64_t key) {
  _profiler->ReportStep(RunConfig::GetEpochFromKey(key), RunConfig::GetStepFromKey(key));
  std::cout.flush();
}

}  // namespace coll_cache_lib
