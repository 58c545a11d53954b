// The process-wide cache manager: same class, methods and argument meaning as coll_cache_lib/facade.h:17-82 of
// the reference.  One CollCache per process, one replica per GPU (this build: one replica).
#pragma once

#include <functional>
#include <memory>
#include <vector>

#include "cache_context.h"
#include "common.h"
#include "freq_recorder.h"
#include "placement.h"
#include "profiler.h"

namespace coll_cache_lib {

using namespace common;

class CollCache : public std::enable_shared_from_this<CollCache> {
 private:
  TensorPtr _nid_to_block;
  TensorPtr _block_density;
  TensorPtr _block_placement;
  TensorPtr _block_access_advise;
  TensorPtr _old_nid_to_block;
  TensorPtr _old_block_density;
  TensorPtr _old_block_placement;
  TensorPtr _old_block_access_advise;
  BarHandle _process_barrier;
  BarHandle _replica_barrier;
  friend class CacheContext;
  friend class RefreshSession;
  friend class ExtractSession;
  std::vector<std::shared_ptr<CacheContext>> _cache_ctx_list;
  std::vector<std::shared_ptr<ExtractSession>> _session_list;
  std::vector<std::shared_ptr<RefreshSession>> _refresh_session_list;
  // defer: the key -> block array is left unwritten and the placement kept as _placed_top_rows / _placed_extra
  // (FreqRankSolver::defer_nid_to_block): the build that follows makes its key list on the device from them
  void solve_impl_master(IdType *ranking_nodes_list_ptr, IdType *ranking_nodes_freq_list_ptr, IdType num_node,
                         bool defer = false);
  void solve_impl_master(ContFreqBuf *freq_rank, IdType num_node, bool defer = false);
  void take_solution(coll_cache::FreqRankSolver &solver, IdType num_node);
  TensorPtr _placed_top_rows;  // set while _nid_to_block is deferred
  size_t _placed_extra = 0;
  IdType _placed_num_node = 0;
  // the key -> block array of the placement in force, written out on first use when the solver deferred it
  TensorPtr EnsureNidToBlock();
  bool HasPartialPlacement() const { return _nid_to_block != nullptr || _placed_top_rows != nullptr; }
  void preserve_old_solution();
  void apply_solution(int replica_id, StreamHandle stream, bool foreground);
  void build_common(int replica_id, std::function<void()> solve, IdType num_node,
                    std::function<MemHandle(size_t)> gpu_mem_allocator, void *cpu_data, DataType dtype, size_t dim,
                    double cache_percentage, StreamHandle stream);

 public:
  CollCache(BarHandle process_barrier, BarHandle replica_barrier)
      : _process_barrier(process_barrier), _replica_barrier(replica_barrier), _profiler(std::make_shared<Profiler>()) {}

  // facade.h:52-54, facade.cc:38-72: builds every replica (here: the one) with the allocator `allocator_builder` makes
  // for it, from the placement the object already holds; a partial cache therefore needs a build_v2 or refresh to have
  // solved before (the reference's own solve() in front of it is dead code), 0 % and 100 % need nothing
  void build(std::function<std::function<MemHandle(size_t)>(int)> allocator_builder, void *cpu_data, DataType dtype,
             size_t dim, double cache_percentage, StreamHandle stream = nullptr);
  // nodes / output are device pointers; blocking: output is complete on return (facade.cc:74-88)
  void lookup(int replica_id, const IdType *nodes, const size_t num_nodes, void *output, StreamHandle stream,
              uint64_t step_key);
  // 64-bit keys, dense ids (extension)
  void lookup64(int replica_id, const Id64Type *nodes, const size_t num_nodes, void *output, StreamHandle stream,
                uint64_t step_key);
  // distinct keys looked up once: rows of the distinct keys + which of them every position holds (extension)
  // lookup + per-sample combination of a multi-hot feature (ExtractSession::ExtractPooled)
  void lookup_pooled(int replica_id, const IdType *nodes, const int64_t *seg_off, const float *weights, size_t num_rows,
                     size_t num_nodes, int combiner, int elem_bytes, void *output, StreamHandle stream,
                     uint64_t step_key);
  void lookup_pooled64(int replica_id, const Id64Type *nodes, const int64_t *seg_off, const float *weights,
                       size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                       StreamHandle stream, uint64_t step_key);
  size_t lookup_unique(int replica_id, const IdType *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                       StreamHandle stream, uint64_t step_key);
  size_t lookup_unique64(int replica_id, const Id64Type *nodes, size_t num_nodes, void *output, uint32_t *inverse_out,
                         StreamHandle stream, uint64_t step_key);

  // rank list + frequency list over all num_node keys (facade.cc:283-381)
  void build_v2(int replica_id, IdType *ranking_nodes_list_ptr, IdType *ranking_nodes_freq_list_ptr, IdType num_node,
                std::function<MemHandle(size_t)> gpu_mem_allocator, void *cpu_data, DataType dtype, size_t dim,
                double cache_percentage, StreamHandle stream = nullptr);
  // observed keys only, in rank order (facade.cc:430-511)
  void build_v2(int replica_id, ContFreqBuf *freq_rank, IdType num_node,
                std::function<MemHandle(size_t)> gpu_mem_allocator, void *cpu_data, DataType dtype, size_t dim,
                double cache_percentage, StreamHandle stream = nullptr);
  // re-place by new hotness, evict + insert (facade.cc:383-428, 513-557)
  void refresh(int replica_id, IdType *ranking_nodes_list_ptr, IdType *ranking_nodes_freq_list_ptr,
               StreamHandle stream = nullptr, bool foreground = false);
  void refresh(int replica_id, ContFreqBuf *freq_rank, StreamHandle stream = nullptr, bool foreground = false);
  // the same refresh with ranking, placement and key lists computed on the device from the hotness the lookups
  // counted there (RunConfig::gpu_refresh); _nid_to_block is not updated by it
  void refresh_on_device(int replica_id, StreamHandle stream = nullptr, bool foreground = false);
  // rows the refreshes of a replica took from the stage of recently missed rows instead of the host table
  uint64_t rows_from_stage(int replica_id) {
    return (size_t)replica_id < _refresh_session_list.size() && _refresh_session_list[replica_id]
               ? _refresh_session_list[replica_id]->RowsFromStage()
               : 0;
  }

  void report_avg();
  void report_last_epoch(uint64_t epoch);
  void report(uint64_t key);
  std::shared_ptr<Profiler> _profiler;

  inline void set_step_profile_value(uint64_t key, LogStepItem item, double val) { _profiler->LogStep(key, item, val); }
  inline void add_epoch_profile_value(uint64_t key, LogEpochItem item, double val) {
    _profiler->LogEpochAdd(key, item, val);
  }

  // drops the per-replica objects (they hold a reference back to this object)
  void release_replicas() {
    _refresh_session_list.clear();
    _session_list.clear();
    _cache_ctx_list.clear();
  }
  // introspection (tests, reports)
  size_t num_replicas_built() const {
    size_t n = 0;
    for (auto &c : _cache_ctx_list) n += c != nullptr;
    return n;
  }
  std::shared_ptr<CacheContext> cache_ctx(int replica_id) { return _cache_ctx_list.at(replica_id); }
  // stream-ordered lookups (ExtractSession::ExtractFeatAsync / Wait); an extension over the reference
  void lookup_async(int replica_id, const IdType *nodes, size_t num_nodes, void *output, StreamHandle stream) {
    _session_list.at(replica_id)->ExtractFeatAsync(nodes, num_nodes, output, stream);
  }
  void lookup_async64(int replica_id, const Id64Type *nodes, size_t num_nodes, void *output, StreamHandle stream) {
    _session_list.at(replica_id)->ExtractFeatAsync64(nodes, num_nodes, output, stream);
  }
  void lookup_pooled_async(int replica_id, const IdType *nodes, const int64_t *seg_off, const float *weights,
                           size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                           StreamHandle stream) {
    _session_list.at(replica_id)->ExtractPooledAsync(nodes, seg_off, weights, num_rows, num_nodes, combiner, elem_bytes,
                                                     output, stream);
  }
  void lookup_pooled_async64(int replica_id, const Id64Type *nodes, const int64_t *seg_off, const float *weights,
                             size_t num_rows, size_t num_nodes, int combiner, int elem_bytes, void *output,
                             StreamHandle stream) {
    _session_list.at(replica_id)->ExtractPooledAsync64(nodes, seg_off, weights, num_rows, num_nodes, combiner,
                                                       elem_bytes, output, stream);
  }
  void segment_offsets(int replica_id, const int64_t *sorted_rows, size_t num_entries, size_t num_rows,
                       int64_t *seg_off, StreamHandle stream) {
    _session_list.at(replica_id)->SegmentOffsets(sorted_rows, num_entries, num_rows, seg_off, stream);
  }
  void lookup_wait(int replica_id, StreamHandle stream) { _session_list.at(replica_id)->Wait(stream); }
  std::shared_ptr<ExtractSession> session(int replica_id) { return _session_list.at(replica_id); }
  TensorPtr nid_to_block() { return EnsureNidToBlock(); }
};

}  // namespace coll_cache_lib
