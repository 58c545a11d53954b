// Frequency-ranked placement for one GPU and its host.
//
// With a single GPU a key has two possible sources, so the reference's MILP over GPUs and links
// (coll_cache/optimal_solver_class.cc) degenerates to "cache the top-K keys by observed frequency".  This
// class keeps the solver interface the facade drives (Build / BuildSingleStream / Solve and the four result
// arrays, optimal_solver_class.h:34-70) and implements the one policy that is left, with the arithmetic of
// RepSolver::Solve (optimal_solver_class.cc:1869-1924):
//   K = (IdType)(num_node * (percent / 100.0));  ranks [0, K) -> block 0 (cached, read from the GPU),
//   ranks [K, num_node) -> block 1 (host).
#pragma once

#include <string>
#include <vector>

#include "common.h"
#include "freq_recorder.h"

namespace coll_cache_lib {
namespace common {
namespace coll_cache {

using PerT = double;

class CollCacheSolver {
 public:
  virtual ~CollCacheSolver() {}
  // rank list + frequency list of all keys, shape [1, num_node]
  virtual void Build(TensorPtr stream_id_list, TensorPtr stream_freq_list, std::vector<int> device_to_stream,
                     const IdType num_node, const TensorPtr nid_to_block_tensor) = 0;
  virtual void BuildSingleStream(ContFreqBuf *freq_rank, std::vector<int> device_to_stream, const IdType num_node,
                                 const TensorPtr nid_to_block_tensor) = 0;
  virtual void Solve(std::vector<int> device_to_stream, std::vector<PerT> device_to_cache_percent, std::string mode,
                     double T_local, double T_cpu) = 0;
  TensorPtr block_density_tensor;  // f64 [num_block], percent of all keys
  TensorPtr block_placement;       // u8  [num_block], bitmask of GPUs holding the block
  TensorPtr block_access_from;     // u8  [num_device, num_block], where each GPU reads the block from
};

class FreqRankSolver : public CollCacheSolver {
 public:
  void Build(TensorPtr stream_id_list, TensorPtr stream_freq_list, std::vector<int> device_to_stream,
             const IdType num_node, const TensorPtr nid_to_block_tensor) override;
  void BuildSingleStream(ContFreqBuf *freq_rank, std::vector<int> device_to_stream, const IdType num_node,
                         const TensorPtr nid_to_block_tensor) override;
  void Solve(std::vector<int> device_to_stream, std::vector<PerT> device_to_cache_percent, std::string mode,
             double T_local, double T_cpu) override;
  // how many of num_node keys a cache of `percent` % holds (optimal_solver_class.cc:1878)
  static IdType NumCachedNodes(IdType num_node, PerT percent) { return (IdType)(num_node * (percent / (double)100)); }

  // Set before Solve: the key -> block array (4 bytes per key of the key space) is not written.  The placement is
  // described by what it was computed from instead: top_rows, the cached keys that were ranked (observed entries, or
  // the head of a full rank list), and num_extra, how many never-observed keys, lowest first, fill the rest of the
  // cache.  A build on one GPU turns that into its key list on the device (CacheContext::build), and Materialize
  // writes the array out for whoever still wants it.
  bool defer_nid_to_block = false;
  TensorPtr top_rows;  // u32 [n], distinct keys
  size_t num_extra = 0;
  static void Materialize(const IdType *top_rows, size_t num_top, size_t num_extra, IdType num_node,
                          IdType *nid_to_block);

 private:
  TensorPtr _rank_keys;  // u32 [num_node]   (Build)
  TensorPtr _rank_freq;  // u32 [num_node]   (Build)
  // BuildSingleStream: the observed keys in rank order; the never-observed keys follow in ascending order
  // (ContFreqBuf::GetLegacyFreqRank) without being written out
  const ContFreqBuf *_cont = nullptr;
  void SolveFromObserved(IdType num_cached_nodes, double *rep_w, double *cpu_w);
  TensorPtr _nid_to_block;
  IdType _num_node = 0;
};

}  // namespace coll_cache
}  // namespace common
}  // namespace coll_cache_lib
