#include "placement.h"

#include <cstring>
#include <iostream>

#include "logging.h"
#include "run_config.h"

namespace coll_cache_lib {
namespace common {
namespace coll_cache {

void FreqRankSolver::Build(TensorPtr stream_id_list, TensorPtr stream_freq_list, std::vector<int> device_to_stream,
                           const IdType num_node, const TensorPtr nid_to_block_tensor) {
  CHECK_NOTNULL(stream_id_list);
  CHECK_NOTNULL(stream_freq_list);
  CHECK_EQ(stream_id_list->NumItem(), (size_t)num_node);
  CHECK_EQ(stream_freq_list->NumItem(), (size_t)num_node);
  _rank_keys = stream_id_list;
  _rank_freq = stream_freq_list;
  _nid_to_block = nid_to_block_tensor;
  _num_node = num_node;
}

void FreqRankSolver::BuildSingleStream(ContFreqBuf *freq_rank, std::vector<int> device_to_stream,
                                       const IdType num_node, const TensorPtr nid_to_block_tensor) {
  CHECK_NOTNULL(freq_rank);
  LegacyFreqBuf legacy;
  freq_rank->GetLegacyFreqRank(&legacy, num_node);
  _rank_keys = Tensor::Empty(kI32, {(size_t)num_node}, CPU_CLIB(), "rank_keys");
  _rank_freq = Tensor::Empty(kI32, {(size_t)num_node}, CPU_CLIB(), "rank_freq");
  memcpy(_rank_keys->MutableData(), legacy.rank_vec.data(), (size_t)num_node * sizeof(IdType));
  memcpy(_rank_freq->MutableData(), legacy.freq_vec.data(), (size_t)num_node * sizeof(IdType));
  _nid_to_block = nid_to_block_tensor;
  _num_node = num_node;
}

void FreqRankSolver::Solve(std::vector<int> device_to_stream, std::vector<PerT> device_to_cache_percent,
                           std::string mode, double T_local, double T_cpu) {
  CHECK_NOTNULL(_nid_to_block);
  const int num_device = (int)device_to_stream.size();
  CHECK_EQ(num_device, 1) << "this build places keys for one GPU and its host";
  const int num_block = 2;
  const IdType num_node = _num_node;
  const IdType num_cached_nodes = (IdType)(num_node * (device_to_cache_percent[0] / (double)100));
  const IdType *rank = _rank_keys->CPtr<IdType>();
  const IdType *freq = _rank_freq->CPtr<IdType>();
  IdType *nid_to_block = _nid_to_block->Ptr<IdType>();
  double rep_w = 0, cpu_w = 0;
#pragma omp parallel for num_threads(RunConfig::omp_thread_num) reduction(+ : rep_w, cpu_w)
  for (IdType r = 0; r < num_node; r++) {
    const IdType key = rank[r];
    if (r < num_cached_nodes) {
      nid_to_block[key] = 0;
      rep_w += freq[r];
    } else {
      nid_to_block[key] = 1;
      cpu_w += freq[r];
    }
  }
  const double total_w = rep_w + cpu_w;
  const IdType cpu_size = num_node - num_cached_nodes;
  std::cout << "coll_cache:optimal_local_storage=" << num_cached_nodes / (double)num_node << "\n";
  std::cout << "coll_cache:optimal_cpu_storage=" << cpu_size / (double)num_node << "\n";
  std::cout << "coll_cache:optimal_local_rate=" << (total_w > 0 ? rep_w / total_w : 0) << "\n";
  std::cout << "coll_cache:optimal_cpu_rate=" << (total_w > 0 ? cpu_w / total_w : 0) << "\n";
  std::cout << "z=" << rep_w * 100 / num_node * T_local + cpu_w * 100 / num_node * T_cpu << "\n";

  block_placement = Tensor::Empty(kU8, {(size_t)num_block}, CPU_CLIB(), "coll_cache_block_placement");
  block_placement->Ptr<uint8_t>()[0] = (uint8_t)((1 << num_device) - 1);
  block_placement->Ptr<uint8_t>()[1] = 0;
  block_access_from = Tensor::Empty(kU8, {(size_t)num_device, (size_t)num_block}, CPU_CLIB(), "coll_cache_advise");
  for (int dev = 0; dev < num_device; dev++) {
    block_access_from->Ptr<uint8_t>()[dev * num_block + 0] = (uint8_t)dev;
    block_access_from->Ptr<uint8_t>()[dev * num_block + 1] = (uint8_t)num_device;
  }
  block_density_tensor = Tensor::Empty(kF64, {(size_t)num_block}, CPU_CLIB(), "coll_cache_block_density");
  block_density_tensor->Ptr<double>()[0] = (double)num_cached_nodes * 100 / (double)num_node;
  block_density_tensor->Ptr<double>()[1] = (double)cpu_size * 100 / (double)num_node;
  (void)mode;
}

}  // namespace coll_cache
}  // namespace common
}  // namespace coll_cache_lib
