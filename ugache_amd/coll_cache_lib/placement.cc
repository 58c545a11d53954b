#include "placement.h"

#include <algorithm>
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
  _cont = nullptr;
  _nid_to_block = nid_to_block_tensor;
  _num_node = num_node;
}

void FreqRankSolver::BuildSingleStream(ContFreqBuf *freq_rank, std::vector<int> device_to_stream,
                                       const IdType num_node, const TensorPtr nid_to_block_tensor) {
  CHECK_NOTNULL(freq_rank);
  CHECK_LE(freq_rank->size(), (size_t)num_node);
  _cont = freq_rank;
  _rank_keys = nullptr;
  _rank_freq = nullptr;
  _nid_to_block = nid_to_block_tensor;
  _num_node = num_node;
}

// Same result as walking the full rank list (observed keys in rank order, then the never-observed keys in
// ascending order), without materialising it: the key space can be hundreds of millions of keys of which a refresh
// has observed a small part.
void FreqRankSolver::Materialize(const IdType *top_rows, size_t num_top, size_t num_extra, IdType num_node_,
                                 IdType *nid_to_block) {
  const size_t num_node = num_node_;
  const int nthr = std::max(1, RunConfig::omp_thread_num);
#pragma omp parallel for num_threads(nthr)
  for (size_t k = 0; k < num_node; k++) nid_to_block[k] = 1;
#pragma omp parallel for num_threads(nthr)
  for (size_t r = 0; r < num_top; r++) nid_to_block[top_rows[r]] = 0;
  if (num_extra == 0) return;
  // the cache is larger than the ranked set: fill it up with the smallest keys that are not in it.  Every ranked key
  // that is cached is block 0 by now; when keys are left over, every ranked key is (the cache holds all of them).
  const size_t chunk = (num_node + nthr - 1) / nthr;
  std::vector<size_t> before(nthr + 1, 0);
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) {
    const size_t lo = std::min(num_node, chunk * t), hi = std::min(num_node, chunk * (t + 1));
    size_t c = 0;
    for (size_t k = lo; k < hi; k++) c += nid_to_block[k] == 1;
    before[t + 1] = c;
  }
  for (int t = 0; t < nthr; t++) before[t + 1] += before[t];
#pragma omp parallel for num_threads(nthr) schedule(static, 1)
  for (int t = 0; t < nthr; t++) {
    const size_t lo = std::min(num_node, chunk * t), hi = std::min(num_node, chunk * (t + 1));
    size_t seen = before[t];
    for (size_t k = lo; k < hi && seen < num_extra; k++)
      if (nid_to_block[k] == 1) {
        nid_to_block[k] = 0;
        seen++;
      }
  }
}

// Same result as walking the full rank list (observed keys in rank order, then the never-observed keys in
// ascending order), without materialising it: the key space can be hundreds of millions of keys of which a refresh
// has observed a small part.
void FreqRankSolver::SolveFromObserved(IdType num_cached_nodes, double *rep_w_out, double *cpu_w_out) {
  const size_t num_node = _num_node, m = _cont->size(), k_cached = num_cached_nodes;
  const auto *e = _cont->buf;
  const int nthr = std::max(1, RunConfig::omp_thread_num);
  double rep_w = 0, cpu_w = 0;
  bool bad = false;
  const size_t top = std::min(m, k_cached);
  top_rows = Tensor::Empty(kI32, {top}, CPU_CLIB(), "placement_top_rows");
  IdType *rows = top_rows->Ptr<IdType>();
#pragma omp parallel for num_threads(nthr) reduction(+ : rep_w, cpu_w) reduction(|| : bad)
  for (size_t r = 0; r < m; r++) {
    if (e[r].key >= num_node) {
      bad = true;
    } else if (r < top) {
      rows[r] = e[r].key;
      rep_w += e[r].cnt;
    } else {
      cpu_w += e[r].cnt;
    }
  }
  CHECK(!bad) << "a ranked key is outside the key space of " << num_node;
  num_extra = k_cached > m ? k_cached - m : 0;
  if (!defer_nid_to_block) Materialize(rows, top, num_extra, _num_node, _nid_to_block->Ptr<IdType>());
  *rep_w_out = rep_w;
  *cpu_w_out = cpu_w;
}

void FreqRankSolver::Solve(std::vector<int> device_to_stream, std::vector<PerT> device_to_cache_percent,
                           std::string mode, double T_local, double T_cpu) {
  const int num_device = (int)device_to_stream.size();
  CHECK_EQ(num_device, 1) << "this build places keys for one GPU and its host";
  const int num_block = 2;
  const IdType num_node = _num_node;
  const IdType num_cached_nodes = NumCachedNodes(num_node, device_to_cache_percent[0]);
  CHECK(defer_nid_to_block || _nid_to_block != nullptr);
  IdType *nid_to_block = _nid_to_block ? _nid_to_block->Ptr<IdType>() : nullptr;
  double rep_w = 0, cpu_w = 0;
  if (_cont != nullptr) {
    SolveFromObserved(num_cached_nodes, &rep_w, &cpu_w);
  } else {
    const IdType *rank = _rank_keys->CPtr<IdType>();
    const IdType *freq = _rank_freq->CPtr<IdType>();
    if (defer_nid_to_block) {
      // the head of the rank list is the cached set; the list is the caller's memory, so the head is copied
      bool bad = false;
#pragma omp parallel for num_threads(RunConfig::omp_thread_num) reduction(+ : rep_w, cpu_w) reduction(|| : bad)
      for (IdType r = 0; r < num_node; r++) {
        bad = bad || rank[r] >= num_node;
        if (r < num_cached_nodes) rep_w += freq[r];
        else cpu_w += freq[r];
      }
      CHECK(!bad) << "a ranked key is outside the key space of " << num_node;
      top_rows = Tensor::CopyBlob(rank, kI32, {(size_t)num_cached_nodes}, CPU_CLIB(), CPU_CLIB(), "placement_top_rows");
      num_extra = 0;
    } else {
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
