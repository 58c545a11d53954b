#include "profiler.h"

#include <algorithm>
#include <cstdio>
#include <iostream>

#include "common.h"
#include "run_config.h"

namespace coll_cache_lib {
namespace common {

void Profiler::LogStep(uint64_t key, LogStepItem item, double val) {
  if (key == 0xffffffffffffffffull) return;
  std::lock_guard<std::mutex> g(_mu);
  Row &r = _steps[key];
  r.v[item] = val;
  r.set_mask[item / 64] |= 1ull << (item % 64);
}

void Profiler::LogStepAdd(uint64_t key, LogStepItem item, double val) {
  if (key == 0xffffffffffffffffull) return;
  std::lock_guard<std::mutex> g(_mu);
  Row &r = _steps[key];
  r.v[item] += val;
  r.set_mask[item / 64] |= 1ull << (item % 64);
}

void Profiler::LogEpochAdd(uint64_t key, LogEpochItem item, double val) {
  if (key == 0xffffffffffffffffull) return;
  std::lock_guard<std::mutex> g(_mu);
  auto &e = _epochs[RunConfig::GetEpochFromKey(key)];
  if (e.empty()) e.assign(kNumLogEpochItems, 0.0);
  e[item] += val;
}

double Profiler::GetStep(uint64_t key, LogStepItem item) {
  std::lock_guard<std::mutex> g(_mu);
  auto it = _steps.find(key);
  return it == _steps.end() ? 0.0 : it->second.v[item];
}

void Profiler::Output(const std::string &type, uint64_t epoch, uint64_t step, const double *v) {
  char buf[1024];
  snprintf(buf, sizeof(buf),
           "    [%s Profiler Level 1 E%llu S%llu]\n"
           "        L1  feature nbytes %10s | miss nbytes  %10s | remote nbytes %10s\n"
           "    [%s Profiler Level 2 E%llu S%llu]\n"
           "        L2  cache feat copy %.6lf\n"
           "    [%s Profiler Level 3 E%llu S%llu]\n"
           "        L3  cache get_index  %.6lf | cache combine_miss %.6lf | cache combine cache %.6lf | "
           "cache combine remote %.6lf\n",
           type.c_str(), (unsigned long long)epoch, (unsigned long long)step,
           ToReadableSize((size_t)v[kLogL1FeatureBytes]).c_str(), ToReadableSize((size_t)v[kLogL1MissBytes]).c_str(),
           ToReadableSize((size_t)v[kLogL1RemoteBytes]).c_str(), type.c_str(), (unsigned long long)epoch,
           (unsigned long long)step, v[kLogL2CacheCopyTime], type.c_str(), (unsigned long long)epoch,
           (unsigned long long)step, v[kLogL3CacheGetIndexTime], v[kLogL3CacheCombineMissTime],
           v[kLogL3CacheCombineCacheTime], v[kLogL3CacheCombineRemoteTime]);
  std::cout << buf;
}

void Profiler::ReportStep(uint64_t epoch, uint64_t step) {
  Row r;
  {
    std::lock_guard<std::mutex> g(_mu);
    auto it = _steps.find(RunConfig::GetBatchKey(epoch, step));
    if (it != _steps.end()) r = it->second;
  }
  Output("Step", epoch, step, r.v);
}

void Profiler::ReportStepAverage(uint64_t epoch, uint64_t step) {
  double sum[kNumLogStepItems] = {0};
  size_t cnt[kNumLogStepItems] = {0};
  const uint64_t last = RunConfig::GetBatchKey(epoch, step);
  {
    std::lock_guard<std::mutex> g(_mu);
    for (auto &kv : _steps) {
      if (kv.first > last) continue;
      for (int i = 0; i < kNumLogStepItems; i++) {
        if (kv.second.set_mask[i / 64] >> (i % 64) & 1) {
          sum[i] += kv.second.v[i];
          cnt[i]++;
        }
      }
    }
  }
  for (int i = 0; i < kNumLogStepItems; i++) sum[i] = cnt[i] ? sum[i] / cnt[i] : 0;
  Output("Step(average)", epoch, step, sum);
}

void Profiler::ReportStepAverageLastEpoch(uint64_t epoch, uint64_t step) { ReportStepAverage(epoch, step); }

void Profiler::ReportStepItemPercentiles(uint64_t epoch, uint64_t step, LogStepItem item,
                                         std::vector<double> percentiles, const std::string &name) {
  std::vector<double> vals;
  const uint64_t last = RunConfig::GetBatchKey(epoch, step);
  {
    std::lock_guard<std::mutex> g(_mu);
    for (auto &kv : _steps)
      if (kv.first <= last && (kv.second.set_mask[item / 64] >> (item % 64) & 1)) vals.push_back(kv.second.v[item]);
  }
  if (vals.empty()) return;
  std::sort(vals.begin(), vals.end());
  for (double p : percentiles) {
    size_t idx = (size_t)(p / 100.0 * vals.size());
    if (idx >= vals.size()) idx = vals.size() - 1;
    char buf[128];
    snprintf(buf, sizeof(buf), "test_result:%s_%g=%.6lf\n", name.c_str(), p, vals[idx]);
    std::cout << buf;
  }
}

}  // namespace common
}  // namespace coll_cache_lib
