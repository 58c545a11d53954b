#include "profiler.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <string>
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

namespace {

// One cell of the step report: "<label><pad><value>".  The layout (labels, column padding, value formats, cells
// per line) is the text the reference prints (profiler.cc:559-760) and its eval scripts split on '|'
// (eval/gnn/common/common_parser.py:311-336); the table below states it, the loop in Output() prints it.
enum CellFmt { kSec10, kSec, kSize10, kCount10 };  // %10.6lf, %.6lf, %10s of a readable size, %10.0lf
struct Cell {
  const char *label;  // with its trailing padding
  int item;           // LogStepItem, or one of the two pseudo items below
  CellFmt fmt;
};
constexpr int kItemSeqDuration = -1, kItemRefreshDuration = -2, kEndOfLine = -3;
#define EOL {nullptr, kEndOfLine, kSec}

const Cell kLevel1[] = {
    {"sample         ", kLogL1SampleTime, kSec10}, {"send         ", kLogL1SendTime, kSec10}, EOL,
    {"recv           ", kLogL1RecvTime, kSec10}, {"copy         ", kLogL1CopyTime, kSec10},
    {"convert time ", kLogL1ConvertTime, kSec}, {"train  ", kLogL1TrainTime, kSec}, EOL,
    {"feature nbytes ", kLogL1FeatureBytes, kSize10}, {"label nbytes ", kLogL1LabelBytes, kSize10}, EOL,
    {"id nbytes      ", kLogL1IdBytes, kSize10}, {"graph nbytes ", kLogL1GraphBytes, kSize10}, EOL,
    {"miss nbytes    ", kLogL1MissBytes, kSize10}, {"remote nbytes ", kLogL1RemoteBytes, kSize10}, EOL,
    {"num nodes      ", kLogL1NumNode, kCount10}, {"num samples  ", kLogL1NumSample, kCount10}, EOL,
    {"seq duration   ", kItemSeqDuration, kSec10}, {"refresh duration ", kItemRefreshDuration, kSec10}, EOL,
};
const Cell kLevel2[] = {
    {"shuffle     ", kLogL2ShuffleTime, kSec}, {"core sample  ", kLogL2CoreSampleTime, kSec},
    {"id remap        ", kLogL2IdRemapTime, kSec}, EOL,
    {"graph copy  ", kLogL2GraphCopyTime, kSec}, {"id copy      ", kLogL2IdCopyTime, kSec},
    {"cache feat copy ", kLogL2CacheCopyTime, kSec}, EOL,
    {"last layer sample time ", kLogL2LastLayerTime, kSec}, {"size ", kLogL2LastLayerSize, kSec}, EOL,
};
const Cell kLevel3[] = {
    {"khop sample coo  ", kLogL3KHopSampleCooTime, kSec}, {"khop sort coo      ", kLogL3KHopSampleSortCooTime, kSec},
    {"khop count edge     ", kLogL3KHopSampleCountEdgeTime, kSec},
    {"khop compact edge ", kLogL3KHopSampleCompactEdgesTime, kSec}, EOL,
    {"walk sample coo  ", kLogL3RandomWalkSampleCooTime, kSec}, {"walk topk total    ", kLogL3RandomWalkTopKTime, kSec},
    {"walk topk step1     ", kLogL3RandomWalkTopKStep1Time, kSec},
    {"walk topk step2   ", kLogL3RandomWalkTopKStep2Time, kSec}, EOL,
    {"walk topk step3  ", kLogL3RandomWalkTopKStep3Time, kSec}, {"walk topk step4    ", kLogL3RandomWalkTopKStep4Time, kSec},
    {"walk topk step5     ", kLogL3RandomWalkTopKStep5Time, kSec}, EOL,
    {"walk topk step6  ", kLogL3RandomWalkTopKStep6Time, kSec}, {"walk topk step7    ", kLogL3RandomWalkTopKStep7Time, kSec},
    EOL,
    {"remap unique     ", kLogL3RemapFillUniqueTime, kSec}, {"remap populate     ", kLogL3RemapPopulateTime, kSec},
    {"remap mapnode       ", kLogL3RemapMapNodeTime, kSec}, {"remap mapedge     ", kLogL3RemapMapEdgeTime, kSec}, EOL,
    {"cache get_index  ", kLogL3CacheGetIndexTime, kSec}, {"cache copy_index   ", KLogL3CacheCopyIndexTime, kSec},
    {"cache extract_miss  ", kLogL3CacheExtractMissTime, kSec}, EOL,
    {"cache copy_miss  ", kLogL3CacheCopyMissTime, kSec}, {"cache combine_miss ", kLogL3CacheCombineMissTime, kSec},
    {"cache combine cache ", kLogL3CacheCombineCacheTime, kSec},
    {"cache combine remote ", kLogL3CacheCombineRemoteTime, kSec}, EOL,
    {"label extract  ", kLogL3LabelExtractTime, kSec}, EOL,
};
#undef EOL

template <size_t N>
void PrintLevel(std::ostream &out, int level, const Cell (&cells)[N], const std::string &type, uint64_t epoch,
                uint64_t step, const double *v, double seq_duration, double refresh_duration) {
  char buf[96];
  snprintf(buf, sizeof(buf), "    [%s Profiler Level %d E%u S%u]\n", type.c_str(), level, (unsigned)epoch,
           (unsigned)step);
  out << buf;
  bool first = true;
  for (const Cell &c : cells) {
    if (c.item == kEndOfLine) {
      out << "\n";
      first = true;
      continue;
    }
    out << (first ? "        L" + std::to_string(level) + "  " : std::string(" | ")) << c.label;
    first = false;
    const double val = c.item == kItemSeqDuration ? seq_duration
                       : c.item == kItemRefreshDuration ? refresh_duration
                                                        : v[c.item];
    switch (c.fmt) {
      case kSec10: snprintf(buf, sizeof(buf), "%10.6lf", val); break;
      case kSec: snprintf(buf, sizeof(buf), "%.6lf", val); break;
      case kCount10: snprintf(buf, sizeof(buf), "%10.0lf", val); break;
      case kSize10: snprintf(buf, sizeof(buf), "%10s", ToReadableSize((size_t)val).c_str()); break;
    }
    out << buf;
  }
}

int ProfileLevel() {
  const char *e = getenv("SAMGRAPH_PROFILE_LEVEL");  // constant.cc:64; anything but 1 or 2 means all three levels
  if (e && std::string(e) == "1") return 1;
  if (e && std::string(e) == "2") return 2;
  return 3;
}

}  // namespace

void Profiler::Output(const std::string &type, uint64_t epoch, uint64_t step, const double *v) {
  const int level = ProfileLevel();
  const double seq = 0, refresh = _refresh_duration;
  PrintLevel(std::cout, 1, kLevel1, type, epoch, step, v, seq, refresh);
  if (level >= 2) PrintLevel(std::cout, 2, kLevel2, type, epoch, step, v, seq, refresh);
  if (level >= 3) PrintLevel(std::cout, 3, kLevel3, type, epoch, step, v, seq, refresh);
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
