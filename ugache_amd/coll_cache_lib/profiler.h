// Per-step metric store behind the LogStep hooks of ExtractFeat / CollCache::lookup.  A small in-process
// stand-in for coll_cache_lib/profiler.{h,cc}: same item ids (profiler.h LogStepItem / LogEpochItem), same
// LogStep / LogEpochAdd / ReportStep / ReportStepAverage entry points, but values live in ordinary memory
// and the report prints only the lines this path feeds.
#pragma once

#include <cstdint>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace coll_cache_lib {
namespace common {

enum LogStepItem {
  kLogL1NumSample = 0, kLogL1NumNode, kLogL1SampleTotalTime, kLogL1SampleTime, kLogL1SendTime, kLogL1RecvTime,
  kLogL1CopyTime, kLogL1ConvertTime, kLogL1TrainTime, kLogL1FeatureBytes, kLogL1LabelBytes, kLogL1IdBytes,
  kLogL1GraphBytes, kLogL1MissBytes, kLogL1RemoteBytes, kLogL1PrefetchAdvanced, kLogL1GetNeighbourTime,
  kLogL1SamplerId,
  kLogL2ShuffleTime, kLogL2LastLayerTime, kLogL2LastLayerSize, kLogL2CoreSampleTime, kLogL2IdRemapTime,
  kLogL2GraphCopyTime, kLogL2IdCopyTime, kLogL2ExtractTime, kLogL2FeatCopyTime, kLogL2CacheCopyTime,
  kLogL3KHopSampleCooTime, kLogL3KHopSampleKernelTime, kLogL3KHopSampleSortCooTime, kLogL3KHopSampleCountEdgeTime,
  kLogL3KHopSampleCompactEdgesTime, kLogL3RandomWalkSampleCooTime, kLogL3RandomWalkTopKTime,
  kLogL3RandomWalkTopKStep1Time, kLogL3RandomWalkTopKStep2Time, kLogL3RandomWalkTopKStep3Time,
  kLogL3RandomWalkTopKStep4Time, kLogL3RandomWalkTopKStep5Time, kLogL3RandomWalkTopKStep6Time,
  kLogL3RandomWalkTopKStep7Time, kLogL3RemapFillUniqueTime, kLogL3RemapPopulateTime, kLogL3RemapMapNodeTime,
  kLogL3RemapMapEdgeTime, kLogL3CacheGetIndexTime, KLogL3CacheCopyIndexTime, kLogL3CacheExtractMissTime,
  kLogL3CacheCopyMissTime, kLogL3CacheCombineMissTime, kLogL3CacheCombineCacheTime, kLogL3CacheCombineRemoteTime,
  kLogL3LabelExtractTime,
  kNumLogStepItems
};

enum LogEpochItem {
  kLogEpochSampleTime = 0, KLogEpochSampleGetCacheMissIndexTime, kLogEpochSampleSendTime, kLogEpochSampleTotalTime,
  kLogEpochCoreSampleTime, kLogEpochSampleCooTime, kLogEpochIdRemapTime, kLogEpochShuffleTime,
  kLogEpochSampleKernelTime, kLogEpochCopyTime, kLogEpochConvertTime, kLogEpochTrainTime, kLogEpochTotalTime,
  kLogEpochFeatureBytes, kLogEpochMissBytes,
  kNumLogEpochItems
};

class Profiler {
 public:
  void LogStep(uint64_t key, LogStepItem item, double val);
  void LogStepAdd(uint64_t key, LogStepItem item, double val);
  void LogEpochAdd(uint64_t key, LogEpochItem item, double val);
  // value of one item at one step key; 0 when never logged
  double GetStep(uint64_t key, LogStepItem item);
  void ReportStep(uint64_t epoch, uint64_t step);
  void ReportStepAverage(uint64_t epoch, uint64_t step);
  void ReportStepItemPercentiles(uint64_t epoch, uint64_t step, LogStepItem item, std::vector<double> percentiles,
                                 const std::string &name);
  void ReportStepAverageLastEpoch(uint64_t epoch, uint64_t step);
  // duration of the last refresh, printed in the level-1 block (profiler.h: _refresh_duration)
  void SetRefreshDuration(double seconds) { _refresh_duration = seconds; }

 private:
  void Output(const std::string &type, uint64_t epoch, uint64_t step, const double *vals);
  std::mutex _mu;
  double _refresh_duration = 0;
  struct Row {
    double v[kNumLogStepItems] = {0};
    uint64_t set_mask[(kNumLogStepItems + 63) / 64] = {0};
  };
  std::unordered_map<uint64_t, Row> _steps;
  std::unordered_map<uint64_t, std::vector<double>> _epochs;
};

}  // namespace common
}  // namespace coll_cache_lib
