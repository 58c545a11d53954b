// Wall-clock stopwatch (coll_cache_lib/timer.h:25-64).
#pragma once
#include <chrono>
namespace coll_cache_lib {
namespace common {
class Timer {
 public:
  Timer() { Reset(); }
  void Reset() { _t0 = std::chrono::steady_clock::now(); }
  double Passed() const { return std::chrono::duration<double>(std::chrono::steady_clock::now() - _t0).count(); }
  double PassedSec() const { return Passed(); }
  double PassedMicro() const { return Passed() * 1e6; }

 private:
  std::chrono::steady_clock::time_point _t0;
};
}  // namespace common
}  // namespace coll_cache_lib
