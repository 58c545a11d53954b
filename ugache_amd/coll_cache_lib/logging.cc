#include "logging.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <iostream>

#include "ugache_hip.h"

namespace coll_cache_lib {
namespace common {

namespace {
const char *kLevelName[] = {"TRACE", "DEBUG", "INFO", "WARNING", "ERROR", "FATAL"};

LogLevel ParseLevel(const char *s) {
  if (!s || !*s) return LogLevel::WARNING;
  for (int i = 0; i <= (int)LogLevel::FATAL; i++) {
    if (strcasecmp(s, kLevelName[i]) == 0) return (LogLevel)i;
  }
  if (strcasecmp(s, "warn") == 0) return LogLevel::WARNING;
  return LogLevel::WARNING;
}
}  // namespace

LogLevel MinLogLevel() {
  static LogLevel lvl = ParseLevel(getenv("SAMGRAPH_LOG_LEVEL"));
  return lvl;
}

LogMessage::LogMessage(const char *file, int line, LogLevel level) : _file(file), _line(line), _level(level) {}

LogMessage::~LogMessage() { Emit(); }

void LogMessage::Emit() {
  if (_emitted) return;
  _emitted = true;
  if (_level < MinLogLevel()) return;
  static const bool hide_time = getenv("SAMGRAPH_LOG_HIDE_TIME") != nullptr;
  std::ostream &os = (_level <= LogLevel::INFO) ? std::cout : std::cerr;
  std::ostringstream head;
  head << '[';
  if (!hide_time) {
    char buf[32];
    time_t now = time(nullptr);
    struct tm tmv;
    localtime_r(&now, &tmv);
    strftime(buf, sizeof(buf), "%F %T", &tmv);
    head << buf << ' ';
  }
  const char *base = strrchr(_file, '/');
  head << (base ? base + 1 : _file) << ':' << _line << "] " << kLevelName[(int)_level] << ": ";
  os << head.str() << str() << std::endl;
}

LogMessageFatal::~LogMessageFatal() {
  Emit();
  std::cout.flush();
  std::cerr.flush();
  abort();
}

void UgkCheckFailed(const char *expr, const char *file, int line) {
  LogMessageFatal(file, line) << "HIP layer call failed: " << expr << ": " << ugk_last_error();
  abort();  // not reached
}

}  // namespace common
}  // namespace coll_cache_lib
