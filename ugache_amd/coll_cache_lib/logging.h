// LOG(level) / CHECK* with the reference's convention (coll_cache_lib/logging.h:32-67, logging.cc:69-113):
// no error codes and no exceptions on the hot path; a failed CHECK or LOG(FATAL) prints and abort()s.
// Level comes from SAMGRAPH_LOG_LEVEL (default WARNING); messages at INFO and below go to stdout.
#pragma once

#include <sstream>
#include <string>

namespace coll_cache_lib {
namespace common {

enum class LogLevel { TRACE = 0, DEBUG, INFO, WARNING, ERROR, FATAL };

class LogMessage : public std::ostringstream {
 public:
  LogMessage(const char *file, int line, LogLevel level);
  ~LogMessage();

 protected:
  void Emit();

 private:
  bool _emitted = false;
  const char *_file;
  int _line;
  LogLevel _level;
};

class LogMessageFatal : public LogMessage {
 public:
  LogMessageFatal(const char *file, int line) : LogMessage(file, line, LogLevel::FATAL) {}
  [[noreturn]] ~LogMessageFatal();
};

LogLevel MinLogLevel();

// Raises a fatal error when a ugk_* call of the HIP C-ABI returns non-zero.
void UgkCheckFailed(const char *expr, const char *file, int line);

}  // namespace common
}  // namespace coll_cache_lib

#define _LOG_TRACE coll_cache_lib::common::LogMessage(__FILE__, __LINE__, coll_cache_lib::common::LogLevel::TRACE)
#define _LOG_DEBUG coll_cache_lib::common::LogMessage(__FILE__, __LINE__, coll_cache_lib::common::LogLevel::DEBUG)
#define _LOG_INFO coll_cache_lib::common::LogMessage(__FILE__, __LINE__, coll_cache_lib::common::LogLevel::INFO)
#define _LOG_WARNING coll_cache_lib::common::LogMessage(__FILE__, __LINE__, coll_cache_lib::common::LogLevel::WARNING)
#define _LOG_ERROR coll_cache_lib::common::LogMessage(__FILE__, __LINE__, coll_cache_lib::common::LogLevel::ERROR)
#define _LOG_FATAL coll_cache_lib::common::LogMessageFatal(__FILE__, __LINE__)
#define LOG(severity) _LOG_##severity

#define CHECK(x) \
  if (!(x)) coll_cache_lib::common::LogMessageFatal(__FILE__, __LINE__) << "Check failed: " #x << ' '
#define CHECK_OP(a, b, op) \
  if (!((a)op(b)))         \
  coll_cache_lib::common::LogMessageFatal(__FILE__, __LINE__) \
      << "Check failed: " #a " " #op " " #b << " (" << (a) << " vs " << (b) << ") "
#define CHECK_LT(a, b) CHECK_OP(a, b, <)
#define CHECK_GT(a, b) CHECK_OP(a, b, >)
#define CHECK_LE(a, b) CHECK_OP(a, b, <=)
#define CHECK_GE(a, b) CHECK_OP(a, b, >=)
#define CHECK_EQ(a, b) CHECK_OP(a, b, ==)
#define CHECK_NE(a, b) CHECK_OP(a, b, !=)
#define CHECK_NOTNULL(x) CHECK((x) != nullptr)

// the counterpart of CUDA_CALL (logging.h:53-58) for the C-ABI over the HIP kernels
#define UGK_CALL(expr)                                                               \
  do {                                                                               \
    if ((expr) != 0) coll_cache_lib::common::UgkCheckFailed(#expr, __FILE__, __LINE__); \
  } while (0)
