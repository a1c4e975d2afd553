// Assertion, logging and namespace helpers shared by every host-side file.
//
// All host code lives in tensorpipe::amd, an inline namespace: source code
// spells tensorpipe::Context exactly as with the reference, while the mangled
// names differ from those of any stock TensorPipe that may be loaded in the
// same process (PyTorch's libtorch_cpu.so carries one).
#pragma once

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>

#define TP_AMD_NAMESPACE_BEGIN \
  namespace tensorpipe {      \
  inline namespace amd {
#define TP_AMD_NAMESPACE_END \
  }                         \
  }

TP_AMD_NAMESPACE_BEGIN

inline const char* tpTrimFilename(const char* path) {
  const char* p = std::strstr(path, "tensorpipe/");
  return p != nullptr ? p : path;
}

// Verbosity is read once from TP_VERBOSE_LOGGING (0 = silent), the same
// switch the reference uses (tensorpipe/common/defs.h:272-286).
inline int tpVerbosity() {
  static const int level = [] {
    const char* e = std::getenv("TP_VERBOSE_LOGGING");
    return e != nullptr ? std::atoi(e) : 0;
  }();
  return level;
}

class LogLine {
 public:
  LogLine(const char* file, int line, char severity) {
    // Monotonic microseconds, so that lines of several processes on one
    // machine can be put on one time axis.
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    char stamp[32];
    snprintf(stamp, sizeof(stamp), "%lld.%03ld", static_cast<long long>(ts.tv_sec) * 1000000 + ts.tv_nsec / 1000, ts.tv_nsec % 1000);
    ss_ << severity << stamp << " " << tpTrimFilename(file) << ":" << line << "] ";
  }
  ~LogLine() {
    ss_ << "\n";
    std::cerr << ss_.str();
  }
  std::ostream& stream() {
    return ss_;
  }

 private:
  std::ostringstream ss_;
};

[[noreturn]] inline void throwAssert(const char* file, int line, const std::string& what) {
  std::ostringstream ss;
  ss << "In " << tpTrimFilename(file) << ":" << line << " \"" << what << "\"";
  throw std::runtime_error(ss.str());
}

TP_AMD_NAMESPACE_END

#define TP_VLOG(level)                     \
  if (::tensorpipe::tpVerbosity() < (level)) \
    ;                                      \
  else                                     \
    ::tensorpipe::LogLine(__FILE__, __LINE__, 'V').stream()

#define TP_LOG_WARNING() ::tensorpipe::LogLine(__FILE__, __LINE__, 'W').stream()

// Programmer errors and failed runtime calls throw std::runtime_error, as the
// reference's TP_THROW_ASSERT does (tensorpipe/common/defs.h:102-105).
#define TP_THROW_ASSERT_IF(cond)                                \
  do {                                                          \
    if (cond) {                                                 \
      ::tensorpipe::throwAssert(__FILE__, __LINE__, #cond);     \
    }                                                           \
  } while (0)

#define TP_THROW_MSG(msg)                                                    \
  do {                                                                       \
    std::ostringstream tp_ss_;                                               \
    tp_ss_ << msg;                                                           \
    ::tensorpipe::throwAssert(__FILE__, __LINE__, tp_ss_.str());             \
  } while (0)

#ifdef NDEBUG
#define TP_DCHECK(cond) \
  do {                  \
  } while (0)
#else
#define TP_DCHECK(cond) TP_THROW_ASSERT_IF(!(cond))
#endif
