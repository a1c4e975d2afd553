#include <cstring>
#include <sstream>

#include <tensorpipe/common/error.h>
#include <tensorpipe/common/hip_api.h>
#include <tensorpipe/common/hip_buffer.h>

TP_AMD_NAMESPACE_BEGIN

const Error Error::kSuccess{};

std::string Error::what() const {
  if (!error_) {
    return "success";
  }
  std::ostringstream ss;
  ss << error_->what() << " (this error originated at " << file_ << ":" << line_ << ")";
  return ss.str();
}

std::string SystemError::what() const {
  std::ostringstream ss;
  ss << syscall_ << ": " << std::strerror(error_);
  return ss.str();
}

std::string ShortReadError::what() const {
  std::ostringstream ss;
  ss << "short read: got " << actual_ << " bytes while expecting to read " << expected_
     << " bytes";
  return ss.str();
}

std::string ShortWriteError::what() const {
  std::ostringstream ss;
  ss << "short write: wrote " << actual_ << " bytes while expecting to write " << expected_
     << " bytes";
  return ss.str();
}

std::string EOFError::what() const {
  return "eof";
}

std::string HipError::what() const {
  std::ostringstream ss;
  ss << call_ << ": [" << code_ << "] " << tphip_strerror(code_);
  return ss.str();
}

int hipDeviceCountNoThrow() {
  int count = 0;
  if (tphip_device_count(&count) != 0) {
    return 0;
  }
  return count;
}

int hipDeviceForPointer(const void* ptr) {
  // With a single visible GPU every device pointer belongs to device 0: skip
  // the driver query, which would otherwise run several times per tensor.
  static const int count = hipDeviceCountNoThrow();
  if (count == 1 && ptr != nullptr) {
    return 0;
  }
  int dev = -1;
  int isHost = 0;
  TP_HIP_CHECK(tphip_device_for_ptr(ptr, &dev, &isHost));
  return isHost ? -1 : dev;
}

Device HipBuffer::getDevice() const {
  int dev = hipDeviceForPointer(ptr);
  TP_THROW_ASSERT_IF(dev < 0);
  return Device{kHipDeviceType, dev};
}

TP_AMD_NAMESPACE_END

#include <tensorpipe/common/stage_timer.h>

#include <cstdio>
#include <cstdlib>

TP_AMD_NAMESPACE_BEGIN

namespace {

struct StageTable {
  std::atomic<uint64_t> nanos[static_cast<int>(Stage::kCount)];
  std::atomic<uint64_t> calls[static_cast<int>(Stage::kCount)];
  bool enabled{false};
  StageTable() {
    for (auto& v : nanos) {
      v.store(0);
    }
    for (auto& v : calls) {
      v.store(0);
    }
    const char* e = std::getenv("TP_STAGE_STATS");
    enabled = e != nullptr && e[0] == '1';
  }
  ~StageTable() {
    if (!enabled) {
      return;
    }
    static const char* const kNames[] = {
        "pipe: encode descriptor", "pipe: write descriptor+payloads", "pipe: issue tensors",
        "pipe: parse descriptor",  "pipe: read request",               "hip_xth: encode descriptor",
        "hip_xth: decode+group",   "hip_xth: launch",                  "harness: make message",
        "harness: stream sync"};
    for (int i = 0; i < static_cast<int>(Stage::kCount); ++i) {
      const uint64_t c = calls[i].load();
      if (c != 0) {
        std::fprintf(
            stderr, "[stage] %-34s %9llu calls  %9.2f us avg\n", kNames[i],
            static_cast<unsigned long long>(c), nanos[i].load() / 1e3 / static_cast<double>(c));
      }
    }
  }
};

StageTable& stageTable() {
  static StageTable t;
  return t;
}

} // namespace

bool stageStatsEnabled() {
  return stageTable().enabled;
}

void stageAdd(Stage s, uint64_t nanos) {
  StageTable& t = stageTable();
  t.nanos[static_cast<int>(s)].fetch_add(nanos, std::memory_order_relaxed);
  t.calls[static_cast<int>(s)].fetch_add(1, std::memory_order_relaxed);
}

TP_AMD_NAMESPACE_END
