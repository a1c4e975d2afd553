// Accumulating wall-clock timers for named stretches of host code, printed at
// process exit when TP_STAGE_STATS=1. Unlike the verbose log they cost two
// clock reads per stretch, so the figures hold for an otherwise unperturbed
// run. The reference has no counterpart.
#pragma once

#include <atomic>
#include <chrono>
#include <cstdint>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

enum class Stage : int {
  kPipeEncodeDescriptor = 0,
  kPipeWriteDescriptor,
  kPipeIssueTensors,
  kPipeParseDescriptor,
  kPipeReadRequest,
  kXthEncode,
  kXthDecode,
  kXthLaunch,
  kHarnessMakeMessage,
  kHarnessSync,
  kCount
};

bool stageStatsEnabled();
void stageAdd(Stage s, uint64_t nanos);

class StageScope {
 public:
  explicit StageScope(Stage s) : stage_(s), on_(stageStatsEnabled()) {
    if (on_) {
      t0_ = std::chrono::steady_clock::now();
    }
  }
  ~StageScope() {
    if (on_) {
      stageAdd(
          stage_,
          static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::nanoseconds>(
                                    std::chrono::steady_clock::now() - t0_)
                                    .count()));
    }
  }

 private:
  const Stage stage_;
  const bool on_;
  std::chrono::steady_clock::time_point t0_;
};

// A timeline of named moments, for finding where the microseconds of a small
// transfer go: TP_TIMELINE=<n> keeps the last n marks of the process (any
// thread) and prints them at exit with their distance from the mark before.
// Costs one relaxed load when switched off.
bool timelineEnabled();
void timelineMark(const char* what);
#define TP_MARK(what)                          \
  do {                                         \
    if (::tensorpipe::timelineEnabled()) {     \
      ::tensorpipe::timelineMark(what);        \
    }                                          \
  } while (0)

TP_AMD_NAMESPACE_END
