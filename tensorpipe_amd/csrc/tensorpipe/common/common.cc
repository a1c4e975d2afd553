#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <map>
#include <mutex>
#include <sstream>

#include <unistd.h>

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

namespace {

// Address ranges the runtime has vouched for, so that the per-tensor question
// "which device owns this pointer" costs a map lookup instead of driver calls
// (the reference asks the driver every time,
// tensorpipe/common/cuda.h:141-166). A range is entered after the runtime has
// named its device, its extent and the id of its allocation; a pointer outside
// every known range goes to the runtime, and one the runtime does not know
// (plain host memory) is reported as such.
//
// An address may be freed and handed out again, to the runtime or to somebody
// else (a plain mmap). So a remembered range is believed only for a while: the
// callers mark the start of every message they handle (hipPointerCheckpoint),
// and the first hit on a range after such a mark asks the runtime whether the
// allocation there is still the one remembered (one query per range and
// message, not per tensor). If it is not, the range is forgotten and the
// pointer is looked up from scratch.
// What a thread remembers: the mark of its current unit of work and the ranges
// it has used last (a message's tensors come from a handful of allocations, and
// a peer's may come from dozens of the caching allocator's segments), sorted by
// address, each with the mark up to which it has been checked. One object, so that a lookup finds the thread's block once.
// TP_POINTER_STATS=1: how often the runtime was asked, printed when the process ends.
struct PointerStats {
  std::atomic<uint64_t> checks{0}, stale{0}, fromScratch{0}, sharedHits{0};
  bool print{false};
  PointerStats() {
    const char* e = std::getenv("TP_POINTER_STATS");
    print = e != nullptr && e[0] == '1';
  }
  ~PointerStats() {
    if (print) {
      std::fprintf(stderr, "[pointers %d] rechecks %llu (stale %llu), looked up from scratch %llu, found in the shared table %llu\n",
                   static_cast<int>(::getpid()), static_cast<unsigned long long>(checks.load()),
                   static_cast<unsigned long long>(stale.load()), static_cast<unsigned long long>(fromScratch.load()),
                   static_cast<unsigned long long>(sharedHits.load()));
    }
  }
};
PointerStats& pointerStats() {
  static PointerStats s;
  return s;
}

struct RecentRange {
  uintptr_t begin{0}, end{0};
  int device{-1};
  uint64_t bufferId{0};
  uint64_t generation{0};
  uint64_t checkedAt{0};
};
constexpr int kRecentRanges = 32;
struct PointerMemo {
  uint64_t epoch{1};
  int scopes{0}; // open HipPointerScopes on this thread
  int hot{-1}; // the entry that answered last
  int used{0};
  RecentRange recent[kRecentRanges]; // sorted by begin
};
thread_local PointerMemo tlsPointerMemo;

class PointerRanges {
 public:
  int lookup(const void* ptr) {
    const uintptr_t p = reinterpret_cast<uintptr_t>(ptr);
    PointerMemo& memo = tlsPointerMemo;
    const uint64_t gen = generation_.load(std::memory_order_acquire);
    int k = -1;
    if (memo.hot >= 0 && p >= memo.recent[memo.hot].begin && p < memo.recent[memo.hot].end) {
      k = memo.hot;
    } else {
      // the last entry that begins at or below p
      int lo = 0, hi = memo.used;
      while (lo < hi) {
        const int mid = (lo + hi) / 2;
        if (memo.recent[mid].begin <= p) {
          lo = mid + 1;
        } else {
          hi = mid;
        }
      }
      if (lo > 0 && p < memo.recent[lo - 1].end) {
        k = lo - 1;
      }
    }
    if (k >= 0) {
      RecentRange& r = memo.recent[k];
      if (r.generation != gen) {
        memo.used = 0; // the shared table has changed under what this thread remembers
        memo.hot = -1;
      } else if (r.checkedAt == memo.epoch) {
        memo.hot = k;
        return r.device;
      } else if (stillThere(ptr, r.bufferId)) {
        r.checkedAt = memo.epoch;
        memo.hot = k;
        return r.device;
      } else {
        forget(r.begin);
        memo.used = 0;
        memo.hot = -1;
      }
    }
    {
      Range found{};
      uintptr_t begin = 0;
      bool hit = false;
      {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = ranges_.upper_bound(p);
        if (it != ranges_.begin()) {
          --it;
          if (p < it->second.end) {
            begin = it->first;
            found = it->second;
            hit = true;
          }
        }
      }
      if (hit) {
        pointerStats().sharedHits.fetch_add(1, std::memory_order_relaxed);
        if (stillThere(ptr, found.bufferId)) {
          const uint64_t now = generation_.load(std::memory_order_acquire);
          if (memo.used == kRecentRanges || (memo.used > 0 && memo.recent[0].generation != now)) {
            memo.used = 0;
          }
          int at = memo.used;
          while (at > 0 && memo.recent[at - 1].begin > begin) {
            memo.recent[at] = memo.recent[at - 1];
            --at;
          }
          memo.recent[at] = RecentRange{begin, found.end, found.device, found.bufferId, now, memo.epoch};
          ++memo.used;
          memo.hot = at;
          return found.device;
        }
        forget(begin);
      }
    }
    pointerStats().fromScratch.fetch_add(1, std::memory_order_relaxed);
    int dev = -1;
    int isHost = 0;
    TP_HIP_CHECK(tphip_device_for_ptr(ptr, &dev, &isHost));
    if (dev < 0) {
      return -1; // memory the runtime has never seen: not something a kernel may touch
    }
    void* base = nullptr;
    size_t size = 0;
    uint64_t id = 0;
    if (tphip_mem_base(ptr, &base, &size) != 0 || base == nullptr || size == 0 ||
        tphip_mem_buffer_id(ptr, &id) != 0 || id == 0) {
      return dev; // known to the runtime, extent or identity unknown: answer, do not remember
    }
    const uintptr_t b = reinterpret_cast<uintptr_t>(base);
    std::lock_guard<std::mutex> lock(mutex_);
    if (ranges_.size() >= 4096) {
      ranges_.clear();
      generation_.fetch_add(1, std::memory_order_acq_rel);
    }
    // whatever overlapped the new range has been freed since
    auto it = ranges_.lower_bound(b);
    if (it != ranges_.begin() && std::prev(it)->second.end > b) {
      --it;
    }
    while (it != ranges_.end() && it->first < b + size) {
      it = ranges_.erase(it);
      generation_.fetch_add(1, std::memory_order_acq_rel);
    }
    ranges_[b] = Range{b + size, dev, id};
    return dev;
  }

 private:
  struct Range {
    uintptr_t end;
    int device;
    uint64_t bufferId;
  };

  // Is the allocation at ptr still the one that was remembered?
  static bool stillThere(const void* ptr, uint64_t bufferId) {
    // TP_POINTER_RECHECK=0: believe remembered ranges for good (for measuring what the check costs)
    static const bool recheck = [] {
      const char* e = std::getenv("TP_POINTER_RECHECK");
      return e == nullptr || e[0] != '0';
    }();
    if (!recheck) {
      return true;
    }
    uint64_t id = 0;
    const bool same = tphip_mem_buffer_id(ptr, &id) == 0 && id != 0 && id == bufferId;
    PointerStats& stats = pointerStats();
    stats.checks.fetch_add(1, std::memory_order_relaxed);
    if (!same) {
      stats.stale.fetch_add(1, std::memory_order_relaxed);
    }
    return same;
  }

  void forget(uintptr_t begin) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (ranges_.erase(begin) != 0) {
      generation_.fetch_add(1, std::memory_order_acq_rel);
    }
  }

  std::mutex mutex_;
  std::map<uintptr_t, Range> ranges_;
  std::atomic<uint64_t> generation_{1};
};

} // namespace

int hipDeviceForPointer(const void* ptr) {
  static PointerRanges* ranges = new PointerRanges();
  return ranges->lookup(ptr);
}

void hipPointerCheckpoint() {
  PointerMemo& memo = tlsPointerMemo;
  if (memo.scopes == 0) {
    ++memo.epoch;
  }
}

HipPointerScope::HipPointerScope() {
  PointerMemo& memo = tlsPointerMemo;
  if (memo.scopes++ == 0) {
    ++memo.epoch;
  }
}

HipPointerScope::~HipPointerScope() {
  --tlsPointerMemo.scopes;
}

Device HipBuffer::getDevice() const {
  int dev = hipDeviceForPointer(ptr);
  TP_THROW_ASSERT_IF(dev < 0);
  return Device{kHipDeviceType, dev};
}

uint32_t HipBuffer::getDeviceKey() const {
  int dev = hipDeviceForPointer(ptr);
  TP_THROW_ASSERT_IF(dev < 0);
  return (2u << 16) | static_cast<uint32_t>(dev & 0xffff);
}

TP_AMD_NAMESPACE_END

#include <tensorpipe/common/stage_timer.h>

#include <cstdio>
#include <cstdlib>
#include <memory>

#include <pthread.h>
#include <unistd.h>

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

namespace {

struct Timeline {
  struct Mark {
    const char* what;
    uint64_t nanos;
    uint64_t thread;
  };
  size_t capacity{0};
  std::unique_ptr<Mark[]> marks;
  std::atomic<uint64_t> next{0};
  Timeline() {
    const char* e = std::getenv("TP_TIMELINE");
    capacity = e != nullptr ? static_cast<size_t>(std::atol(e)) : 0;
    if (capacity > 0) {
      marks.reset(new Mark[capacity]());
    }
  }
  ~Timeline() {
    if (capacity == 0) {
      return;
    }
    const uint64_t end = next.load();
    const uint64_t begin = end > capacity ? end - capacity : 0;
    uint64_t prev = 0;
    for (uint64_t i = begin; i < end; ++i) {
      const Mark& m = marks[i % capacity];
      if (m.what == nullptr) {
        continue;
      }
      std::fprintf(
          stderr, "[timeline %d] %12.2f us  +%8.2f  thread %04llx  %s\n", static_cast<int>(::getpid()),
          m.nanos / 1e3, prev == 0 ? 0.0 : (static_cast<double>(m.nanos) - static_cast<double>(prev)) / 1e3,
          static_cast<unsigned long long>(m.thread & 0xffff), m.what);
      prev = m.nanos;
    }
  }
};

Timeline& timeline() {
  static Timeline t;
  return t;
}

} // namespace

bool timelineEnabled() {
  return timeline().capacity != 0;
}

void timelineMark(const char* what) {
  Timeline& t = timeline();
  const uint64_t i = t.next.fetch_add(1, std::memory_order_relaxed);
  Timeline::Mark& m = t.marks[i % t.capacity];
  m.nanos = static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::nanoseconds>(
                                      std::chrono::steady_clock::now().time_since_epoch())
                                      .count());
  m.thread = static_cast<uint64_t>(reinterpret_cast<uintptr_t>(pthread_self()) >> 12);
  m.what = what;
}

bool stageStatsEnabled() {
  return stageTable().enabled;
}

void stageAdd(Stage s, uint64_t nanos) {
  StageTable& t = stageTable();
  t.nanos[static_cast<int>(s)].fetch_add(nanos, std::memory_order_relaxed);
  t.calls[static_cast<int>(s)].fetch_add(1, std::memory_order_relaxed);
}

TP_AMD_NAMESPACE_END
