// Pieces shared by the three HIP channels: the process identity used in
// device descriptors, a completion poller for HIP events, and the helper that
// turns a list of (src, dst, bytes) into ONE batched copy launch.
#pragma once

#include <array>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <atomic>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <tuple>
#include <vector>

#include <tensorpipe/common/error.h>
#include <tensorpipe/common/hip_api.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {

// "<boot id>_<pid>_<nonce>": equal in two contexts iff they live in the same
// process (tensorpipe/channel/cuda_xth/context_impl.cc:28-73 builds the same
// kind of string from boot id, pid namespace and pid).
const std::string& processIdentity();
// "<boot id>": equal iff same machine boot.
const std::string& bootIdentity();

// Thread that watches HIP events and runs a callback once an event's captured
// work has finished. Replaces the stream-callback thread of the reference
// (tensorpipe/common/cuda_loop.cc:62-124) with event polling, which completes
// within a microsecond or two of the GPU instead of a runtime callback hop.
// Callbacks run on the poller thread and must hop to their own loop.
class HipEventPoller {
 public:
  using TCallback = std::function<void(const Error&)>;

  HipEventPoller();
  ~HipEventPoller();

  // `event` must have been recorded already; ownership moves to the poller
  // until the callback has run, then back to `pool` (if given).
  void watch(std::unique_ptr<HipEvent> event, HipEventPool* pool, TCallback fn);

  // The same for anything else the host can only find out by looking: a
  // signal word in shared pinned memory, a ticket of the copy agent. `check`
  // sets *done once the awaited thing has happened and returns 0, or returns a
  // tphip error code; it runs on the poller thread, again and again.
  using TCheck = std::function<int(bool* done)>;
  void watchCondition(TCheck check, TCallback fn);

  void join();

 private:
  struct Item {
    std::unique_ptr<HipEvent> event; // or
    TCheck check;
    HipEventPool* pool;
    TCallback fn;
  };

  void run();

  std::mutex mutex_;
  std::condition_variable cv_;
  std::deque<Item> incoming_;
  // Set whenever incoming_ may be non-empty or the thread must look at stopping_.
  std::atomic<bool> incomingPending_{false};
  bool stopping_{false};
  std::thread thread_;
};

using HandleBytes = std::array<uint8_t, TPHIP_IPC_HANDLE_BYTES>;

// Process-wide identifiers for things this process exports to peers (tensor
// allocations, staging slabs, pinned rings). A peer keys its mapping on
// (exporting process, identifier), never on the handle bytes: an address that
// is freed and handed out again may come with the very same handle.
uint64_t nextExportId();

// Mappings of peer memory, shared by the channels of this process and counted:
// every acquire() is paired with a release(), the last one unmaps. Mapping a
// handle costs a few hundred microseconds, so a mapping lives as long as any
// channel uses it.
class HipIpcImports {
 public:
  static HipIpcImports& get();
  // `peer` is the exporter's processIdentity(), `id` its nextExportId() value
  // for the allocation, `handle` what tphip_ipc_mem_export gave it, `base` and
  // `size` the allocation's address range in the exporter. Returns a tphip
  // error code. An older mapping from the same process whose range overlaps
  // the new one belongs to memory the exporter has freed since (two live
  // allocations of a process never overlap) and is unmapped first; the handle
  // bytes themselves cannot tell, their tail differs from one export of the
  // same allocation to the next.
  int acquire(
      int device,
      const std::string& peer,
      uint64_t id,
      const HandleBytes& handle,
      uint64_t base,
      uint64_t size,
      void** out);
  void release(int device, const std::string& peer, uint64_t id);

 private:
  struct Entry {
    void* ptr{nullptr};
    uint64_t base{0};
    uint64_t size{0};
    size_t refs{0};
    bool mapped{false};
  };
  using Key = std::tuple<int, std::string, uint64_t>;
  std::mutex mutex_;
  std::map<Key, Entry> entries_;
};

// "Is there anything pending on this stream?", asked only while asking is
// cheap. hipStreamQuery answers in about 0.1 us when the last thing on the
// stream was an event marker that has completed (a ping-pong through these
// channels: the stream's last work was the channel's own copy and marker), and
// lets a channel skip an event round trip of about 10 us. When the last thing
// was a kernel -- finished or not -- the runtime has to enqueue a marker of
// its own to find out: the call takes about 12 us and answers "busy" anyway.
// A stream whose query turned out slow and said "busy" is therefore treated as
// busy, without asking, for the next 63 calls. Use from one loop.
class StreamIdleProbe {
 public:
  bool idle(int device, void* stream) {
    if (states_.size() > 256) {
      states_.clear(); // streams come and go; what is remembered here is only a hint
    }
    State& st = states_[std::make_pair(device, stream)];
    if (st.skip > 0) {
      --st.skip;
      return false;
    }
    const auto t0 = std::chrono::steady_clock::now();
    int idle = 0;
    const int rc = tphip_stream_query(device, stream, &idle);
    const auto took = std::chrono::steady_clock::now() - t0;
    const bool isIdle = rc == 0 && idle != 0;
    if (!isIdle && took > std::chrono::microseconds(6)) {
      st.skip = skipCount();
    }
    return isIdle;
  }

 private:
  // TP_HIP_IDLE_PROBE_SKIP: calls answered "busy" without asking after a slow
  // query (default 63; 0 asks every time).
  static uint32_t skipCount() {
    static const uint32_t v = [] {
      const char* e = std::getenv("TP_HIP_IDLE_PROBE_SKIP");
      return e != nullptr ? static_cast<uint32_t>(std::atoi(e)) : 63u;
    }();
    return v;
  }
  struct State {
    uint32_t skip{0};
  };
  std::map<std::pair<int, void*>, State> states_;
};

// Enqueue one batched copy on (device, stream); throws on a failed launch.
void hipBatchedCopy(int device, void* stream, const std::vector<tphip_copy_desc>& table);

// The same, and `done` is recorded behind the copy. With `signalOnKernel` the
// event is the completion signal of the copy kernel itself where possible: a
// polling host sees it about 2.5 us sooner than a marker enqueued after the
// kernel. Returns true when that is what happened. A marker must then still
// follow on the stream at some point: after a kernel without one the runtime
// does not know when the stream has drained, and the next hipStreamQuery or
// hipStreamSynchronize on it (the user's, or a channel's idle check) takes
// 12-20 us instead of 0.1. StreamMarkers below decides when. Channels that ask a
// stream whether it is idle right after their own copy (hip_ipc, before
// announcing a tensor) pass false and poll a marker, recorded at once.
// TP_HIP_SIGNAL_ON_KERNEL=0 does that everywhere. `blocks` workgroups (0 = the
// library's choice) and `nontemporal` mask (-1 = the library's choice) as for
// tphip_batched_copy_tuned.
bool hipBatchedCopy(
    int device,
    void* stream,
    const std::vector<tphip_copy_desc>& table,
    HipEvent& done,
    bool signalOnKernel,
    uint32_t blocks = 0,
    int nontemporal = -1);

// When the marker behind a kernel whose own signal is polled gets recorded. On
// a quiet stream: at once, right behind the kernel, off everybody's path (the
// kernel is still running). When the stream already has an unfinished copy of
// ours in front -- several transfers in flight -- not yet: a marker between
// two queued kernels would only hold the second one back (24-26 us instead of
// ~21 per 64 MiB copy); the thread that sees the kernel finish records it
// then, if nothing newer has been launched on the stream meanwhile. Shared
// between the loop (launched) and the poller thread (finished).
class StreamMarkers {
 public:
  struct Launch {
    uint64_t id{0};
    bool markerOwed{false}; // not recorded at launch: due when the kernel has finished
  };

  // Loop: a kernel without a marker behind it has just been launched.
  Launch launched(int device, void* stream, HipEventPool& pool) {
    Launch l;
    {
      std::lock_guard<std::mutex> lock(mutex_);
      if (streams_.size() > 256) {
        for (auto it = streams_.begin(); it != streams_.end();) {
          it = it->second.outstanding == 0 ? streams_.erase(it) : std::next(it);
        }
      }
      State& st = streams_[std::make_pair(device, stream)];
      l.id = ++st.last;
      l.markerOwed = st.outstanding > 0;
      ++st.outstanding;
    }
    if (!l.markerOwed) {
      record(device, stream, pool);
    }
    return l;
  }

  // Any thread: that kernel has finished.
  void finished(int device, void* stream, const Launch& l, HipEventPool& pool) {
    bool due = false;
    {
      std::lock_guard<std::mutex> lock(mutex_);
      auto it = streams_.find(std::make_pair(device, stream));
      if (it != streams_.end()) {
        if (it->second.outstanding > 0) {
          --it->second.outstanding;
        }
        due = l.markerOwed && it->second.last == l.id;
      }
    }
    if (due) {
      record(device, stream, pool);
    }
  }

 private:
  static void record(int device, void* stream, HipEventPool& pool) {
    try {
      auto marker = pool.get(device, stream);
      marker->record(stream);
      pool.put(std::move(marker)); // nobody waits for it
    } catch (const std::exception&) {
      // without the marker the next query of the stream is slow, nothing more
    }
  }

  struct State {
    uint64_t last{0};
    uint32_t outstanding{0};
  };
  std::mutex mutex_;
  std::map<std::pair<int, void*>, State> streams_;
};

} // namespace channel
TP_AMD_NAMESPACE_END
