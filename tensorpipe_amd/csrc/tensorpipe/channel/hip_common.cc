#include <tensorpipe/channel/hip_common.h>

#include <tensorpipe/common/loop.h>

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <fstream>
#include <random>
#include <sstream>

#include <unistd.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {

const std::string& bootIdentity() {
  static const std::string id = [] {
    std::ifstream f("/proc/sys/kernel/random/boot_id");
    std::string s;
    std::getline(f, s);
    return s;
  }();
  return id;
}

const std::string& processIdentity() {
  static const std::string id = [] {
    std::random_device rd;
    std::ostringstream ss;
    ss << bootIdentity() << "_" << ::getpid() << "_" << std::hex << rd() << rd();
    return ss.str();
  }();
  return id;
}

HipEventPoller::HipEventPoller() {
  thread_ = std::thread([this] { run(); });
}

HipEventPoller::~HipEventPoller() {
  join();
}

void HipEventPoller::watch(std::unique_ptr<HipEvent> event, HipEventPool* pool, TCallback fn) {
  {
    std::unique_lock<std::mutex> lock(mutex_);
    if (!stopping_) {
      incoming_.push_back(Item{std::move(event), nullptr, pool, std::move(fn)});
      incomingPending_.store(true, std::memory_order_release);
      lock.unlock();
      cv_.notify_one();
      return;
    }
  }
  // The thread is on its way out and may never look again: the caller waits
  // for the GPU itself. Every callback still runs exactly once.
  int rc = 0;
  for (int done = 0; rc == 0 && done == 0;) {
    rc = tphip_event_query(event->device(), event->raw(), &done);
    if (rc == 0 && done == 0) {
      std::this_thread::yield();
    }
  }
  fn(rc != 0 ? TP_CREATE_ERROR(HipError, "tphip_event_query", rc) : Error::kSuccess);
  if (pool != nullptr) {
    pool->put(std::move(event));
  }
}

void HipEventPoller::watchCondition(TCheck check, TCallback fn) {
  {
    std::unique_lock<std::mutex> lock(mutex_);
    if (!stopping_) {
      incoming_.push_back(Item{nullptr, std::move(check), nullptr, std::move(fn)});
      incomingPending_.store(true, std::memory_order_release);
      lock.unlock();
      cv_.notify_one();
      return;
    }
  }
  // Nobody is left to keep looking, and what is awaited may depend on a peer:
  // one look, then the operation fails.
  bool happened = false;
  const int rc = check(&happened);
  if (rc == 0 && happened) {
    fn(Error::kSuccess);
  } else {
    fn(TP_CREATE_ERROR(HipError, "completion check after the context was joined", rc != 0 ? rc : TPHIP_ERR_BUSY));
  }
}

void HipEventPoller::join() {
  {
    std::lock_guard<std::mutex> lock(mutex_);
    if (stopping_) {
      return;
    }
    stopping_ = true;
    incomingPending_.store(true, std::memory_order_release);
  }
  cv_.notify_one();
  if (thread_.joinable()) {
    thread_.join();
  }
}

namespace {
int pollGapNanos() {
  static const int v = [] {
    const char* e = std::getenv("TP_HIP_POLL_GAP_NS");
    return e != nullptr ? std::atoi(e) : 0;
  }();
  return v;
}
} // namespace

void HipEventPoller::run() {
  thisIsLibraryThread() = true;
  using Clock = std::chrono::steady_clock;
  std::deque<Item> active;
  auto lastBusy = Clock::now();
  const auto hot = std::chrono::microseconds(runsOnFewCpus() ? 0 : 300);
  for (;;) {
    // Idle and hot: watch one flag, leave the mutex to the threads that post.
    if (active.empty() && !incomingPending_.load(std::memory_order_acquire) &&
        Clock::now() - lastBusy < hot) {
#if defined(__x86_64__)
      __builtin_ia32_pause();
#endif
      continue;
    }
    {
      std::unique_lock<std::mutex> lock(mutex_);
      if (active.empty() && incoming_.empty() && !stopping_) {
        // Stay hot for a short while after the last event: in a ping-pong the
        // next one arrives within microseconds and a sleeping thread would add
        // its wake-up time to every transfer.
        if (Clock::now() - lastBusy < hot) {
          lock.unlock();
#if defined(__x86_64__)
          __builtin_ia32_pause();
#endif
          continue;
        }
        cv_.wait(lock, [this] { return stopping_ || !incoming_.empty(); });
      }
      while (!incoming_.empty()) {
        active.push_back(std::move(incoming_.front()));
        incoming_.pop_front();
      }
      incomingPending_.store(false, std::memory_order_relaxed);
      if (stopping_ && active.empty()) {
        return;
      }
    }
    bool any = false;
    for (auto it = active.begin(); it != active.end();) {
      int done = 0;
      int rc = 0;
      if (it->event) {
        rc = tphip_event_query(it->event->device(), it->event->raw(), &done);
      } else {
        bool happened = false;
        rc = it->check(&happened);
        done = happened ? 1 : 0;
      }
      if (rc != 0 || done) {
        Item item = std::move(*it);
        it = active.erase(it);
        any = true;
        if (rc != 0) {
          item.fn(TP_CREATE_ERROR(HipError, item.event ? "tphip_event_query" : "completion check", rc));
        } else {
          item.fn(Error::kSuccess);
        }
        if (item.pool != nullptr && item.event) {
          item.pool->put(std::move(item.event));
        }
      } else {
        ++it;
      }
    }
    if (any || !active.empty()) {
      lastBusy = Clock::now();
    }
    if (!any) {
      // Leave the runtime's locks alone for a moment between rounds: the
      // threads that launch the next copies need them too.
      if (runsOnFewCpus()) {
        // The copy's launcher and the callbacks' consumers need this CPU.
        ::sched_yield();
        continue;
      }
      const auto until = Clock::now() + std::chrono::nanoseconds(pollGapNanos());
      do {
#if defined(__x86_64__)
        __builtin_ia32_pause();
#endif
      } while (Clock::now() < until);
    }
  }
}

uint64_t nextExportId() {
  static std::atomic<uint64_t> next{1};
  return next.fetch_add(1, std::memory_order_relaxed);
}

HipIpcImports& HipIpcImports::get() {
  static HipIpcImports* r = new HipIpcImports();
  return *r;
}

int HipIpcImports::acquire(
    int device,
    const std::string& peer,
    uint64_t id,
    const HandleBytes& handle,
    uint64_t base,
    uint64_t size,
    void** out) {
  std::lock_guard<std::mutex> lock(mutex_);
  const Key key{device, peer, id};
  auto it = entries_.find(key);
  if (it != entries_.end() && it->second.mapped) {
    ++it->second.refs;
    *out = it->second.ptr;
    return 0;
  }
  // The same address range of the same process under another identifier:
  // stale, unmap before mapping anew.
  size_t staleClosed = 0;
  for (auto& kv : entries_) {
    if (std::get<0>(kv.first) == device && std::get<1>(kv.first) == peer && kv.second.mapped &&
        kv.second.base < base + size && base < kv.second.base + kv.second.size) {
      int crc = tphip_ipc_mem_close(device, kv.second.ptr);
      TP_VLOG(5) << "IPC imports: unmapped stale " << std::get<1>(kv.first) << "#"
                 << std::get<2>(kv.first) << " (rc " << crc << ") for #" << id;
      kv.second.mapped = false;
      kv.second.ptr = nullptr;
      ++staleClosed;
    }
  }
  void* ptr = nullptr;
  int rc = tphip_ipc_mem_open(device, handle.data(), &ptr);
  if (rc != 0) {
    TP_LOG_WARNING() << "IPC imports: cannot map " << peer << "#" << id << ": " << tphip_strerror(rc)
                     << " (" << entries_.size() << " entries, " << staleClosed
                     << " stale unmapped, re-acquire of a known id: " << (it != entries_.end()) << ")";
    return rc;
  }
  TP_VLOG(5) << "IPC imports: mapped " << peer << "#" << id << " at " << ptr;
  Entry& e = entries_[key];
  e.ptr = ptr;
  e.base = base;
  e.size = size;
  e.mapped = true;
  ++e.refs;
  *out = ptr;
  return 0;
}

void HipIpcImports::release(int device, const std::string& peer, uint64_t id) {
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = entries_.find(Key{device, peer, id});
  if (it == entries_.end()) {
    return;
  }
  if (it->second.refs > 0) {
    --it->second.refs;
  }
  if (it->second.refs == 0) {
    if (it->second.mapped) {
      tphip_ipc_mem_close(device, it->second.ptr);
    }
    entries_.erase(it);
  }
}

void hipBatchedCopy(int device, void* stream, const std::vector<tphip_copy_desc>& table) {
  size_t off = 0;
  while (off < table.size()) {
    const size_t n = table.size() - off < TPHIP_MAX_BATCH ? table.size() - off : TPHIP_MAX_BATCH;
    TP_HIP_CHECK(tphip_batched_copy(device, table.data() + off, static_cast<uint32_t>(n), stream));
    off += n;
  }
}

bool hipBatchedCopy(
    int device,
    void* stream,
    const std::vector<tphip_copy_desc>& table,
    HipEvent& done,
    bool signalOnKernel,
    uint32_t blocks,
    int nontemporal) {
  static const bool onKernel = [] {
    const char* e = std::getenv("TP_HIP_SIGNAL_ON_KERNEL");
    return e == nullptr || std::atoi(e) != 0;
  }();
  const bool tuned = blocks != 0 || nontemporal >= 0;
  if (!signalOnKernel || !onKernel || table.empty() || table.size() > TPHIP_MAX_BATCH ||
      done.device() != device) {
    size_t off = 0;
    while (off < table.size()) {
      const size_t n = std::min<size_t>(table.size() - off, TPHIP_MAX_BATCH);
      if (tuned) {
        TP_HIP_CHECK(tphip_batched_copy_tuned(
            device, table.data() + off, static_cast<uint32_t>(n), stream, 4, blocks,
            nontemporal < 0 ? 3 : nontemporal));
      } else {
        TP_HIP_CHECK(
            tphip_batched_copy(device, table.data() + off, static_cast<uint32_t>(n), stream));
      }
      off += n;
    }
    done.record(stream);
    return false;
  }
  TP_HIP_CHECK(tphip_batched_copy_signal(
      device, table.data(), static_cast<uint32_t>(table.size()), stream, done.raw(),
      tuned ? 4 : 0, blocks, nontemporal));
  return true;
}

} // namespace channel
TP_AMD_NAMESPACE_END
