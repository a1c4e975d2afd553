// A host-only stand-in for libtphip.so: the same C ABI (include/tphip.h) with
// no GPU behind it, so that the host logic of the three device channels --
// loops, state machines, control messages, slot rings, signal words -- can run
// on the CPU, under ThreadSanitizer / AddressSanitizer and inside a stock
// TensorPipe, where no GPU is present. Test infrastructure only: nothing in
// the product links against it; the C++ test programs pick it up when
// LD_LIBRARY_PATH puts its directory ahead of the real library's.
//
//  "device" memory and "pinned" memory are anonymous shared-memory files
//      (memfd): an inter-process handle names the owner's descriptor, the
//      opening process maps the same pages at an address of its own, as a real
//      handle does. Nothing is left behind in /dev/shm when a process dies.
//  a stream is a thread with a queue: work runs in order, asynchronously to
//      the caller, and overlaps with other streams. The null stream is a
//      stream like any other.
//  an event completes when the stream reaches the marker its record() queued.
//  copies are memcpy on the stream's thread; the gate, the signal word and the
//      copy agent follow the rules stated in tphip.h (bounded wait, words
//      raised behind the work, notify behind the copy).
//
// One device (index 0). Every pointer handed to a copy must lie in an
// allocation made or opened here or be plain host memory of the caller's; a
// copy that touches an allocation after it was freed aborts with a message,
// which is the closest a CPU run comes to a GPU memory fault.
#include <tphip.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include <fcntl.h>
#include <sys/mman.h>
#include <unistd.h>

namespace {

using Clock = std::chrono::steady_clock;

// ---- allocations ---------------------------------------------------------------

struct Allocation {
  uint8_t* base{nullptr};
  size_t size{0};
  size_t mapped{0};
  uint64_t id{0};
  bool host{false};
  bool imported{false};
  int fd{-1};
};

std::mutex gAllocMutex;
std::map<uintptr_t, Allocation> gAllocs; // by base address
std::atomic<uint64_t> gNextBufferId{1};

size_t roundUp(size_t v, size_t to) {
  return (v + to - 1) / to * to;
}

// mutex held
Allocation* findLocked(const void* ptr) {
  const uintptr_t p = reinterpret_cast<uintptr_t>(ptr);
  auto it = gAllocs.upper_bound(p);
  if (it == gAllocs.begin()) {
    return nullptr;
  }
  --it;
  if (p < it->first + it->second.mapped) {
    return &it->second;
  }
  return nullptr;
}

int allocate(size_t bytes, bool host, void** out) {
  if (out == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  const size_t mapped = roundUp(bytes == 0 ? 1 : bytes, 4096);
  const int fd = ::memfd_create(host ? "tphip_fake_pinned" : "tphip_fake_device", MFD_CLOEXEC);
  if (fd < 0 || ::ftruncate(fd, static_cast<off_t>(mapped)) != 0) {
    if (fd >= 0) {
      ::close(fd);
    }
    return 2; // hipErrorOutOfMemory
  }
  void* p = ::mmap(nullptr, mapped, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  if (p == MAP_FAILED) {
    ::close(fd);
    return 2;
  }
  Allocation a;
  a.base = static_cast<uint8_t*>(p);
  a.size = bytes;
  a.mapped = mapped;
  a.id = gNextBufferId++;
  a.host = host;
  a.fd = fd;
  std::lock_guard<std::mutex> lock(gAllocMutex);
  gAllocs[reinterpret_cast<uintptr_t>(p)] = a;
  *out = p;
  return 0;
}

int release(void* ptr, bool wantImported) {
  Allocation a;
  {
    std::lock_guard<std::mutex> lock(gAllocMutex);
    auto it = gAllocs.find(reinterpret_cast<uintptr_t>(ptr));
    if (it == gAllocs.end() || it->second.imported != wantImported) {
      return 1; // hipErrorInvalidValue
    }
    a = it->second;
    gAllocs.erase(it);
  }
  // The pages stay mapped, unreadable: a late copy faults loudly instead of
  // scribbling over whatever the address is handed to next.
  ::mprotect(a.base, a.mapped, PROT_NONE);
  if (a.fd >= 0) {
    ::close(a.fd);
  }
  return 0;
}

struct WireHandle { // fits TPHIP_IPC_HANDLE_BYTES
  uint32_t magic;
  int32_t pid;
  int32_t fd;
  uint32_t pad;
  uint64_t mapped;
  uint64_t size;
  uint64_t id;
  uint64_t host;
};
static_assert(sizeof(WireHandle) <= TPHIP_IPC_HANDLE_BYTES, "handle too large");
constexpr uint32_t kMagic = 0x7fa4e001u;

// ---- streams -------------------------------------------------------------------

class Stream {
 public:
  Stream() {
    thread_ = std::thread([this] { run(); });
  }
  ~Stream() {
    {
      std::lock_guard<std::mutex> lock(m_);
      stop_ = true;
    }
    cv_.notify_all();
    thread_.join();
  }
  void push(std::function<void()> fn) {
    {
      std::lock_guard<std::mutex> lock(m_);
      q_.push_back(std::move(fn));
      ++queued_;
    }
    cv_.notify_all();
  }
  bool idle() {
    std::lock_guard<std::mutex> lock(m_);
    return done_ == queued_;
  }
  void sync() {
    std::unique_lock<std::mutex> lock(m_);
    const uint64_t target = queued_;
    idleCv_.wait(lock, [&] { return done_ >= target; });
  }

 private:
  void run() {
    std::unique_lock<std::mutex> lock(m_);
    for (;;) {
      cv_.wait(lock, [this] { return stop_ || !q_.empty(); });
      if (q_.empty()) {
        return;
      }
      auto fn = std::move(q_.front());
      q_.pop_front();
      lock.unlock();
      fn();
      fn = nullptr;
      lock.lock();
      ++done_;
      idleCv_.notify_all();
    }
  }
  std::mutex m_;
  std::condition_variable cv_, idleCv_;
  std::deque<std::function<void()>> q_;
  uint64_t queued_{0}, done_{0};
  bool stop_{false};
  std::thread thread_;
};

// Never destroyed: work may still be queued when static destructors run.
Stream& nullStream() {
  static Stream* s = new Stream();
  return *s;
}

Stream& streamOf(void* handle) {
  return handle == nullptr ? nullStream() : *static_cast<Stream*>(handle);
}

// ---- events --------------------------------------------------------------------

struct EventState {
  std::mutex m;
  std::condition_variable cv;
  uint64_t recorded{0};
  uint64_t completed{0};
  Clock::time_point when{};
};

// An event may be destroyed while a stream still has its marker queued, as
// with the real runtime: the queued work holds the state alive.
using EventRef = std::shared_ptr<EventState>;
struct Event {
  EventRef state{std::make_shared<EventState>()};
};

EventRef ref(void* event) {
  return event != nullptr ? static_cast<Event*>(event)->state : nullptr;
}

// ---- copies --------------------------------------------------------------------

[[noreturn]] void fault(const char* what, const void* p, uint64_t n) {
  std::fprintf(stderr, "fake tphip: memory access fault: %s %p (+%llu bytes) is not in a live allocation\n",
               what, p, static_cast<unsigned long long>(n));
  std::fflush(stderr);
  std::abort();
}

// Plain host memory of the caller's is fine (tests read results into it);
// what lies inside a known allocation must not run past its end.
void checkRange(const char* what, const void* p, uint64_t n) {
  if (n == 0) {
    return;
  }
  std::lock_guard<std::mutex> lock(gAllocMutex);
  Allocation* a = findLocked(p);
  if (a != nullptr) {
    const uintptr_t off = reinterpret_cast<uintptr_t>(p) - reinterpret_cast<uintptr_t>(a->base);
    if (off + n > a->mapped) {
      fault(what, p, n);
    }
  }
}

std::vector<tphip_copy_desc> snapshot(const tphip_copy_desc* table, uint32_t n) {
  std::vector<tphip_copy_desc> t;
  for (uint32_t i = 0; i < n; ++i) {
    if (table[i].bytes != 0) {
      t.push_back(table[i]);
    }
  }
  return t;
}

void runCopies(const std::vector<tphip_copy_desc>& t) {
  for (const auto& d : t) {
    checkRange("source", d.src, d.bytes);
    checkRange("destination", d.dst, d.bytes);
    std::memcpy(d.dst, d.src, d.bytes);
  }
}

void completeEvent(const EventRef& ev, uint64_t seq) {
  std::lock_guard<std::mutex> lock(ev->m);
  if (seq > ev->completed) {
    ev->completed = seq;
    ev->when = Clock::now();
  }
  ev->cv.notify_all();
}

uint64_t beginRecord(const EventRef& ev) {
  std::lock_guard<std::mutex> lock(ev->m);
  return ++ev->recorded;
}

std::atomic<uint64_t>* word(void* p) {
  return reinterpret_cast<std::atomic<uint64_t>*>(p);
}
const std::atomic<uint64_t>* word(const void* p) {
  return reinterpret_cast<const std::atomic<uint64_t>*>(p);
}

// ---- the copy agent -------------------------------------------------------------

struct Agent {
  static constexpr uint64_t kRing = 64;
  struct Command {
    tphip_copy_desc d;
    void* notify;
    uint64_t value;
  };
  std::mutex m;
  std::condition_variable cv;
  std::deque<Command> q;
  uint64_t next{1};
  std::atomic<uint64_t> done{0};
  bool stop{false};
  std::thread thread;

  Agent() {
    thread = std::thread([this] {
      std::unique_lock<std::mutex> lock(m);
      for (;;) {
        cv.wait(lock, [this] { return stop || !q.empty(); });
        if (q.empty()) {
          return;
        }
        Command c = q.front();
        q.pop_front();
        lock.unlock();
        runCopies({c.d});
        if (c.notify != nullptr) {
          word(c.notify)->store(c.value, std::memory_order_release);
        }
        done.fetch_add(1, std::memory_order_release);
        lock.lock();
      }
    });
  }
};

} // namespace

extern "C" {

const char* tphip_strerror(int err) {
  switch (err) {
    case 0:
      return "success";
    case TPHIP_ERR_INVALID_ARG:
      return "invalid argument";
    case TPHIP_ERR_TOO_LARGE:
      return "too large";
    case TPHIP_ERR_NO_DEVICE:
      return "no such device";
    case TPHIP_ERR_CAPTURING:
      return "stream is capturing";
    case TPHIP_ERR_BUSY:
      return "busy";
    default:
      return "error of the stand-in runtime";
  }
}

int tphip_device_count(int* count) {
  if (count == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  *count = 1;
  return 0;
}

int tphip_device_uuid(int dev, char out[TPHIP_UUID_STRLEN + 1]) {
  if (dev != 0) {
    return TPHIP_ERR_NO_DEVICE;
  }
  std::snprintf(out, TPHIP_UUID_STRLEN + 1, "%s", "fa4efa4e-0000-4000-8000-00000000cafe");
  return 0;
}

int tphip_device_for_ptr(const void* ptr, int* dev, int* is_host) {
  if (dev == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  std::lock_guard<std::mutex> lock(gAllocMutex);
  Allocation* a = findLocked(ptr);
  if (a == nullptr) {
    *dev = -1;
    if (is_host != nullptr) {
      *is_host = 1;
    }
    return 0;
  }
  *dev = 0;
  if (is_host != nullptr) {
    *is_host = a->host ? 1 : 0;
  }
  return 0;
}

int tphip_mem_base(const void* ptr, void** base, size_t* size) {
  std::lock_guard<std::mutex> lock(gAllocMutex);
  Allocation* a = findLocked(ptr);
  if (a == nullptr) {
    return 1;
  }
  if (base != nullptr) {
    *base = a->base;
  }
  if (size != nullptr) {
    *size = a->size;
  }
  return 0;
}

int tphip_mem_buffer_id(const void* ptr, uint64_t* id) {
  if (id == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  std::lock_guard<std::mutex> lock(gAllocMutex);
  Allocation* a = findLocked(ptr);
  *id = a != nullptr ? a->id : 0;
  return 0;
}

int tphip_malloc(int dev, size_t bytes, void** ptr) {
  return dev != 0 ? TPHIP_ERR_NO_DEVICE : allocate(bytes, false, ptr);
}

int tphip_free(int dev, void* ptr) {
  return ptr == nullptr ? 0 : release(ptr, false);
}

int tphip_host_alloc(int dev, size_t bytes, void** host_ptr, void** dev_ptr) {
  if (dev != 0) {
    return TPHIP_ERR_NO_DEVICE;
  }
  const int rc = allocate(bytes, true, host_ptr);
  if (rc == 0 && dev_ptr != nullptr) {
    *dev_ptr = *host_ptr;
  }
  return rc;
}

int tphip_host_free(void* host_ptr) {
  return host_ptr == nullptr ? 0 : release(host_ptr, false);
}

int tphip_stream_create(int dev, void** stream) {
  if (dev != 0 || stream == nullptr) {
    return TPHIP_ERR_NO_DEVICE;
  }
  *stream = new Stream();
  return 0;
}

int tphip_stream_destroy(int dev, void* stream) {
  delete static_cast<Stream*>(stream);
  return 0;
}

int tphip_stream_sync(int dev, void* stream) {
  streamOf(stream).sync();
  return 0;
}

int tphip_stream_query(int dev, void* stream, int* done) {
  *done = streamOf(stream).idle() ? 1 : 0;
  return 0;
}

int tphip_event_create(int dev, int interprocess, void** event) {
  if (dev != 0 || event == nullptr) {
    return TPHIP_ERR_NO_DEVICE;
  }
  *event = new Event();
  return 0;
}

int tphip_event_create_timed(int dev, void** event) {
  return tphip_event_create(dev, 0, event);
}

int tphip_event_destroy(int dev, void* event) {
  delete static_cast<Event*>(event);
  return 0;
}

int tphip_event_record(int dev, void* event, void* stream) {
  auto ev = ref(event);
  const uint64_t seq = beginRecord(ev);
  streamOf(stream).push([ev, seq] { completeEvent(ev, seq); });
  return 0;
}

int tphip_stream_wait_event(int dev, void* stream, void* event) {
  auto ev = ref(event);
  uint64_t target;
  {
    std::lock_guard<std::mutex> lock(ev->m);
    target = ev->recorded;
  }
  if (target == 0) {
    return 0;
  }
  streamOf(stream).push([ev, target] {
    std::unique_lock<std::mutex> lock(ev->m);
    ev->cv.wait(lock, [&] { return ev->completed >= target; });
  });
  return 0;
}

int tphip_event_query(int dev, void* event, int* done) {
  auto ev = ref(event);
  std::lock_guard<std::mutex> lock(ev->m);
  *done = ev->completed >= ev->recorded ? 1 : 0;
  return 0;
}

int tphip_event_sync(int dev, void* event) {
  auto ev = ref(event);
  std::unique_lock<std::mutex> lock(ev->m);
  const uint64_t target = ev->recorded;
  ev->cv.wait(lock, [&] { return ev->completed >= target; });
  return 0;
}

int tphip_event_elapsed_ms(void* start, void* stop, float* ms) {
  auto a = ref(start);
  auto b = ref(stop);
  *ms = std::chrono::duration<float, std::milli>(b->when - a->when).count();
  return 0;
}

int tphip_stream_on_complete(int dev, void* stream, tphip_host_fn fn, void* arg) {
  streamOf(stream).push([fn, arg] { fn(arg, 0); });
  return 0;
}

int tphip_ipc_mem_export(int dev, void* base, uint8_t out[TPHIP_IPC_HANDLE_BYTES]) {
  std::lock_guard<std::mutex> lock(gAllocMutex);
  auto it = gAllocs.find(reinterpret_cast<uintptr_t>(base));
  if (it == gAllocs.end() || it->second.imported) {
    return 1;
  }
  WireHandle h{};
  h.magic = kMagic;
  h.pid = static_cast<int32_t>(::getpid());
  h.fd = it->second.fd;
  h.mapped = it->second.mapped;
  h.size = it->second.size;
  h.id = it->second.id;
  h.host = it->second.host ? 1 : 0;
  std::memset(out, 0, TPHIP_IPC_HANDLE_BYTES);
  std::memcpy(out, &h, sizeof(h));
  return 0;
}

int tphip_ipc_mem_open(int dev, const uint8_t handle[TPHIP_IPC_HANDLE_BYTES], void** ptr) {
  WireHandle h;
  std::memcpy(&h, handle, sizeof(h));
  if (h.magic != kMagic || ptr == nullptr) {
    return 1;
  }
  if (h.pid == static_cast<int32_t>(::getpid())) {
    return 1; // a process cannot open its own handle (hipErrorInvalidValue / context)
  }
  char path[64];
  std::snprintf(path, sizeof(path), "/proc/%d/fd/%d", h.pid, h.fd);
  const int fd = ::open(path, O_RDWR | O_CLOEXEC);
  if (fd < 0) {
    return 17; // hipErrorInvalidDevicePointer: the exporter is gone or freed it
  }
  void* p = ::mmap(nullptr, h.mapped, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  if (p == MAP_FAILED) {
    ::close(fd);
    return 2;
  }
  Allocation a;
  a.base = static_cast<uint8_t*>(p);
  a.size = h.size;
  a.mapped = h.mapped;
  a.id = gNextBufferId++;
  a.host = h.host != 0;
  a.imported = true;
  a.fd = fd;
  std::lock_guard<std::mutex> lock(gAllocMutex);
  gAllocs[reinterpret_cast<uintptr_t>(p)] = a;
  *ptr = p;
  return 0;
}

int tphip_ipc_mem_close(int dev, void* ptr) {
  return release(ptr, true);
}

int tphip_ipc_event_export(int dev, void* event, uint8_t out[TPHIP_IPC_HANDLE_BYTES]) {
  return 1; // refused, as on the machines this library is deployed on
}

int tphip_ipc_event_open(int dev, const uint8_t handle[TPHIP_IPC_HANDLE_BYTES], void** event) {
  return 1;
}

int tphip_batched_copy_signal(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                              void* event, int unroll, uint32_t blocks, int nontemporal) {
  if (dev != 0) {
    return TPHIP_ERR_NO_DEVICE;
  }
  if (n > TPHIP_MAX_BATCH) {
    return TPHIP_ERR_TOO_LARGE;
  }
  auto t = snapshot(table, n);
  auto ev = ref(event);
  const uint64_t seq = ev != nullptr ? beginRecord(ev) : 0;
  if (t.empty() && ev == nullptr) {
    return 0;
  }
  streamOf(stream).push([t{std::move(t)}, ev, seq] {
    runCopies(t);
    if (ev != nullptr) {
      completeEvent(ev, seq);
    }
  });
  return 0;
}

int tphip_batched_copy(int dev, const tphip_copy_desc* table, uint32_t n, void* stream) {
  return tphip_batched_copy_signal(dev, table, n, stream, nullptr, 0, 0, -1);
}

int tphip_batched_copy_noalloc(int dev, const tphip_copy_desc* table, uint32_t n, void* stream) {
  if (n > TPHIP_NOALLOC_MAX_BATCH) {
    return TPHIP_ERR_TOO_LARGE;
  }
  return tphip_batched_copy_signal(dev, table, n, stream, nullptr, 0, 0, -1);
}

int tphip_batched_copy_tuned(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                             int unroll, uint32_t blocks, int nontemporal) {
  return tphip_batched_copy_signal(dev, table, n, stream, nullptr, unroll, blocks, nontemporal);
}

int tphip_copy(int dev, void* dst, const void* src, uint64_t bytes, void* stream) {
  tphip_copy_desc d{src, dst, bytes};
  return tphip_batched_copy(dev, &d, 1, stream);
}

int tphip_memcpy_async(int dev, void* dst, const void* src, uint64_t bytes, void* stream) {
  return tphip_copy(dev, dst, src, bytes, stream);
}

int tphip_stream_signal(int dev, void* stream, void* w, uint64_t value) {
  if (w == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  streamOf(stream).push([w, value] { word(w)->store(value, std::memory_order_release); });
  return 0;
}

int tphip_batched_copy_gated(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                             void* event, const void* gate_word, uint64_t gate_value,
                             uint32_t max_wait_us, void* expired_word) {
  if (dev != 0 || gate_word == nullptr || expired_word == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  auto t = snapshot(table, n);
  auto ev = ref(event);
  const uint64_t seq = ev != nullptr ? beginRecord(ev) : 0;
  streamOf(stream).push([t{std::move(t)}, ev, seq, gate_word, gate_value, max_wait_us, expired_word] {
    const auto until = Clock::now() + std::chrono::microseconds(max_wait_us);
    bool open = false;
    for (;;) {
      if (word(gate_word)->load(std::memory_order_acquire) >= gate_value) {
        open = true;
        break;
      }
      if (Clock::now() > until) {
        break;
      }
      std::this_thread::yield();
    }
    if (open) {
      runCopies(t);
    } else {
      word(expired_word)->store(1, std::memory_order_release);
    }
    if (ev != nullptr) {
      completeEvent(ev, seq);
    }
  });
  return 0;
}

int tphip_agent_create(int dev, void** agent) {
  if (dev != 0 || agent == nullptr) {
    return TPHIP_ERR_NO_DEVICE;
  }
  *agent = new Agent();
  return 0;
}

int tphip_agent_destroy(void* agent) {
  auto* a = static_cast<Agent*>(agent);
  if (a == nullptr) {
    return 0;
  }
  {
    std::lock_guard<std::mutex> lock(a->m);
    a->stop = true;
  }
  a->cv.notify_all();
  a->thread.join(); // serves what is queued first
  delete a;
  return 0;
}

int tphip_agent_submit(void* agent, const tphip_copy_desc* table, uint32_t n, void* notify,
                       uint64_t notify_value, uint64_t* ticket) {
  auto* a = static_cast<Agent*>(agent);
  if (a == nullptr || table == nullptr || n == 0 || n > 32 || ticket == nullptr ||
      notify_value >= (uint64_t(1) << 48)) {
    return TPHIP_ERR_INVALID_ARG;
  }
  auto t = snapshot(table, n);
  if (t.empty()) {
    return TPHIP_ERR_INVALID_ARG;
  }
  std::lock_guard<std::mutex> lock(a->m);
  if (a->stop) {
    return TPHIP_ERR_INVALID_ARG;
  }
  const uint64_t outstanding = (a->next - 1) - a->done.load(std::memory_order_acquire);
  if (outstanding + t.size() > Agent::kRing) {
    return TPHIP_ERR_BUSY;
  }
  for (size_t i = 0; i < t.size(); ++i) {
    const bool last = i + 1 == t.size();
    a->q.push_back(Agent::Command{t[i], last ? notify : nullptr, notify_value});
    *ticket = a->next++;
  }
  a->cv.notify_all();
  return 0;
}

int tphip_agent_done(void* agent, uint64_t ticket, int* done) {
  auto* a = static_cast<Agent*>(agent);
  if (a == nullptr || done == nullptr) {
    return TPHIP_ERR_INVALID_ARG;
  }
  *done = a->done.load(std::memory_order_acquire) >= ticket ? 1 : 0;
  return 0;
}

size_t tphip_ring_scratch_bytes(uint32_t num_slots) {
  return 256;
}

} // extern "C"

namespace {

// The ring kernels of the real library, one chunk after the other on the
// stream's thread: wait (bounded) for the other side's counter, copy, raise
// this side's. The scratch holds what this end has completed, as the kernels
// keep it.
int ringTransfer(bool push, const tphip_ring_end* ring, const void* user, uint64_t bytes,
                 uint64_t firstSeq, uint32_t yieldUs, void* stream, void* event) {
  if (ring == nullptr || ring->slots == nullptr || ring->slot_bytes == 0 || ring->slot_bytes % 16 != 0 ||
      ring->num_slots == 0 || ring->produced == nullptr || ring->consumed == nullptr ||
      ring->scratch == nullptr || ring->status == nullptr || ring->abort == nullptr || user == nullptr ||
      bytes == 0) {
    return TPHIP_ERR_INVALID_ARG;
  }
  const tphip_ring_end r = *ring;
  auto ev = ref(event);
  const uint64_t evSeq = ev != nullptr ? beginRecord(ev) : 0;
  streamOf(stream).push([=] {
    auto* published = word(r.scratch);
    const auto* awaited = word(push ? r.consumed : r.produced);
    auto* raised = word(push ? r.produced : r.consumed);
    const uint64_t nChunks = (bytes + r.slot_bytes - 1) / r.slot_bytes;
    bool yielded = false;
    for (uint64_t k = 0; k < nChunks && !yielded; ++k) {
      const uint64_t seq = firstSeq + k;
      const uint64_t slot = seq % r.num_slots;
      const uint64_t need = push ? (seq >= r.num_slots ? seq - r.num_slots + 1 : 0) : seq + 1;
      const auto until = Clock::now() + std::chrono::microseconds(yieldUs);
      while (awaited->load(std::memory_order_acquire) < need) {
        if (Clock::now() > until || word(r.abort)->load(std::memory_order_acquire) != 0) {
          yielded = true;
          break;
        }
        std::this_thread::yield();
      }
      if (yielded) {
        break;
      }
      const uint64_t off = k * r.slot_bytes;
      const uint64_t len = std::min<uint64_t>(bytes - off, r.slot_bytes);
      char* slotPtr = static_cast<char*>(r.slots) + slot * r.slot_bytes;
      char* userPtr = static_cast<char*>(const_cast<void*>(user)) + off;
      runCopies({push ? tphip_copy_desc{userPtr, slotPtr, len} : tphip_copy_desc{slotPtr, userPtr, len}});
      if (published->load(std::memory_order_relaxed) != seq) {
        std::fprintf(stderr, "fake tphip: ring call out of sequence (%llu complete, chunk %llu)\n",
                     static_cast<unsigned long long>(published->load()), static_cast<unsigned long long>(seq));
        std::abort();
      }
      published->store(seq + 1, std::memory_order_relaxed);
      raised->store(seq + 1, std::memory_order_release);
    }
    word(r.status)->store(published->load(std::memory_order_relaxed) | (yielded ? TPHIP_RING_YIELDED : 0),
                          std::memory_order_release);
    if (ev != nullptr) {
      completeEvent(ev, evSeq);
    }
  });
  return 0;
}

} // namespace

extern "C" {

int tphip_ring_push(int dev, const tphip_ring_end* ring, const void* src, uint64_t bytes,
                    uint64_t first_seq, uint32_t yield_us, uint32_t blocks, void* stream, void* event) {
  return dev != 0 ? TPHIP_ERR_NO_DEVICE : ringTransfer(true, ring, src, bytes, first_seq, yield_us, stream, event);
}

int tphip_ring_pull(int dev, const tphip_ring_end* ring, void* dst, uint64_t bytes,
                    uint64_t first_seq, uint32_t yield_us, uint32_t blocks, void* stream, void* event) {
  return dev != 0 ? TPHIP_ERR_NO_DEVICE : ringTransfer(false, ring, dst, bytes, first_seq, yield_us, stream, event);
}

int tphip_profile_start(int dev, uint32_t max_launches) {
  return 0;
}

int tphip_profile_stop(int dev, uint32_t* launches, double* total_ms, uint64_t* total_bytes) {
  if (launches != nullptr) {
    *launches = 0;
  }
  if (total_ms != nullptr) {
    *total_ms = 0;
  }
  if (total_bytes != nullptr) {
    *total_bytes = 0;
  }
  return 0;
}

int tphip_bench_stream(int dev, int write, void* ptr, uint64_t bytes, void* stream) {
  if (write != 0) {
    return tphip_fill(dev, ptr, 0x5b, bytes, stream);
  }
  return 0;
}

int tphip_fill(int dev, void* ptr, int value, uint64_t bytes, void* stream) {
  streamOf(stream).push([ptr, value, bytes] {
    checkRange("fill target", ptr, bytes);
    std::memset(ptr, value, bytes);
  });
  return 0;
}

int tphip_test_set_table_limit(uint64_t vectors) {
  return 0;
}

// Keeps the stream busy for a while and leaves garbage behind, as the kernel does.
int tphip_test_slow_kernel(int dev, void* ptr, uint64_t n, void* stream) {
  streamOf(stream).push([ptr, n] {
    checkRange("slow kernel target", ptr, n);
    for (int round = 0; round < 20; ++round) {
      std::memset(ptr, 0x5a + round, n);
      std::this_thread::sleep_for(std::chrono::milliseconds(2));
    }
  });
  return 0;
}

} // extern "C"
