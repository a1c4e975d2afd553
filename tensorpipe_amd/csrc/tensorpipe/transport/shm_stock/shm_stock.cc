// Shared-memory transport in the protocol of the reference's shm transport, so
// that the other end may be an unmodified TensorPipe on the same host.
//
// What the two ends must agree on, and where the reference defines it:
//  * Listener and connection meet on a Unix stream socket with an abstract
//    address (tensorpipe/transport/shm/sockaddr.cc:23-46, listener_impl.cc:39-70).
//  * Every connection owns an inbox: a byte ring whose header and data are two
//    shared-memory segments (tensorpipe/common/shm_ringbuffer.h:23-52). A header
//    is {data size, data size - 1, two one-byte transaction flags, two 64-bit
//    markers}; marker 0 counts the bytes ever consumed, marker 1 the bytes ever
//    produced, and a side holds its flag while it moves its marker
//    (tensorpipe/common/ringbuffer.h:50-140, ringbuffer_role.h:50-150). The
//    header segment is exactly as large as the header, the data segment as
//    large as the header says (shm_ringbuffer.h:66-82).
//  * Every context owns a reactor: a ring of the same kind, 4 MiB, that carries
//    32-bit tokens; whoever wants a function of that context run writes its
//    token there (tensorpipe/transport/shm/reactor.cc:20-42,109-135), and the
//    context's thread polls the ring. There is no other wake-up.
//  * At set-up each end sends ONE message over the socket: two tokens (run
//    this when you have written into my inbox / when you have read from your
//    inbox, which is my outbox) and four descriptors by SCM_RIGHTS: reactor
//    header, reactor data, inbox header, inbox data
//    (tensorpipe/transport/shm/connection_impl.cc:231-291, common/socket.h:59-165).
//    After that the socket only says when the peer has gone.
//  * A message in a ring is a 32-bit length and then the bytes, streamed in as
//    many pieces as the ring's room demands
//    (tensorpipe/common/ringbuffer_read_write_ops.h:136-189,223-266).
//
// Own design around that: one thread per context polls the token ring, the
// sockets (epoll) and the task queue; it spins while anything happens and naps
// 100 us at a time once nothing has for a while (the reference's reactor spins
// for as long as the context lives). A peer that hangs up still has what it
// wrote before delivered.

#include <tensorpipe/transport/shm_stock/factory.h>

#include <fcntl.h>
#include <poll.h>
#include <sys/epoll.h>
#include <sys/eventfd.h>
#include <sys/mman.h>
#include <sys/socket.h>
#include <sys/stat.h>
#include <sys/syscall.h>
#include <sys/un.h>
#include <unistd.h>

#include <sched.h>

#include <atomic>
#include <cerrno>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <fstream>
#include <mutex>
#include <new>
#include <set>
#include <sstream>
#include <stdexcept>
#include <thread>
#include <vector>

#include <tensorpipe/common/defs.h>
#include <tensorpipe/common/loop.h>
#include <tensorpipe/transport/connection.h>
#include <tensorpipe/transport/error.h>
#include <tensorpipe/transport/listener.h>

TP_AMD_NAMESPACE_BEGIN
namespace transport {
namespace shm_stock {

namespace {

constexpr size_t kInboxBytes = 2 * 1024 * 1024; // tensorpipe/transport/shm/connection_impl.h:38
constexpr size_t kReactorBytes = 4 * 1024 * 1024; // tensorpipe/transport/shm/reactor.h:38
constexpr size_t kLengthPrefix = 4;

// ThreadSanitizer keys happens-before on virtual addresses; the two ends of a
// ring inside one process see the same markers at different addresses.
#if defined(__SANITIZE_THREAD__)
extern "C" void __tsan_acquire(void* addr);
extern "C" void __tsan_release(void* addr);
char gTsanRingToken;
#define TP_TSAN_RING_RELEASE() __tsan_release(&gTsanRingToken)
#define TP_TSAN_RING_ACQUIRE() __tsan_acquire(&gTsanRingToken)
#else
#define TP_TSAN_RING_RELEASE() ((void)0)
#define TP_TSAN_RING_ACQUIRE() ((void)0)
#endif

// The bytes of tensorpipe::RingBufferHeader<2> as libstdc++ lays them out on
// x86-64 (std::atomic_flag is one byte there).
struct RingHeader {
  uint64_t dataBytes;
  uint64_t dataMask;
  std::atomic<uint8_t> inTransaction[2]; // 0: the consumer, 1: a producer
  std::atomic<uint64_t> marker[2]; // 0: bytes consumed, 1: bytes produced
};
static_assert(sizeof(RingHeader) == 40, "must match the reference's header");
static_assert(offsetof(RingHeader, inTransaction) == 16, "must match the reference's header");
static_assert(offsetof(RingHeader, marker) == 24, "must match the reference's header");

// A memory-backed file of an exact size, mapped.
class Segment {
 public:
  Segment() = default;
  Segment(const Segment&) = delete;
  Segment& operator=(const Segment&) = delete;
  ~Segment() {
    reset();
  }

  // tensorpipe/common/shm_segment.cc:48-75,118-143
  bool create(size_t bytes) {
    reset();
    fd_ = static_cast<int>(::syscall(SYS_memfd_create, "tensorpipe_shm", MFD_CLOEXEC));
    if (fd_ < 0 || ::ftruncate(fd_, static_cast<off_t>(bytes)) != 0) {
      reset();
      return false;
    }
    return map(bytes);
  }

  // Takes the descriptor over. tensorpipe/common/shm_segment.cc:145-166
  bool open(int fd) {
    reset();
    fd_ = fd;
    struct stat sb;
    if (::fstat(fd_, &sb) != 0 || sb.st_size <= 0) {
      reset();
      return false;
    }
    return map(static_cast<size_t>(sb.st_size));
  }

  int fd() const {
    return fd_;
  }
  size_t size() const {
    return bytes_;
  }
  uint8_t* data() const {
    return static_cast<uint8_t*>(ptr_);
  }

  void reset() {
    if (ptr_ != nullptr) {
      ::munmap(ptr_, bytes_);
      ptr_ = nullptr;
    }
    if (fd_ >= 0) {
      ::close(fd_);
      fd_ = -1;
    }
    bytes_ = 0;
  }

 private:
  bool map(size_t bytes) {
    void* p = ::mmap(nullptr, bytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd_, 0);
    if (p == MAP_FAILED) {
      reset();
      return false;
    }
    ptr_ = p;
    bytes_ = bytes;
    return true;
  }

  int fd_{-1};
  void* ptr_{nullptr};
  size_t bytes_{0};
};

// One ring: a header segment and a data segment.
class Ring {
 public:
  bool create(size_t dataBytes) {
    size_t pow2 = 2;
    while (pow2 < dataBytes) {
      pow2 <<= 1;
    }
    if (!header_.create(sizeof(RingHeader)) || !data_.create(pow2)) {
      return false;
    }
    RingHeader* h = new (header_.data()) RingHeader();
    h->dataBytes = pow2;
    h->dataMask = pow2 - 1;
    for (int r = 0; r < 2; ++r) {
      h->inTransaction[r].store(0, std::memory_order_relaxed);
      h->marker[r].store(0, std::memory_order_relaxed);
    }
    bytes_ = pow2;
    return true;
  }

  // The peer's ring, from the two descriptors it sent (both are taken over).
  bool open(int headerFd, int dataFd) {
    const bool okHeader = header_.open(headerFd);
    const bool okData = data_.open(dataFd);
    if (!okHeader || !okData || header_.size() != sizeof(RingHeader)) {
      return false;
    }
    const RingHeader* h = header();
    const uint64_t bytes = h->dataBytes;
    if (bytes < 2 || (bytes & (bytes - 1)) != 0 || h->dataMask != bytes - 1 || data_.size() != bytes) {
      return false;
    }
    bytes_ = bytes; // the header is memory that the peer can write: never read the size from it again
    return true;
  }

  // The markers said something that no ring of this size can be in: the peer
  // (or whoever else maps the header) has scribbled over it.
  bool corrupt() const {
    return corrupt_;
  }

  RingHeader* header() const {
    return reinterpret_cast<RingHeader*>(header_.data());
  }
  int headerFd() const {
    return header_.fd();
  }
  int dataFd() const {
    return data_.fd();
  }
  bool valid() const {
    return header_.data() != nullptr && data_.data() != nullptr;
  }

  // ---- the consumer's side (one consumer per ring, always the same thread)

  // Bytes that can be read now.
  uint64_t readable() const {
    const RingHeader* h = header();
    return h->marker[1].load(std::memory_order_acquire) - h->marker[0].load(std::memory_order_relaxed);
  }

  // Copies out up to `n` bytes (all of them or none unless `partial`) and gives
  // their room back; returns how many.
  size_t consume(void* dst, size_t n, bool partial) {
    RingHeader* h = header();
    if (h->inTransaction[0].exchange(1, std::memory_order_acquire) != 0) {
      return 0; // not ours to take: a single consumer never meets this
    }
    TP_TSAN_RING_ACQUIRE();
    const uint64_t tail = h->marker[0].load(std::memory_order_relaxed);
    const uint64_t avail = h->marker[1].load(std::memory_order_acquire) - tail;
    size_t take = 0;
    if (avail > bytes_) {
      corrupt_ = true;
    } else if (avail >= n) {
      take = n;
    } else if (partial) {
      take = static_cast<size_t>(avail);
    }
    if (take > 0) {
      const uint64_t start = tail & (bytes_ - 1);
      const size_t first = static_cast<size_t>(std::min<uint64_t>(take, bytes_ - start));
      std::memcpy(dst, data_.data() + start, first);
      std::memcpy(static_cast<uint8_t*>(dst) + first, data_.data(), take - first);
      TP_TSAN_RING_RELEASE();
      h->marker[0].fetch_add(take, std::memory_order_release);
    }
    h->inTransaction[0].store(0, std::memory_order_release);
    return take;
  }

  // ---- a producer's side

  enum class Put { kDone, kBusy, kFull };

  // Copies in up to `n` bytes (all or none unless `partial`); `*put` says how
  // many. kBusy: another producer holds the ring (only rings with several
  // producers, the reactors', ever say so).
  Put produce(const void* src, size_t n, bool partial, size_t* put) {
    *put = 0;
    RingHeader* h = header();
    if (h->inTransaction[1].exchange(1, std::memory_order_acquire) != 0) {
      return Put::kBusy;
    }
    TP_TSAN_RING_ACQUIRE();
    const uint64_t head = h->marker[1].load(std::memory_order_relaxed);
    const uint64_t room = h->marker[0].load(std::memory_order_acquire) + bytes_ - head;
    size_t take = 0;
    if (room > bytes_) {
      corrupt_ = true;
    } else if (room >= n) {
      take = n;
    } else if (partial) {
      take = static_cast<size_t>(room);
    }
    if (take > 0) {
      const uint64_t start = head & (bytes_ - 1);
      const size_t first = static_cast<size_t>(std::min<uint64_t>(take, bytes_ - start));
      std::memcpy(data_.data() + start, src, first);
      std::memcpy(data_.data(), static_cast<const uint8_t*>(src) + first, take - first);
      TP_TSAN_RING_RELEASE();
      h->marker[1].fetch_add(take, std::memory_order_release);
    }
    h->inTransaction[1].store(0, std::memory_order_release);
    *put = take;
    return take > 0 || n == 0 ? Put::kDone : Put::kFull;
  }

 private:
  Segment header_;
  Segment data_;
  uint64_t bytes_{0}; // of the data segment, as checked when the ring was made or opened
  bool corrupt_{false};
};

std::string readLine(const char* path) {
  std::ifstream f(path);
  std::string v;
  if (f.is_open()) {
    std::getline(f, v);
  }
  return v;
}

// tensorpipe/transport/shm/context_impl.cc:29-47: "shm:" + boot id + '_' + the
// network namespace as the reference names it (device and inode of
// /proc/self/ns/net, both in hex; tensorpipe/common/system.cc:166-200).
std::string makeDomainDescriptor() {
  const std::string boot = readLine("/proc/sys/kernel/random/boot_id");
  struct stat link;
  struct stat target;
  if (boot.empty() || ::lstat("/proc/self/ns/net", &link) != 0 || !S_ISLNK(link.st_mode) ||
      ::stat("/proc/self/ns/net", &target) != 0) {
    return std::string();
  }
  std::ostringstream oss;
  oss << "shm:" << boot << '_' << std::hex << target.st_dev << '_' << target.st_ino;
  return oss.str();
}

// tensorpipe/transport/shm/sockaddr.cc:23-46
socklen_t abstractAddress(const std::string& name, sockaddr_un* sun) {
  std::memset(sun, 0, sizeof(*sun));
  sun->sun_family = AF_UNIX;
  if (name.empty()) {
    return sizeof(sun->sun_family); // the kernel picks a name
  }
  const size_t len = std::min(sizeof(sun->sun_path) - 1, name.size());
  std::memcpy(&sun->sun_path[1], name.data(), len);
  return static_cast<socklen_t>(sizeof(sun->sun_family) + 1 + len);
}

class FdHandler {
 public:
  virtual void onEvents(uint32_t events) = 0;
  virtual void shutdownFromLoop() = 0;
  virtual ~FdHandler() = default;
};

// The context's thread: token ring, sockets, tasks.
class Reactor final : public std::enable_shared_from_this<Reactor> {
 public:
  using Token = uint32_t;

  Reactor() {
    epollFd_ = ::epoll_create1(EPOLL_CLOEXEC);
    wakeFd_ = ::eventfd(0, EFD_NONBLOCK | EFD_CLOEXEC);
    TP_THROW_ASSERT_IF(epollFd_ < 0 || wakeFd_ < 0);
    TP_THROW_ASSERT_IF(!ring_.create(kReactorBytes));
    epoll_event ev{};
    ev.events = EPOLLIN;
    ev.data.ptr = nullptr; // the wake-up fd
    ::epoll_ctl(epollFd_, EPOLL_CTL_ADD, wakeFd_, &ev);
    thread_ = std::thread([this] { run(); });
  }

  ~Reactor() {
    join();
    ::close(epollFd_);
    ::close(wakeFd_);
  }

  int ringHeaderFd() const {
    return ring_.headerFd();
  }
  int ringDataFd() const {
    return ring_.dataFd();
  }

  void defer(std::function<void()> fn) {
    {
      std::lock_guard<std::mutex> lock(mutex_);
      if (stopped_) {
        lateTasks_.push_back(std::move(fn));
        if (lateRunning_) {
          return;
        }
        lateRunning_ = true;
      } else {
        tasks_.push_back(std::move(fn));
        pendingTasks_.fetch_add(1); // sequentially consistent, as the look at napping_ after it
        if (napping_.load()) {
          const uint64_t one = 1;
          (void)!::write(wakeFd_, &one, sizeof(one));
        }
        return;
      }
    }
    for (;;) {
      std::function<void()> task;
      {
        std::lock_guard<std::mutex> lock(mutex_);
        if (lateTasks_.empty()) {
          lateRunning_ = false;
          return;
        }
        task = std::move(lateTasks_.front());
        lateTasks_.pop_front();
      }
      task();
    }
  }

  // Loop only: a function that a token written into the ring runs
  // (tensorpipe/transport/shm/reactor.cc:66-99: the lowest free token is used again).
  Token addReaction(std::function<void()> fn) {
    Token token;
    if (!freeTokens_.empty()) {
      token = *freeTokens_.begin();
      freeTokens_.erase(freeTokens_.begin());
    } else {
      token = static_cast<Token>(reactions_.size());
      reactions_.emplace_back();
    }
    reactions_[token] = std::move(fn);
    return token;
  }
  void removeReaction(Token token) {
    reactions_[token] = nullptr;
    freeTokens_.insert(token);
  }

  void setInterest(int fd, FdHandler* handler, uint32_t events, bool* registered) {
    epoll_event ev{};
    ev.events = events;
    ev.data.ptr = handler;
    ::epoll_ctl(epollFd_, *registered ? EPOLL_CTL_MOD : EPOLL_CTL_ADD, fd, &ev);
    *registered = true;
  }
  void forget(int fd) {
    ::epoll_ctl(epollFd_, EPOLL_CTL_DEL, fd, nullptr);
  }
  void enroll(std::shared_ptr<FdHandler> h) {
    live_.insert(std::move(h));
  }
  void unenroll(const std::shared_ptr<FdHandler>& h) {
    live_.erase(h);
  }
  void touched() {
    lastActivity_ = std::chrono::steady_clock::now();
  }

  bool closed() const {
    return closed_.load(std::memory_order_acquire);
  }

  void close() {
    if (closed_.exchange(true)) {
      return;
    }
    auto self = shared_from_this();
    defer([self] {
      auto live = self->live_;
      for (auto& h : live) {
        h->shutdownFromLoop();
      }
    });
  }

  void join() {
    close();
    {
      std::lock_guard<std::mutex> lock(mutex_);
      if (joined_) {
        return;
      }
      joined_ = true;
    }
    auto self = this;
    defer([self] { self->stop_ = true; });
    if (thread_.joinable()) {
      thread_.join();
    }
  }

 private:
  void run() {
    thisIsLibraryThread() = true;
    std::vector<epoll_event> events(64);
    const auto spinFor = std::chrono::microseconds([] {
      const char* e = std::getenv("TP_SHM_STOCK_SPIN_US");
      long v = e != nullptr ? std::atol(e) : 500;
      cpu_set_t set;
      CPU_ZERO(&set);
      if (::sched_getaffinity(0, sizeof(set), &set) == 0 && CPU_COUNT(&set) < 4) {
        v = 0;
      }
      return v;
    }());
    lastActivity_ = std::chrono::steady_clock::now();
    uint32_t sinceSockets = 0;
    while (!stop_) {
      bool progressed = false;
      // tokens
      for (int k = 0; k < 64; ++k) {
        Token token = 0;
        if (ring_.consume(&token, sizeof(token), /*partial=*/false) != sizeof(token)) {
          break;
        }
        progressed = true;
        if (token < reactions_.size() && reactions_[token]) {
          auto fn = reactions_[token]; // a reaction may remove itself
          fn();
        }
      }
      // tasks
      if (pendingTasks_.load(std::memory_order_acquire) > 0) {
        progressed |= runTasks();
      }
      // sockets: rare (set-up, hang-up), so looked at every so often while busy
      if (!progressed || ++sinceSockets >= 256) {
        sinceSockets = 0;
        progressed |= pollSockets(events, 0);
      }
      if (progressed) {
        lastActivity_ = std::chrono::steady_clock::now();
        continue;
      }
      if (std::chrono::steady_clock::now() - lastActivity_ < spinFor) {
        std::this_thread::yield();
        continue;
      }
      // Nothing for a while: nap, woken by sockets and tasks at once and by the
      // clock for the token ring, which has no way to wake anybody.
      napping_.store(true); // sequentially consistent with defer(): one of the two sees the other
      if (pendingTasks_.load() == 0 && ring_.readable() < sizeof(Token)) {
        pollfd pfd{};
        pfd.fd = epollFd_;
        pfd.events = POLLIN;
        timespec ts{0, 100 * 1000};
        (void)::ppoll(&pfd, 1, &ts, nullptr);
      }
      napping_.store(false, std::memory_order_release);
    }
    auto live = live_;
    for (auto& h : live) {
      h->shutdownFromLoop();
    }
    runTasks();
    live_.clear();
    std::lock_guard<std::mutex> lock(mutex_);
    stopped_ = true;
    for (auto& t : tasks_) {
      lateTasks_.push_back(std::move(t));
    }
    tasks_.clear();
  }

  bool pollSockets(std::vector<epoll_event>& events, int timeoutMs) {
    const int n = ::epoll_wait(epollFd_, events.data(), static_cast<int>(events.size()), timeoutMs);
    for (int i = 0; i < n; ++i) {
      if (events[i].data.ptr == nullptr) {
        uint64_t v;
        (void)!::read(wakeFd_, &v, sizeof(v));
        continue;
      }
      FdHandler* h = static_cast<FdHandler*>(events[i].data.ptr);
      const auto it = live_.find(std::shared_ptr<FdHandler>(std::shared_ptr<FdHandler>(), h));
      if (it != live_.end()) {
        std::shared_ptr<FdHandler> keep = *it;
        keep->onEvents(events[i].events);
      }
    }
    return n > 0;
  }

  bool runTasks() {
    bool any = false;
    for (;;) {
      std::deque<std::function<void()>> batch;
      {
        std::lock_guard<std::mutex> lock(mutex_);
        batch.swap(tasks_);
        pendingTasks_.store(0, std::memory_order_release);
      }
      if (batch.empty()) {
        return any;
      }
      any = true;
      for (auto& t : batch) {
        t();
      }
    }
  }

  int epollFd_{-1};
  int wakeFd_{-1};
  Ring ring_;
  std::thread thread_;
  std::mutex mutex_;
  std::deque<std::function<void()>> tasks_;
  std::deque<std::function<void()>> lateTasks_;
  std::atomic<int64_t> pendingTasks_{0};
  std::atomic<bool> napping_{false};
  bool lateRunning_{false};
  bool stopped_{false};
  bool joined_{false};
  bool stop_{false}; // loop only
  std::atomic<bool> closed_{false};
  std::set<std::shared_ptr<FdHandler>> live_; // loop only
  std::vector<std::function<void()>> reactions_; // loop only
  std::set<Token> freeTokens_; // loop only
  std::chrono::steady_clock::time_point lastActivity_; // loop only
};

class ConnectionImpl final : public FdHandler, public std::enable_shared_from_this<ConnectionImpl> {
 public:
  using read_callback_fn = Connection::read_callback_fn;
  using write_callback_fn = Connection::write_callback_fn;

  ConnectionImpl(std::shared_ptr<Reactor> reactor, std::string addr)
      : reactor_(std::move(reactor)), addr_(std::move(addr)) {}
  ConnectionImpl(std::shared_ptr<Reactor> reactor, int fd) : reactor_(std::move(reactor)), fd_(fd) {}

  ~ConnectionImpl() override {
    if (fd_ >= 0) {
      ::close(fd_);
    }
  }

  void init() {
    auto self = shared_from_this();
    reactor_->defer([self] { self->initFromLoop(); });
  }

  void read(read_callback_fn fn) {
    auto self = shared_from_this();
    reactor_->defer([self, fn{std::move(fn)}]() mutable {
      self->enqueueRead(ReadOp{nullptr, 0, false, std::move(fn)});
    });
  }
  void read(void* ptr, size_t length, read_callback_fn fn) {
    auto self = shared_from_this();
    reactor_->defer([self, ptr, length, fn{std::move(fn)}]() mutable {
      self->enqueueRead(ReadOp{static_cast<uint8_t*>(ptr), length, true, std::move(fn)});
    });
  }
  void write(const void* ptr, size_t length, write_callback_fn fn) {
    auto self = shared_from_this();
    reactor_->defer([self, ptr, length, fn{std::move(fn)}]() mutable {
      if (self->error_) {
        fn(self->error_);
        return;
      }
      if (length > 0xffffffffull) {
        fn(TP_CREATE_ERROR(SystemError, "a message of this transport carries a 32-bit length", EMSGSIZE));
        return;
      }
      if (self->peerGone_) {
        fn(TP_CREATE_ERROR(EOFError));
        self->fail(TP_CREATE_ERROR(EOFError));
        return;
      }
      WriteOp op;
      op.ptr = static_cast<const uint8_t*>(ptr);
      op.length = length;
      op.fn = std::move(fn);
      self->writes_.push_back(std::move(op));
      self->pumpWrites();
    });
  }
  void setId(std::string id) {
    auto self = shared_from_this();
    reactor_->defer([self, id{std::move(id)}]() mutable { self->id_ = std::move(id); });
  }
  void close() {
    auto self = shared_from_this();
    reactor_->defer([self] { self->fail(TP_CREATE_ERROR(ConnectionClosedError)); });
  }

  // tensorpipe/transport/shm/connection_impl.cc:168-291
  void onEvents(uint32_t events) override {
    if (error_) {
      return;
    }
    if (state_ == State::kSendDescriptors && (events & EPOLLOUT)) {
      sendDescriptors();
      return;
    }
    if (state_ == State::kRecvDescriptors && (events & EPOLLIN)) {
      recvDescriptors();
      return;
    }
    if (events & (EPOLLIN | EPOLLRDHUP | EPOLLHUP | EPOLLERR)) {
      // Nothing is ever sent on the socket after set-up: the peer has gone.
      // What it wrote before leaving is in the inbox and is still delivered, to
      // reads posted by now and to later ones; whatever needs the peer fails.
      if (state_ != State::kEstablished) {
        fail(TP_CREATE_ERROR(EOFError));
        return;
      }
      peerGone_ = true;
      if (registered_) {
        reactor_->forget(fd_); // epoll would report the hang-up for ever
        registered_ = false;
      }
      pumpReads();
      if (!error_ && !writes_.empty()) {
        fail(TP_CREATE_ERROR(EOFError));
      }
    }
  }

  void shutdownFromLoop() override {
    fail(TP_CREATE_ERROR(ContextClosedError));
  }

 private:
  enum class State { kInitializing, kSendDescriptors, kRecvDescriptors, kEstablished };

  struct ReadOp {
    uint8_t* ptr;
    size_t length;
    bool exact; // into the caller's buffer, which must be exactly the message's size
    read_callback_fn fn;
  };
  struct WriteOp {
    const uint8_t* ptr{nullptr};
    size_t length{0};
    bool lengthWritten{false};
    size_t done{0};
    write_callback_fn fn;
  };

  void initFromLoop() {
    auto self = shared_from_this();
    reactor_->enroll(self);
    if (reactor_->closed()) {
      fail(TP_CREATE_ERROR(ContextClosedError));
      return;
    }
    if (fd_ < 0) {
      fd_ = ::socket(AF_UNIX, SOCK_STREAM | SOCK_NONBLOCK | SOCK_CLOEXEC, 0);
      if (fd_ < 0) {
        fail(TP_CREATE_ERROR(SystemError, "socket", errno));
        return;
      }
      sockaddr_un sun;
      const socklen_t len = abstractAddress(addr_, &sun);
      if (::connect(fd_, reinterpret_cast<sockaddr*>(&sun), len) != 0) {
        fail(TP_CREATE_ERROR(SystemError, "connect", errno));
        return;
      }
    } else {
      const int flags = ::fcntl(fd_, F_GETFL, 0);
      ::fcntl(fd_, F_SETFL, flags | O_NONBLOCK);
    }
    if (!inbox_.create(kInboxBytes)) {
      fail(TP_CREATE_ERROR(SystemError, "shared memory for the inbox", errno));
      return;
    }
    std::weak_ptr<ConnectionImpl> weak = self;
    inboxToken_ = reactor_->addReaction([weak] {
      if (auto me = weak.lock()) {
        me->pumpReads(); // the peer wrote into our inbox
      }
    });
    outboxToken_ = reactor_->addReaction([weak] {
      if (auto me = weak.lock()) {
        me->pumpWrites(); // the peer read from our outbox
      }
    });
    haveTokens_ = true;
    state_ = State::kSendDescriptors;
    reactor_->setInterest(fd_, this, EPOLLOUT, &registered_);
  }

  // One message: our two tokens, and the reactor's and the inbox's segments by
  // SCM_RIGHTS (tensorpipe/common/socket.h:59-113).
  void sendDescriptors() {
    uint32_t tokens[2] = {inboxToken_, outboxToken_};
    int fds[4] = {reactor_->ringHeaderFd(), reactor_->ringDataFd(), inbox_.headerFd(), inbox_.dataFd()};
    iovec iov{};
    iov.iov_base = tokens;
    iov.iov_len = sizeof(tokens);
    alignas(cmsghdr) char control[CMSG_SPACE(sizeof(fds))];
    std::memset(control, 0, sizeof(control));
    msghdr msg{};
    msg.msg_iov = &iov;
    msg.msg_iovlen = 1;
    msg.msg_control = control;
    msg.msg_controllen = sizeof(control);
    cmsghdr* cmsg = CMSG_FIRSTHDR(&msg);
    cmsg->cmsg_level = SOL_SOCKET;
    cmsg->cmsg_type = SCM_RIGHTS;
    cmsg->cmsg_len = CMSG_LEN(sizeof(fds));
    std::memcpy(CMSG_DATA(cmsg), fds, sizeof(fds));
    ssize_t rv;
    do {
      rv = ::sendmsg(fd_, &msg, MSG_NOSIGNAL);
    } while (rv < 0 && errno == EINTR);
    if (rv < 0 && (errno == EAGAIN || errno == EWOULDBLOCK)) {
      return; // asked again when writable
    }
    if (rv != static_cast<ssize_t>(sizeof(tokens))) {
      fail(TP_CREATE_ERROR(SystemError, "sendmsg", rv < 0 ? errno : EIO));
      return;
    }
    state_ = State::kRecvDescriptors;
    reactor_->setInterest(fd_, this, EPOLLIN, &registered_);
  }

  // tensorpipe/common/socket.h:115-165, tensorpipe/transport/shm/connection_impl.cc:214-252
  void recvDescriptors() {
    uint32_t tokens[2] = {0, 0};
    iovec iov{};
    iov.iov_base = tokens;
    iov.iov_len = sizeof(tokens);
    alignas(cmsghdr) char control[CMSG_SPACE(4 * sizeof(int))];
    std::memset(control, 0, sizeof(control));
    msghdr msg{};
    msg.msg_iov = &iov;
    msg.msg_iovlen = 1;
    msg.msg_control = control;
    msg.msg_controllen = sizeof(control);
    ssize_t rv;
    do {
      rv = ::recvmsg(fd_, &msg, MSG_CMSG_CLOEXEC);
    } while (rv < 0 && errno == EINTR);
    if (rv < 0 && (errno == EAGAIN || errno == EWOULDBLOCK)) {
      return;
    }
    int fds[4] = {-1, -1, -1, -1};
    int nfds = 0;
    for (cmsghdr* cmsg = CMSG_FIRSTHDR(&msg); cmsg != nullptr; cmsg = CMSG_NXTHDR(&msg, cmsg)) {
      if (cmsg->cmsg_level != SOL_SOCKET || cmsg->cmsg_type != SCM_RIGHTS) {
        continue;
      }
      const size_t count = (cmsg->cmsg_len - CMSG_LEN(0)) / sizeof(int);
      for (size_t i = 0; i < count; ++i) {
        int fd;
        std::memcpy(&fd, CMSG_DATA(cmsg) + i * sizeof(int), sizeof(int));
        if (nfds < 4) {
          fds[nfds++] = fd;
        } else {
          ::close(fd);
        }
      }
    }
    if (rv == 0) {
      fail(TP_CREATE_ERROR(EOFError));
      return;
    }
    if (rv != static_cast<ssize_t>(sizeof(tokens)) || nfds != 4) {
      for (int i = 0; i < nfds; ++i) {
        ::close(fds[i]);
      }
      fail(TP_CREATE_ERROR(ShortReadError, static_cast<ssize_t>(sizeof(tokens)), rv));
      return;
    }
    const bool okReactor = peerReactor_.open(fds[0], fds[1]);
    const bool okOutbox = outbox_.open(fds[2], fds[3]);
    if (!okReactor || !okOutbox) {
      fail(TP_CREATE_ERROR(SystemError, "the peer's rings are not what this transport expects", EPROTO));
      return;
    }
    peerInboxToken_ = tokens[0];
    peerOutboxToken_ = tokens[1];
    state_ = State::kEstablished;
    // the socket stays in the set for its hang-up
    reactor_->setInterest(fd_, this, EPOLLIN | EPOLLRDHUP, &registered_);
    pumpWrites();
    if (!error_) {
      pumpReads();
    }
  }

  void enqueueRead(ReadOp op) {
    if (error_) {
      op.fn(error_, nullptr, 0);
      return;
    }
    reads_.push_back(std::move(op));
    pumpReads();
  }

  // Writes `token` into the peer's reactor ring
  // (tensorpipe/transport/shm/reactor.cc:20-42). Other connections, of this and of
  // other processes, write there too.
  bool trigger(uint32_t token) {
    const auto giveUp = std::chrono::steady_clock::now() + std::chrono::seconds(5);
    for (uint32_t spins = 0;; ++spins) {
      size_t put = 0;
      if (peerReactor_.produce(&token, sizeof(token), /*partial=*/false, &put) == Ring::Put::kDone) {
        return true;
      }
      if (peerReactor_.corrupt()) {
        fail(TP_CREATE_ERROR(SystemError, "the header of the peer's reactor ring makes no sense", EPROTO));
        return false;
      }
      // held by another producer for a few instructions, or full of tokens that
      // the peer's thread has not got to yet
      std::this_thread::yield();
      if ((spins & 1023) == 1023 && std::chrono::steady_clock::now() > giveUp) {
        fail(TP_CREATE_ERROR(SystemError, "the peer's reactor takes no tokens", ETIMEDOUT));
        return false;
      }
    }
  }

  // tensorpipe/common/ringbuffer_read_write_ops.h:136-189 and
  // tensorpipe/transport/shm/connection_impl.cc:293-314
  void pumpReads() {
    if (state_ != State::kEstablished) {
      return;
    }
    while (!reads_.empty() && !error_) {
      ReadOp& op = reads_.front();
      size_t now = 0;
      if (!lengthKnown_) {
        uint32_t length = 0;
        if (inbox_.consume(&length, kLengthPrefix, /*partial=*/false) != kLengthPrefix) {
          if (inbox_.corrupt()) {
            failCorrupt();
          } else if (peerGone_) {
            fail(TP_CREATE_ERROR(EOFError));
          }
          return;
        }
        now += kLengthPrefix;
        lengthKnown_ = true;
        messageLength_ = length;
        payloadDone_ = 0;
        if (op.exact) {
          if (messageLength_ != op.length) {
            fail(TP_CREATE_ERROR(
                ShortReadError, static_cast<ssize_t>(op.length), static_cast<ssize_t>(messageLength_)));
            return;
          }
        } else {
          try {
            scratch_.resize(messageLength_);
          } catch (const std::bad_alloc&) {
            fail(TP_CREATE_ERROR(SystemError, "no memory for a message of the announced length", ENOMEM));
            return;
          }
        }
      }
      uint8_t* dst = op.exact ? op.ptr : scratch_.data();
      if (payloadDone_ < messageLength_) {
        const size_t got =
            inbox_.consume(dst + payloadDone_, messageLength_ - payloadDone_, /*partial=*/true);
        payloadDone_ += got;
        now += got;
        if (inbox_.corrupt()) {
          failCorrupt();
          return;
        }
      }
      if (now > 0 && !peerGone_) {
        reactor_->touched();
        if (!trigger(peerOutboxToken_)) { // the peer's outbox has room again
          return;
        }
      }
      if (payloadDone_ < messageLength_) {
        if (peerGone_ && now == 0) {
          fail(TP_CREATE_ERROR(EOFError)); // the rest will never come
        } else if (peerGone_) {
          continue; // took something: look again before giving up
        }
        return; // the rest is not there yet
      }
      ReadOp finished = std::move(op);
      reads_.pop_front();
      lengthKnown_ = false;
      finished.fn(Error::kSuccess, dst, messageLength_);
    }
  }

  // tensorpipe/common/ringbuffer_read_write_ops.h:223-266 and
  // tensorpipe/transport/shm/connection_impl.cc:316-336
  void pumpWrites() {
    if (state_ != State::kEstablished) {
      return;
    }
    while (!writes_.empty() && !error_) {
      WriteOp& op = writes_.front();
      size_t now = 0;
      size_t put = 0;
      if (!op.lengthWritten) {
        const uint32_t length = static_cast<uint32_t>(op.length);
        if (outbox_.produce(&length, kLengthPrefix, /*partial=*/false, &put) != Ring::Put::kDone) {
          if (outbox_.corrupt()) {
            failCorrupt();
          }
          return; // no room for the length: the peer's read will run this again
        }
        op.lengthWritten = true;
        now += put;
      }
      if (op.done < op.length) {
        (void)outbox_.produce(op.ptr + op.done, op.length - op.done, /*partial=*/true, &put);
        op.done += put;
        now += put;
        if (outbox_.corrupt()) {
          failCorrupt();
          return;
        }
      }
      if (now > 0) {
        reactor_->touched();
        if (!trigger(peerInboxToken_)) {
          return;
        }
      }
      if (op.done < op.length) {
        return; // the ring is full
      }
      WriteOp finished = std::move(op);
      writes_.pop_front();
      finished.fn(Error::kSuccess);
    }
  }

  void failCorrupt() {
    fail(TP_CREATE_ERROR(SystemError, "the markers of a ring shared with the peer make no sense", EPROTO));
  }

  void fail(Error error) {
    if (error_) {
      return;
    }
    error_ = std::move(error);
    TP_VLOG(8) << "Connection " << id_ << " is failing: " << error_.what();
    if (haveTokens_) {
      reactor_->removeReaction(inboxToken_);
      reactor_->removeReaction(outboxToken_);
      haveTokens_ = false;
    }
    if (fd_ >= 0) {
      if (registered_) {
        reactor_->forget(fd_);
      }
      ::shutdown(fd_, SHUT_RDWR);
      ::close(fd_);
      fd_ = -1;
    }
    auto reads = std::move(reads_);
    reads_.clear();
    auto writes = std::move(writes_);
    writes_.clear();
    for (auto& op : reads) {
      op.fn(error_, nullptr, 0);
    }
    for (auto& op : writes) {
      op.fn(error_);
    }
    reactor_->unenroll(shared_from_this());
  }

  std::shared_ptr<Reactor> reactor_;
  const std::string addr_;
  std::string id_{"N/A"};
  int fd_{-1};
  bool registered_{false};
  State state_{State::kInitializing};
  Error error_;
  Ring inbox_; // ours; the peer produces
  Ring outbox_; // the peer's inbox; we produce
  Ring peerReactor_;
  bool haveTokens_{false};
  bool peerGone_{false}; // the socket hung up; the inbox may still hold what the peer wrote
  uint32_t inboxToken_{0}, outboxToken_{0};
  uint32_t peerInboxToken_{0}, peerOutboxToken_{0};
  std::deque<ReadOp> reads_;
  std::deque<WriteOp> writes_;
  bool lengthKnown_{false};
  size_t messageLength_{0};
  size_t payloadDone_{0};
  std::vector<uint8_t> scratch_;
};

class ShmStockConnection final : public Connection {
 public:
  explicit ShmStockConnection(std::shared_ptr<ConnectionImpl> impl) : impl_(std::move(impl)) {}
  ~ShmStockConnection() override {
    impl_->close();
  }
  void read(read_callback_fn fn) override {
    impl_->read(std::move(fn));
  }
  void read(void* ptr, size_t length, read_callback_fn fn) override {
    impl_->read(ptr, length, std::move(fn));
  }
  void write(const void* ptr, size_t length, write_callback_fn fn) override {
    impl_->write(ptr, length, std::move(fn));
  }
  void read(AbstractNopHolder& object, read_nop_callback_fn fn) override {
    impl_->read([&object, fn{std::move(fn)}](const Error& error, const void* ptr, size_t len) {
      if (!error && !object.deserialize(static_cast<const uint8_t*>(ptr), len)) {
        fn(TP_CREATE_ERROR(ShortReadError, -1, static_cast<ssize_t>(len)));
        return;
      }
      fn(error);
    });
  }
  void write(const AbstractNopHolder& object, write_callback_fn fn) override {
    auto buf = std::make_shared<std::vector<uint8_t>>(object.getSize());
    object.serialize(buf->data(), buf->size());
    impl_->write(buf->data(), buf->size(), [buf, fn{std::move(fn)}](const Error& error) { fn(error); });
  }
  void setId(std::string id) override {
    impl_->setId(std::move(id));
  }
  void close() override {
    impl_->close();
  }

 private:
  std::shared_ptr<ConnectionImpl> impl_;
};

// tensorpipe/transport/shm/listener_impl.cc:39-150
class ListenerImpl final : public FdHandler, public std::enable_shared_from_this<ListenerImpl> {
 public:
  using accept_callback_fn = Listener::accept_callback_fn;

  ListenerImpl(std::shared_ptr<Reactor> reactor, const std::string& name) : reactor_(std::move(reactor)) {
    fd_ = ::socket(AF_UNIX, SOCK_STREAM | SOCK_NONBLOCK | SOCK_CLOEXEC, 0);
    TP_THROW_ASSERT_IF(fd_ < 0);
    sockaddr_un sun;
    const socklen_t len = abstractAddress(name, &sun);
    if (::bind(fd_, reinterpret_cast<sockaddr*>(&sun), len) != 0 || ::listen(fd_, 128) != 0) {
      const int err = errno;
      ::close(fd_);
      fd_ = -1;
      throw std::runtime_error("cannot listen on shm://" + name + ": " + std::strerror(err));
    }
    sockaddr_un bound;
    socklen_t boundLen = sizeof(bound);
    std::memset(&bound, 0, sizeof(bound));
    ::getsockname(fd_, reinterpret_cast<sockaddr*>(&bound), &boundLen);
    // an abstract name: everything after the leading NUL (tensorpipe/transport/shm/sockaddr.cc:57-69)
    if (boundLen > sizeof(bound.sun_family) + 1) {
      addr_.assign(&bound.sun_path[1], boundLen - sizeof(bound.sun_family) - 1);
    }
  }

  ~ListenerImpl() override {
    if (fd_ >= 0) {
      ::close(fd_);
    }
  }

  void init() {
    auto self = shared_from_this();
    reactor_->defer([self] {
      self->reactor_->enroll(self);
      if (self->reactor_->closed()) {
        self->fail(TP_CREATE_ERROR(ContextClosedError));
      }
    });
  }

  void accept(accept_callback_fn fn) {
    auto self = shared_from_this();
    reactor_->defer([self, fn{std::move(fn)}]() mutable {
      if (self->error_) {
        fn(self->error_, nullptr);
        return;
      }
      self->acceptors_.push_back(std::move(fn));
      self->drain();
      self->updateInterest();
    });
  }

  const std::string& addr() const {
    return addr_;
  }

  void close() {
    auto self = shared_from_this();
    reactor_->defer([self] { self->fail(TP_CREATE_ERROR(ListenerClosedError)); });
  }

  void onEvents(uint32_t /*events*/) override {
    drain();
    updateInterest();
  }

  void shutdownFromLoop() override {
    fail(TP_CREATE_ERROR(ContextClosedError));
  }

 private:
  void updateInterest() {
    if (fd_ < 0 || error_) {
      return;
    }
    const uint32_t want = acceptors_.empty() ? 0u : static_cast<uint32_t>(EPOLLIN);
    if (!registered_ || want != interest_) {
      reactor_->setInterest(fd_, this, want, &registered_);
      interest_ = want;
    }
  }

  void drain() {
    while (!acceptors_.empty() && !error_) {
      const int fd = ::accept4(fd_, nullptr, nullptr, SOCK_CLOEXEC | SOCK_NONBLOCK);
      if (fd < 0) {
        if (errno == EAGAIN || errno == EWOULDBLOCK || errno == EINTR || errno == ECONNABORTED) {
          return;
        }
        fail(TP_CREATE_ERROR(SystemError, "accept", errno));
        return;
      }
      auto fn = std::move(acceptors_.front());
      acceptors_.pop_front();
      auto conn = std::make_shared<ConnectionImpl>(reactor_, fd);
      conn->init();
      fn(Error::kSuccess, std::make_shared<ShmStockConnection>(std::move(conn)));
    }
  }

  void fail(Error error) {
    if (error_) {
      return;
    }
    error_ = std::move(error);
    if (fd_ >= 0) {
      if (registered_) {
        reactor_->forget(fd_);
      }
      ::close(fd_);
      fd_ = -1;
    }
    auto acceptors = std::move(acceptors_);
    acceptors_.clear();
    for (auto& fn : acceptors) {
      fn(error_, nullptr);
    }
    reactor_->unenroll(shared_from_this());
  }

  std::shared_ptr<Reactor> reactor_;
  std::string addr_;
  int fd_{-1};
  bool registered_{false};
  uint32_t interest_{0};
  Error error_;
  std::deque<accept_callback_fn> acceptors_;
};

class ShmStockListener final : public Listener {
 public:
  explicit ShmStockListener(std::shared_ptr<ListenerImpl> impl) : impl_(std::move(impl)) {}
  ~ShmStockListener() override {
    impl_->close();
  }
  void accept(accept_callback_fn fn) override {
    impl_->accept(std::move(fn));
  }
  std::string addr() const override {
    return impl_->addr();
  }
  void setId(std::string /*id*/) override {}
  void close() override {
    impl_->close();
  }

 private:
  std::shared_ptr<ListenerImpl> impl_;
};

class ShmStockContext final : public Context {
 public:
  ShmStockContext() : domain_(makeDomainDescriptor()) {
    Segment probe; // tensorpipe/transport/shm/context_impl.cc:49-58: can such memory be had at all?
    viable_ = !domain_.empty() && probe.create(1024 * 1024);
    if (viable_) {
      reactor_ = std::make_shared<Reactor>();
    }
  }
  ~ShmStockContext() override {
    if (reactor_) {
      reactor_->join();
    }
  }
  std::shared_ptr<Connection> connect(std::string addr) override {
    TP_THROW_ASSERT_IF(!viable_);
    auto conn = std::make_shared<ConnectionImpl>(reactor_, std::move(addr));
    conn->init();
    return std::make_shared<ShmStockConnection>(std::move(conn));
  }
  std::shared_ptr<Listener> listen(std::string addr) override {
    TP_THROW_ASSERT_IF(!viable_);
    auto l = std::make_shared<ListenerImpl>(reactor_, addr);
    l->init();
    return std::make_shared<ShmStockListener>(std::move(l));
  }
  bool isViable() const override {
    return viable_;
  }
  const std::string& domainDescriptor() const override {
    return domain_;
  }
  void setId(std::string /*id*/) override {}
  void close() override {
    if (reactor_) {
      reactor_->close();
    }
  }
  void join() override {
    if (reactor_) {
      reactor_->join();
    }
  }

 private:
  const std::string domain_;
  bool viable_{false};
  std::shared_ptr<Reactor> reactor_;
};

} // namespace

std::shared_ptr<Context> create() {
  return std::make_shared<ShmStockContext>();
}

} // namespace shm_stock
} // namespace transport
TP_AMD_NAMESPACE_END
