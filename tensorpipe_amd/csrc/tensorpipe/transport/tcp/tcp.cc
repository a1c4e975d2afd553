// TCP transport, wire-compatible with the reference's uv transport: a message
// is an 8-byte little-endian length and then the bytes
// (tensorpipe/common/stream_read_write_ops.h:30-65,146-188). One reactor thread
// per context (epoll, level-triggered) runs every socket of that context; a
// socket asks for readability only while a read is posted and for writability
// only while bytes are queued, so an idle connection costs nothing. Own design;
// the reference drives libuv (tensorpipe/transport/uv/*).

#include <tensorpipe/transport/tcp/factory.h>

#include <arpa/inet.h>
#include <fcntl.h>
#include <netinet/in.h>
#include <netinet/tcp.h>
#include <sys/epoll.h>
#include <sys/eventfd.h>
#include <sys/socket.h>
#include <unistd.h>

#include <sched.h>

#include <algorithm>
#include <atomic>
#include <cerrno>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <mutex>
#include <set>
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
namespace tcp {

namespace {

constexpr size_t kHeader = 8;
constexpr uint64_t kGrowBytes = 1 << 20; // step in which the buffer of an unsized read grows

class FdHandler {
 public:
  virtual void onEvents(uint32_t events) = 0;
  virtual void shutdownFromLoop() = 0;
  virtual ~FdHandler() = default;
};

// "a.b.c.d:port", "a.b.c.d", "[v6 address]:port" or "[v6 address]", as the
// reference's uv transport writes its addresses (tensorpipe/transport/uv/sockaddr.cc).
bool parseAddr(const std::string& addr, sockaddr_storage* out, socklen_t* len) {
  std::memset(out, 0, sizeof(*out));
  if (!addr.empty() && addr[0] == '[') {
    const size_t close = addr.find(']');
    if (close == std::string::npos) {
      return false;
    }
    int port = 0;
    if (close + 1 < addr.size()) {
      if (addr[close + 1] != ':') {
        return false;
      }
      port = std::atoi(addr.c_str() + close + 2);
    }
    auto* sa = reinterpret_cast<sockaddr_in6*>(out);
    sa->sin6_family = AF_INET6;
    sa->sin6_port = htons(static_cast<uint16_t>(port));
    *len = sizeof(sockaddr_in6);
    return ::inet_pton(AF_INET6, addr.substr(1, close - 1).c_str(), &sa->sin6_addr) == 1;
  }
  std::string host = addr;
  int port = 0;
  const size_t colon = addr.rfind(':');
  if (colon != std::string::npos) {
    host = addr.substr(0, colon);
    port = std::atoi(addr.c_str() + colon + 1);
  }
  auto* sa = reinterpret_cast<sockaddr_in*>(out);
  sa->sin_family = AF_INET;
  sa->sin_port = htons(static_cast<uint16_t>(port));
  *len = sizeof(sockaddr_in);
  return ::inet_pton(AF_INET, host.c_str(), &sa->sin_addr) == 1;
}

std::string formatAddr(const sockaddr_storage& ss) {
  char host[INET6_ADDRSTRLEN] = {0};
  if (ss.ss_family == AF_INET6) {
    const auto* sa = reinterpret_cast<const sockaddr_in6*>(&ss);
    ::inet_ntop(AF_INET6, &sa->sin6_addr, host, sizeof(host));
    return "[" + std::string(host) + "]:" + std::to_string(ntohs(sa->sin6_port));
  }
  const auto* sa = reinterpret_cast<const sockaddr_in*>(&ss);
  ::inet_ntop(AF_INET, &sa->sin_addr, host, sizeof(host));
  return std::string(host) + ":" + std::to_string(ntohs(sa->sin_port));
}

class Reactor final : public std::enable_shared_from_this<Reactor> {
 public:
  Reactor() {
    epollFd_ = ::epoll_create1(EPOLL_CLOEXEC);
    wakeFd_ = ::eventfd(0, EFD_NONBLOCK | EFD_CLOEXEC);
    TP_THROW_ASSERT_IF(epollFd_ < 0 || wakeFd_ < 0);
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

  bool inLoop() const {
    return std::this_thread::get_id() == thread_.get_id();
  }

  void defer(std::function<void()> fn) {
    {
      std::lock_guard<std::mutex> lock(mutex_);
      if (stopped_) {
        // The thread is gone: run late tasks (closes, callbacks with errors)
        // one at a time on whoever brings them.
        lateTasks_.push_back(std::move(fn));
        if (lateRunning_) {
          return;
        }
        lateRunning_ = true;
      } else {
        tasks_.push_back(std::move(fn));
        const uint64_t one = 1;
        (void)!::write(wakeFd_, &one, sizeof(one));
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

  // Loop only.
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
    // After an event the loop keeps asking without sleeping for a short while:
    // in a ping-pong the next message is a few microseconds away, and a wake-up
    // from epoll costs more than that (TP_TCP_SPIN_US, 0 = always sleep; no
    // spinning where the process has fewer than four CPUs to run on).
    const long spinUs = [] {
      const char* e = std::getenv("TP_TCP_SPIN_US");
      long v = e != nullptr ? std::atol(e) : 100;
      cpu_set_t set;
      CPU_ZERO(&set);
      if (::sched_getaffinity(0, sizeof(set), &set) == 0 && CPU_COUNT(&set) < 4) {
        v = 0;
      }
      return v;
    }();
    auto lastEvent = std::chrono::steady_clock::now() - std::chrono::seconds(1);
    while (!stop_) {
      const bool spin = spinUs > 0 &&
          std::chrono::steady_clock::now() - lastEvent < std::chrono::microseconds(spinUs);
      const int n = ::epoll_wait(epollFd_, events.data(), static_cast<int>(events.size()), spin ? 0 : -1);
      if (n > 0) {
        lastEvent = std::chrono::steady_clock::now();
      }
      for (int i = 0; i < n; ++i) {
        if (events[i].data.ptr == nullptr) {
          uint64_t v;
          (void)!::read(wakeFd_, &v, sizeof(v));
          continue;
        }
        // A handler may be destroyed by an earlier event of this batch: only
        // those still enrolled are called.
        FdHandler* h = static_cast<FdHandler*>(events[i].data.ptr);
        // (the set orders its members by address: an owner-less pointer to the
        // same address finds the member)
        const auto it = live_.find(std::shared_ptr<FdHandler>(std::shared_ptr<FdHandler>(), h));
        if (it != live_.end()) {
          std::shared_ptr<FdHandler> keep = *it;
          keep->onEvents(events[i].events);
        }
      }
      runTasks();
    }
    // Whatever is still enrolled goes down with the loop.
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

  void runTasks() {
    for (;;) {
      std::deque<std::function<void()>> batch;
      {
        std::lock_guard<std::mutex> lock(mutex_);
        batch.swap(tasks_);
      }
      if (batch.empty()) {
        return;
      }
      for (auto& t : batch) {
        t();
      }
    }
  }

  int epollFd_{-1};
  int wakeFd_{-1};
  std::thread thread_;
  std::mutex mutex_;
  std::deque<std::function<void()>> tasks_;
  std::deque<std::function<void()>> lateTasks_;
  bool lateRunning_{false};
  bool stopped_{false};
  bool joined_{false};
  bool stop_{false}; // loop only
  std::atomic<bool> closed_{false};
  std::set<std::shared_ptr<FdHandler>> live_; // loop only
};

class ConnectionImpl final : public FdHandler, public std::enable_shared_from_this<ConnectionImpl> {
 public:
  using read_callback_fn = Connection::read_callback_fn;
  using write_callback_fn = Connection::write_callback_fn;

  // Client end: connects from the loop.
  ConnectionImpl(std::shared_ptr<Reactor> reactor, std::string addr)
      : reactor_(std::move(reactor)), addr_(std::move(addr)) {}
  // Accepted end.
  ConnectionImpl(std::shared_ptr<Reactor> reactor, int fd) : reactor_(std::move(reactor)), fd_(fd), connected_(true) {}

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
      WriteOp op;
      for (size_t i = 0; i < kHeader; ++i) {
        op.header[i] = static_cast<uint8_t>(static_cast<uint64_t>(length) >> (8 * i));
      }
      op.ptr = static_cast<const uint8_t*>(ptr);
      op.length = length;
      op.fn = std::move(fn);
      if (self->error_) {
        op.fn(self->error_);
        return;
      }
      self->writes_.push_back(std::move(op));
      self->pumpWrites();
      self->updateInterest();
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

  void onEvents(uint32_t events) override {
    if (error_) {
      return;
    }
    if (!connected_) {
      if (events & (EPOLLOUT | EPOLLERR | EPOLLHUP)) {
        int err = 0;
        socklen_t len = sizeof(err);
        ::getsockopt(fd_, SOL_SOCKET, SO_ERROR, &err, &len);
        if (err != 0) {
          fail(TP_CREATE_ERROR(SystemError, "connect", err));
          return;
        }
        connected_ = true;
      } else {
        return;
      }
    }
    if (events & (EPOLLIN | EPOLLRDHUP | EPOLLHUP | EPOLLERR)) {
      if (events & (EPOLLRDHUP | EPOLLHUP | EPOLLERR)) {
        peerClosed_ = true; // what it sent before leaving is still delivered
      }
      if (events & (EPOLLHUP | EPOLLERR)) {
        // epoll reports these two whatever was asked for, and keeps reporting
        // them: the socket leaves the set, and from here on reads and writes
        // find out what the socket holds when they are posted.
        hungUp_ = true;
        if (registered_) {
          reactor_->forget(fd_);
          registered_ = false;
        }
      }
      pumpReads(); // with nobody reading, the hang-up is remembered and no longer asked about
    }
    if (!error_ && (events & EPOLLOUT)) {
      pumpWrites();
    }
    if (!error_) {
      updateInterest();
    }
  }

  void shutdownFromLoop() override {
    fail(TP_CREATE_ERROR(ContextClosedError));
  }

 private:
  struct ReadOp {
    uint8_t* ptr;
    size_t length;
    bool exact; // into the caller's buffer, which must be exactly the message's size
    read_callback_fn fn;
  };
  struct WriteOp {
    uint8_t header[kHeader];
    const uint8_t* ptr{nullptr};
    size_t length{0};
    size_t done{0}; // of header + payload
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
      sockaddr_storage sa;
      socklen_t salen = 0;
      if (!parseAddr(addr_, &sa, &salen)) {
        fail(TP_CREATE_ERROR(SystemError, "inet_pton", EINVAL));
        return;
      }
      fd_ = ::socket(sa.ss_family, SOCK_STREAM | SOCK_NONBLOCK | SOCK_CLOEXEC, 0);
      if (fd_ < 0) {
        fail(TP_CREATE_ERROR(SystemError, "socket", errno));
        return;
      }
      const int rc = ::connect(fd_, reinterpret_cast<sockaddr*>(&sa), salen);
      if (rc != 0 && errno != EINPROGRESS) {
        fail(TP_CREATE_ERROR(SystemError, "connect", errno));
        return;
      }
      connected_ = rc == 0;
    } else {
      const int flags = ::fcntl(fd_, F_GETFL, 0);
      ::fcntl(fd_, F_SETFL, flags | O_NONBLOCK);
    }
    int one = 1;
    ::setsockopt(fd_, IPPROTO_TCP, TCP_NODELAY, &one, sizeof(one));
    updateInterest();
    if (connected_) {
      pumpWrites();
      pumpReads();
      if (!error_) {
        updateInterest();
      }
    }
  }

  void updateInterest() {
    if (fd_ < 0 || error_ || hungUp_) {
      return;
    }
    uint32_t want = 0;
    if (!connected_) {
      want = EPOLLOUT;
    } else {
      if (!reads_.empty()) {
        want |= EPOLLIN;
      }
      if (!writes_.empty()) {
        want |= EPOLLOUT;
      }
      if (!peerClosed_) {
        want |= EPOLLRDHUP;
      }
    }
    if (!registered_ || want != interest_) {
      reactor_->setInterest(fd_, this, want, &registered_);
      interest_ = want;
    }
  }

  void enqueueRead(ReadOp op) {
    if (error_) {
      op.fn(error_, nullptr, 0);
      return;
    }
    reads_.push_back(std::move(op));
    if (connected_) {
      pumpReads();
    }
    if (!error_) {
      updateInterest();
    }
  }

  // Moves what the socket holds into the read at the head of the queue; calls
  // back for every message completed.
  void pumpReads() {
    while (!reads_.empty() && !error_) {
      ReadOp& op = reads_.front();
      if (headerDone_ < kHeader) {
        const ssize_t r = recvRetrying(header_ + headerDone_, kHeader - headerDone_);
        if (!absorb(r)) {
          return;
        }
        headerDone_ += static_cast<size_t>(r);
        if (headerDone_ < kHeader) {
          continue;
        }
        messageLength_ = 0;
        for (size_t i = 0; i < kHeader; ++i) {
          messageLength_ |= static_cast<uint64_t>(header_[i]) << (8 * i);
        }
        payloadDone_ = 0;
        if (op.exact) {
          if (messageLength_ != op.length) {
            fail(TP_CREATE_ERROR(
                ShortReadError, static_cast<ssize_t>(op.length), static_cast<ssize_t>(messageLength_)));
            return;
          }
        } else {
          if (messageLength_ > (uint64_t(1) << 40)) {
            fail(TP_CREATE_ERROR(ShortReadError, -1, static_cast<ssize_t>(messageLength_)));
            return;
          }
          scratch_.clear();
        }
      }
      while (payloadDone_ < messageLength_) {
        uint64_t room = messageLength_ - payloadDone_;
        if (!op.exact) {
          // The length is the peer's word: the buffer grows with the bytes
          // that really arrive, not with the announcement.
          room = std::min<uint64_t>(room, kGrowBytes);
          if (scratch_.size() < payloadDone_ + room) {
            scratch_.resize(static_cast<size_t>(payloadDone_ + room));
          }
        }
        uint8_t* dst = op.exact ? op.ptr : scratch_.data();
        const ssize_t r = recvRetrying(dst + payloadDone_, static_cast<size_t>(room));
        if (!absorb(r)) {
          return;
        }
        payloadDone_ += static_cast<size_t>(r);
      }
      uint8_t* dst = op.exact ? op.ptr : scratch_.data();
      ReadOp finished = std::move(op);
      reads_.pop_front();
      headerDone_ = 0;
      finished.fn(Error::kSuccess, dst, static_cast<size_t>(messageLength_));
    }
  }

  // recv() that starts over when a signal cut it short: after the hang-up has
  // taken the socket out of the epoll set nothing else would ask again.
  ssize_t recvRetrying(uint8_t* dst, size_t room) {
    for (;;) {
      const ssize_t r = ::recv(fd_, dst, room, 0);
      if (r >= 0 || errno != EINTR) {
        return r;
      }
    }
  }

  // Whether recv's result is bytes to use; EOF and errors fail the connection,
  // "nothing yet" just returns false.
  bool absorb(ssize_t r) {
    if (r > 0) {
      return true;
    }
    if (r == 0) {
      fail(TP_CREATE_ERROR(EOFError));
      return false;
    }
    if (errno == EAGAIN || errno == EWOULDBLOCK) {
      if (peerClosed_) {
        // the hang-up was seen and the socket is drained
        fail(TP_CREATE_ERROR(EOFError));
      }
      return false;
    }
    fail(TP_CREATE_ERROR(SystemError, "recv", errno));
    return false;
  }

  void pumpWrites() {
    if (!connected_) {
      return;
    }
    while (!writes_.empty() && !error_) {
      WriteOp& op = writes_.front();
      const size_t total = kHeader + op.length;
      while (op.done < total) {
        ssize_t r;
        if (op.done < kHeader) {
          iovec iov[2];
          iov[0].iov_base = op.header + op.done;
          iov[0].iov_len = kHeader - op.done;
          iov[1].iov_base = const_cast<uint8_t*>(op.ptr);
          iov[1].iov_len = op.length;
          msghdr msg{};
          msg.msg_iov = iov;
          msg.msg_iovlen = op.length > 0 ? 2 : 1;
          r = ::sendmsg(fd_, &msg, MSG_NOSIGNAL);
        } else {
          r = ::send(fd_, op.ptr + (op.done - kHeader), total - op.done, MSG_NOSIGNAL);
        }
        if (r < 0) {
          if (errno == EAGAIN || errno == EWOULDBLOCK) {
            if (hungUp_) {
              fail(TP_CREATE_ERROR(EOFError)); // nobody will ever say "writable" again
            }
            return;
          }
          if (errno == EINTR) {
            continue;
          }
          fail(TP_CREATE_ERROR(SystemError, "send", errno));
          return;
        }
        op.done += static_cast<size_t>(r);
      }
      WriteOp finished = std::move(op);
      writes_.pop_front();
      finished.fn(Error::kSuccess);
    }
  }

  void fail(Error error) {
    if (error_) {
      return;
    }
    error_ = std::move(error);
    TP_VLOG(8) << "Connection " << id_ << " is failing: " << error_.what();
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
  bool connected_{false};
  bool registered_{false};
  bool peerClosed_{false};
  bool hungUp_{false}; // EPOLLHUP or EPOLLERR was seen; the socket is out of the epoll set
  uint32_t interest_{0};
  Error error_;
  std::deque<ReadOp> reads_;
  std::deque<WriteOp> writes_;
  uint8_t header_[kHeader];
  size_t headerDone_{0};
  uint64_t messageLength_{0};
  uint64_t payloadDone_{0};
  std::vector<uint8_t> scratch_;
};

class TcpConnection final : public Connection {
 public:
  explicit TcpConnection(std::shared_ptr<ConnectionImpl> impl) : impl_(std::move(impl)) {}
  ~TcpConnection() override {
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

class ListenerImpl final : public FdHandler, public std::enable_shared_from_this<ListenerImpl> {
 public:
  using accept_callback_fn = Listener::accept_callback_fn;

  // Binds at once, so that the address is known when listen() returns.
  ListenerImpl(std::shared_ptr<Reactor> reactor, const std::string& addr) : reactor_(std::move(reactor)) {
    sockaddr_storage sa;
    socklen_t salen = 0;
    TP_THROW_ASSERT_IF(!parseAddr(addr, &sa, &salen));
    fd_ = ::socket(sa.ss_family, SOCK_STREAM | SOCK_NONBLOCK | SOCK_CLOEXEC, 0);
    TP_THROW_ASSERT_IF(fd_ < 0);
    int one = 1;
    ::setsockopt(fd_, SOL_SOCKET, SO_REUSEADDR, &one, sizeof(one));
    if (::bind(fd_, reinterpret_cast<sockaddr*>(&sa), salen) != 0 || ::listen(fd_, 128) != 0) {
      const int err = errno;
      ::close(fd_);
      fd_ = -1;
      throw std::runtime_error("cannot listen on " + addr + ": " + std::strerror(err));
    }
    socklen_t len = sizeof(sa);
    ::getsockname(fd_, reinterpret_cast<sockaddr*>(&sa), &len);
    addr_ = formatAddr(sa);
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
      fn(Error::kSuccess, std::make_shared<TcpConnection>(std::move(conn)));
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

class TcpListener final : public Listener {
 public:
  explicit TcpListener(std::shared_ptr<ListenerImpl> impl) : impl_(std::move(impl)) {}
  ~TcpListener() override {
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

class TcpContext final : public Context {
 public:
  TcpContext() : reactor_(std::make_shared<Reactor>()) {}
  ~TcpContext() override {
    reactor_->join();
  }
  std::shared_ptr<Connection> connect(std::string addr) override {
    auto conn = std::make_shared<ConnectionImpl>(reactor_, std::move(addr));
    conn->init();
    return std::make_shared<TcpConnection>(std::move(conn));
  }
  std::shared_ptr<Listener> listen(std::string addr) override {
    if (addr.empty()) {
      addr = "127.0.0.1:0";
    }
    auto l = std::make_shared<ListenerImpl>(reactor_, addr);
    l->init();
    return std::make_shared<TcpListener>(std::move(l));
  }
  bool isViable() const override {
    return true;
  }
  const std::string& domainDescriptor() const override {
    // What the reference's uv context announces
    // (tensorpipe/transport/uv/context_impl.cc: "uv:*").
    static const std::string d = "uv:*";
    return d;
  }
  void setId(std::string /*id*/) override {}
  void close() override {
    reactor_->close();
  }
  void join() override {
    reactor_->join();
  }

 private:
  std::shared_ptr<Reactor> reactor_;
};

} // namespace

std::shared_ptr<Context> create() {
  return std::make_shared<TcpContext>();
}

} // namespace tcp
} // namespace transport
TP_AMD_NAMESPACE_END
