// Shared scaffolding of the C++ test programs: a tiny case registry with
// EXPECT-style checks, a two-endpoint runner (two threads of one process, or
// two processes started by an orchestrator that never touches the GPU), and
// helpers that wrap host and device memory for the tests.
//
// The test programs exercise the product's C++ API (channel::Context /
// channel::Channel, Context / Listener / Pipe) exactly where a user of the
// reference would call it; the cases follow tensorpipe/test/channel/*.cc and
// tensorpipe/test/core/pipe_cuda_test.cc (cited at each case).
#pragma once

#include <dirent.h>
#include <execinfo.h>
#include <signal.h>
#include <sys/syscall.h>
#include <sys/types.h>
#include <sys/wait.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <future>
#include <memory>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include <tensorpipe/channel/channel.h>
#include <tensorpipe/tensorpipe.h>
#include <tensorpipe/tensorpipe_hip.h>
#include <tensorpipe/transport/connection.h>
#include <tensorpipe/transport/listener.h>
#include <tphip.h>

namespace tptest {

using namespace tensorpipe;

constexpr int kWaitSeconds = 30;

// ---- where a stuck program's threads are --------------------------------------
// `kill -USR1 <pid>` (or `timeout -s USR1 ...`) makes every thread write its
// call stack to stderr as module + offset lines (addr2line names them): what a
// program that hangs once in a hundred runs is asked when no debugger is at hand.

inline void writeOwnStack(int) {
  void* frames[64];
  const int n = ::backtrace(frames, 64);
  char head[64];
  const int len = std::snprintf(head, sizeof(head), "--- stack of thread %ld\n", static_cast<long>(::syscall(SYS_gettid)));
  (void)!::write(2, head, static_cast<size_t>(len));
  ::backtrace_symbols_fd(frames, n, 2);
}

inline void askEveryThreadForItsStack(int) {
  DIR* dir = ::opendir("/proc/self/task");
  if (dir == nullptr) {
    return;
  }
  while (dirent* entry = ::readdir(dir)) {
    const long tid = std::atol(entry->d_name);
    if (tid > 0) {
      ::syscall(SYS_tgkill, ::getpid(), tid, SIGUSR2);
      ::usleep(20000); // one stack at a time keeps the lines together
    }
  }
  ::closedir(dir);
}

inline void installStackDumper() {
  void* warm[2];
  (void)::backtrace(warm, 2); // loads what backtrace() needs outside a handler
  struct sigaction own {};
  own.sa_handler = writeOwnStack;
  ::sigaction(SIGUSR2, &own, nullptr);
  struct sigaction all {};
  all.sa_handler = askEveryThreadForItsStack;
  ::sigaction(SIGUSR1, &all, nullptr);
}

// ---- failure bookkeeping ----------------------------------------------------

struct Failures {
  std::mutex mutex;
  std::vector<std::string> messages;
  void add(const std::string& m) {
    std::lock_guard<std::mutex> lock(mutex);
    messages.push_back(m);
  }
  bool any() {
    std::lock_guard<std::mutex> lock(mutex);
    return !messages.empty();
  }
  std::string joined() {
    std::lock_guard<std::mutex> lock(mutex);
    std::string s;
    for (auto& m : messages) {
      s += (s.empty() ? "" : "; ") + m;
    }
    return s;
  }
  void clear() {
    std::lock_guard<std::mutex> lock(mutex);
    messages.clear();
  }
};

inline Failures& failures() {
  static Failures f;
  return f;
}

// Raised when going on would leave the two endpoints out of step (a wait timed
// out): ends the case and every case after it.
struct Fatal : std::runtime_error {
  using std::runtime_error::runtime_error;
};

#define TPT_STR2(x) #x
#define TPT_STR(x) TPT_STR2(x)
#define EXPECT_TRUE(cond)                                                         \
  do {                                                                            \
    if (!(cond)) {                                                                \
      ::tptest::failures().add(__FILE__ ":" TPT_STR(__LINE__) " expected " #cond); \
    }                                                                             \
  } while (0)
#define EXPECT_FALSE(cond) EXPECT_TRUE(!(cond))
#define EXPECT_EQ(a, b)                                                              \
  do {                                                                               \
    auto va_ = (a);                                                                  \
    auto vb_ = (b);                                                                  \
    if (!(va_ == vb_)) {                                                             \
      std::ostringstream ss_;                                                        \
      ss_ << __FILE__ ":" TPT_STR(__LINE__) " expected " #a " == " #b " (" << va_    \
          << " vs " << vb_ << ")";                                                   \
      ::tptest::failures().add(ss_.str());                                           \
    }                                                                                \
  } while (0)
#define EXPECT_OK(err)                                                                     \
  do {                                                                                     \
    const ::tensorpipe::Error& e_ = (err);                                                 \
    if (e_) {                                                                              \
      ::tptest::failures().add(__FILE__ ":" TPT_STR(__LINE__) " unexpected error: " + e_.what()); \
    }                                                                                      \
  } while (0)
#define HIP_OK(call)                                                                    \
  do {                                                                                  \
    int rc_ = (call);                                                                   \
    if (rc_ != 0) {                                                                     \
      throw ::tptest::Fatal(std::string(#call " failed: ") + tphip_strerror(rc_));      \
    }                                                                                   \
  } while (0)

template <typename T>
T waitFor(std::future<T>& f, const char* what) {
  if (f.wait_for(std::chrono::seconds(kWaitSeconds)) != std::future_status::ready) {
    throw Fatal(std::string("timed out waiting for ") + what);
  }
  return f.get();
}

// ---- memory -----------------------------------------------------------------

// Host or device bytes behind one interface (the role of DataWrapper in
// tensorpipe/test/channel/channel_test.h:31-37).
class Data {
 public:
  virtual Buffer buffer() = 0;
  virtual size_t size() const = 0;
  virtual std::vector<uint8_t> bytes() = 0;
  virtual ~Data() = default;
};

class CpuData final : public Data {
 public:
  explicit CpuData(size_t n) : v_(n, 0) {}
  explicit CpuData(std::vector<uint8_t> v) : v_(std::move(v)) {}
  Buffer buffer() override {
    return CpuBuffer{v_.data()};
  }
  size_t size() const override {
    return v_.size();
  }
  std::vector<uint8_t> bytes() override {
    return v_;
  }

 private:
  std::vector<uint8_t> v_;
};

// Device allocations of the tests are at least this large, as the segments of
// a framework's caching allocator are; a case that wants the exact size (the
// runtime then carves the allocation out of a block it shares with others)
// holds an ExactGpuAllocations while it allocates.
inline std::atomic<int>& exactGpuAllocationHolders() {
  static std::atomic<int> n{0};
  return n;
}
inline size_t minGpuAllocation() {
  return exactGpuAllocationHolders().load() > 0 ? size_t(1) : size_t(2) << 20;
}
struct ExactGpuAllocations {
  ExactGpuAllocations() {
    ++exactGpuAllocationHolders();
  }
  ~ExactGpuAllocations() {
    --exactGpuAllocationHolders();
  }
};

class GpuData final : public Data {
 public:
  // `offset` bytes of 0xff precede the payload inside the allocation.
  explicit GpuData(size_t n, size_t offset = 0) : n_(n), offset_(offset) {
    HIP_OK(tphip_malloc(0, std::max(n + offset, minGpuAllocation()), &base_));
    HIP_OK(tphip_stream_create(0, &stream_));
    HIP_OK(tphip_fill(0, base_, 0xff, n + offset, stream_));
    HIP_OK(tphip_stream_sync(0, stream_));
  }
  explicit GpuData(const std::vector<uint8_t>& v, size_t offset = 0) : GpuData(v.size(), offset) {
    if (!v.empty()) {
      HIP_OK(tphip_memcpy_async(0, ptr(), v.data(), v.size(), stream_));
      HIP_OK(tphip_stream_sync(0, stream_));
    }
  }
  ~GpuData() override {
    tphip_stream_sync(0, stream_);
    tphip_stream_destroy(0, stream_);
    tphip_free(0, base_);
  }
  void* ptr() {
    return static_cast<uint8_t*>(base_) + offset_;
  }
  void* stream() {
    return stream_;
  }
  Buffer buffer() override {
    return HipBuffer{ptr(), stream_};
  }
  size_t size() const override {
    return n_;
  }
  std::vector<uint8_t> bytes() override {
    std::vector<uint8_t> out(n_);
    if (n_ > 0) {
      HIP_OK(tphip_memcpy_async(0, out.data(), ptr(), n_, stream_));
    }
    HIP_OK(tphip_stream_sync(0, stream_));
    return out;
  }

 private:
  size_t n_;
  size_t offset_;
  void* base_{nullptr};
  void* stream_{nullptr};
};

inline std::unique_ptr<Data> makeData(bool gpu, size_t n) {
  if (gpu) {
    return std::make_unique<GpuData>(n);
  }
  return std::make_unique<CpuData>(n);
}

inline std::unique_ptr<Data> makeData(bool gpu, const std::vector<uint8_t>& v) {
  if (gpu) {
    return std::make_unique<GpuData>(v);
  }
  return std::make_unique<CpuData>(v);
}

inline std::vector<uint8_t> iota(size_t n) {
  std::vector<uint8_t> v(n);
  for (size_t i = 0; i < n; ++i) {
    v[i] = static_cast<uint8_t>(i);
  }
  return v;
}

// ---- transport plumbing -------------------------------------------------------

inline std::shared_ptr<transport::Connection> acceptOne(transport::Listener& l) {
  auto p = std::make_shared<std::promise<std::pair<Error, std::shared_ptr<transport::Connection>>>>();
  auto f = p->get_future();
  l.accept([p](const Error& e, std::shared_ptr<transport::Connection> c) {
    p->set_value({e, std::move(c)});
  });
  auto r = waitFor(f, "accept");
  if (r.first) {
    throw Fatal("accept failed: " + r.first.what());
  }
  return r.second;
}

inline void writeByte(transport::Connection& c, uint8_t b) {
  auto p = std::make_shared<std::promise<Error>>();
  auto f = p->get_future();
  auto holder = std::make_shared<uint8_t>(b);
  c.write(holder.get(), 1, [p, holder](const Error& e) { p->set_value(e); });
  Error e = waitFor(f, "control write");
  if (e) {
    throw Fatal("control write failed: " + e.what());
  }
}

inline uint8_t readByte(transport::Connection& c) {
  auto p = std::make_shared<std::promise<Error>>();
  auto f = p->get_future();
  auto holder = std::make_shared<uint8_t>(0);
  c.read(holder.get(), 1, [p, holder](const Error& e, const void*, size_t) { p->set_value(e); });
  Error e = waitFor(f, "control read");
  if (e) {
    throw Fatal("control read failed: " + e.what());
  }
  return *holder;
}

enum class Role { kServer, kClient };

inline const char* roleName(Role r) {
  return r == Role::kServer ? "server" : "client";
}

// One endpoint's view of a test run: the persistent control connection to the
// peer plus a way to open `n` fresh, index-matched connections per case.
class Endpoint {
 public:
  Endpoint(Role role, std::string baseAddr) : role_(role), baseAddr_(std::move(baseAddr)) {
    transport_ = transport::shm::create();
  }

  ~Endpoint() {
    control_.reset();
    controlListener_.reset();
    transport_->join();
  }

  Role role() const {
    return role_;
  }
  bool isServer() const {
    return role_ == Role::kServer;
  }
  std::shared_ptr<transport::Context> transport() {
    return transport_;
  }

  // Server: start listening for the control connection (call before the
  // client exists). Client: nothing.
  void prepare() {
    if (isServer()) {
      controlListener_ = transport_->listen(baseAddr_ + "_ctl");
    }
  }

  void establishControl() {
    if (isServer()) {
      control_ = acceptOne(*controlListener_);
    } else {
      control_ = transport_->connect(baseAddr_ + "_ctl");
    }
    // One byte each way proves that the connection works.
    writeByte(*control_, 'H');
    if (readByte(*control_) != 'H') {
      throw Fatal("control handshake failed");
    }
  }

  // Address for the next rendezvous; both endpoints draw the same sequence.
  std::string freshAddr() {
    return baseAddr_ + "_c" + std::to_string(caseCounter_++);
  }
  // Server: "I listen at the address drawn last". Client: wait for that.
  void signalListening() {
    writeByte(*control_, 'L');
  }
  void awaitListening() {
    if (readByte(*control_) != 'L') {
      throw Fatal("expected the listening notice");
    }
  }

  // A small number from one endpoint to the other (a port that the listening
  // side only learns once it is bound).
  void sendNumber(uint16_t v) {
    writeByte(*control_, static_cast<uint8_t>(v >> 8));
    writeByte(*control_, static_cast<uint8_t>(v & 0xff));
  }
  uint16_t recvNumber() {
    const uint16_t hi = readByte(*control_);
    return static_cast<uint16_t>(hi << 8 | readByte(*control_));
  }

  // `n` connections whose i-th ends pair up on both sides.
  std::vector<std::shared_ptr<transport::Connection>> openConnections(size_t n) {
    const std::string addr = freshAddr();
    std::vector<std::shared_ptr<transport::Connection>> conns(n);
    if (isServer()) {
      auto listener = transport_->listen(addr);
      signalListening(); // the client may connect now
      for (size_t i = 0; i < n; ++i) {
        auto c = acceptOne(*listener);
        const uint8_t idx = readByte(*c);
        if (idx >= n || conns[idx]) {
          throw Fatal("bad connection index");
        }
        conns[idx] = std::move(c);
      }
      listener->close();
    } else {
      awaitListening();
      for (size_t i = 0; i < n; ++i) {
        conns[i] = transport_->connect(addr);
        writeByte(*conns[i], static_cast<uint8_t>(i));
      }
    }
    return conns;
  }

  // Both endpoints call this before tearing a case down; returns once the
  // peer got there too (PeerGroup::done + join in the reference's harness).
  void barrier() {
    writeByte(*control_, 'B');
    if (readByte(*control_) != 'B') {
      throw Fatal("barrier out of step");
    }
  }

 private:
  const Role role_;
  const std::string baseAddr_;
  std::shared_ptr<transport::Context> transport_;
  std::shared_ptr<transport::Listener> controlListener_;
  std::shared_ptr<transport::Connection> control_;
  int caseCounter_{0};
};

// ---- case registry and runner -------------------------------------------------

struct Case {
  std::string name;
  std::function<void(Endpoint&)> server;
  std::function<void(Endpoint&)> client;
};

inline void runRole(Endpoint& ep, const std::vector<Case>& cases, const std::string& filter) {
  bool aborted = false;
  for (auto& c : cases) {
    if (!filter.empty() && c.name.find(filter) == std::string::npos) {
      continue;
    }
    if (aborted) {
      std::printf("RESULT %s %s SKIPPED (earlier case left the endpoints out of step)\n",
                  roleName(ep.role()), c.name.c_str());
      std::fflush(stdout);
      continue;
    }
    failures().clear();
    std::printf("RUN %s %s\n", roleName(ep.role()), c.name.c_str());
    std::fflush(stdout);
    try {
      (ep.isServer() ? c.server : c.client)(ep);
    } catch (const Fatal& f) {
      failures().add(std::string("fatal: ") + f.what());
      aborted = true;
    } catch (const std::exception& e) {
      failures().add(std::string("exception: ") + e.what());
      aborted = true;
    }
    if (failures().any()) {
      std::printf("RESULT %s %s FAIL %s\n", roleName(ep.role()), c.name.c_str(),
                  failures().joined().c_str());
    } else {
      std::printf("RESULT %s %s OK\n", roleName(ep.role()), c.name.c_str());
    }
    std::fflush(stdout);
  }
}

// In one process, two threads. Failures are shared, so a case fails if either
// endpoint fails; results are printed per role all the same.
inline int runBoth(const std::vector<Case>& cases, const std::string& filter,
                   const std::string& baseAddr) {
  // One case at a time so that the shared failure list belongs to that case.
  int failed = 0;
  for (auto& c : cases) {
    if (!filter.empty() && c.name.find(filter) == std::string::npos) {
      continue;
    }
    failures().clear();
    std::printf("RUN both %s\n", c.name.c_str());
    std::fflush(stdout);
    std::string fatal;
    std::mutex fatalMutex;
    {
      Endpoint server(Role::kServer, baseAddr + "_" + std::to_string(failed) + c.name);
      Endpoint client(Role::kClient, baseAddr + "_" + std::to_string(failed) + c.name);
      server.prepare();
      auto body = [&](Endpoint& ep, const std::function<void(Endpoint&)>& fn) {
        try {
          ep.establishControl();
          fn(ep);
        } catch (const std::exception& e) {
          std::lock_guard<std::mutex> lock(fatalMutex);
          fatal += std::string(roleName(ep.role())) + ": " + e.what() + "; ";
        }
      };
      std::thread st([&] { body(server, c.server); });
      std::thread ct([&] { body(client, c.client); });
      st.join();
      ct.join();
    }
    if (!fatal.empty()) {
      failures().add(fatal);
    }
    if (failures().any()) {
      ++failed;
      std::printf("RESULT both %s FAIL %s\n", c.name.c_str(), failures().joined().c_str());
    } else {
      std::printf("RESULT both %s OK\n", c.name.c_str());
    }
    std::fflush(stdout);
  }
  return failed == 0 ? 0 : 1;
}

inline int runSingleRole(Role role, const std::vector<Case>& cases, const std::string& filter,
                         const std::string& baseAddr, int readyFd) {
  Endpoint ep(role, baseAddr);
  ep.prepare();
  if (readyFd >= 0) {
    char b = 'R';
    ssize_t rc = ::write(readyFd, &b, 1);
    (void)rc;
    ::close(readyFd);
  }
  try {
    ep.establishControl();
  } catch (const std::exception& e) {
    std::printf("RESULT %s <setup> FAIL %s\n", roleName(role), e.what());
    std::fflush(stdout);
    return 1;
  }
  runRole(ep, cases, filter);
  return 0;
}

// Starts this program again as server and as client. The orchestrating process
// makes no GPU call, so starting children from it is safe.
inline int orchestrate(const char* self, const std::vector<std::string>& passThrough,
                       const std::string& baseAddr) {
  int readyPipe[2];
  if (::pipe(readyPipe) != 0) {
    std::perror("pipe");
    return 2;
  }
  auto spawn = [&](const char* role, int readyFd) -> pid_t {
    pid_t pid = ::fork();
    if (pid == 0) {
      std::vector<std::string> args = {self, "--role", role, "--addr", baseAddr};
      if (readyFd >= 0) {
        args.push_back("--ready-fd");
        args.push_back(std::to_string(readyFd));
      } else {
        ::close(readyPipe[1]);
      }
      ::close(readyPipe[0]);
      for (auto& a : passThrough) {
        args.push_back(a);
      }
      std::vector<char*> argv;
      for (auto& a : args) {
        argv.push_back(const_cast<char*>(a.c_str()));
      }
      argv.push_back(nullptr);
      ::execv("/proc/self/exe", argv.data());
      std::perror("execv");
      ::_exit(127);
    }
    return pid;
  };
  pid_t server = spawn("server", readyPipe[1]);
  ::close(readyPipe[1]);
  char b = 0;
  // Blocks until the server listens (or died: read returns 0).
  ssize_t rc = ::read(readyPipe[0], &b, 1);
  ::close(readyPipe[0]);
  if (rc != 1) {
    int st = 0;
    ::waitpid(server, &st, 0);
    std::printf("RESULT server <setup> FAIL server ended before listening\n");
    return 1;
  }
  pid_t client = spawn("client", -1);
  int st1 = 0, st2 = 0;
  ::waitpid(server, &st1, 0);
  ::waitpid(client, &st2, 0);
  const bool ok = WIFEXITED(st1) && WEXITSTATUS(st1) == 0 && WIFEXITED(st2) && WEXITSTATUS(st2) == 0;
  if (!ok) {
    std::printf("RESULT both <processes> FAIL exit statuses %d %d\n", st1, st2);
  }
  return ok ? 0 : 1;
}

struct Args {
  std::string role; // "", "server", "client", "both"
  std::string addr;
  std::string filter;
  std::string suite;
  int readyFd{-1};
  bool list{false};
};

inline Args parseArgs(int argc, char** argv) {
  installStackDumper();
  Args a;
  for (int i = 1; i < argc; ++i) {
    std::string s = argv[i];
    auto next = [&]() -> std::string {
      if (i + 1 >= argc) {
        std::fprintf(stderr, "missing value after %s\n", s.c_str());
        std::exit(2);
      }
      return argv[++i];
    };
    if (s == "--role") {
      a.role = next();
    } else if (s == "--addr") {
      a.addr = next();
    } else if (s == "--case") {
      a.filter = next();
    } else if (s == "--suite") {
      a.suite = next();
    } else if (s == "--ready-fd") {
      a.readyFd = std::atoi(next().c_str());
    } else if (s == "--list") {
      a.list = true;
    } else {
      std::fprintf(stderr, "unknown argument %s\n", s.c_str());
      std::exit(2);
    }
  }
  return a;
}

} // namespace tptest
