// C harness API (include/tensorpipe_c.h) over the C++ pipe/channel layer.

#include <tensorpipe_c.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <functional>
#include <future>
#include <mutex>
#include <sstream>
#include <string>
#include <thread>
#include <vector>

#include <tensorpipe/common/stage_timer.h>
#include <tensorpipe/tensorpipe.h>
#include <tensorpipe/tensorpipe_hip.h>
#include <tensorpipe/common/hip_api.h>

using namespace tensorpipe;

namespace {

thread_local std::string gLastError;

void setLastError(const std::string& what) {
  gLastError = what;
}

// One-shot completion slot shared between a callback and a waiter.
struct Completion {
  std::mutex mutex;
  std::condition_variable cv;
  bool done{false};
  std::atomic<bool> flag{false};
  Error error;

  void set(const Error& e) {
    {
      std::lock_guard<std::mutex> lock(mutex);
      error = e;
      done = true;
      flag.store(true, std::memory_order_release);
    }
    cv.notify_all();
  }

  // 0 ok, TPC_ERR_FAILED, TPC_ERR_TIMEOUT. Spins briefly before blocking: the
  // callbacks of a transfer in flight arrive within microseconds.
  int wait(int timeoutMs) {
    const auto spinUntil = std::chrono::steady_clock::now() + std::chrono::microseconds(200);
    while (!flag.load(std::memory_order_acquire) &&
           std::chrono::steady_clock::now() < spinUntil) {
#if defined(__x86_64__)
      __builtin_ia32_pause();
#endif
    }
    std::unique_lock<std::mutex> lock(mutex);
    if (timeoutMs < 0) {
      cv.wait(lock, [this] { return done; });
    } else if (!cv.wait_for(lock, std::chrono::milliseconds(timeoutMs), [this] { return done; })) {
      setLastError("timed out");
      return TPC_ERR_TIMEOUT;
    }
    if (error) {
      setLastError(error.what());
      return TPC_ERR_FAILED;
    }
    return 0;
  }
};

std::vector<std::pair<std::string, int64_t>> parseList(const char* spec) {
  std::vector<std::pair<std::string, int64_t>> out;
  if (spec == nullptr) {
    return out;
  }
  std::stringstream ss(spec);
  std::string item;
  while (std::getline(ss, item, ',')) {
    if (item.empty()) {
      continue;
    }
    auto pos = item.find(':');
    std::string name = item.substr(0, pos);
    int64_t prio = pos == std::string::npos ? static_cast<int64_t>(out.size())
                                            : std::stoll(item.substr(pos + 1));
    out.emplace_back(name, prio);
  }
  return out;
}

Buffer bufferFromC(const tpc_tensor& t) {
  if (t.device_type == TPC_DEVICE_HIP) {
    return HipBuffer{t.ptr, t.stream};
  }
  return CpuBuffer{t.ptr};
}

Message makeMessage(
    const char* metadata,
    const tpc_payload* payloads,
    uint32_t numPayloads,
    const tpc_tensor* tensors,
    uint32_t numTensors) {
  Message m;
  m.metadata = metadata != nullptr ? metadata : "";
  for (uint32_t i = 0; i < numPayloads; ++i) {
    Message::Payload p;
    p.data = payloads[i].ptr;
    p.length = payloads[i].length;
    m.payloads.push_back(std::move(p));
  }
  m.tensors.resize(numTensors);
  for (uint32_t i = 0; i < numTensors; ++i) {
    Message::Tensor& t = m.tensors[i];
    t.buffer = bufferFromC(tensors[i]);
    t.length = tensors[i].length;
    if (tensors[i].target_type != TPC_NO_TARGET) {
      t.targetDevice.emplace(
          tensors[i].target_type == TPC_DEVICE_HIP ? kHipDeviceType : kCpuDeviceType,
          tensors[i].target_index);
    }
  }
  return m;
}

Allocation makeAllocation(
    void* const* payloadPtrs,
    uint32_t numPayloads,
    const tpc_tensor* tensors,
    uint32_t numTensors) {
  Allocation a;
  a.payloads.resize(numPayloads);
  for (uint32_t i = 0; i < numPayloads; ++i) {
    a.payloads[i].data = payloadPtrs[i];
  }
  a.tensors.resize(numTensors);
  for (uint32_t i = 0; i < numTensors; ++i) {
    a.tensors[i].buffer = bufferFromC(tensors[i]);
  }
  return a;
}

void syncRecvStreams(const tpc_tensor* tensors, uint32_t n) {
  std::vector<void*> seen;
  for (uint32_t i = 0; i < n; ++i) {
    if (tensors[i].device_type != TPC_DEVICE_HIP || tensors[i].length == 0) {
      continue;
    }
    bool dup = false;
    for (void* s : seen) {
      dup |= s == tensors[i].stream;
    }
    if (dup) {
      continue;
    }
    seen.push_back(tensors[i].stream);
    int dev = hipDeviceForPointer(tensors[i].ptr);
    dev = dev < 0 ? 0 : dev;
    // Poll rather than block: the blocking wait of the runtime adds several
    // microseconds of wake-up latency to every step.
    int done = 0;
    const auto spinUntil = std::chrono::steady_clock::now() + std::chrono::milliseconds(2);
    while (!done && std::chrono::steady_clock::now() < spinUntil) {
      TP_HIP_CHECK(tphip_stream_query(dev, tensors[i].stream, &done));
    }
    if (!done) {
      TP_HIP_CHECK(tphip_stream_sync(dev, tensors[i].stream));
    }
  }
}

} // namespace

struct tpc_context {
  std::shared_ptr<Context> ctx;
  std::vector<std::string> channels;
};

struct tpc_listener {
  std::shared_ptr<Listener> listener;
};

struct tpc_pipe {
  std::shared_ptr<Pipe> pipe;
};

struct tpc_op {
  std::shared_ptr<Completion> completion;
};

#define TPC_GUARD_BEGIN try {
#define TPC_GUARD_END(failure)            \
  }                                       \
  catch (const std::exception& e) {       \
    setLastError(e.what());               \
    return failure;                       \
  }

extern "C" {

const char* tpc_last_error(void) {
  return gLastError.c_str();
}

tpc_context* tpc_context_create(const char* name, const char* transports, const char* channels) {
  return tpc_context_create_ex(name, transports, channels, -1);
}

tpc_context* tpc_context_create_ex(const char* name, const char* transports, const char* channels, int stock_wire) {
  TPC_GUARD_BEGIN
  auto out = std::make_unique<tpc_context>();
  out->ctx = stock_wire < 0
      ? std::make_shared<Context>(ContextOptions().name(name != nullptr ? name : ""))
      : std::make_shared<Context>(ContextOptions().name(name != nullptr ? name : "").stockWireFormat(stock_wire != 0));
  for (auto& t : parseList(transports)) {
    if (t.first == "shm") {
      out->ctx->registerTransport(t.second, "shm", transport::shm::create());
    } else if (t.first == "uv") {
      out->ctx->registerTransport(t.second, "uv", transport::tcp::create());
    } else if (t.first == "shm_stock") {
      // the reference's shm protocol, under the name its contexts know it by
      out->ctx->registerTransport(t.second, "shm", transport::shm_stock::create());
    } else {
      setLastError("unknown transport " + t.first);
      return nullptr;
    }
  }
  for (auto& c : parseList(channels)) {
    std::shared_ptr<channel::Context> cctx;
    if (c.first == "basic") {
      cctx = channel::basic::create();
    } else if (c.first == "xth") {
      cctx = channel::xth::create();
    } else if (c.first == "hip_xth") {
      cctx = channel::hip_xth::create();
    } else if (c.first == "hip_ipc") {
      cctx = channel::hip_ipc::create();
    } else if (c.first == "hip_basic") {
      cctx = channel::hip_basic::create(channel::basic::create());
    } else {
      setLastError("unknown channel " + c.first);
      return nullptr;
    }
    if (cctx->isViable()) {
      out->channels.push_back(c.first);
    }
    out->ctx->registerChannel(c.second, c.first, std::move(cctx));
  }
  return out.release();
  TPC_GUARD_END(nullptr)
}

void tpc_context_close(tpc_context* ctx) {
  if (ctx != nullptr) {
    ctx->ctx->close();
  }
}

void tpc_context_destroy(tpc_context* ctx) {
  if (ctx != nullptr) {
    ctx->ctx->join();
    delete ctx;
  }
}

int tpc_context_has_channel(tpc_context* ctx, const char* name) {
  for (auto& c : ctx->channels) {
    if (c == name) {
      return 1;
    }
  }
  return 0;
}

tpc_listener* tpc_listen(tpc_context* ctx, const char* url) {
  TPC_GUARD_BEGIN
  auto out = std::make_unique<tpc_listener>();
  // one URL, or several separated by commas (one per transport)
  std::vector<std::string> urls;
  std::string rest(url);
  for (size_t at; (at = rest.find(',')) != std::string::npos; rest = rest.substr(at + 1)) {
    urls.push_back(rest.substr(0, at));
  }
  urls.push_back(rest);
  out->listener = ctx->ctx->listen(urls);
  return out.release();
  TPC_GUARD_END(nullptr)
}

int tpc_listener_url(tpc_listener* l, const char* transport, char* out, size_t outLen) {
  TPC_GUARD_BEGIN
  std::string url = l->listener->url(transport);
  if (url.size() + 1 > outLen) {
    setLastError("buffer too small");
    return TPC_ERR_FAILED;
  }
  std::memcpy(out, url.c_str(), url.size() + 1);
  return 0;
  TPC_GUARD_END(TPC_ERR_FAILED)
}

tpc_pipe* tpc_accept(tpc_listener* l, int timeoutMs) {
  TPC_GUARD_BEGIN
  auto completion = std::make_shared<Completion>();
  auto slot = std::make_shared<std::shared_ptr<Pipe>>();
  l->listener->accept([completion, slot](const Error& error, std::shared_ptr<Pipe> pipe) {
    *slot = std::move(pipe);
    completion->set(error);
  });
  if (completion->wait(timeoutMs) != 0) {
    return nullptr;
  }
  auto out = std::make_unique<tpc_pipe>();
  out->pipe = std::move(*slot);
  return out.release();
  TPC_GUARD_END(nullptr)
}

void tpc_listener_destroy(tpc_listener* l) {
  delete l;
}

tpc_pipe* tpc_connect(tpc_context* ctx, const char* url) {
  TPC_GUARD_BEGIN
  auto out = std::make_unique<tpc_pipe>();
  out->pipe = ctx->ctx->connect(url);
  return out.release();
  TPC_GUARD_END(nullptr)
}

void tpc_pipe_close(tpc_pipe* p) {
  if (p != nullptr) {
    p->pipe->close();
  }
}

void tpc_pipe_destroy(tpc_pipe* p) {
  delete p;
}

int tpc_pipe_remote_name(tpc_pipe* p, char* out, size_t outLen) {
  const std::string& n = p->pipe->getRemoteName();
  if (n.size() + 1 > outLen) {
    return TPC_ERR_FAILED;
  }
  std::memcpy(out, n.c_str(), n.size() + 1);
  return 0;
}

int tpc_pipe_transport(tpc_pipe* p, char* out, size_t outLen) {
  TPC_GUARD_BEGIN
  const std::string n = p->pipe->transportInUse();
  if (n.size() + 1 > outLen) {
    return TPC_ERR_FAILED;
  }
  std::memcpy(out, n.c_str(), n.size() + 1);
  return 0;
  TPC_GUARD_END(TPC_ERR_FAILED)
}

tpc_op* tpc_write_async(
    tpc_pipe* p,
    const char* metadata,
    const tpc_payload* payloads,
    uint32_t numPayloads,
    const tpc_tensor* tensors,
    uint32_t numTensors) {
  TPC_GUARD_BEGIN
  auto op = std::make_unique<tpc_op>();
  op->completion = std::make_shared<Completion>();
  auto completion = op->completion;
  p->pipe->write(
      makeMessage(metadata, payloads, numPayloads, tensors, numTensors),
      [completion](const Error& error) { completion->set(error); });
  return op.release();
  TPC_GUARD_END(nullptr)
}

int tpc_read_descriptor(tpc_pipe* p, tpc_descriptor* out, int timeoutMs) {
  TPC_GUARD_BEGIN
  auto completion = std::make_shared<Completion>();
  auto slot = std::make_shared<Descriptor>();
  p->pipe->readDescriptor([completion, slot](const Error& error, Descriptor d) {
    *slot = std::move(d);
    completion->set(error);
  });
  int rc = completion->wait(timeoutMs);
  if (rc != 0) {
    return rc;
  }
  const Descriptor& d = *slot;
  if (d.payloads.size() > 64 || d.tensors.size() > TPC_MAX_DESC_ITEMS ||
      d.metadata.size() >= sizeof(out->metadata)) {
    setLastError("descriptor too large for tpc_descriptor");
    return TPC_ERR_FAILED;
  }
  std::memset(out->metadata, 0, sizeof(out->metadata));
  std::memcpy(out->metadata, d.metadata.data(), d.metadata.size());
  out->num_payloads = static_cast<uint32_t>(d.payloads.size());
  out->num_tensors = static_cast<uint32_t>(d.tensors.size());
  for (size_t i = 0; i < d.payloads.size(); ++i) {
    out->payload_lengths[i] = d.payloads[i].length;
  }
  for (size_t i = 0; i < d.tensors.size(); ++i) {
    const auto& t = d.tensors[i];
    out->tensor_lengths[i] = t.length;
    out->tensor_source_type[i] = t.sourceDevice.type == kCpuDeviceType ? TPC_DEVICE_CPU : TPC_DEVICE_HIP;
    out->tensor_source_index[i] = t.sourceDevice.index;
    if (t.targetDevice.has_value()) {
      out->tensor_target_type[i] =
          t.targetDevice->type == kCpuDeviceType ? TPC_DEVICE_CPU : TPC_DEVICE_HIP;
      out->tensor_target_index[i] = t.targetDevice->index;
    } else {
      out->tensor_target_type[i] = TPC_NO_TARGET;
      out->tensor_target_index[i] = 0;
    }
  }
  return 0;
  TPC_GUARD_END(TPC_ERR_FAILED)
}

tpc_op* tpc_read_async(
    tpc_pipe* p,
    void* const* payloadPtrs,
    uint32_t numPayloads,
    const tpc_tensor* tensors,
    uint32_t numTensors) {
  TPC_GUARD_BEGIN
  auto op = std::make_unique<tpc_op>();
  op->completion = std::make_shared<Completion>();
  auto completion = op->completion;
  p->pipe->read(
      makeAllocation(payloadPtrs, numPayloads, tensors, numTensors),
      [completion](const Error& error) { completion->set(error); });
  return op.release();
  TPC_GUARD_END(nullptr)
}

int tpc_op_wait(tpc_op* op, int timeoutMs) {
  if (op == nullptr) {
    return TPC_ERR_FAILED;
  }
  int rc = op->completion->wait(timeoutMs);
  if (rc != TPC_ERR_TIMEOUT) {
    delete op;
  }
  return rc;
}

// One-way transfers between two pipe endpoints of this process, chained through
// callbacks like the reference's own benchmark
// (tensorpipe/benchmark/benchmark_pipe.cc:463-468,571-577): the write of step
// k+1 is issued from whichever callback of step k (write done, read done) fires
// last, on the library's threads. The caller only waits for the end.
// One message after the other from `sender` to `receiver`. Each end carries on
// from its own callback -- the sender writes message k+1 when its write of
// message k has completed, the receiver asks for descriptor k+1 when its read
// of message k has completed -- so that each end's work stays on the threads
// that serve that end, as it would between two programs (issuing both from
// whichever callback came last puts the sender's work on the receiver's thread
// half of the time). A round is over when both of its halves are.
struct TransferChain : std::enable_shared_from_this<TransferChain> {
  using Clock = std::chrono::steady_clock;
  std::shared_ptr<Pipe> sender, receiver;
  std::vector<tpc_payload> payloads;
  std::vector<void*> recvPayloadPtrs;
  std::vector<tpc_tensor> sendTensors, recvTensors;
  uint32_t warmup{0}, iters{0};
  double* perIterUs{nullptr};
  Clock::time_point begin, end;
  std::vector<Clock::time_point> issued;
  std::unique_ptr<std::atomic<int>[]> halves; // per round: completed halves
  Completion finished;
  std::atomic<bool> failed{false};

  uint32_t total() const {
    return warmup + iters;
  }

  void fail(const Error& e) {
    if (!failed.exchange(true)) {
      finished.set(e);
    }
  }

  void start() {
    issued.resize(total());
    halves.reset(new std::atomic<int>[total() > 0 ? total() : 1]);
    for (uint32_t r = 0; r < total(); ++r) {
      halves[r].store(0, std::memory_order_relaxed);
    }
    if (total() == 0) {
      begin = end = Clock::now();
      finished.set(Error::kSuccess);
      return;
    }
    armRead(0);
    issueWrite(0);
  }

  void halfDone(uint32_t round) {
    if (halves[round].fetch_add(1, std::memory_order_acq_rel) != 1) {
      return;
    }
    const auto now = Clock::now();
    if (round >= warmup && perIterUs != nullptr) {
      perIterUs[round - warmup] = std::chrono::duration<double, std::micro>(now - issued[round]).count();
    }
    TP_MARK("harness: step over");
    if (round + 1 == total()) {
      end = now;
      finished.set(Error::kSuccess);
    }
  }

  void issueWrite(uint32_t round) {
    auto self = shared_from_this();
    issued[round] = Clock::now();
    if (round == warmup) {
      begin = issued[round];
    }
    optional<StageScope> makeTimer;
    makeTimer.emplace(Stage::kHarnessMakeMessage);
    Message message = makeMessage(
        "", payloads.data(), static_cast<uint32_t>(payloads.size()), sendTensors.data(),
        static_cast<uint32_t>(sendTensors.size()));
    makeTimer.reset();
    sender->write(std::move(message), [self, round](const Error& e) {
      if (e) {
        self->fail(e);
        return;
      }
      self->halfDone(round);
      if (round + 1 < self->total() && !self->failed.load()) {
        self->issueWrite(round + 1);
      }
    });
  }

  void armRead(uint32_t round) {
    auto self = shared_from_this();
    receiver->readDescriptor([self, round](const Error& e, Descriptor) {
      if (e) {
        self->fail(e);
        return;
      }
      self->receiver->read(
          makeAllocation(
              self->recvPayloadPtrs.data(), static_cast<uint32_t>(self->recvPayloadPtrs.size()),
              self->recvTensors.data(), static_cast<uint32_t>(self->recvTensors.size())),
          [self, round](const Error& e2) {
            if (e2) {
              self->fail(e2);
              return;
            }
            try {
              // the bytes are where a reader of these buffers would look before the round counts
              StageScope syncTimer(Stage::kHarnessSync);
              syncRecvStreams(self->recvTensors.data(), static_cast<uint32_t>(self->recvTensors.size()));
            } catch (const std::exception&) {
              self->fail(TP_CREATE_ERROR(HipError, "stream sync", TPHIP_ERR_INVALID_ARG));
              return;
            }
            self->halfDone(round);
            if (round + 1 < self->total() && !self->failed.load()) {
              self->armRead(round + 1);
            }
          });
    });
  }
};

int tpc_bench_transfer(
    tpc_pipe* sender,
    tpc_pipe* receiver,
    const tpc_payload* payloads,
    uint32_t numPayloads,
    void* const* recvPayloadPtrs,
    const tpc_tensor* sendTensors,
    const tpc_tensor* recvTensors,
    uint32_t numTensors,
    uint32_t warmup,
    uint32_t iters,
    double* perIterUs,
    double* totalSeconds) {
  TPC_GUARD_BEGIN
  auto chain = std::make_shared<TransferChain>();
  chain->sender = sender->pipe;
  chain->receiver = receiver->pipe;
  chain->payloads.assign(payloads, payloads + numPayloads);
  chain->recvPayloadPtrs.assign(recvPayloadPtrs, recvPayloadPtrs + numPayloads);
  chain->sendTensors.assign(sendTensors, sendTensors + numTensors);
  chain->recvTensors.assign(recvTensors, recvTensors + numTensors);
  chain->warmup = warmup;
  chain->iters = iters;
  chain->perIterUs = perIterUs;
  chain->start();
  int rc = chain->finished.wait(600000);
  if (rc != 0) {
    return rc;
  }
  if (totalSeconds != nullptr) {
    *totalSeconds = std::chrono::duration<double>(chain->end - chain->begin).count();
  }
  return 0;
  TPC_GUARD_END(TPC_ERR_FAILED)
}

// Callback-chained ping-pong, the shape of the reference's own benchmark
// (tensorpipe/benchmark/benchmark_pipe.cc:463-468,571-577): every step is
// issued from the callback of the previous one on the library's threads, so
// no thread hand-off is on the clock. The caller only waits for the end.
struct PingPong : std::enable_shared_from_this<PingPong> {
  using Clock = std::chrono::steady_clock;
  std::shared_ptr<Pipe> pipe;
  bool initiator{false};
  std::vector<tpc_payload> payloads;
  std::vector<void*> recvPayloadPtrs;
  std::vector<tpc_tensor> sendTensors, recvTensors;
  uint32_t warmup{0}, iters{0}, round{0};
  double* perIterUs{nullptr};
  Clock::time_point begin, end, t0;
  Completion finished;
  std::atomic<bool> failed{false};
  // With several chains side by side on one context the initiator's wait for
  // its receive stream may not sit on the context's thread (every chain's
  // messages pass through it): a thread of the chain's own waits instead.
  bool syncOffLoop{false};
  std::thread syncThread;
  std::mutex syncMutex;
  std::condition_variable syncCv;
  bool syncPending{false}, syncQuit{false};

  void fail(const Error& e) {
    if (!failed.exchange(true)) {
      finished.set(e);
    }
  }

  // The initiator's end of a round: the bytes are in place, the round counts,
  // the next one starts.
  void roundTripOver() {
    try {
      syncRecvStreams(recvTensors.data(), static_cast<uint32_t>(recvTensors.size()));
    } catch (const std::exception&) {
      fail(TP_CREATE_ERROR(HipError, "stream sync", TPHIP_ERR_INVALID_ARG));
      return;
    }
    if (round >= warmup && perIterUs != nullptr) {
      perIterUs[round - warmup] = std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
    }
    ++round;
    step();
  }

  void startSyncThread() {
    syncOffLoop = true;
    syncThread = std::thread([this] {
      std::unique_lock<std::mutex> lock(syncMutex);
      for (;;) {
        syncCv.wait(lock, [this] { return syncPending || syncQuit; });
        if (syncQuit) {
          return;
        }
        syncPending = false;
        lock.unlock();
        roundTripOver();
        lock.lock();
      }
    });
  }

  void stopSyncThread() {
    if (!syncThread.joinable()) {
      return;
    }
    {
      std::lock_guard<std::mutex> lock(syncMutex);
      syncQuit = true;
    }
    syncCv.notify_one();
    syncThread.join();
  }

  void doWrite(std::function<void()> next) {
    auto self = shared_from_this();
    pipe->write(
        makeMessage(
            "", payloads.data(), static_cast<uint32_t>(payloads.size()), sendTensors.data(),
            static_cast<uint32_t>(sendTensors.size())),
        [self, next{std::move(next)}](const Error& e) {
          if (e) {
            self->fail(e);
          } else if (next) {
            next();
          }
        });
  }

  void doRead(std::function<void()> next) {
    auto self = shared_from_this();
    pipe->readDescriptor([self, next{std::move(next)}](const Error& e, Descriptor) {
      if (e) {
        self->fail(e);
        return;
      }
      self->pipe->read(
          makeAllocation(
              self->recvPayloadPtrs.data(), static_cast<uint32_t>(self->recvPayloadPtrs.size()),
              self->recvTensors.data(), static_cast<uint32_t>(self->recvTensors.size())),
          [self, next](const Error& e2) {
            if (e2) {
              self->fail(e2);
            } else {
              next();
            }
          });
    });
  }

  void step() {
    if (round == warmup + iters) {
      end = Clock::now();
      finished.set(Error::kSuccess);
      return;
    }
    if (round == warmup) {
      begin = Clock::now();
    }
    auto self = shared_from_this();
    if (initiator) {
      t0 = Clock::now();
      doWrite(nullptr);
      doRead([self] {
        if (!self->syncOffLoop) {
          self->roundTripOver();
          return;
        }
        {
          std::lock_guard<std::mutex> lock(self->syncMutex);
          self->syncPending = true;
        }
        self->syncCv.notify_one();
      });
    } else {
      // The echo leaves from the buffers the message arrived in; a channel
      // whose recv callback means "enqueued" keeps the two ordered on the
      // buffers' stream.
      doRead([self] {
        self->doWrite([self] {
          ++self->round;
          self->step();
        });
      });
    }
  }
};

int tpc_bench_pingpong(
    tpc_pipe* p,
    int initiator,
    const tpc_payload* payloads,
    uint32_t numPayloads,
    void* const* recvPayloadPtrs,
    const tpc_tensor* sendTensors,
    const tpc_tensor* recvTensors,
    uint32_t numTensors,
    uint32_t warmup,
    uint32_t iters,
    double* perIterUs,
    double* totalSeconds) {
  TPC_GUARD_BEGIN
  auto pp = std::make_shared<PingPong>();
  pp->pipe = p->pipe;
  pp->initiator = initiator != 0;
  if (initiator == 2) {
    pp->startSyncThread();
  }
  pp->payloads.assign(payloads, payloads + numPayloads);
  pp->recvPayloadPtrs.assign(recvPayloadPtrs, recvPayloadPtrs + numPayloads);
  pp->sendTensors.assign(sendTensors, sendTensors + numTensors);
  pp->recvTensors.assign(recvTensors, recvTensors + numTensors);
  pp->warmup = warmup;
  pp->iters = iters;
  pp->perIterUs = perIterUs;
  pp->step();
  int rc = pp->finished.wait(600000);
  pp->stopSyncThread();
  if (rc != 0) {
    return rc;
  }
  if (totalSeconds != nullptr) {
    *totalSeconds = std::chrono::duration<double>(pp->end - pp->begin).count();
  }
  return 0;
  TPC_GUARD_END(TPC_ERR_FAILED)
}

} // extern "C"
