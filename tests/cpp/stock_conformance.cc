// This library's channels registered in an UNMODIFIED TensorPipe: the build
// that PyTorch ships inside libtorch_cpu.so, driven through its public headers
// (torch/include/tensorpipe). Its Context, Listener, Pipe, shm transport and
// basic channel are the stock ones; the only thing added is
// tensorpipe_amd_bridge::createChannelContext(...) handed to
// Context::registerChannel, as tensorpipe/test/core/pipe_test.h:300-316 does
// with the CUDA channels. A message with a payload, a CPU tensor and GPU
// tensors then travels between two stock contexts and every byte is checked.
//
//   stock_conformance same_process   hip_xth between two contexts of this process
//   stock_conformance two_process    hip_ipc and hip_basic between this process and a child
//   stock_conformance to_self <channel> <rounds>
//       ONE context with a pipe to itself, as an RPC agent has for calls to its
//       own rank, messages travelling both ways at the same moment from
//       threads of the application: with hip_basic every GPU tensor then takes
//       the route through the wrapped CPU channel, whose loop and the staged
//       channel's own loop are both driven by whichever thread comes by
//
// Prints "RESULT <case> OK" or "RESULT <case> FAIL <why>" per case.
#include <tensorpipe/tensorpipe.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <future>
#include <string>
#include <vector>

#include <sys/wait.h>
#include <unistd.h>

#include <tphip.h>

#include <bridge/stock_adapter.h>
#include <tensorpipe_c.h>

using namespace tensorpipe;
using tensorpipe_amd_bridge::HipBuffer;

#define CHECK_HIP(x)                                                           \
  do {                                                                         \
    int rc_ = (x);                                                             \
    if (rc_ != 0) {                                                            \
      std::fprintf(stderr, "%s failed: %s\n", #x, tphip_strerror(rc_));        \
      std::exit(3);                                                            \
    }                                                                          \
  } while (0)

static std::shared_ptr<Context> makeContext(const char* name, const std::vector<std::string>& channels, bool withUv = false, bool alsoShm = false) {
  auto ctx = std::make_shared<Context>(ContextOptions().name(name));
  if (withUv) {
    ctx->registerTransport(0, "uv", transport::uv::create());
    if (alsoShm) {
      ctx->registerTransport(1, "shm", transport::shm::create()); // preferred where the peer speaks it
    }
  } else {
    ctx->registerTransport(0, "shm", transport::shm::create());
  }
  ctx->registerChannel(0, "basic", channel::basic::create());
  int priority = 10;
  for (auto& c : channels) {
    auto cc = tensorpipe_amd_bridge::createChannelContext(c);
    if (!cc || !cc->isViable()) {
      std::fprintf(stderr, "channel %s is not viable here\n", c.c_str());
      std::exit(3);
    }
    ctx->registerChannel(priority++, c, std::move(cc));
  }
  return ctx;
}

static uint8_t pattern(size_t i, int salt) {
  return static_cast<uint8_t>((i * 7 + (i >> 9) * 13 + static_cast<size_t>(salt) * 101) % 251);
}

struct GpuTensor {
  void* dev{nullptr};
  size_t bytes{0};
  void* stream{nullptr};
  void fill(int salt) {
    std::vector<uint8_t> host(bytes);
    for (size_t i = 0; i < bytes; ++i) {
      host[i] = pattern(i, salt);
    }
    void* pinned = nullptr;
    void* pinnedDev = nullptr;
    CHECK_HIP(tphip_host_alloc(0, bytes, &pinned, &pinnedDev));
    std::memcpy(pinned, host.data(), bytes);
    CHECK_HIP(tphip_copy(0, dev, pinnedDev, bytes, stream));
    CHECK_HIP(tphip_stream_sync(0, stream));
    CHECK_HIP(tphip_host_free(pinned));
  }
  std::string check(int salt) {
    void* pinned = nullptr;
    void* pinnedDev = nullptr;
    CHECK_HIP(tphip_host_alloc(0, bytes, &pinned, &pinnedDev));
    CHECK_HIP(tphip_stream_sync(0, stream));
    CHECK_HIP(tphip_copy(0, pinnedDev, dev, bytes, stream));
    CHECK_HIP(tphip_stream_sync(0, stream));
    std::string bad;
    const uint8_t* got = static_cast<const uint8_t*>(pinned);
    for (size_t i = 0; i < bytes; ++i) {
      if (got[i] != pattern(i, salt)) {
        bad = "byte " + std::to_string(i) + " of a GPU tensor differs";
        break;
      }
    }
    CHECK_HIP(tphip_host_free(pinned));
    return bad;
  }
};

// Frees the tensors of a message when the function that made them returns.
struct GpuTensors : std::vector<GpuTensor> {
  GpuTensors() = default;
  GpuTensors(const GpuTensors&) = delete;
  ~GpuTensors() {
    for (auto& t : *this) {
      tphip_stream_sync(0, t.stream);
      tphip_free(0, t.dev);
      tphip_stream_destroy(0, t.stream);
    }
  }
};

static GpuTensor makeGpu(size_t bytes) {
  GpuTensor t;
  t.bytes = bytes;
  CHECK_HIP(tphip_malloc(0, bytes, &t.dev));
  CHECK_HIP(tphip_stream_create(0, &t.stream));
  CHECK_HIP(tphip_fill(0, t.dev, 0xEE, bytes, t.stream));
  CHECK_HIP(tphip_stream_sync(0, t.stream));
  return t;
}

static const std::vector<size_t> kGpuSizes = {4096, (3u << 20) + 17, 256};
static const size_t kCpuBytes = 70001;
static const std::string kPayload = "payload #1";

// Sends the test message on `pipe` and waits for the write callback.
static std::string sendMessage(Pipe& pipe, int salt) {
  GpuTensors gpus;
  std::vector<uint8_t> cpu(kCpuBytes);
  for (size_t i = 0; i < cpu.size(); ++i) {
    cpu[i] = pattern(i, salt + 50);
  }
  Message m;
  m.metadata = "conformance";
  Message::Payload p;
  std::string payload = kPayload;
  p.data = payload.data();
  p.length = payload.size();
  m.payloads.push_back(std::move(p));
  for (size_t k = 0; k < kGpuSizes.size(); ++k) {
    gpus.push_back(makeGpu(kGpuSizes[k]));
    gpus.back().fill(salt + static_cast<int>(k));
    Message::Tensor t;
    t.buffer = HipBuffer{gpus.back().dev, gpus.back().stream, 0};
    t.length = gpus.back().bytes;
    t.targetDevice = Device{"cuda", 0};
    m.tensors.push_back(std::move(t));
  }
  Message::Tensor ct;
  ct.buffer = CpuBuffer{cpu.data()};
  ct.length = cpu.size();
  m.tensors.push_back(std::move(ct));
  std::promise<std::string> done;
  pipe.write(std::move(m), [&done](const Error& e) { done.set_value(e ? e.what() : std::string()); });
  auto f = done.get_future();
  if (f.wait_for(std::chrono::seconds(60)) != std::future_status::ready) {
    return "write never completed";
  }
  return f.get();
}

static std::string recvMessage(Pipe& pipe, int salt) {
  std::promise<std::string> done;
  GpuTensors gpus;
  std::vector<uint8_t> cpu;
  std::string payload;
  pipe.readDescriptor([&](const Error& e, Descriptor d) {
    if (e) {
      done.set_value("readDescriptor: " + e.what());
      return;
    }
    if (d.metadata != "conformance" || d.payloads.size() != 1 || d.tensors.size() != kGpuSizes.size() + 1) {
      done.set_value("unexpected descriptor");
      return;
    }
    Allocation a;
    payload.resize(d.payloads[0].length);
    a.payloads.resize(1);
    a.payloads[0].data = &payload[0];
    a.tensors.resize(d.tensors.size());
    for (size_t k = 0; k < kGpuSizes.size(); ++k) {
      if (d.tensors[k].length != kGpuSizes[k] || d.tensors[k].sourceDevice.type != "cuda") {
        done.set_value("unexpected GPU tensor in the descriptor");
        return;
      }
      gpus.push_back(makeGpu(kGpuSizes[k]));
      a.tensors[k].buffer = HipBuffer{gpus.back().dev, gpus.back().stream, 0};
    }
    cpu.assign(d.tensors.back().length, 0);
    a.tensors.back().buffer = CpuBuffer{cpu.data()};
    pipe.read(std::move(a), [&done](const Error& e2) { done.set_value(e2 ? "read: " + e2.what() : std::string()); });
  });
  auto f = done.get_future();
  if (f.wait_for(std::chrono::seconds(60)) != std::future_status::ready) {
    return "read never completed";
  }
  std::string err = f.get();
  if (!err.empty()) {
    return err;
  }
  if (payload != kPayload) {
    return "payload differs";
  }
  for (size_t k = 0; k < gpus.size(); ++k) {
    std::string bad = gpus[k].check(salt + static_cast<int>(k));
    if (!bad.empty()) {
      return bad;
    }
  }
  if (cpu.size() != kCpuBytes) {
    return "CPU tensor has the wrong length";
  }
  for (size_t i = 0; i < cpu.size(); ++i) {
    if (cpu[i] != pattern(i, salt + 50)) {
      return "byte " + std::to_string(i) + " of the CPU tensor differs";
    }
  }
  return "";
}

static void report(const std::string& name, const std::string& problem) {
  if (problem.empty()) {
    std::printf("RESULT %s OK\n", name.c_str());
  } else {
    std::printf("RESULT %s FAIL %s\n", name.c_str(), problem.c_str());
  }
  std::fflush(stdout);
}

static std::shared_ptr<Pipe> acceptOne(Listener& listener) {
  std::promise<std::shared_ptr<Pipe>> pp;
  listener.accept([&pp](const Error& e, std::shared_ptr<Pipe> pipe) {
    if (e) {
      std::fprintf(stderr, "accept: %s\n", e.what().c_str());
    }
    pp.set_value(std::move(pipe));
  });
  return pp.get_future().get();
}

static int sameProcess() {
  const std::string addr = "shm://tpamd_conf_" + std::to_string(::getpid());
  auto server = makeContext("server", {"hip_xth"});
  auto client = makeContext("client", {"hip_xth"});
  auto listener = server->listen({addr});
  auto cpipe = client->connect(listener->url("shm"));
  auto spipe = acceptOne(*listener);
  std::string problem;
  for (int round = 0; round < 3 && problem.empty(); ++round) {
    auto sent = std::async(std::launch::async, [&] { return sendMessage(*cpipe, 10 * round); });
    problem = recvMessage(*spipe, 10 * round);
    const std::string w = sent.get();
    if (problem.empty()) {
      problem = w;
    }
    // and back
    if (problem.empty()) {
      auto sent2 = std::async(std::launch::async, [&] { return sendMessage(*spipe, 10 * round + 5); });
      problem = recvMessage(*cpipe, 10 * round + 5);
      const std::string w2 = sent2.get();
      if (problem.empty()) {
        problem = w2;
      }
    }
  }
  if (problem.empty() && tensorpipe_amd_bridge::gpuOperationsServed() != 3 * 2 * 3 * 2) {
    problem = "the GPU tensors did not all travel on this library's channel: " +
        std::to_string(tensorpipe_amd_bridge::gpuOperationsServed()) + " operations served";
  }
  report("hip_xth_in_stock_context", problem);
  cpipe.reset();
  spipe.reset();
  listener.reset();
  client->join();
  server->join();
  return problem.empty() ? 0 : 1;
}


// One context talking to itself, both directions busy at once, `rounds` times.
// Every thread here is the application's: the host's transport threads and the
// four below are all strangers to this library's loops.
static int toSelf(const std::string& channel, int rounds) {
  const std::string addr = "shm://tpamd_conf_self_" + std::to_string(::getpid());
  auto ctx = makeContext("self", {channel});
  auto listener = ctx->listen({addr});
  auto cpipe = ctx->connect(listener->url("shm"));
  auto spipe = acceptOne(*listener);
  std::string problem = spipe ? std::string() : std::string("accept failed");
  for (int round = 0; round < rounds && problem.empty(); ++round) {
    auto w1 = std::async(std::launch::async, [&] { return sendMessage(*cpipe, 10 * round); });
    auto w2 = std::async(std::launch::async, [&] { return sendMessage(*spipe, 10 * round + 5); });
    auto r1 = std::async(std::launch::async, [&] { return recvMessage(*spipe, 10 * round); });
    auto r2 = std::async(std::launch::async, [&] { return recvMessage(*cpipe, 10 * round + 5); });
    for (auto* f : {&w1, &w2, &r1, &r2}) {
      const std::string p = f->get();
      if (problem.empty()) {
        problem = p;
      }
    }
  }
  const size_t expected = static_cast<size_t>(rounds) * 2 * kGpuSizes.size() * 2;
  if (problem.empty() && tensorpipe_amd_bridge::gpuOperationsServed() != expected) {
    problem = "the GPU tensors did not all travel on this library's channel: " +
        std::to_string(tensorpipe_amd_bridge::gpuOperationsServed()) + " operations served";
  }
  report(channel + "_to_self_in_stock_context", problem);
  cpipe.reset();
  spipe.reset();
  listener.reset();
  ctx->join();
  return problem.empty() ? 0 : 1;
}

static int twoProcess(const std::string& channel) {
  const std::string addr = "shm://tpamd_conf2_" + channel + "_" + std::to_string(::getpid());
  int go[2], over[2];
  if (::pipe(go) != 0 || ::pipe(over) != 0) {
    return 3;
  }
  pid_t pid = ::fork(); // before anything has touched the GPU
  if (pid == 0) {
    char byte = 0;
    if (::read(go[0], &byte, 1) != 1) { // the parent is listening now
      ::_exit(2);
    }
    auto ctx = makeContext("peer", {channel});
    auto pipe = ctx->connect(addr);
    std::string problem = recvMessage(*pipe, 1);
    if (problem.empty()) {
      problem = sendMessage(*pipe, 2);
    }
    // A write is over when its bytes have been handed on, which on a route through the host's
    // transport is before the other end has read them: the pipe stays open until the parent has
    // the message (the reference's tests end their peers behind a barrier for the same reason).
    if (::read(over[0], &byte, 1) != 1) {
      problem = problem.empty() ? "the parent left early" : problem;
    }
    if (problem.empty() && tensorpipe_amd_bridge::gpuOperationsServed() != 6) {
      problem = "the GPU tensors did not all travel on this library's channel";
    }
    if (!problem.empty()) {
      std::fprintf(stderr, "[peer] %s\n", problem.c_str());
    }
    pipe.reset();
    ctx->join();
    ::_exit(problem.empty() ? 0 : 1);
  }
  auto ctx = makeContext("main", {channel});
  auto listener = ctx->listen({addr});
  const char byte = 1;
  if (::write(go[1], &byte, 1) != 1) {
    return 3;
  }
  auto pipe = acceptOne(*listener);
  std::string problem = pipe ? sendMessage(*pipe, 1) : std::string("accept failed");
  if (problem.empty()) {
    problem = recvMessage(*pipe, 2);
  }
  if (::write(over[1], &byte, 1) != 1) {
    problem = problem.empty() ? "cannot tell the peer that the exchange is over" : problem;
  }
  int status = 0;
  ::waitpid(pid, &status, 0);
  if (problem.empty() && !(WIFEXITED(status) && WEXITSTATUS(status) == 0)) {
    problem = "the peer process reported a failure";
  }
  if (problem.empty() && tensorpipe_amd_bridge::gpuOperationsServed() != 6) {
    problem = "the GPU tensors did not all travel on this library's channel: " +
        std::to_string(tensorpipe_amd_bridge::gpuOperationsServed()) + " operations served";
  }
  report(channel + "_in_stock_context", problem);
  pipe.reset();
  listener.reset();
  ctx->join();
  return problem.empty() ? 0 : 1;
}

// A message of one payload and one CPU tensor: what an endpoint with the HIP
// channels registered can exchange with a peer that has none of them.
static std::string sendCpuMessage(Pipe& pipe, int salt) {
  std::vector<uint8_t> cpu(kCpuBytes);
  for (size_t i = 0; i < cpu.size(); ++i) {
    cpu[i] = pattern(i, salt);
  }
  Message m;
  m.metadata = "cpu only";
  Message::Payload p;
  std::string payload = kPayload;
  p.data = payload.data();
  p.length = payload.size();
  m.payloads.push_back(std::move(p));
  Message::Tensor ct;
  ct.buffer = CpuBuffer{cpu.data()};
  ct.length = cpu.size();
  m.tensors.push_back(std::move(ct));
  std::promise<std::string> done;
  pipe.write(std::move(m), [&done](const Error& e) { done.set_value(e ? e.what() : std::string()); });
  auto f = done.get_future();
  if (f.wait_for(std::chrono::seconds(60)) != std::future_status::ready) {
    return "write never completed";
  }
  return f.get();
}

static std::string recvCpuMessage(Pipe& pipe, int salt) {
  std::promise<std::string> done;
  std::vector<uint8_t> cpu;
  std::string payload;
  pipe.readDescriptor([&](const Error& e, Descriptor d) {
    if (e) {
      done.set_value("readDescriptor: " + e.what());
      return;
    }
    if (d.metadata != "cpu only" || d.payloads.size() != 1 || d.tensors.size() != 1) {
      done.set_value("unexpected descriptor");
      return;
    }
    Allocation a;
    payload.resize(d.payloads[0].length);
    a.payloads.resize(1);
    a.payloads[0].data = &payload[0];
    a.tensors.resize(1);
    cpu.assign(d.tensors[0].length, 0);
    a.tensors[0].buffer = CpuBuffer{cpu.data()};
    pipe.read(std::move(a), [&done](const Error& e2) { done.set_value(e2 ? "read: " + e2.what() : std::string()); });
  });
  auto f = done.get_future();
  if (f.wait_for(std::chrono::seconds(60)) != std::future_status::ready) {
    return "read never completed";
  }
  std::string err = f.get();
  if (!err.empty()) {
    return err;
  }
  if (payload != kPayload || cpu.size() != kCpuBytes) {
    return "payload or tensor length differs";
  }
  for (size_t i = 0; i < cpu.size(); ++i) {
    if (cpu[i] != pattern(i, salt)) {
      return "byte " + std::to_string(i) + " of the CPU tensor differs";
    }
  }
  return "";
}

// One end has the three HIP channels registered next to the stock ones, the
// other is an unmodified TensorPipe endpoint: channel selection must skip what
// only one side offers and the two must still talk.
static int unmodifiedPeer() {
  const std::string addr = "shm://tpamd_conf3_" + std::to_string(::getpid());
  auto server = makeContext("server", {"hip_xth", "hip_ipc", "hip_basic"});
  auto client = makeContext("unmodified", {});
  auto listener = server->listen({addr});
  auto cpipe = client->connect(listener->url("shm"));
  auto spipe = acceptOne(*listener);
  std::string problem = spipe ? std::string() : std::string("accept failed");
  for (int round = 0; round < 3 && problem.empty(); ++round) {
    auto sent = std::async(std::launch::async, [&] { return sendCpuMessage(*spipe, 7 * round); });
    problem = recvCpuMessage(*cpipe, 7 * round);
    const std::string w = sent.get();
    if (problem.empty()) {
      problem = w;
    }
    if (problem.empty()) {
      auto sent2 = std::async(std::launch::async, [&] { return sendCpuMessage(*cpipe, 7 * round + 3); });
      problem = recvCpuMessage(*spipe, 7 * round + 3);
      const std::string w2 = sent2.get();
      if (problem.empty()) {
        problem = w2;
      }
    }
  }
  report("hip_channels_registered_beside_an_unmodified_peer", problem);
  cpipe.reset();
  spipe.reset();
  listener.reset();
  client->join();
  server->join();
  return problem.empty() ? 0 : 1;
}

// Timing, not a test: one GPU tensor of `bytes` bytes per message over hip_xth
// between two stock contexts of this process, one message at a time, the next
// write issued by the thread that saw both callbacks of the previous one.
static int timeSameProcess(size_t bytes, int iters, size_t pieces) {
  const std::string addr = "shm://tpamd_conf4_" + std::to_string(::getpid());
  auto server = makeContext("server", {"hip_xth"});
  auto client = makeContext("client", {"hip_xth"});
  auto listener = server->listen({addr});
  auto cpipe = client->connect(listener->url("shm"));
  auto spipe = acceptOne(*listener);
  GpuTensor src = makeGpu(bytes);
  GpuTensor dst = makeGpu(bytes);
  src.fill(3);
  std::vector<double> us;
  std::string problem;
  for (int it = 0; it < iters + 10 && problem.empty(); ++it) {
    std::promise<std::string> wrote, read;
    const auto t0 = std::chrono::steady_clock::now();
    // the bytes as `pieces` tensors of one message, cut at odd places
    Message m;
    const size_t each = bytes / pieces;
    for (size_t k = 0; k < pieces; ++k) {
      Message::Tensor t;
      t.buffer = HipBuffer{static_cast<char*>(src.dev) + k * each, src.stream, 0};
      t.length = k + 1 == pieces ? bytes - k * each : each;
      t.targetDevice = Device{"cuda", 0};
      m.tensors.push_back(std::move(t));
    }
    spipe->readDescriptor([&](const Error& e, Descriptor d) {
      if (e || d.tensors.size() != pieces) {
        read.set_value("readDescriptor failed");
        return;
      }
      Allocation a;
      a.tensors.resize(pieces);
      for (size_t k = 0; k < pieces; ++k) {
        a.tensors[k].buffer = HipBuffer{static_cast<char*>(dst.dev) + k * each, dst.stream, 0};
      }
      spipe->read(std::move(a), [&read](const Error& e2) { read.set_value(e2 ? e2.what() : std::string()); });
    });
    cpipe->write(std::move(m), [&wrote](const Error& e) { wrote.set_value(e ? e.what() : std::string()); });
    problem = read.get_future().get();
    const std::string w = wrote.get_future().get();
    if (problem.empty()) {
      problem = w;
    }
    const auto t1 = std::chrono::steady_clock::now();
    if (it >= 10) {
      us.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count());
    }
  }
  if (problem.empty()) {
    problem = dst.check(3);
  }
  std::sort(us.begin(), us.end());
  if (problem.empty() && !us.empty()) {
    const double p50 = us[us.size() / 2];
    std::printf("TIMING hip_xth in stock contexts: %zu bytes in %zu tensors, %d messages, p50 %.1f us per message, %.1f GB/s payload\n",
                bytes, pieces, iters, p50, static_cast<double>(bytes) / p50 / 1e3);
  }
  report("timing_hip_xth_in_stock_context", problem);
  cpipe.reset();
  spipe.reset();
  listener.reset();
  client->join();
  server->join();
  return problem.empty() ? 0 : 1;
}

// ---- this library's own pipe as the peer -----------------------------------------
//
// One end is a context of this library in stock wire format (its pipe, its TCP
// transport under the name "uv", its channels natively), driven through the C
// harness API; the other end is the stock TensorPipe with the same channel
// registered through the bridge. The two were built from different headers and
// meet on the wire only.

static std::string nativeSend(tpc_pipe* pipe, int salt) {
  std::vector<GpuTensor> gpus;
  std::vector<uint8_t> cpu(kCpuBytes);
  for (size_t i = 0; i < cpu.size(); ++i) {
    cpu[i] = pattern(i, salt + 50);
  }
  std::string payload = kPayload;
  tpc_payload p{&payload[0], payload.size()};
  std::vector<tpc_tensor> tensors;
  for (size_t k = 0; k < kGpuSizes.size(); ++k) {
    gpus.push_back(makeGpu(kGpuSizes[k]));
    gpus.back().fill(salt + static_cast<int>(k));
    tpc_tensor t{};
    t.ptr = gpus.back().dev;
    t.length = gpus.back().bytes;
    t.device_type = TPC_DEVICE_HIP;
    t.target_type = TPC_DEVICE_HIP;
    t.target_index = 0;
    t.stream = gpus.back().stream;
    tensors.push_back(t);
  }
  tpc_tensor ct{};
  ct.ptr = cpu.data();
  ct.length = cpu.size();
  ct.device_type = TPC_DEVICE_CPU;
  ct.target_type = TPC_NO_TARGET;
  tensors.push_back(ct);
  tpc_op* op = tpc_write_async(pipe, "conformance", &p, 1, tensors.data(), static_cast<uint32_t>(tensors.size()));
  if (op == nullptr || tpc_op_wait(op, 60000) != 0) {
    return std::string("native write: ") + tpc_last_error();
  }
  return "";
}

static std::string nativeRecv(tpc_pipe* pipe, int salt) {
  auto d = std::make_unique<tpc_descriptor>();
  if (tpc_read_descriptor(pipe, d.get(), 60000) != 0) {
    return std::string("native readDescriptor: ") + tpc_last_error();
  }
  if (std::string(d->metadata) != "conformance" || d->num_payloads != 1 || d->num_tensors != kGpuSizes.size() + 1) {
    return "unexpected descriptor on the native end";
  }
  std::string payload(d->payload_lengths[0], '\0');
  void* payloadPtr = &payload[0];
  std::vector<GpuTensor> gpus;
  std::vector<uint8_t> cpu(d->tensor_lengths[kGpuSizes.size()]);
  std::vector<tpc_tensor> tensors;
  for (size_t k = 0; k < kGpuSizes.size(); ++k) {
    if (d->tensor_lengths[k] != kGpuSizes[k] || d->tensor_source_type[k] != TPC_DEVICE_HIP) {
      return "unexpected GPU tensor in the descriptor on the native end";
    }
    gpus.push_back(makeGpu(kGpuSizes[k]));
    tpc_tensor t{};
    t.ptr = gpus.back().dev;
    t.length = gpus.back().bytes;
    t.device_type = TPC_DEVICE_HIP;
    t.target_type = TPC_NO_TARGET;
    t.stream = gpus.back().stream;
    tensors.push_back(t);
  }
  tpc_tensor ct{};
  ct.ptr = cpu.data();
  ct.length = cpu.size();
  ct.device_type = TPC_DEVICE_CPU;
  ct.target_type = TPC_NO_TARGET;
  tensors.push_back(ct);
  tpc_op* op = tpc_read_async(pipe, &payloadPtr, 1, tensors.data(), static_cast<uint32_t>(tensors.size()));
  if (op == nullptr || tpc_op_wait(op, 60000) != 0) {
    return std::string("native read: ") + tpc_last_error();
  }
  if (payload != kPayload) {
    return "payload differs on the native end";
  }
  for (size_t k = 0; k < gpus.size(); ++k) {
    std::string bad = gpus[k].check(salt + static_cast<int>(k));
    if (!bad.empty()) {
      return bad + " (native end)";
    }
  }
  if (cpu.size() != kCpuBytes) {
    return "CPU tensor has the wrong length on the native end";
  }
  for (size_t i = 0; i < cpu.size(); ++i) {
    if (cpu[i] != pattern(i, salt + 50)) {
      return "byte " + std::to_string(i) + " of the CPU tensor differs on the native end";
    }
  }
  return "";
}

// hip_xth needs both ends in one process: a native server and a stock client.
static int nativePeerSameProcess() {
  tpc_context* native = tpc_context_create_ex("native_server", "uv:0", "basic:0,hip_xth:12", 1);
  tpc_listener* listener = native != nullptr ? tpc_listen(native, "uv://127.0.0.1") : nullptr;
  char url[256] = {0};
  if (listener == nullptr || tpc_listener_url(listener, "uv", url, sizeof(url)) != 0) {
    report("native_hip_xth_with_stock_peer", std::string("native listen: ") + tpc_last_error());
    return 1;
  }
  auto ctx = makeContext("stock_client", {"hip_xth"}, /*withUv=*/true);
  auto stock = ctx->connect(url);
  tpc_pipe* pipe = tpc_accept(listener, 30000);
  std::string problem = pipe != nullptr ? std::string() : std::string("native accept: ") + tpc_last_error();
  const unsigned long long before = tensorpipe_amd_bridge::gpuOperationsServed();
  for (int round = 0; round < 3 && problem.empty(); ++round) {
    auto sent = std::async(std::launch::async, [&] { return nativeSend(pipe, 20 * round); });
    problem = recvMessage(*stock, 20 * round);
    const std::string w = sent.get();
    if (problem.empty()) {
      problem = w;
    }
    if (problem.empty()) {
      auto sent2 = std::async(std::launch::async, [&] { return sendMessage(*stock, 20 * round + 7); });
      problem = nativeRecv(pipe, 20 * round + 7);
      const std::string w2 = sent2.get();
      if (problem.empty()) {
        problem = w2;
      }
    }
  }
  if (problem.empty() && tensorpipe_amd_bridge::gpuOperationsServed() - before != 3 * 2 * 3) {
    problem = "the GPU tensors did not all travel on this library's channel on the stock end";
  }
  report("native_hip_xth_with_stock_peer", problem);
  stock.reset();
  if (pipe != nullptr) {
    tpc_pipe_destroy(pipe);
  }
  tpc_listener_destroy(listener);
  tpc_context_destroy(native);
  ctx->join();
  return problem.empty() ? 0 : 1;
}

// hip_ipc / hip_basic: the native end in a child process, the stock end here.
// overShm: both ends also hold the reference's shm transport (the native end
// through transport/shm_stock), preferred; the stock end connects over uv and
// the pipe moves to shm before the first message.
static int nativePeerTwoProcess(const std::string& channel, bool overShm) {
  int toChild[2], toParent[2];
  if (::pipe(toChild) != 0 || ::pipe(toParent) != 0) {
    return 3;
  }
  pid_t pid = ::fork(); // before anything has touched the GPU
  if (pid == 0) {
    const std::string channels = "basic:0," + channel + ":10";
    tpc_context* native = tpc_context_create_ex("native_peer", overShm ? "uv:0,shm_stock:1" : "uv:0", channels.c_str(), 1);
    tpc_listener* listener =
        native != nullptr ? tpc_listen(native, overShm ? "uv://127.0.0.1,shm://" : "uv://127.0.0.1") : nullptr;
    char url[256] = {0};
    if (listener == nullptr || tpc_listener_url(listener, "uv", url, sizeof(url)) != 0) {
      std::fprintf(stderr, "[native] listen: %s\n", tpc_last_error());
      ::_exit(2);
    }
    if (::write(toParent[1], url, sizeof(url)) != static_cast<ssize_t>(sizeof(url))) {
      ::_exit(2);
    }
    tpc_pipe* pipe = tpc_accept(listener, 30000);
    std::string problem = pipe != nullptr ? std::string() : std::string("accept: ") + tpc_last_error();
    if (problem.empty()) {
      problem = nativeRecv(pipe, 1);
    }
    if (problem.empty()) {
      problem = nativeSend(pipe, 2);
    }
    if (problem.empty()) {
      char transport[64] = {0};
      const std::string expected = overShm ? "shm" : "uv";
      if (tpc_pipe_transport(pipe, transport, sizeof(transport)) != 0 || expected != transport) {
        problem = std::string("the pipe runs on transport \"") + transport + "\", not on " + expected;
      }
    }
    if (!problem.empty()) {
      std::fprintf(stderr, "[native] %s\n", problem.c_str());
    }
    char byte = 0;
    (void)!::read(toChild[0], &byte, 1); // the stock end has checked what it received
    if (pipe != nullptr) {
      tpc_pipe_destroy(pipe);
    }
    tpc_listener_destroy(listener);
    tpc_context_destroy(native);
    ::_exit(problem.empty() ? 0 : 1);
  }
  char url[256] = {0};
  if (::read(toParent[0], url, sizeof(url)) != static_cast<ssize_t>(sizeof(url))) {
    report("native_" + channel + "_with_stock_peer", "the native process did not come up");
    return 1;
  }
  auto ctx = makeContext("stock_main", {channel}, /*withUv=*/true, /*alsoShm=*/overShm);
  auto pipe = ctx->connect(url);
  std::string problem = sendMessage(*pipe, 1);
  if (problem.empty()) {
    problem = recvMessage(*pipe, 2);
  }
  if (problem.empty() && tensorpipe_amd_bridge::gpuOperationsServed() != 6) {
    problem = "the GPU tensors did not all travel on this library's channel on the stock end";
  }
  const char byte = 1;
  (void)!::write(toChild[1], &byte, 1);
  int status = 0;
  ::waitpid(pid, &status, 0);
  if (problem.empty() && !(WIFEXITED(status) && WEXITSTATUS(status) == 0)) {
    problem = "the native process reported a failure";
  }
  report("native_" + channel + "_with_stock_peer", problem);
  pipe.reset();
  ctx->join();
  return problem.empty() ? 0 : 1;
}

int main(int argc, char** argv) {
  if (argc == 2 && std::strcmp(argv[1], "same_process") == 0) {
    return sameProcess();
  }
  if (argc == 3 && std::strcmp(argv[1], "two_process") == 0) {
    return twoProcess(argv[2]);
  }
  if (argc == 4 && std::strcmp(argv[1], "to_self") == 0) {
    return toSelf(argv[2], std::atoi(argv[3]));
  }
  if (argc == 2 && std::strcmp(argv[1], "unmodified_peer") == 0) {
    return unmodifiedPeer();
  }
  if ((argc == 3 || argc == 4) && std::strcmp(argv[1], "native_peer") == 0) {
    const bool overShm = argc == 4 && std::strcmp(argv[3], "shm") == 0;
    return std::strcmp(argv[2], "hip_xth") == 0 ? nativePeerSameProcess() : nativePeerTwoProcess(argv[2], overShm);
  }
  if ((argc == 4 || argc == 5) && std::strcmp(argv[1], "time_same_process") == 0) {
    const size_t pieces = argc == 5 ? std::strtoull(argv[4], nullptr, 10) : 1;
    const size_t bytes = std::strtoull(argv[2], nullptr, 10);
    if (pieces == 0 || bytes < pieces) {
      std::fprintf(stderr, "need at least one byte per tensor\n");
      return 2;
    }
    return timeSameProcess(bytes, std::atoi(argv[3]), pieces);
  }
  std::fprintf(stderr, "usage: %s same_process | two_process hip_ipc|hip_basic | to_self <channel> <rounds> | unmodified_peer | native_peer hip_xth|hip_ipc|hip_basic [shm] | time_same_process <bytes> <messages> [tensors per message]\n", argv[0]);
  return 2;
}
