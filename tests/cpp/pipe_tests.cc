// Pipe-level tests of messages that mix CPU and GPU tensors, through
// Context::registerChannel + Pipe::write / readDescriptor / read, with the
// channel set and priorities of the reference's test context
// (tensorpipe/test/core/pipe_test.h:292-316): basic 100, hip_basic 10,
// hip_ipc 11, hip_xth 12 over the shm transport.
//
//   pipe_tests --suite [cpu_]two_process|[cpu_]same_process [--case SUBSTRING] [--list]
//
// The cpu_ suites run the same messages with every tensor in host memory and
// only the CPU channels (basic 100, xth 101) registered.
//
// The messages are those of tensorpipe/test/core/pipe_cuda_test.cc:13-262:
// three payloads "payload #k", tensors "tensor #k" with per-item metadata,
// sources and targets on cpu:0 / the GPU in every combination, received into
// freshly allocated buffers on the devices the test names; checked as
// expectDescriptorAndStorageMatchMessage does (pipe_test.h:225-280).
#include <algorithm>
#include <thread>

#include "support.h"

using namespace tptest;

namespace {

// Without a GPU (the cpu_* suites) every "GPU" tensor of the messages below
// becomes a CPU tensor and only the CPU channels are registered.
bool gHaveGpu = true;
const Device kCpu{kCpuDeviceType, 0};
Device kGpu{kHipDeviceType, 0};

struct InlineTensor {
  std::string data;
  std::string metadata;
  Device device;
  optional<Device> target;
};

struct InlineMessage {
  std::vector<std::pair<std::string, std::string>> payloads; // data, metadata
  std::vector<InlineTensor> tensors;
  std::string metadata;
};

std::shared_ptr<Context> makeContext(const char* name) {
  auto ctx = std::make_shared<Context>(ContextOptions().name(name));
  ctx->registerTransport(1, "shm", transport::shm::create());
  ctx->registerChannel(100, "basic", channel::basic::create());
  ctx->registerChannel(101, "xth", channel::xth::create());
  if (!gHaveGpu) {
    return ctx;
  }
  ctx->registerChannel(10, "hip_basic", channel::hip_basic::create(channel::basic::create()));
  ctx->registerChannel(11, "hip_ipc", channel::hip_ipc::create());
  ctx->registerChannel(12, "hip_xth", channel::hip_xth::create());
  return ctx;
}

std::vector<uint8_t> toBytes(const std::string& s) {
  return std::vector<uint8_t>(s.begin(), s.end());
}

// The same kind of buffer as `d`'s, `offset` bytes further into its memory.
Buffer subBuffer(Data& d, size_t offset) {
  Buffer whole = d.buffer();
  if (whole.device().type == kCpuDeviceType) {
    return CpuBuffer{static_cast<uint8_t*>(whole.unwrap<CpuBuffer>().ptr) + offset};
  }
  HipBuffer hb = whole.unwrap<HipBuffer>();
  hb.ptr = static_cast<uint8_t*>(hb.ptr) + offset;
  return hb;
}

// Owns the memory a Message refers to.
struct Storage {
  std::vector<std::vector<uint8_t>> payloads;
  std::vector<std::unique_ptr<Data>> tensors;
};

Message buildMessage(const InlineMessage& im, Storage* storage) {
  Message m;
  m.metadata = im.metadata;
  for (auto& p : im.payloads) {
    storage->payloads.push_back(toBytes(p.first));
    Message::Payload mp;
    mp.data = storage->payloads.back().data();
    mp.length = storage->payloads.back().size();
    mp.metadata = p.second;
    m.payloads.push_back(std::move(mp));
  }
  for (auto& t : im.tensors) {
    storage->tensors.push_back(makeData(gHaveGpu && t.device == kGpu, toBytes(t.data)));
    Message::Tensor mt;
    mt.buffer = storage->tensors.back()->buffer();
    mt.length = t.data.size();
    mt.targetDevice = t.target;
    mt.metadata = t.metadata;
    m.tensors.push_back(std::move(mt));
  }
  return m;
}

void writeMessage(Pipe& pipe, const InlineMessage& im) {
  Storage storage;
  Message m = buildMessage(im, &storage);
  auto p = std::make_shared<std::promise<Error>>();
  auto f = p->get_future();
  pipe.write(std::move(m), [p](const Error& e) { p->set_value(e); });
  EXPECT_OK(waitFor(f, "write"));
}

// readDescriptor, allocate on `devices`, read, compare with `im`.
void readAndCheck(Pipe& pipe, const InlineMessage& im, const std::vector<Device>& devices) {
  auto pd = std::make_shared<std::promise<std::pair<Error, Descriptor>>>();
  auto fd = pd->get_future();
  pipe.readDescriptor([pd](const Error& e, Descriptor d) { pd->set_value({e, std::move(d)}); });
  auto rd = waitFor(fd, "readDescriptor");
  EXPECT_OK(rd.first);
  if (rd.first) {
    return;
  }
  const Descriptor& d = rd.second;
  EXPECT_EQ(d.metadata, im.metadata);
  EXPECT_EQ(d.payloads.size(), im.payloads.size());
  EXPECT_EQ(d.tensors.size(), im.tensors.size());
  EXPECT_EQ(d.tensors.size(), devices.size());
  if (failures().any()) {
    throw Fatal("descriptor does not match the message; not reading");
  }

  Storage storage;
  Allocation a;
  for (auto& p : d.payloads) {
    storage.payloads.emplace_back(p.length, 0);
    Allocation::Payload ap;
    ap.data = storage.payloads.back().data();
    a.payloads.push_back(ap);
  }
  for (size_t i = 0; i < d.tensors.size(); ++i) {
    storage.tensors.push_back(makeData(gHaveGpu && devices[i] == kGpu, d.tensors[i].length));
    Allocation::Tensor at;
    at.buffer = storage.tensors.back()->buffer();
    a.tensors.push_back(std::move(at));
  }
  auto pr = std::make_shared<std::promise<Error>>();
  auto fr = pr->get_future();
  pipe.read(std::move(a), [pr](const Error& e) { pr->set_value(e); });
  EXPECT_OK(waitFor(fr, "read"));

  for (size_t i = 0; i < im.payloads.size(); ++i) {
    EXPECT_EQ(d.payloads[i].metadata, im.payloads[i].second);
    EXPECT_EQ(d.payloads[i].length, im.payloads[i].first.size());
    EXPECT_EQ(std::string(storage.payloads[i].begin(), storage.payloads[i].end()), im.payloads[i].first);
  }
  for (size_t i = 0; i < im.tensors.size(); ++i) {
    EXPECT_TRUE(d.tensors[i].sourceDevice == im.tensors[i].device);
    EXPECT_EQ(d.tensors[i].metadata, im.tensors[i].metadata);
    EXPECT_EQ(d.tensors[i].targetDevice.has_value(), im.tensors[i].target.has_value());
    if (d.tensors[i].targetDevice.has_value() && im.tensors[i].target.has_value()) {
      EXPECT_TRUE(*d.tensors[i].targetDevice == *im.tensors[i].target);
      EXPECT_TRUE(*im.tensors[i].target == devices[i]);
    }
    EXPECT_EQ(d.tensors[i].length, im.tensors[i].data.size());
    std::vector<uint8_t> got = storage.tensors[i]->bytes();
    EXPECT_EQ(std::string(got.begin(), got.end()), im.tensors[i].data);
  }
}

struct PipeEnd {
  std::shared_ptr<Context> ctx;
  std::shared_ptr<Listener> listener;
  std::shared_ptr<Pipe> pipe;
  ~PipeEnd() {
    pipe.reset();
    listener.reset();
    if (ctx) {
      ctx->join();
    }
  }
};

std::unique_ptr<PipeEnd> openPipe(Endpoint& ep) {
  auto e = std::make_unique<PipeEnd>();
  const std::string url = "shm://" + ep.freshAddr();
  if (ep.isServer()) {
    e->ctx = makeContext("server");
    e->listener = e->ctx->listen({url});
    ep.signalListening();
    auto p = std::make_shared<std::promise<std::pair<Error, std::shared_ptr<Pipe>>>>();
    auto f = p->get_future();
    e->listener->accept([p](const Error& err, std::shared_ptr<Pipe> pipe) {
      p->set_value({err, std::move(pipe)});
    });
    auto r = waitFor(f, "accept");
    if (r.first) {
      throw Fatal("accept failed: " + r.first.what());
    }
    e->pipe = std::move(r.second);
  } else {
    e->ctx = makeContext("client");
    ep.awaitListening();
    e->pipe = e->ctx->connect(url);
  }
  return e;
}

InlineMessage messageWith(std::vector<InlineTensor> tensors) {
  InlineMessage im;
  im.payloads = {{"payload #1", "payload metadata #1"},
                 {"payload #2", "payload metadata #2"},
                 {"payload #3", "payload metadata #3"}};
  im.tensors = std::move(tensors);
  im.metadata = "pipe metadata";
  return im;
}

// The server writes `im`; the client reads it onto `devices`.
Case oneWay(std::string name, InlineMessage im, std::vector<Device> devices) {
  return Case{std::move(name),
              [im](Endpoint& ep) {
                auto e = openPipe(ep);
                writeMessage(*e->pipe, im);
                ep.barrier();
              },
              [im, devices](Endpoint& ep) {
                auto e = openPipe(ep);
                readAndCheck(*e->pipe, im, devices);
                ep.barrier();
              }};
}


// ---- many messages in flight ----------------------------------------------------

// Deterministic content of tensor `t` of message `m` travelling in direction `dir`.
std::vector<uint8_t> patterned(uint32_t dir, uint32_t m, uint32_t t, size_t n) {
  std::vector<uint8_t> v(n);
  uint64_t x = 0x9E3779B97F4A7C15ull * (1 + dir + 7 * m + 131 * t) + n;
  for (size_t i = 0; i < n; ++i) {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    v[i] = static_cast<uint8_t>(x >> 11);
  }
  return v;
}

// Shape of message `m` in direction `dir`: tensor lengths and devices, derived
// from the indices alone so that both endpoints agree without talking.
struct Shape {
  std::vector<size_t> lengths;
  std::vector<bool> gpu;
};

Shape shapeOf(uint32_t dir, uint32_t m) {
  Shape s;
  uint64_t x = 0xD1B54A32D192ED03ull * (3 + dir + 2 * m);
  const uint32_t n = static_cast<uint32_t>((x >> 60) % 6); // 0..5 tensors
  for (uint32_t t = 0; t < n; ++t) {
    x = x * 6364136223846793005ull + 1442695040888963407ull;
    const uint32_t cls = static_cast<uint32_t>((x >> 33) % 5);
    size_t len = 0;
    switch (cls) {
      case 0: len = 0; break;
      case 1: len = 1 + (x >> 40) % 63; break;
      case 2: len = 4096 + (x >> 40) % 4096; break;
      case 3: len = (256u << 10) + (x >> 40) % 1000; break;
      default: len = (2u << 20) + (x >> 40) % 100000; break;
    }
    s.lengths.push_back(len);
    s.gpu.push_back(((x >> 20) & 1) != 0);
  }
  return s;
}

// Writes `count` messages without waiting in between and reads `count`
// messages of the opposite direction at the same time; every callback must
// fire exactly once, in order, with the right bytes.
// `lane` separates the contents of pipes that run side by side.
void exchangeMany(Pipe& pipe, uint32_t myRole, uint32_t count, uint32_t lane = 0) {
  const uint32_t myDir = myRole + 2 * lane;
  struct Outgoing {
    Storage storage;
    std::future<Error> done;
  };
  std::vector<std::unique_ptr<Outgoing>> outs;
  auto writeFires = std::make_shared<std::vector<int>>(count, 0);
  for (uint32_t m = 0; m < count; ++m) {
    Shape sh = shapeOf(myDir, m);
    auto o = std::make_unique<Outgoing>();
    Message msg;
    msg.metadata = "m" + std::to_string(m);
    for (size_t t = 0; t < sh.lengths.size(); ++t) {
      o->storage.tensors.push_back(
          makeData(gHaveGpu && sh.gpu[t], patterned(myDir, m, static_cast<uint32_t>(t), sh.lengths[t])));
      Message::Tensor mt;
      mt.buffer = o->storage.tensors.back()->buffer();
      mt.length = sh.lengths[t];
      mt.metadata = "t" + std::to_string(t);
      msg.tensors.push_back(std::move(mt));
    }
    auto p = std::make_shared<std::promise<Error>>();
    o->done = p->get_future();
    pipe.write(std::move(msg), [p, writeFires, m](const Error& e) {
      if (++(*writeFires)[m] == 1) {
        p->set_value(e);
      }
    });
    outs.push_back(std::move(o));
  }

  const uint32_t theirDir = (1 - myRole) + 2 * lane;
  for (uint32_t m = 0; m < count; ++m) {
    Shape sh = shapeOf(theirDir, m);
    auto pd = std::make_shared<std::promise<std::pair<Error, Descriptor>>>();
    auto fd = pd->get_future();
    pipe.readDescriptor([pd](const Error& e, Descriptor d) { pd->set_value({e, std::move(d)}); });
    auto rd = waitFor(fd, "readDescriptor");
    EXPECT_OK(rd.first);
    if (rd.first) {
      throw Fatal("readDescriptor failed in the middle of the exchange");
    }
    const Descriptor& d = rd.second;
    EXPECT_EQ(d.metadata, "m" + std::to_string(m)); // messages arrive in the order written
    EXPECT_EQ(d.tensors.size(), sh.lengths.size());
    if (d.tensors.size() != sh.lengths.size()) {
      throw Fatal("unexpected message shape");
    }
    Storage storage;
    Allocation a;
    for (size_t t = 0; t < d.tensors.size(); ++t) {
      EXPECT_EQ(d.tensors[t].length, sh.lengths[t]);
      // receive on the other kind of device than the one it was sent from
      storage.tensors.push_back(makeData(gHaveGpu && !sh.gpu[t], d.tensors[t].length));
      Allocation::Tensor at;
      at.buffer = storage.tensors.back()->buffer();
      a.tensors.push_back(std::move(at));
    }
    auto pr = std::make_shared<std::promise<Error>>();
    auto fr = pr->get_future();
    pipe.read(std::move(a), [pr](const Error& e) { pr->set_value(e); });
    EXPECT_OK(waitFor(fr, "read"));
    for (size_t t = 0; t < d.tensors.size(); ++t) {
      if (storage.tensors[t]->bytes() != patterned(theirDir, m, static_cast<uint32_t>(t), sh.lengths[t])) {
        failures().add("message " + std::to_string(m) + " tensor " + std::to_string(t) + " differs");
      }
    }
  }
  for (uint32_t m = 0; m < count; ++m) {
    EXPECT_OK(waitFor(outs[m]->done, "write"));
  }
  for (uint32_t m = 0; m < count; ++m) {
    EXPECT_EQ((*writeFires)[m], 1);
  }
}

// Posts one readDescriptor -> read chain per expected message before anything
// has arrived (pipeReadWithFuture of pipe_test.h, several at once), then checks
// what each of them received.
void readPostedAhead(Pipe& pipe, const std::vector<InlineMessage>& expected,
                     const std::vector<std::vector<Device>>& devices) {
  struct Got {
    Descriptor descriptor;
    Storage storage;
  };
  const size_t n = expected.size();
  auto got = std::make_shared<std::vector<Got>>(n);
  auto left = std::make_shared<std::atomic<int>>(static_cast<int>(n));
  auto done = std::make_shared<std::promise<std::string>>();
  auto fDone = done->get_future();
  auto finish = [done](const std::string& what) {
    try {
      done->set_value(what);
    } catch (const std::future_error&) {
    }
  };
  Pipe* p = &pipe;
  for (size_t i = 0; i < n; ++i) {
    const std::vector<Device> onto = devices[i];
    p->readDescriptor([p, got, left, finish, i, onto](const Error& err, Descriptor d) {
      if (err) {
        finish("readDescriptor: " + err.what());
        return;
      }
      if (d.tensors.size() != onto.size()) {
        finish("message " + std::to_string(i) + " has " + std::to_string(d.tensors.size()) + " tensors");
        return;
      }
      Got& g = (*got)[i];
      Allocation a;
      for (auto& pl : d.payloads) {
        g.storage.payloads.emplace_back(pl.length, 0);
        Allocation::Payload ap;
        ap.data = g.storage.payloads.back().data();
        a.payloads.push_back(ap);
      }
      for (size_t t = 0; t < d.tensors.size(); ++t) {
        g.storage.tensors.push_back(makeData(gHaveGpu && onto[t] == kGpu, d.tensors[t].length));
        Allocation::Tensor at;
        at.buffer = g.storage.tensors.back()->buffer();
        a.tensors.push_back(std::move(at));
      }
      g.descriptor = std::move(d);
      p->read(std::move(a), [left, finish](const Error& err2) {
        if (err2) {
          finish("read: " + err2.what());
        } else if (left->fetch_sub(1) == 1) {
          finish("");
        }
      });
    });
  }
  const std::string problem = waitFor(fDone, "reads posted ahead");
  EXPECT_EQ(problem, std::string());
  if (!problem.empty()) {
    return;
  }
  for (size_t i = 0; i < n; ++i) {
    const InlineMessage& im = expected[i];
    const Got& g = (*got)[i];
    EXPECT_EQ(g.descriptor.metadata, im.metadata);
    EXPECT_EQ(g.descriptor.payloads.size(), im.payloads.size());
    EXPECT_EQ(g.descriptor.tensors.size(), im.tensors.size());
    for (size_t k = 0; k < g.storage.payloads.size() && k < im.payloads.size(); ++k) {
      EXPECT_EQ(g.descriptor.payloads[k].metadata, im.payloads[k].second);
      EXPECT_EQ(std::string(g.storage.payloads[k].begin(), g.storage.payloads[k].end()), im.payloads[k].first);
    }
    for (size_t k = 0; k < g.storage.tensors.size() && k < im.tensors.size(); ++k) {
      std::vector<uint8_t> b = g.storage.tensors[k]->bytes();
      EXPECT_EQ(std::string(b.begin(), b.end()), im.tensors[k].data);
      EXPECT_EQ(g.descriptor.tensors[k].metadata, im.tensors[k].metadata);
      EXPECT_TRUE(g.descriptor.tensors[k].sourceDevice == im.tensors[k].device);
      EXPECT_EQ(g.descriptor.tensors[k].targetDevice.has_value(), im.tensors[k].target.has_value());
    }
  }
}

// The server writes both messages without waiting in between; the client has
// both reads posted.
Case twoInFlight(std::string name, InlineMessage im1, InlineMessage im2, std::vector<Device> onto1,
                 std::vector<Device> onto2) {
  return Case{std::move(name),
              [im1, im2](Endpoint& ep) {
                auto e = openPipe(ep);
                Storage s1, s2;
                auto p1 = std::make_shared<std::promise<Error>>();
                auto p2 = std::make_shared<std::promise<Error>>();
                auto f1 = p1->get_future();
                auto f2 = p2->get_future();
                e->pipe->write(buildMessage(im1, &s1), [p1](const Error& err) { p1->set_value(err); });
                e->pipe->write(buildMessage(im2, &s2), [p2](const Error& err) { p2->set_value(err); });
                EXPECT_OK(waitFor(f1, "first write"));
                EXPECT_OK(waitFor(f2, "second write"));
                ep.barrier();
              },
              [im1, im2, onto1, onto2](Endpoint& ep) {
                auto e = openPipe(ep);
                readPostedAhead(*e->pipe, {im1, im2}, {onto1, onto2});
                ep.barrier();
              }};
}

std::vector<Case> makeCases() {
  std::vector<Case> cases;

  // pipe_test.cc:20-70 (SimpleWriteRead; context_test.cc ClientPingSerial sends
  // the same kind of message once): payloads and three CPU tensors.
  cases.push_back(oneWay(
      "SimpleWriteRead",
      messageWith({{"tensor #1", "tensor metadata #1", kCpu, nullopt},
                   {"tensor #2", "tensor metadata #2", kCpu, nullopt},
                   {"tensor #3", "tensor metadata #3", kCpu, nullopt}}),
      {kCpu, kCpu, kCpu}));

  // pipe_cuda_test.cc:13-81
  cases.push_back(oneWay(
      "SimpleWriteReadWithAllTargetDevices",
      messageWith({{"tensor #1", "tensor metadata #1", kGpu, kGpu},
                   {"tensor #2", "tensor metadata #2", kCpu, kGpu},
                   {"tensor #3", "tensor metadata #3", kGpu, kCpu},
                   {"tensor #4", "tensor metadata #4", kCpu, kCpu}}),
      {kGpu, kGpu, kCpu, kCpu}));

  // pipe_cuda_test.cc:83-142
  cases.push_back(oneWay(
      "SimpleWriteReadWithSomeTargetDevices",
      messageWith({{"tensor #1", "tensor metadata #1", kGpu, kGpu},
                   {"tensor #2", "tensor metadata #2", kGpu, nullopt},
                   {"tensor #3", "tensor metadata #3", kCpu, nullopt}}),
      {kGpu, kCpu, kCpu}));

  // pipe_cuda_test.cc:144-208
  cases.push_back(oneWay(
      "SimpleWriteReadWithoutTargetDevice",
      messageWith({{"tensor #1", "tensor metadata #1", kCpu, nullopt},
                   {"tensor #2", "tensor metadata #2", kCpu, nullopt},
                   {"tensor #3", "tensor metadata #3", kGpu, nullopt},
                   {"tensor #4", "tensor metadata #4", kGpu, nullopt}}),
      {kCpu, kGpu, kCpu, kGpu}));

  // pipe_test.cc:72-105: a message of payloads alone.
  {
    InlineMessage im = messageWith({});
    cases.push_back(oneWay("SimpleWriteReadPayloadsOnly", im, {}));
  }

  // pipe_test.cc:107-160: a message of tensors alone.
  {
    InlineMessage im = messageWith({{"tensor #1", "tensor metadata #1", kGpu, nullopt},
                                    {"tensor #2", "tensor metadata #2", kCpu, nullopt}});
    im.payloads.clear();
    cases.push_back(oneWay("SimpleWriteReadTensorsOnly", im, {kGpu, kCpu}));
  }

  // context_test.cc:468-632 (ServerPingPongTwice): two pings written back to
  // back; every later step (readDescriptor, read, the pong's write) is issued
  // from inside the callback of the one before, and the rounds finish in order.
  {
    struct Round {
      Storage out;
      Storage in;
      Descriptor descriptor;
    };
    auto pingPong = [](Endpoint& ep) {
      auto e = openPipe(ep);
      const bool server = ep.isServer();
      const InlineMessage im = messageWith({{"tensor #1", "tensor metadata #1", kGpu, nullopt},
                                            {"tensor #2", "tensor metadata #2", kCpu, nullopt}});
      Pipe* pipe = e->pipe.get();
      auto rounds = std::make_shared<std::vector<Round>>(2);
      auto finished = std::make_shared<std::atomic<int>>(0);
      auto done = std::make_shared<std::promise<std::string>>();
      auto fDone = done->get_future();
      auto settle = [done, finished](int i, const Error& err, const char* what) {
        // a failure ends the case at once; success needs both rounds, in order
        if (err) {
          try {
            done->set_value(std::string(what) + ": " + err.what());
          } catch (const std::future_error&) {
          }
          return false;
        }
        (void)i;
        return true;
      };
      // readDescriptor -> read, then `then(i)`
      auto readOne = [pipe, rounds, settle](int i, std::function<void(int)> then) {
        pipe->readDescriptor([pipe, rounds, settle, i, then](const Error& err, Descriptor d) {
          if (!settle(i, err, "readDescriptor")) {
            return;
          }
          Round& r = (*rounds)[i];
          Allocation a;
          for (auto& p : d.payloads) {
            r.in.payloads.emplace_back(p.length, 0);
            Allocation::Payload ap;
            ap.data = r.in.payloads.back().data();
            a.payloads.push_back(ap);
          }
          for (auto& t : d.tensors) {
            r.in.tensors.push_back(makeData(gHaveGpu && t.sourceDevice == kGpu, t.length));
            Allocation::Tensor at;
            at.buffer = r.in.tensors.back()->buffer();
            a.tensors.push_back(std::move(at));
          }
          r.descriptor = std::move(d);
          pipe->read(std::move(a), [settle, i, then](const Error& err2) {
            if (settle(i, err2, "read")) {
              then(i);
            }
          });
        });
      };
      auto roundOver = [finished, done](int i) {
        const int before = finished->fetch_add(1);
        if (before != i) {
          try {
            done->set_value("round " + std::to_string(i) + " finished out of order");
          } catch (const std::future_error&) {
          }
        } else if (before == 1) {
          try {
            done->set_value("");
          } catch (const std::future_error&) {
          }
        }
      };
      for (int i = 0; i < 2; ++i) {
        if (server) {
          // ping; from its callback: read the pong
          Message m = buildMessage(im, &(*rounds)[i].out);
          pipe->write(std::move(m), [settle, readOne, roundOver, i](const Error& err) {
            if (settle(i, err, "write")) {
              readOne(i, roundOver);
            }
          });
        } else {
          // read the ping; from the read's callback: write the pong
          readOne(i, [pipe, rounds, im, settle, roundOver](int k) {
            Message m = buildMessage(im, &(*rounds)[k].out);
            pipe->write(std::move(m), [settle, roundOver, k](const Error& err) {
              if (settle(k, err, "write")) {
                roundOver(k);
              }
            });
          });
        }
      }
      const std::string problem = waitFor(fDone, "two chained rounds");
      EXPECT_EQ(problem, std::string());
      for (int i = 0; i < 2 && problem.empty(); ++i) {
        Round& r = (*rounds)[i];
        EXPECT_EQ(r.descriptor.metadata, im.metadata);
        EXPECT_EQ(r.descriptor.payloads.size(), im.payloads.size());
        EXPECT_EQ(r.descriptor.tensors.size(), im.tensors.size());
        for (size_t k = 0; k < r.in.payloads.size() && k < im.payloads.size(); ++k) {
          EXPECT_EQ(std::string(r.in.payloads[k].begin(), r.in.payloads[k].end()), im.payloads[k].first);
        }
        for (size_t k = 0; k < r.in.tensors.size() && k < im.tensors.size(); ++k) {
          std::vector<uint8_t> got = r.in.tensors[k]->bytes();
          EXPECT_EQ(std::string(got.begin(), got.end()), im.tensors[k].data);
          EXPECT_EQ(r.descriptor.tensors[k].metadata, im.tensors[k].metadata);
        }
      }
      ep.barrier();
    };
    cases.push_back({"ServerPingPongTwice", pingPong, pingPong});
  }

  // pipe_test.cc:286-364 (MultipleWriteRead) and :366-446
  // (MultipleWriteReadWithSomeTargetDevices), and the same with a GPU tensor.
  {
    InlineMessage m1, m2;
    m1.metadata = m2.metadata = "message metadata";
    m1.payloads = {{"payload #1.1", "payload metadata #1.1"}};
    m2.payloads = {{"payload #2.1", "payload metadata #2.1"}};
    m1.tensors = {{"tensor #1.1", "tensor metadata #1.1", kCpu, nullopt}};
    m2.tensors = {{"tensor #2.1", "tensor metadata #2.1", kCpu, nullopt}};
    cases.push_back(twoInFlight("MultipleWriteRead", m1, m2, {kCpu}, {kCpu}));
    m2.tensors = {{"tensor #2.1", "tensor metadata #2.1", kCpu, kCpu}};
    cases.push_back(twoInFlight("MultipleWriteReadWithSomeTargetDevices", m1, m2, {kCpu}, {kCpu}));
    m1.tensors = {{"tensor #1.1", "tensor metadata #1.1", kGpu, nullopt}};
    m2.tensors = {{"tensor #2.1", "tensor metadata #2.1", kGpu, kGpu},
                  {"tensor #2.2", "tensor metadata #2.2", kCpu, nullopt}};
    cases.push_back(twoInFlight("MultipleWriteReadWithGpuTensors", m1, m2, {kCpu}, {kGpu, kGpu}));
  }

  // Two messages in flight whose GPU tensors each take several wire units in
  // the cross-process channel (outbox route, 1 MiB slots): the second read is
  // posted while the first tensor's chunks are still arriving.
  if (gHaveGpu) {
    auto big = [](int k) {
      std::string v(3 * 1024 * 1024 + 300 * 1024 + 5, '\0');
      for (size_t j = 0; j < v.size(); ++j) {
        v[j] = static_cast<char>((j * 13 + static_cast<size_t>(k) * 101 + (j >> 11)) % 253);
      }
      return v;
    };
    InlineMessage m1, m2;
    m1.metadata = m2.metadata = "message metadata";
    m1.tensors = {{big(1), "tensor metadata #1.1", kGpu, kGpu}, {big(2), "tensor metadata #1.2", kGpu, kGpu}};
    m2.tensors = {{big(3), "tensor metadata #2.1", kGpu, kGpu}};
    Case inner = twoInFlight("ChunkedGpuTensorsTwoInFlight", m1, m2, {kGpu, kGpu}, {kGpu});
    auto staged = [](std::function<void(Endpoint&)> fn) {
      return [fn](Endpoint& ep) {
        ::setenv("TP_HIP_IPC_MODE", "outbox", 1);
        ::setenv("TP_HIP_IPC_SLOT_BYTES", "1048576", 1);
        ::setenv("TP_HIP_IPC_NUM_SLOTS", "3", 1);
        try {
          fn(ep);
        } catch (...) {
          ::unsetenv("TP_HIP_IPC_MODE");
          ::unsetenv("TP_HIP_IPC_SLOT_BYTES");
          ::unsetenv("TP_HIP_IPC_NUM_SLOTS");
          throw;
        }
        ::unsetenv("TP_HIP_IPC_MODE");
        ::unsetenv("TP_HIP_IPC_SLOT_BYTES");
        ::unsetenv("TP_HIP_IPC_NUM_SLOTS");
      };
    };
    cases.push_back({inner.name, staged(inner.server), staged(inner.client)});
  }

  // context_test.cc:634-738 (MixedTensorMessage): two reads are posted before
  // anything arrives; a message with payloads and tensors is followed by one
  // with nothing in it at all.
  cases.push_back(
      {"MixedTensorMessage",
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         Pipe* pipe = e->pipe.get();
         struct Got {
           Descriptor descriptor;
           Storage storage;
         };
         auto got = std::make_shared<std::vector<Got>>(2);
         auto left = std::make_shared<std::atomic<int>>(2);
         auto done = std::make_shared<std::promise<std::string>>();
         auto fDone = done->get_future();
         auto finish = [done](const std::string& what) {
           try {
             done->set_value(what);
           } catch (const std::future_error&) {
           }
         };
         for (int i = 0; i < 2; ++i) {
           pipe->readDescriptor([pipe, got, left, finish, i](const Error& err, Descriptor d) {
             if (err) {
               finish("readDescriptor: " + err.what());
               return;
             }
             Got& g = (*got)[i];
             Allocation a;
             for (auto& p : d.payloads) {
               g.storage.payloads.emplace_back(p.length, 0);
               Allocation::Payload ap;
               ap.data = g.storage.payloads.back().data();
               a.payloads.push_back(ap);
             }
             for (auto& t : d.tensors) {
               g.storage.tensors.push_back(makeData(gHaveGpu && t.sourceDevice == kGpu, t.length));
               Allocation::Tensor at;
               at.buffer = g.storage.tensors.back()->buffer();
               a.tensors.push_back(std::move(at));
             }
             g.descriptor = std::move(d);
             pipe->read(std::move(a), [left, finish](const Error& err2) {
               if (err2) {
                 finish("read: " + err2.what());
               } else if (left->fetch_sub(1) == 1) {
                 finish("");
               }
             });
           });
         }
         ep.barrier(); // both reads are posted; now the peer writes
         EXPECT_EQ(waitFor(fDone, "two posted reads"), std::string());
         const InlineMessage im = messageWith({{"tensor #1", "tensor metadata #1", kGpu, nullopt},
                                               {"tensor #2", "tensor metadata #2", kCpu, nullopt}});
         const Got& first = (*got)[0];
         EXPECT_EQ(first.descriptor.metadata, im.metadata);
         EXPECT_EQ(first.descriptor.payloads.size(), im.payloads.size());
         EXPECT_EQ(first.descriptor.tensors.size(), im.tensors.size());
         for (size_t k = 0; k < first.storage.payloads.size() && k < im.payloads.size(); ++k) {
           EXPECT_EQ(std::string(first.storage.payloads[k].begin(), first.storage.payloads[k].end()),
                     im.payloads[k].first);
         }
         for (size_t k = 0; k < first.storage.tensors.size() && k < im.tensors.size(); ++k) {
           std::vector<uint8_t> b = first.storage.tensors[k]->bytes();
           EXPECT_EQ(std::string(b.begin(), b.end()), im.tensors[k].data);
         }
         const Got& second = (*got)[1];
         EXPECT_EQ(second.descriptor.metadata, std::string());
         EXPECT_EQ(second.descriptor.payloads.size(), size_t(0));
         EXPECT_EQ(second.descriptor.tensors.size(), size_t(0));
         ep.barrier();
       },
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         ep.barrier();
         writeMessage(*e->pipe, messageWith({{"tensor #1", "tensor metadata #1", kGpu, nullopt},
                                              {"tensor #2", "tensor metadata #2", kCpu, nullopt}}));
         InlineMessage nothing;
         writeMessage(*e->pipe, nothing);
         ep.barrier();
       }});

  // Several messages back to back, each answered, with tensors large enough to
  // go through more than one staging slot.
  cases.push_back(
      {"MixedMessagesBothDirections",
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         for (int k = 0; k < 5; ++k) {
           InlineMessage out = messageWith(
               {{std::string(3 * 1024 * 1024 + k, char('a' + k)), "big", kGpu, kGpu},
                {std::string(100 + k, char('A' + k)), "small", kCpu, nullopt},
                {"", "empty", kGpu, nullopt}});
           writeMessage(*e->pipe, out);
           InlineMessage in = messageWith(
               {{std::string(2 * 1024 * 1024 + k, char('k' + k)), "reply", kGpu, nullopt}});
           readAndCheck(*e->pipe, in, {kCpu});
         }
         ep.barrier();
       },
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         for (int k = 0; k < 5; ++k) {
           InlineMessage in = messageWith(
               {{std::string(3 * 1024 * 1024 + k, char('a' + k)), "big", kGpu, kGpu},
                {std::string(100 + k, char('A' + k)), "small", kCpu, nullopt},
                {"", "empty", kGpu, nullopt}});
           readAndCheck(*e->pipe, in, {kGpu, kGpu, kGpu});
           InlineMessage out = messageWith(
               {{std::string(2 * 1024 * 1024 + k, char('k' + k)), "reply", kGpu, nullopt}});
           writeMessage(*e->pipe, out);
         }
         ep.barrier();
       }});

  // context_test.cc:384-466 (ClientPingInline): read() issued from inside the
  // readDescriptor callback, on the library's thread.
  cases.push_back(
      {"ReadInsideDescriptorCallback",
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         auto done = std::make_shared<std::promise<Error>>();
         auto fDone = done->get_future();
         auto storage = std::make_shared<Storage>();
         auto got = std::make_shared<Descriptor>();
         Pipe* pipe = e->pipe.get();
         pipe->readDescriptor([pipe, done, storage, got](const Error& err, Descriptor d) {
           if (err) {
             done->set_value(err);
             return;
           }
           Allocation a;
           for (auto& p : d.payloads) {
             storage->payloads.emplace_back(p.length, 0);
             Allocation::Payload ap;
             ap.data = storage->payloads.back().data();
             a.payloads.push_back(ap);
           }
           for (auto& t : d.tensors) {
             storage->tensors.push_back(makeData(gHaveGpu && t.sourceDevice == kGpu, t.length));
             Allocation::Tensor at;
             at.buffer = storage->tensors.back()->buffer();
             a.tensors.push_back(std::move(at));
           }
           *got = std::move(d);
           pipe->read(std::move(a), [done](const Error& err2) { done->set_value(err2); });
         });
         EXPECT_OK(waitFor(fDone, "read chained to readDescriptor"));
         EXPECT_EQ(got->tensors.size(), size_t(2));
         if (got->tensors.size() == 2) {
           std::vector<uint8_t> b0 = storage->tensors[0]->bytes();
           std::vector<uint8_t> b1 = storage->tensors[1]->bytes();
           EXPECT_EQ(std::string(b0.begin(), b0.end()), std::string("tensor #1"));
           EXPECT_EQ(std::string(b1.begin(), b1.end()), std::string("tensor #2"));
         }
         ep.barrier();
       },
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         writeMessage(*e->pipe, messageWith({{"tensor #1", "tensor metadata #1", kGpu, nullopt},
                                              {"tensor #2", "tensor metadata #2", kCpu, nullopt}}));
         ep.barrier();
       }});

  // pipe_test.cc:525-600 (WriteFromBothThenRead): each endpoint writes before it
  // reads; neither write may wait for the local read.
  auto writeThenRead = [](Endpoint& ep) {
    auto e = openPipe(ep);
    const char mine = ep.isServer() ? 'S' : 'C';
    const char theirs = ep.isServer() ? 'C' : 'S';
    InlineMessage out = messageWith({{std::string(300000, mine), "from me", kGpu, nullopt},
                                     {std::string(17, mine), "small", kCpu, nullopt}});
    InlineMessage in = messageWith({{std::string(300000, theirs), "from me", kGpu, nullopt},
                                    {std::string(17, theirs), "small", kCpu, nullopt}});
    Storage storage;
    Message m = buildMessage(out, &storage);
    auto p = std::make_shared<std::promise<Error>>();
    auto f = p->get_future();
    e->pipe->write(std::move(m), [p](const Error& err) { p->set_value(err); });
    readAndCheck(*e->pipe, in, {kGpu, kCpu});
    EXPECT_OK(waitFor(f, "write"));
    ep.barrier();
  };
  cases.push_back({"WriteFromBothThenRead", writeThenRead, writeThenRead});

  // tensorpipe/core/pipe_impl.cc:987-1042,1108-1125: a pipe opened over TCP
  // between two contexts that both hold shm, preferred, moves there during the
  // handshake; messages then flow both ways (CPU tensors: the case is about
  // the pipe's own connections).
  auto movesToShm = [](Endpoint& ep) {
    auto e = std::make_unique<PipeEnd>();
    e->ctx = std::make_shared<Context>(ContextOptions().name(ep.isServer() ? "server" : "client"));
    e->ctx->registerTransport(1, "uv", transport::tcp::create());
    e->ctx->registerTransport(2, "shm", transport::shm::create());
    e->ctx->registerChannel(100, "basic", channel::basic::create());
    const std::string shmUrl = "shm://" + ep.freshAddr();
    InlineMessage im;
    im.metadata = "after the move";
    im.payloads = {{"payload #1", "payload metadata #1"}};
    im.tensors = {{std::string(300000, 'x'), "tensor metadata #1", kCpu, nullopt},
                  {"tensor #2", "", kCpu, kCpu}};
    if (ep.isServer()) {
      e->listener = e->ctx->listen({"uv://127.0.0.1:0", shmUrl});
      const std::string url = e->listener->url("uv");
      ep.sendNumber(static_cast<uint16_t>(std::stoi(url.substr(url.rfind(':') + 1))));
      auto p = std::make_shared<std::promise<std::pair<Error, std::shared_ptr<Pipe>>>>();
      auto f = p->get_future();
      e->listener->accept([p](const Error& err, std::shared_ptr<Pipe> pipe) {
        p->set_value({err, std::move(pipe)});
      });
      auto r = waitFor(f, "accept");
      if (r.first) {
        throw Fatal("accept failed: " + r.first.what());
      }
      e->pipe = std::move(r.second);
      writeMessage(*e->pipe, im);
      readAndCheck(*e->pipe, im, {kCpu, kCpu});
    } else {
      e->pipe = e->ctx->connect("uv://127.0.0.1:" + std::to_string(ep.recvNumber()));
      readAndCheck(*e->pipe, im, {kCpu, kCpu});
      writeMessage(*e->pipe, im);
    }
    EXPECT_EQ(e->pipe->transportInUse(), std::string("shm"));
    ep.barrier();
  };
  cases.push_back({"PipeOpenedOverTcpMovesToShm", movesToShm, movesToShm});

  // listener_test.cc:21-60 (ClosingAbortsOperations): an accept that is pending
  // when the listener closes fails, once.
  auto listenerClose = [](Endpoint& ep) {
    auto ctx = makeContext(ep.isServer() ? "server" : "client");
    auto listener = ctx->listen({"shm://" + ep.freshAddr() + (ep.isServer() ? "_s" : "_c")});
    auto fires = std::make_shared<std::atomic<int>>(0);
    auto p = std::make_shared<std::promise<Error>>();
    auto f = p->get_future();
    listener->accept([p, fires](const Error& err, std::shared_ptr<Pipe>) {
      if (fires->fetch_add(1) == 0) {
        p->set_value(err);
      }
    });
    listener->close();
    Error err = waitFor(f, "accept that must fail");
    EXPECT_TRUE(static_cast<bool>(err));
    listener.reset();
    ctx->join();
    EXPECT_EQ(fires->load(), 1);
  };
  cases.push_back({"ListenerClosingAbortsAccept", listenerClose, listenerClose});

  // Sixty messages of random shape each way, all writes issued up front.
  cases.push_back({"ManyMessagesBothDirections",
                   [](Endpoint& ep) {
                     auto e = openPipe(ep);
                     exchangeMany(*e->pipe, 0, 60);
                     ep.barrier();
                   },
                   [](Endpoint& ep) {
                     auto e = openPipe(ep);
                     exchangeMany(*e->pipe, 1, 60);
                     ep.barrier();
                   }});

  // The same with every GPU tensor in a device allocation of exactly its own
  // size, freed when its message is done (the runtime packs such allocations
  // several to a block).
  cases.push_back({"ManyMessagesSmallAllocations",
                   [](Endpoint& ep) {
                     ExactGpuAllocations guard;
                     auto e = openPipe(ep);
                     exchangeMany(*e->pipe, 0, 60);
                     ep.barrier();
                   },
                   [](Endpoint& ep) {
                     ExactGpuAllocations guard;
                     auto e = openPipe(ep);
                     exchangeMany(*e->pipe, 1, 60);
                     ep.barrier();
                   }});

  // One message with more tensors than a copy table holds (4096): the channels
  // cut it into several launches, the pipe into nothing. 5000 tensors of 1 to
  // 200 bytes, carved at odd offsets out of one allocation on each side.
  {
    const uint32_t count = 5000;
    auto lengthOf = [](uint32_t t) { return size_t(1 + (t * 37u) % 200u); };
    auto layout = [lengthOf](std::vector<size_t>* offsets) {
      size_t off = 3;
      for (uint32_t t = 0; t < count; ++t) {
        offsets->push_back(off);
        off += lengthOf(t) + 1 + (t % 5);
      }
      return off;
    };
    cases.push_back(
        {"FiveThousandTensorsInOneMessage",
         [lengthOf, layout](Endpoint& ep) {
           auto e = openPipe(ep);
           std::vector<size_t> offsets;
           const size_t total = layout(&offsets);
           auto arena = makeData(gHaveGpu, patterned(0, 0, 0, total));
           Message msg;
           msg.metadata = "many";
           for (uint32_t t = 0; t < count; ++t) {
             Message::Tensor mt;
             mt.buffer = subBuffer(*arena, offsets[t]);
             mt.length = lengthOf(t);
             msg.tensors.push_back(std::move(mt));
           }
           auto p = std::make_shared<std::promise<Error>>();
           auto f = p->get_future();
           e->pipe->write(std::move(msg), [p](const Error& err) { p->set_value(err); });
           EXPECT_OK(waitFor(f, "write"));
           ep.barrier();
         },
         [lengthOf, layout](Endpoint& ep) {
           auto e = openPipe(ep);
           std::vector<size_t> offsets;
           const size_t total = layout(&offsets);
           auto pd = std::make_shared<std::promise<std::pair<Error, Descriptor>>>();
           auto fd = pd->get_future();
           e->pipe->readDescriptor(
               [pd](const Error& err, Descriptor d) { pd->set_value({err, std::move(d)}); });
           auto rd = waitFor(fd, "readDescriptor");
           EXPECT_OK(rd.first);
           EXPECT_EQ(rd.second.tensors.size(), size_t(count));
           if (rd.first || rd.second.tensors.size() != count) {
             throw Fatal("unexpected descriptor");
           }
           auto arena = makeData(gHaveGpu, std::vector<uint8_t>(total, 0xEE));
           Allocation a;
           for (uint32_t t = 0; t < count; ++t) {
             EXPECT_EQ(rd.second.tensors[t].length, lengthOf(t));
             Allocation::Tensor at;
             at.buffer = subBuffer(*arena, offsets[t]);
             a.tensors.push_back(std::move(at));
           }
           auto pr = std::make_shared<std::promise<Error>>();
           auto fr = pr->get_future();
           e->pipe->read(std::move(a), [pr](const Error& err) { pr->set_value(err); });
           EXPECT_OK(waitFor(fr, "read"));
           // every tensor arrived, and the gaps between them are untouched
           std::vector<uint8_t> want(total, 0xEE);
           const std::vector<uint8_t> sent = patterned(0, 0, 0, total);
           for (uint32_t t = 0; t < count; ++t) {
             std::copy(sent.begin() + offsets[t], sent.begin() + offsets[t] + lengthOf(t),
                       want.begin() + offsets[t]);
           }
           if (arena->bytes() != want) {
             failures().add("received arena differs");
           }
           ep.barrier();
         }});
  }

  // Four pipes between the same two contexts, each exchanging messages of
  // random shape both ways from a thread of its own: the channels of a context
  // share its staging slots, pinned rings, mapped peer allocations and event
  // poller.
  cases.push_back(
      {"SeveralPipesAtOnce",
       [](Endpoint& ep) {
         const uint32_t lanes = 4, count = 25;
         PipeEnd e;
         const std::string url = "shm://" + ep.freshAddr();
         e.ctx = makeContext("server");
         e.listener = e.ctx->listen({url});
         ep.signalListening();
         // Pipes are accepted in any order: the first message names the lane.
         std::vector<std::shared_ptr<Pipe>> pipes(lanes);
         for (uint32_t k = 0; k < lanes; ++k) {
           auto p = std::make_shared<std::promise<std::pair<Error, std::shared_ptr<Pipe>>>>();
           auto f = p->get_future();
           e.listener->accept([p](const Error& err, std::shared_ptr<Pipe> pipe) {
             p->set_value({err, std::move(pipe)});
           });
           auto r = waitFor(f, "accept");
           if (r.first) {
             throw Fatal("accept failed: " + r.first.what());
           }
           auto pd = std::make_shared<std::promise<std::pair<Error, Descriptor>>>();
           auto fd = pd->get_future();
           r.second->readDescriptor(
               [pd](const Error& err, Descriptor d) { pd->set_value({err, std::move(d)}); });
           auto rd = waitFor(fd, "lane announcement");
           if (rd.first) {
             throw Fatal("lane announcement failed: " + rd.first.what());
           }
           auto pr = std::make_shared<std::promise<Error>>();
           auto fr = pr->get_future();
           r.second->read(Allocation{}, [pr](const Error& err) { pr->set_value(err); });
           EXPECT_OK(waitFor(fr, "read of the lane announcement"));
           const uint32_t lane = static_cast<uint32_t>(std::stoul(rd.second.metadata));
           if (lane >= lanes || pipes[lane]) {
             throw Fatal("unexpected lane " + rd.second.metadata);
           }
           pipes[lane] = std::move(r.second);
         }
         std::vector<std::thread> threads;
         for (uint32_t k = 0; k < lanes; ++k) {
           threads.emplace_back([&pipes, k] {
             try {
               exchangeMany(*pipes[k], 0, count, k);
             } catch (const std::exception& ex) {
               failures().add("lane " + std::to_string(k) + ": " + ex.what());
             }
           });
         }
         for (auto& t : threads) {
           t.join();
         }
         ep.barrier();
         pipes.clear();
       },
       [](Endpoint& ep) {
         const uint32_t lanes = 4, count = 25;
         PipeEnd e;
         const std::string url = "shm://" + ep.freshAddr();
         e.ctx = makeContext("client");
         ep.awaitListening();
         std::vector<std::shared_ptr<Pipe>> pipes;
         for (uint32_t k = 0; k < lanes; ++k) {
           pipes.push_back(e.ctx->connect(url));
           Message msg;
           msg.metadata = std::to_string(k);
           auto p = std::make_shared<std::promise<Error>>();
           auto f = p->get_future();
           pipes.back()->write(std::move(msg), [p](const Error& err) { p->set_value(err); });
           EXPECT_OK(waitFor(f, "lane announcement"));
         }
         std::vector<std::thread> threads;
         for (uint32_t k = 0; k < lanes; ++k) {
           threads.emplace_back([&pipes, k] {
             try {
               exchangeMany(*pipes[k], 1, count, k);
             } catch (const std::exception& ex) {
               failures().add("lane " + std::to_string(k) + ": " + ex.what());
             }
           });
         }
         for (auto& t : threads) {
           t.join();
         }
         ep.barrier();
         pipes.clear();
       }});

  // Writes that are still queued or in flight when the pipe is closed complete
  // with an error or with success, but every one of them completes, once.
  cases.push_back(
      {"CloseWithWritesInFlight",
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         ep.barrier();
         const int count = 40;
         auto fires = std::make_shared<std::vector<std::atomic<int>>>(count);
         auto remaining = std::make_shared<std::atomic<int>>(count);
         auto all = std::make_shared<std::promise<void>>();
         auto fAll = all->get_future();
         std::vector<std::unique_ptr<Data>> keep;
         for (int m = 0; m < count; ++m) {
           keep.push_back(makeData(gHaveGpu && (m & 1), patterned(0, m, 0, (1u << 20) + m)));
           Message msg;
           Message::Tensor mt;
           mt.buffer = keep.back()->buffer();
           mt.length = keep.back()->size();
           msg.tensors.push_back(std::move(mt));
           e->pipe->write(std::move(msg), [fires, remaining, all, m](const Error&) {
             (*fires)[m].fetch_add(1);
             if (remaining->fetch_sub(1) == 1) {
               all->set_value();
             }
           });
           if (m == count / 2) {
             e->pipe->close();
           }
         }
         if (fAll.wait_for(std::chrono::seconds(kWaitSeconds)) != std::future_status::ready) {
           throw Fatal("not every write callback fired after close");
         }
         for (int m = 0; m < count; ++m) {
           EXPECT_EQ((*fires)[m].load(), 1);
         }
         ep.barrier();
       },
       [](Endpoint& ep) {
         auto e = openPipe(ep);
         ep.barrier();
         // Read whatever arrives until the pipe fails.
         for (;;) {
           auto pd = std::make_shared<std::promise<std::pair<Error, Descriptor>>>();
           auto fd = pd->get_future();
           e->pipe->readDescriptor(
               [pd](const Error& err, Descriptor d) { pd->set_value({err, std::move(d)}); });
           auto rd = waitFor(fd, "readDescriptor");
           if (rd.first) {
             break;
           }
           Storage storage;
           Allocation a;
           for (auto& t : rd.second.tensors) {
             storage.tensors.push_back(makeData(gHaveGpu, t.length));
             Allocation::Tensor at;
             at.buffer = storage.tensors.back()->buffer();
             a.tensors.push_back(std::move(at));
           }
           auto pr = std::make_shared<std::promise<Error>>();
           auto fr = pr->get_future();
           e->pipe->read(std::move(a), [pr](const Error& err) { pr->set_value(err); });
           if (waitFor(fr, "read")) {
             break;
           }
         }
         ep.barrier();
       }});

  // A pipe that is closed fails what is pending and what comes later.
  cases.push_back({"CloseFailsPendingRead",
                   [](Endpoint& ep) {
                     auto e = openPipe(ep);
                     auto pd = std::make_shared<std::promise<Error>>();
                     auto fd = pd->get_future();
                     e->pipe->readDescriptor(
                         [pd](const Error& err, Descriptor) { pd->set_value(err); });
                     ep.barrier(); // the client closes its end now
                     Error err = waitFor(fd, "readDescriptor that must fail");
                     EXPECT_TRUE(static_cast<bool>(err));
                     ep.barrier();
                   },
                   [](Endpoint& ep) {
                     auto e = openPipe(ep);
                     // make sure the pipe is fully established before closing
                     ep.barrier();
                     e->pipe->close();
                     ep.barrier();
                   }});

  return cases;
}

} // namespace

int main(int argc, char** argv) {
  Args args = parseArgs(argc, argv);
  const bool cpuOnly = args.suite.rfind("cpu_", 0) == 0;
  const std::string shape = cpuOnly ? args.suite.substr(4) : args.suite;
  if (shape != "two_process" && shape != "same_process") {
    std::fprintf(
        stderr, "usage: %s --suite [cpu_]two_process|[cpu_]same_process [--case S] [--list]\n",
        argv[0]);
    return 2;
  }
  if (cpuOnly) {
    gHaveGpu = false;
    kGpu = kCpu;
  }
  std::vector<Case> cases = makeCases();
  if (args.list) {
    for (auto& c : cases) {
      std::printf("%s\n", c.name.c_str());
    }
    return 0;
  }
  const std::string addr =
      args.addr.empty() ? "tppipe_" + std::to_string(::getpid()) + "_" + args.suite : args.addr;
  if (args.role == "server") {
    return runSingleRole(Role::kServer, cases, args.filter, addr, args.readyFd);
  }
  if (args.role == "client") {
    return runSingleRole(Role::kClient, cases, args.filter, addr, -1);
  }
  if (shape == "same_process") {
    return runBoth(cases, args.filter, addr);
  }
  std::vector<std::string> pass = {"--suite", args.suite};
  if (!args.filter.empty()) {
    pass.push_back("--case");
    pass.push_back(args.filter);
  }
  return orchestrate(argv[0], pass, addr);
}
