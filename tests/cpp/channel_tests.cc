// Channel-level tests of hip_xth, hip_ipc and hip_basic, driven through the
// plugin surface itself: channel::Context::createChannel over raw transport
// connections, then Channel::send / recv with Buffer{HipBuffer|CpuBuffer}.
//
//   channel_tests --suite hip_xth|hip_ipc|hip_ipc_outbox|hip_ipc_gated|hip_ipc_messages|hip_basic|hip_basic_host_ring|hip_basic_small_ring|basic|xth [--case SUBSTRING] [--list]
//
// hip_xth and xth run both endpoints as two threads of this process; hip_ipc,
// hip_basic and basic run them as two processes. The CPU channels (basic, xth)
// go through the same cases with host memory. Each case prints one
// "RESULT <role> <case> OK|FAIL ..." line per endpoint.
//
// Cases and data follow the reference's suites:
//   tensorpipe/test/channel/channel_test.cc:19-336        (generic)
//   tensorpipe/test/channel/channel_test_cuda.cc:19-139   (stream ordering, offsets)
//   tensorpipe/test/channel/channel_test_cuda_xdtt.cc:19-195 (CPU <-> GPU)
//   tensorpipe/test/channel/cuda_ipc/cuda_ipc_test.cc:37-57
//   tensorpipe/test/channel/cuda_basic/cuda_basic_test.cc:40-62
#include "support.h"

using namespace tptest;

namespace {

std::string gSuite;
bool gGpu = true; // whether the suite's tensors live on the GPU

bool knownSuite(const std::string& s) {
  return s == "hip_xth" || s == "hip_ipc" || s == "hip_ipc_outbox" || s == "hip_ipc_gated" ||
      s == "hip_ipc_messages" || s == "hip_basic" || s == "hip_basic_host_ring" ||
      s == "hip_basic_small_ring" || s == "basic" || s == "xth";
}

bool twoProcessSuite(const std::string& s) {
  return s == "hip_ipc" || s == "hip_ipc_outbox" || s == "hip_ipc_gated" || s == "hip_ipc_messages" ||
      s == "hip_basic" || s == "hip_basic_host_ring" || s == "hip_basic_small_ring" || s == "basic";
}

Buffer nullBuffer() {
  if (gGpu) {
    return HipBuffer{nullptr, nullptr};
  }
  return CpuBuffer{nullptr};
}

std::shared_ptr<channel::Context> makeContext() {
  if (gSuite == "hip_xth") {
    return channel::hip_xth::create();
  }
  if (gSuite == "hip_ipc" || gSuite == "hip_ipc_outbox" || gSuite == "hip_ipc_gated" ||
      gSuite == "hip_ipc_messages") {
    return channel::hip_ipc::create();
  }
  if (gSuite.rfind("hip_basic", 0) == 0) {
    return channel::hip_basic::create(channel::basic::create());
  }
  if (gSuite == "basic") {
    return channel::basic::create();
  }
  if (gSuite == "xth") {
    return channel::xth::create();
  }
  throw Fatal("unknown suite " + gSuite);
}

struct Opened {
  std::shared_ptr<channel::Context> ctx;
  std::shared_ptr<channel::Channel> ch;
  // Channel first, then the context (joined), as the reference's harness does.
  ~Opened() {
    ch.reset();
    if (ctx) {
      ctx->join();
    }
  }
};

std::unique_ptr<Opened> open(Endpoint& ep) {
  auto o = std::make_unique<Opened>();
  o->ctx = makeContext();
  o->ctx->setId(std::string(roleName(ep.role())) + "_ctx");
  if (!o->ctx->isViable()) {
    throw Fatal("context is not viable");
  }
  auto conns = ep.openConnections(o->ctx->numConnectionsNeeded());
  o->ch = o->ctx->createChannel(
      std::move(conns), ep.isServer() ? channel::Endpoint::kListen : channel::Endpoint::kConnect);
  return o;
}

std::future<Error> sendF(channel::Channel& ch, Buffer b, size_t n) {
  auto p = std::make_shared<std::promise<Error>>();
  auto f = p->get_future();
  ch.send(std::move(b), n, [p](const Error& e) { p->set_value(e); });
  return f;
}

std::future<Error> recvF(channel::Channel& ch, Buffer b, size_t n) {
  auto p = std::make_shared<std::promise<Error>>();
  auto f = p->get_future();
  ch.recv(std::move(b), n, [p](const Error& e) { p->set_value(e); });
  return f;
}

void expectBytes(Data& d, const std::vector<uint8_t>& want, const char* what) {
  std::vector<uint8_t> got = d.bytes();
  if (got.size() != want.size()) {
    failures().add(std::string(what) + ": size differs");
    return;
  }
  for (size_t i = 0; i < got.size(); ++i) {
    if (got[i] != want[i]) {
      failures().add(
          std::string(what) + ": byte " + std::to_string(i) + " is " + std::to_string(got[i]) +
          ", expected " + std::to_string(want[i]));
      return;
    }
  }
}

// A transfer of `data` from the sending endpoint to the receiving one.
void sender(Endpoint& ep, bool gpu, const std::vector<uint8_t>& data) {
  auto o = open(ep);
  auto d = makeData(gpu, data);
  auto f = sendF(*o->ch, d->buffer(), d->size());
  EXPECT_OK(waitFor(f, "send"));
  ep.barrier();
}

void receiver(Endpoint& ep, bool gpu, const std::vector<uint8_t>& want) {
  auto o = open(ep);
  auto d = makeData(gpu, want.size());
  auto f = recvF(*o->ch, d->buffer(), d->size());
  EXPECT_OK(waitFor(f, "recv"));
  expectBytes(*d, want, "received data");
  ep.barrier();
}

std::vector<Case> makeCases() {
  std::vector<Case> cases;
  const bool staged = gSuite.rfind("hip_basic", 0) == 0;

  // channel_test.cc:19-43
  auto descriptors = [](Endpoint&) {
    auto c1 = makeContext();
    auto c2 = makeContext();
    const auto& d1 = c1->deviceDescriptors();
    const auto& d2 = c2->deviceDescriptors();
    EXPECT_FALSE(d1.empty());
    EXPECT_EQ(d1.size(), d2.size());
    EXPECT_EQ(d1.count(gGpu ? Device{kHipDeviceType, 0} : Device{kCpuDeviceType, 0}), size_t(1));
    for (auto& kv : d1) {
      EXPECT_FALSE(kv.second.empty());
      EXPECT_EQ(d2.count(kv.first), size_t(1));
      if (d2.count(kv.first) == 1) {
        EXPECT_EQ(kv.second, d2.at(kv.first));
      }
    }
    c1->join();
    c2->join();
  };
  cases.push_back({"DeviceDescriptors", descriptors, descriptors});

  // channel_test.cc:45-125: 256 sequential bytes, each direction.
  cases.push_back({"ServerToClient",
                   [](Endpoint& ep) { sender(ep, gGpu, iota(256)); },
                   [](Endpoint& ep) { receiver(ep, gGpu, iota(256)); }});
  cases.push_back({"ClientToServer",
                   [](Endpoint& ep) { receiver(ep, gGpu, iota(256)); },
                   [](Endpoint& ep) { sender(ep, gGpu, iota(256)); }});

  // channel_test.cc:127-189: 100 tensors of 256 KiB holding i % 256, all posted
  // before any is awaited.
  cases.push_back(
      {"SendMultipleTensors",
       [](Endpoint& ep) {
         auto o = open(ep);
         auto d = makeData(gGpu, iota(256 * 1024));
         std::vector<std::future<Error>> fs;
         for (int i = 0; i < 100; ++i) {
           fs.push_back(sendF(*o->ch, d->buffer(), d->size()));
         }
         for (auto& f : fs) {
           EXPECT_OK(waitFor(f, "send"));
         }
         ep.barrier();
       },
       [](Endpoint& ep) {
         auto o = open(ep);
         std::vector<std::unique_ptr<Data>> ds;
         std::vector<std::future<Error>> fs;
         for (int i = 0; i < 100; ++i) {
           ds.push_back(makeData(gGpu, 256 * 1024));
           fs.push_back(recvF(*o->ch, ds.back()->buffer(), ds.back()->size()));
         }
         for (auto& f : fs) {
           EXPECT_OK(waitFor(f, "recv"));
         }
         const auto want = iota(256 * 1024);
         for (auto& d : ds) {
           expectBytes(*d, want, "tensor");
         }
         ep.barrier();
       }});

  // Several receives posted ahead of tensors that take several wire units each
  // (3.5 MiB against the 1 MiB staging slots of the chunking suites), every
  // tensor with bytes of its own: a unit handed to the wrong operation shows.
  {
    auto pattern = [](int k) {
      std::vector<uint8_t> v(3 * 1024 * 1024 + 512 * 1024 + 17);
      for (size_t j = 0; j < v.size(); ++j) {
        v[j] = static_cast<uint8_t>((j * 7 + static_cast<size_t>(k) * 37 + (j >> 12)) % 251);
      }
      return v;
    };
    cases.push_back(
        {"SeveralChunkedTensorsPostedAhead",
         [pattern](Endpoint& ep) {
           auto o = open(ep);
           std::vector<std::unique_ptr<Data>> ds;
           std::vector<std::future<Error>> fs;
           for (int k = 0; k < 4; ++k) {
             ds.push_back(makeData(gGpu, pattern(k)));
             fs.push_back(sendF(*o->ch, ds.back()->buffer(), ds.back()->size()));
           }
           for (auto& f : fs) {
             EXPECT_OK(waitFor(f, "send"));
           }
           ep.barrier();
         },
         [pattern](Endpoint& ep) {
           auto o = open(ep);
           std::vector<std::unique_ptr<Data>> ds;
           std::vector<std::future<Error>> fs;
           for (int k = 0; k < 4; ++k) {
             ds.push_back(makeData(gGpu, pattern(k).size()));
             fs.push_back(recvF(*o->ch, ds.back()->buffer(), ds.back()->size()));
           }
           for (auto& f : fs) {
             EXPECT_OK(waitFor(f, "recv"));
           }
           for (int k = 0; k < 4; ++k) {
             expectBytes(*ds[k], pattern(k), "tensor");
           }
           ep.barrier();
         }});
  }

  // Many small tensors of different sizes, each with bytes of its own, all
  // posted before any is awaited: a channel that lets ready receives share a
  // launch (or a unit) must still put every byte where it belongs.
  {
    auto sizeOf = [](int k) { return static_cast<size_t>(1 + (k * 7919) % 40000 + (k % 5 == 0 ? 70000 : 0)); };
    auto pattern = [sizeOf](int k) {
      std::vector<uint8_t> v(sizeOf(k));
      for (size_t j = 0; j < v.size(); ++j) {
        v[j] = static_cast<uint8_t>((j * 13 + static_cast<size_t>(k) * 101 + (j >> 9)) % 253);
      }
      return v;
    };
    constexpr int kTensors = 160;
    cases.push_back(
        {"ManySmallTensorsEachItsOwn",
         [pattern](Endpoint& ep) {
           auto o = open(ep);
           std::vector<std::unique_ptr<Data>> ds;
           std::vector<std::future<Error>> fs;
           for (int k = 0; k < kTensors; ++k) {
             ds.push_back(makeData(gGpu, pattern(k)));
           }
           for (int k = 0; k < kTensors; ++k) {
             fs.push_back(sendF(*o->ch, ds[k]->buffer(), ds[k]->size()));
           }
           for (auto& f : fs) {
             EXPECT_OK(waitFor(f, "send"));
           }
           ep.barrier();
         },
         [pattern, sizeOf](Endpoint& ep) {
           auto o = open(ep);
           std::vector<std::unique_ptr<Data>> ds;
           std::vector<std::future<Error>> fs;
           for (int k = 0; k < kTensors; ++k) {
             ds.push_back(makeData(gGpu, sizeOf(k)));
           }
           for (int k = 0; k < kTensors; ++k) {
             fs.push_back(recvF(*o->ch, ds[k]->buffer(), ds[k]->size()));
           }
           for (auto& f : fs) {
             EXPECT_OK(waitFor(f, "recv"));
           }
           for (int k = 0; k < kTensors; ++k) {
             expectBytes(*ds[k], pattern(k), "tensor");
           }
           ep.barrier();
         }});
  }

  // Traffic in both directions from one seeded schedule that both ends know:
  // sizes from nothing to a few MiB, directions mixed, up to sixteen
  // operations in flight on each end. Every tensor has bytes of its own.
  {
    struct Step {
      bool fromServer;
      size_t size;
    };
    auto schedule = [] {
      std::vector<Step> steps;
      uint64_t x = 0x9e3779b97f4a7c15ull; // splitmix64
      auto next = [&x] {
        x += 0x9e3779b97f4a7c15ull;
        uint64_t z = x;
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
      };
      for (int i = 0; i < 96; ++i) {
        const uint64_t r = next();
        size_t size;
        switch (r % 8) {
          case 0:
            size = 0;
            break;
          case 1:
          case 2:
            size = 1 + (r >> 8) % 300;
            break;
          case 3:
          case 4:
          case 5:
            size = 4000 + (r >> 8) % 200000;
            break;
          case 6:
            size = (1u << 20) + (r >> 8) % 4096;
            break;
          default:
            size = (2u << 20) + (1u << 19) + (r >> 8) % 77777;
        }
        steps.push_back(Step{((r >> 40) & 1) != 0, size});
      }
      return steps;
    };
    auto pattern = [](int k, size_t size) {
      std::vector<uint8_t> v(size);
      for (size_t j = 0; j < size; ++j) {
        v[j] = static_cast<uint8_t>((j * 31 + static_cast<size_t>(k) * 59 + (j >> 10) * 7) % 251);
      }
      return v;
    };
    auto side = [schedule, pattern](Endpoint& ep) {
      auto o = open(ep);
      const auto steps = schedule();
      std::vector<std::unique_ptr<Data>> ds(steps.size());
      std::vector<std::future<Error>> fs(steps.size());
      const size_t window = 16;
      auto settle = [&](size_t k) {
        const bool mine = steps[k].fromServer == ep.isServer();
        EXPECT_OK(waitFor(fs[k], mine ? "send" : "recv"));
        if (!mine) {
          expectBytes(*ds[k], pattern(static_cast<int>(k), steps[k].size), "tensor");
        }
        ds[k].reset();
      };
      for (size_t k = 0; k < steps.size(); ++k) {
        if (k >= window) {
          settle(k - window);
        }
        const bool mine = steps[k].fromServer == ep.isServer();
        if (mine) {
          ds[k] = makeData(gGpu, pattern(static_cast<int>(k), steps[k].size));
          fs[k] = sendF(*o->ch, ds[k]->buffer(), ds[k]->size());
        } else {
          ds[k] = makeData(gGpu, steps[k].size);
          fs[k] = recvF(*o->ch, ds[k]->buffer(), ds[k]->size());
        }
      }
      for (size_t k = steps.size() > window ? steps.size() - window : 0; k < steps.size(); ++k) {
        settle(k);
      }
      ep.barrier();
    };
    cases.push_back({"SeededTrafficBothWays", side, side});
    // The same with every tensor in a device allocation of exactly its size,
    // allocated for the operation and freed when it completes: allocations
    // that the runtime packs several to a block come and go while transfers
    // of their neighbours are still under way.
    auto exact = [side](Endpoint& ep) {
      ExactGpuAllocations guard;
      side(ep);
    };
    cases.push_back({"SeededTrafficSmallAllocations", exact, exact});
  }

  // Both ends of a channel on ONE context: a process that talks to itself (an
  // RPC worker calling itself does). Tensors go both ways at once; the context
  // shares its loop, its staging rings and its poller between the two ends.
  if (gSuite != "hip_ipc" && gSuite.rfind("hip_ipc_", 0) != 0) {
    auto sizeOf = [](int k) {
      static const size_t sizes[] = {(1u << 20) + 1, (3u << 20) + 5, 100, 0, 65536, (2u << 20) + (1u << 19)};
      return sizes[k % 6] + static_cast<size_t>(k / 6) * 4099;
    };
    auto pattern = [sizeOf](int k, int dir) {
      std::vector<uint8_t> v(sizeOf(k));
      for (size_t j = 0; j < v.size(); ++j) {
        v[j] = static_cast<uint8_t>((j * 17 + static_cast<size_t>(k) * 29 + static_cast<size_t>(dir) * 7 + (j >> 11)) % 249);
      }
      return v;
    };
    auto oneContext = [sizeOf, pattern](Endpoint& ep) {
      const std::string base = ep.freshAddr(); // drawn by both ends: they count addresses in step
      if (ep.isServer()) {
        auto ctx = makeContext();
        ctx->setId("talks_to_itself");
        if (!ctx->isViable()) {
          throw Fatal("context is not viable");
        }
        const size_t n = ctx->numConnectionsNeeded();
        const std::string addr = base + "_self";
        auto listener = ep.transport()->listen(addr);
        std::vector<std::shared_ptr<transport::Connection>> connecting(n), accepted(n);
        for (size_t i = 0; i < n; ++i) {
          // one at a time, so that the i-th ends belong together
          connecting[i] = ep.transport()->connect(addr);
          accepted[i] = acceptOne(*listener);
          writeByte(*connecting[i], static_cast<uint8_t>(i));
          if (readByte(*accepted[i]) != i) {
            throw Fatal("connections paired out of order");
          }
        }
        listener->close();
        {
          auto a = ctx->createChannel(std::move(accepted), channel::Endpoint::kListen);
          auto b = ctx->createChannel(std::move(connecting), channel::Endpoint::kConnect);
          constexpr int kTensors = 18;
          std::vector<std::unique_ptr<Data>> out[2], in[2];
          std::vector<std::future<Error>> sends, recvs;
          for (int k = 0; k < kTensors; ++k) {
            for (int dir = 0; dir < 2; ++dir) {
              out[dir].push_back(makeData(gGpu, pattern(k, dir)));
              in[dir].push_back(makeData(gGpu, sizeOf(k)));
            }
          }
          for (int k = 0; k < kTensors; ++k) {
            // dir 0: a -> b, dir 1: b -> a; receives posted now and then ahead of the sends
            if (k % 3 == 0) {
              recvs.push_back(recvF(*b, in[0][k]->buffer(), in[0][k]->size()));
              recvs.push_back(recvF(*a, in[1][k]->buffer(), in[1][k]->size()));
            }
            sends.push_back(sendF(*a, out[0][k]->buffer(), out[0][k]->size()));
            sends.push_back(sendF(*b, out[1][k]->buffer(), out[1][k]->size()));
            if (k % 3 != 0) {
              recvs.push_back(recvF(*b, in[0][k]->buffer(), in[0][k]->size()));
              recvs.push_back(recvF(*a, in[1][k]->buffer(), in[1][k]->size()));
            }
          }
          for (auto& f : sends) {
            EXPECT_OK(waitFor(f, "send"));
          }
          for (auto& f : recvs) {
            EXPECT_OK(waitFor(f, "recv"));
          }
          for (int k = 0; k < kTensors; ++k) {
            for (int dir = 0; dir < 2; ++dir) {
              expectBytes(*in[dir][k], pattern(k, dir), "tensor");
            }
          }
        }
        ctx->join();
      }
      ep.barrier();
    };
    cases.push_back({"BothEndsOnOneContext", oneContext, oneContext});
  }

  // Two channels of one context carrying tensors the SAME way, receives and
  // sends posted crosswise: the first channel's receive is posted before
  // anything is sent on it, the second channel's send (far more than the
  // connection buffers and the staging slots hold) before its receive. A
  // receiver that took its landing slots when the receive was posted would hold
  // them all for the first channel while the second one's sends hold every send
  // slot: the reference takes a receive buffer only for a chunk that is on its
  // way (tensorpipe/channel/cuda_basic/channel_impl.cc:413-441).
  if (gSuite != "hip_ipc" && gSuite.rfind("hip_ipc_", 0) != 0) {
    auto crosswise = [](Endpoint& ep) {
      const std::string base = ep.freshAddr();
      if (ep.isServer()) {
        auto ctx = makeContext();
        ctx->setId("two_flows_one_way");
        if (!ctx->isViable()) {
          throw Fatal("context is not viable");
        }
        const size_t n = ctx->numConnectionsNeeded();
        const std::string addr = base + "_flows";
        auto listener = ep.transport()->listen(addr);
        std::shared_ptr<channel::Channel> from[2], to[2];
        for (int flow = 0; flow < 2; ++flow) {
          std::vector<std::shared_ptr<transport::Connection>> connecting(n), accepted(n);
          for (size_t i = 0; i < n; ++i) {
            connecting[i] = ep.transport()->connect(addr);
            accepted[i] = acceptOne(*listener);
            writeByte(*connecting[i], static_cast<uint8_t>(i));
            if (readByte(*accepted[i]) != i) {
              throw Fatal("connections paired out of order");
            }
          }
          from[flow] = ctx->createChannel(std::move(accepted), channel::Endpoint::kListen);
          to[flow] = ctx->createChannel(std::move(connecting), channel::Endpoint::kConnect);
        }
        listener->close();
        {
          auto fill = [](size_t bytes, int salt) {
            std::vector<uint8_t> v(bytes);
            for (size_t j = 0; j < v.size(); ++j) {
              v[j] = static_cast<uint8_t>((j * 23 + static_cast<size_t>(salt) * 31 + (j >> 13)) % 241);
            }
            return v;
          };
          const size_t small = 6 * 65536 + 17, large = (5u << 20) + 3;
          auto out0 = makeData(gGpu, fill(small, 1)), out1 = makeData(gGpu, fill(large, 2));
          auto in0 = makeData(gGpu, small), in1 = makeData(gGpu, large);
          std::vector<std::future<Error>> fs;
          fs.push_back(recvF(*to[0], in0->buffer(), small));
          fs.push_back(sendF(*from[1], out1->buffer(), large));
          std::this_thread::sleep_for(std::chrono::milliseconds(100)); // the second flow fills what it can
          fs.push_back(sendF(*from[0], out0->buffer(), small));
          std::this_thread::sleep_for(std::chrono::milliseconds(100)); // the first flow's receiver has heard of it
          fs.push_back(recvF(*to[1], in1->buffer(), large));
          for (auto& f : fs) {
            EXPECT_OK(waitFor(f, "transfer"));
          }
          expectBytes(*in0, fill(small, 1), "first flow");
          expectBytes(*in1, fill(large, 2), "second flow");
        }
        for (int flow = 0; flow < 2; ++flow) {
          from[flow].reset();
          to[flow].reset();
        }
        ctx->join();
      }
      ep.barrier();
    };
    cases.push_back({"TwoFlowsOneWayPostedCrosswise", crosswise, crosswise});
  }

  // Two channels between the same two contexts at once (two pipes between two
  // workers, as RPC agents open them), traffic flowing the opposite way on each:
  // they share each context's loop, poller and staging rings, and one tensor is
  // larger than a whole ring.
  {
    auto sizeOf = [](int k) {
      static const size_t sizes[] = {70000, (1u << 20) + 3, 333, (20u << 20) + 11, 4096, (2u << 20) + 77};
      return sizes[k % 6] + static_cast<size_t>(k / 6) * 1031;
    };
    auto pattern = [sizeOf](int k, int lane) {
      std::vector<uint8_t> v(sizeOf(k));
      for (size_t j = 0; j < v.size(); ++j) {
        v[j] = static_cast<uint8_t>((j * 19 + static_cast<size_t>(k) * 23 + static_cast<size_t>(lane) * 5 + (j >> 12)) % 247);
      }
      return v;
    };
    auto side = [sizeOf, pattern](Endpoint& ep) {
      auto ctx = makeContext();
      ctx->setId(std::string(roleName(ep.role())) + "_ctx");
      if (!ctx->isViable()) {
        throw Fatal("context is not viable");
      }
      const auto end = ep.isServer() ? channel::Endpoint::kListen : channel::Endpoint::kConnect;
      {
        auto first = ctx->createChannel(ep.openConnections(ctx->numConnectionsNeeded()), end);
        auto second = ctx->createChannel(ep.openConnections(ctx->numConnectionsNeeded()), end);
        // the server sends on the first and receives on the second, the client the other way round
        auto& outCh = ep.isServer() ? *first : *second;
        auto& inCh = ep.isServer() ? *second : *first;
        const int outLane = ep.isServer() ? 0 : 1;
        constexpr int kTensors = 12;
        std::vector<std::unique_ptr<Data>> out, in;
        std::vector<std::future<Error>> fs;
        for (int k = 0; k < kTensors; ++k) {
          out.push_back(makeData(gGpu, pattern(k, outLane)));
          in.push_back(makeData(gGpu, sizeOf(k)));
        }
        for (int k = 0; k < kTensors; ++k) {
          fs.push_back(sendF(outCh, out[k]->buffer(), out[k]->size()));
          fs.push_back(recvF(inCh, in[k]->buffer(), in[k]->size()));
        }
        for (auto& f : fs) {
          EXPECT_OK(waitFor(f, "transfer"));
        }
        for (int k = 0; k < kTensors; ++k) {
          expectBytes(*in[k], pattern(k, 1 - outLane), "tensor");
        }
        ep.barrier();
      }
      ctx->join();
    };
    cases.push_back({"TwoChannelsShareTheContexts", side, side});
  }

  // channel_test.cc:191-259: one send and one recv in flight on each side.
  auto bothWays = [](Endpoint& ep) {
    auto o = open(ep);
    std::vector<uint8_t> mine(256, ep.isServer() ? 0x11 : 0x22);
    std::vector<uint8_t> theirs(256, ep.isServer() ? 0x22 : 0x11);
    auto out = makeData(gGpu, mine);
    auto in = makeData(gGpu, 256);
    auto fs = sendF(*o->ch, out->buffer(), out->size());
    auto fr = recvF(*o->ch, in->buffer(), in->size());
    EXPECT_OK(waitFor(fs, "send"));
    EXPECT_OK(waitFor(fr, "recv"));
    expectBytes(*in, theirs, "received data");
    ep.barrier();
  };
  cases.push_back({"SendTensorsBothWays", bothWays, bothWays});

  // channel_test.cc:262-293 and channel_test_cpu.cc:19-43 (NullPointer): zero
  // bytes at a null pointer complete at once.
  cases.push_back({"EmptyTensor",
                   [](Endpoint& ep) {
                     auto o = open(ep);
                     auto f = sendF(*o->ch, nullBuffer(), 0);
                     EXPECT_OK(waitFor(f, "send"));
                     ep.barrier();
                   },
                   [](Endpoint& ep) {
                     auto o = open(ep);
                     auto f = recvF(*o->ch, nullBuffer(), 0);
                     EXPECT_OK(waitFor(f, "recv"));
                     ep.barrier();
                   }});

  // channel_test.cc:295-336: lengths 1, 0, 1 keep their order.
  cases.push_back(
      {"EmptyAndNonEmptyTensors",
       [](Endpoint& ep) {
         auto o = open(ep);
         auto a = makeData(gGpu, std::vector<uint8_t>{0xA1});
         auto c = makeData(gGpu, std::vector<uint8_t>{0xC3});
         auto f1 = sendF(*o->ch, a->buffer(), 1);
         auto f2 = sendF(*o->ch, nullBuffer(), 0);
         auto f3 = sendF(*o->ch, c->buffer(), 1);
         EXPECT_OK(waitFor(f1, "send 1"));
         EXPECT_OK(waitFor(f2, "send 2"));
         EXPECT_OK(waitFor(f3, "send 3"));
         ep.barrier();
       },
       [](Endpoint& ep) {
         auto o = open(ep);
         auto a = makeData(gGpu, 1);
         auto c = makeData(gGpu, 1);
         auto f1 = recvF(*o->ch, a->buffer(), 1);
         auto f2 = recvF(*o->ch, nullBuffer(), 0);
         auto f3 = recvF(*o->ch, c->buffer(), 1);
         EXPECT_OK(waitFor(f1, "recv 1"));
         EXPECT_OK(waitFor(f2, "recv 2"));
         EXPECT_OK(waitFor(f3, "recv 3"));
         expectBytes(*a, {0xA1}, "first");
         expectBytes(*c, {0xC3}, "third");
         ep.barrier();
       }});

  if (gGpu) {
  // channel_test_cuda.cc:19-94: the source is still being produced on the send
  // stream when send() is called (a slow kernel scribbles over it, then a fill
  // writes 0x42); the receiver must see the 0x42s.
  cases.push_back(
      {"ReceiverWaitsForStartEvent",
       [](Endpoint& ep) {
         auto o = open(ep);
         GpuData d(1024);
         HIP_OK(tphip_test_slow_kernel(0, d.ptr(), 1024, d.stream()));
         HIP_OK(tphip_fill(0, d.ptr(), 0x42, 1024, d.stream()));
         auto f = sendF(*o->ch, d.buffer(), 1024);
         EXPECT_OK(waitFor(f, "send"));
         ep.barrier();
       },
       [](Endpoint& ep) { receiver(ep, true, std::vector<uint8_t>(1024, 0x42)); }});

  // channel_test_cuda.cc:96-139: the tensor starts 128 bytes into its
  // allocation (matters for handles that name the allocation base).
  cases.push_back({"SendOffsetAllocation",
                   [](Endpoint& ep) {
                     auto o = open(ep);
                     GpuData d(std::vector<uint8_t>(256, 0x42), /*offset=*/128);
                     auto f = sendF(*o->ch, d.buffer(), 256);
                     EXPECT_OK(waitFor(f, "send"));
                     ep.barrier();
                   },
                   [](Endpoint& ep) { receiver(ep, true, std::vector<uint8_t>(256, 0x42)); }});
  } // gGpu

  // Sizes around the chunking and vector-width boundaries of the copy paths.
  for (size_t n : {size_t(1), size_t(15), size_t(4097), size_t(1) << 20, (size_t(8) << 20) + 5,
                   size_t(20) << 20}) {
    std::vector<uint8_t> v(n);
    uint64_t x = 0x9E3779B97F4A7C15ull * (n + 1);
    for (size_t i = 0; i < n; ++i) {
      x ^= x << 13;
      x ^= x >> 7;
      x ^= x << 17;
      v[i] = static_cast<uint8_t>(x);
    }
    cases.push_back({"Size" + std::to_string(n),
                     [v](Endpoint& ep) { sender(ep, gGpu, v); },
                     [v](Endpoint& ep) { receiver(ep, gGpu, v); }});
  }

  // Memory that is freed and allocated again between sends (the allocator
  // tends to hand the same address back): the receiver must see the bytes of
  // the allocation that is live now, never those of a mapping it kept from an
  // earlier one.
  cases.push_back({"SourceFreedAndAllocatedAgain",
                   [](Endpoint& ep) {
                     auto o = open(ep);
                     for (int k = 0; k < 12; ++k) {
                       auto d = makeData(gGpu, std::vector<uint8_t>((1 << 20) + 64 * k, uint8_t(k + 1)));
                       auto f = sendF(*o->ch, d->buffer(), d->size());
                       EXPECT_OK(waitFor(f, "send"));
                       ep.barrier(); // the receiver has checked; free the source now
                     }
                     ep.barrier();
                   },
                   [](Endpoint& ep) {
                     auto o = open(ep);
                     for (int k = 0; k < 12; ++k) {
                       const size_t n = (1 << 20) + 64 * k;
                       auto d = makeData(gGpu, n);
                       auto f = recvF(*o->ch, d->buffer(), n);
                       EXPECT_OK(waitFor(f, "recv"));
                       expectBytes(*d, std::vector<uint8_t>(n, uint8_t(k + 1)), "round");
                       ep.barrier();
                     }
                     ep.barrier();
                   }});

  if (staged) {
    // channel_test_cuda_xdtt.cc:19-143: 1024 bytes of 0x42 across device types.
    cases.push_back({"SendFromCpuToGpu",
                     [](Endpoint& ep) { sender(ep, false, std::vector<uint8_t>(1024, 0x42)); },
                     [](Endpoint& ep) { receiver(ep, true, std::vector<uint8_t>(1024, 0x42)); }});
    cases.push_back({"SendFromGpuToCpu",
                     [](Endpoint& ep) { sender(ep, true, std::vector<uint8_t>(1024, 0x42)); },
                     [](Endpoint& ep) { receiver(ep, false, std::vector<uint8_t>(1024, 0x42)); }});
    // channel_test_cuda_xdtt.cc:145-195: the channel is never chosen for a pair of
    // CPU endpoints, yet carries CPU memory both ways when asked to.
    cases.push_back({"SendFromCpuToCpu",
                     [](Endpoint& ep) { sender(ep, false, std::vector<uint8_t>(1024, 0x42)); },
                     [](Endpoint& ep) { receiver(ep, false, std::vector<uint8_t>(1024, 0x42)); }});
    // The same over several chunks, with a ragged end.
    cases.push_back({"SendFromCpuToCpuSeveralChunks",
                     [](Endpoint& ep) { sender(ep, false, iota(3 * 1024 * 1024 + 5)); },
                     [](Endpoint& ep) { receiver(ep, false, iota(3 * 1024 * 1024 + 5)); }});
    // A GPU tensor of several chunks landing in CPU memory (on the GPU-driven
    // route the receiver's GPU cannot write the target itself).
    cases.push_back({"SendFromGpuToCpuSeveralChunks",
                     [](Endpoint& ep) { sender(ep, true, iota(5 * 1024 * 1024 + 3)); },
                     [](Endpoint& ep) { receiver(ep, false, iota(5 * 1024 * 1024 + 3)); }});
    // Tensors of several chunks in both directions at the same moment, three
    // in a row each way with a one-chunk tensor in between: every end pushes
    // into its own ring while it pulls from the peer's.
    auto chunkedBothWays = [](Endpoint& ep) {
      auto o = open(ep);
      const int salt = ep.isServer() ? 3 : 11;
      const size_t sizes[] = {6 * 1024 * 1024 + 17, 4096, 9 * 1024 * 1024, 3 * 1024 * 1024 + 1};
      std::vector<std::unique_ptr<Data>> out, in;
      std::vector<std::future<Error>> fs;
      for (size_t n : sizes) {
        std::vector<uint8_t> bytes(n);
        for (size_t i = 0; i < n; ++i) {
          bytes[i] = static_cast<uint8_t>((i * 31 + (i >> 11) + salt + n) & 0xff);
        }
        out.push_back(makeData(true, bytes));
        in.push_back(makeData(true, n));
      }
      for (size_t k = 0; k < out.size(); ++k) {
        fs.push_back(recvF(*o->ch, in[k]->buffer(), in[k]->size()));
        fs.push_back(sendF(*o->ch, out[k]->buffer(), out[k]->size()));
      }
      for (auto& f : fs) {
        EXPECT_OK(waitFor(f, "transfer"));
      }
      const int peerSalt = ep.isServer() ? 11 : 3;
      for (size_t k = 0; k < in.size(); ++k) {
        const size_t n = in[k]->size();
        std::vector<uint8_t> want(n);
        for (size_t i = 0; i < n; ++i) {
          want[i] = static_cast<uint8_t>((i * 31 + (i >> 11) + peerSalt + n) & 0xff);
        }
        expectBytes(*in[k], want, "tensor from the peer");
      }
      ep.barrier();
    };
    cases.push_back({"ChunkedTensorsBothWaysAtOnce", chunkedBothWays, chunkedBothWays});
    // cuda_basic_test.cc:40-62: a pair of CPU endpoints is left to CPU channels.
    auto cpuToCpu = [](Endpoint&) {
      auto c = makeContext();
      const auto& d = c->deviceDescriptors();
      const Device cpu{kCpuDeviceType, 0};
      const Device gpu{kHipDeviceType, 0};
      EXPECT_EQ(d.count(cpu), size_t(1));
      EXPECT_EQ(d.count(gpu), size_t(1));
      if (d.count(cpu) == 1 && d.count(gpu) == 1) {
        EXPECT_FALSE(c->canCommunicateWithRemote(d.at(cpu), d.at(cpu)));
        EXPECT_TRUE(c->canCommunicateWithRemote(d.at(cpu), d.at(gpu)));
        EXPECT_TRUE(c->canCommunicateWithRemote(d.at(gpu), d.at(cpu)));
        EXPECT_TRUE(c->canCommunicateWithRemote(d.at(gpu), d.at(gpu)));
      }
      c->join();
    };
    cases.push_back({"CannotCommunicateCpuToCpu", cpuToCpu, cpuToCpu});
  }

  if (gSuite == "hip_ipc" || gSuite == "hip_ipc_outbox" || gSuite == "hip_ipc_gated" ||
      gSuite == "hip_ipc_messages") {
    // cuda_ipc_test.cc:37-57: two contexts of one process must not pick IPC.
    auto sameProcess = [](Endpoint&) {
      auto c1 = makeContext();
      auto c2 = makeContext();
      const Device gpu{kHipDeviceType, 0};
      const auto& d1 = c1->deviceDescriptors();
      const auto& d2 = c2->deviceDescriptors();
      EXPECT_EQ(d1.count(gpu), size_t(1));
      EXPECT_EQ(d2.count(gpu), size_t(1));
      if (d1.count(gpu) == 1 && d2.count(gpu) == 1) {
        EXPECT_FALSE(c1->canCommunicateWithRemote(d1.at(gpu), d2.at(gpu)));
      }
      c1->join();
      c2->join();
    };
    cases.push_back({"CannotCommunicateInSameProcess", sameProcess, sameProcess});
  }

  if (gSuite == "hip_ipc") {
    // An allocation at or above the export limit is not mapped by the peer but
    // staged through the outbox, and so is one below the size at which the
    // runtime gives an allocation a block of its own. The two routes are told
    // apart by when the send completes: a staged send once its bytes sit in
    // the outbox, before the peer has posted its recv; a direct send only
    // after the peer's copy.
    auto pattern = [](size_t n, uint8_t salt) {
      std::vector<uint8_t> v(n);
      for (size_t i = 0; i < n; ++i) {
        v[i] = static_cast<uint8_t>((i >> 8) ^ (i & 0xff) ^ salt);
      }
      return v;
    };
    const size_t direct = 4096; // inside an allocation of 2 MiB, as all allocations of these tests
    // staged: how many bytes, and whether the allocation is exactly that large
    auto sendSide = [=](Endpoint& ep, size_t staged, bool exact) {
      ::setenv("TP_HIP_IPC_MAX_EXPORT_BYTES", "3145728", 1);
      auto o = open(ep);
      ::unsetenv("TP_HIP_IPC_MAX_EXPORT_BYTES");
      std::unique_ptr<GpuData> other;
      {
        std::unique_ptr<ExactGpuAllocations> guard;
        if (exact) {
          guard = std::make_unique<ExactGpuAllocations>();
        }
        other = std::make_unique<GpuData>(pattern(staged, 1));
      }
      GpuData below(pattern(direct, 2));
      auto fa = sendF(*o->ch, other->buffer(), other->size());
      EXPECT_OK(waitFor(fa, "staged send before the peer's recv"));
      auto fb = sendF(*o->ch, below.buffer(), below.size());
      EXPECT_TRUE(fb.wait_for(std::chrono::milliseconds(300)) == std::future_status::timeout);
      ep.barrier(); // the peer posts its recvs now
      EXPECT_OK(waitFor(fb, "direct send"));
      ep.barrier();
    };
    auto recvSide = [=](Endpoint& ep, size_t staged) {
      auto o = open(ep);
      GpuData a(staged), b(direct);
      ep.barrier();
      auto fa = recvF(*o->ch, a.buffer(), a.size());
      auto fb = recvF(*o->ch, b.buffer(), b.size());
      EXPECT_OK(waitFor(fa, "recv of the staged tensor"));
      EXPECT_OK(waitFor(fb, "recv of the direct tensor"));
      expectBytes(a, pattern(staged, 1), "staged tensor");
      expectBytes(b, pattern(direct, 2), "direct tensor");
      ep.barrier();
    };
    const size_t big = 4 * 1024 * 1024, little = 256 * 1024;
    cases.push_back({"AllocationsAboveExportLimitAreStaged",
                     [=](Endpoint& ep) { sendSide(ep, big, false); },
                     [=](Endpoint& ep) { recvSide(ep, big); }});
    cases.push_back({"AllocationsBelowBlockSizeAreStaged",
                     [=](Endpoint& ep) { sendSide(ep, little, true); },
                     [=](Endpoint& ep) { recvSide(ep, little); }});
  }

  if (gSuite == "hip_ipc") {
    // A receiver keeps the peer allocations it has mapped up to a limit and
    // drops the least recently used ones beyond it; a tensor out of an
    // allocation that was dropped is mapped again when it comes by. Thirty
    // allocations of 512 KiB, all alive at once, against a limit of 1 MiB.
    const size_t bytes = 512 * 1024;
    const int allocations = 30;
    auto pattern = [](size_t n, uint8_t salt) {
      std::vector<uint8_t> v(n);
      for (size_t i = 0; i < n; ++i) {
        v[i] = static_cast<uint8_t>((i * 13) ^ (i >> 9) ^ salt);
      }
      return v;
    };
    // the order both sides follow: every allocation once, then back to old ones
    auto order = [allocations] {
      std::vector<int> o;
      for (int i = 0; i < allocations; ++i) {
        o.push_back(i);
      }
      for (int i : {0, 1, 29, 0, 15, 2}) {
        o.push_back(i);
      }
      return o;
    };
    auto sendSide = [=](Endpoint& ep) {
      auto o = open(ep);
      std::vector<std::unique_ptr<GpuData>> sources;
      for (int i = 0; i < allocations; ++i) {
        sources.push_back(std::make_unique<GpuData>(pattern(bytes, static_cast<uint8_t>(i))));
      }
      ep.barrier();
      for (int i : order()) {
        auto f = sendF(*o->ch, sources[i]->buffer(), bytes);
        EXPECT_OK(waitFor(f, "send"));
      }
      ep.barrier();
    };
    auto recvSide = [=](Endpoint& ep) {
      ::setenv("TP_HIP_IPC_MAX_MAPPED_BYTES", "1048576", 1);
      auto o = open(ep);
      ::unsetenv("TP_HIP_IPC_MAX_MAPPED_BYTES");
      ep.barrier();
      GpuData d(bytes);
      for (int i : order()) {
        auto f = recvF(*o->ch, d.buffer(), bytes);
        EXPECT_OK(waitFor(f, "recv"));
        expectBytes(d, pattern(bytes, static_cast<uint8_t>(i)), "received data");
      }
      ep.barrier();
    };
    cases.push_back({"MappingsBeyondTheLimitAreDropped", sendSide, recvSide});
  }

  if (gSuite == "hip_xth") {
    auto sameProcess = [](Endpoint&) {
      auto c1 = makeContext();
      auto c2 = makeContext();
      const Device gpu{kHipDeviceType, 0};
      EXPECT_TRUE(c1->canCommunicateWithRemote(
          c1->deviceDescriptors().at(gpu), c2->deviceDescriptors().at(gpu)));
      // Same boot, another process: refused.
      std::string other = c2->deviceDescriptors().at(gpu) + "9";
      EXPECT_FALSE(c1->canCommunicateWithRemote(c1->deviceDescriptors().at(gpu), other));
      c1->join();
      c2->join();
    };
    cases.push_back({"CommunicatesOnlyInSameProcess", sameProcess, sameProcess});
  }

  // channel_test_cpu.cc:44-109: the callback does not run inside send()/recv()
  // on the caller's stack (it would deadlock on the caller's mutex here). The
  // reference asks this of its CPU channels only. hip_basic is left out: its
  // recv callback means "copy enqueued", which can be true before recv()
  // returns when the sender's chunk notice is already waiting.
  if (!staged)
  cases.push_back(
      {"CallbacksAreDeferred",
       [](Endpoint& ep) {
         auto o = open(ep);
         auto d = makeData(gGpu, iota(256));
         auto p = std::make_shared<std::promise<Error>>();
         auto f = p->get_future();
         auto mutex = std::make_shared<std::mutex>();
         {
           std::unique_lock<std::mutex> callerLock(*mutex);
           o->ch->send(d->buffer(), 256, [p, mutex](const Error& e) {
             std::unique_lock<std::mutex> calleeLock(*mutex);
             p->set_value(e);
           });
         }
         EXPECT_OK(waitFor(f, "send"));
         ep.barrier();
       },
       [](Endpoint& ep) {
         auto o = open(ep);
         auto d = makeData(gGpu, 256);
         auto p = std::make_shared<std::promise<Error>>();
         auto f = p->get_future();
         auto mutex = std::make_shared<std::mutex>();
         {
           std::unique_lock<std::mutex> callerLock(*mutex);
           o->ch->recv(d->buffer(), 256, [p, mutex](const Error& e) {
             std::unique_lock<std::mutex> calleeLock(*mutex);
             p->set_value(e);
           });
         }
         EXPECT_OK(waitFor(f, "recv"));
         expectBytes(*d, iota(256), "received data");
         ep.barrier();
       }});

  // ---- closing and errors (channel_impl_boilerplate.h:189-192, error.h:18-37) --

  // After close() every new operation fails with ChannelClosedError, through
  // its callback, exactly once. The server closes first; the client, whose
  // channel may already have seen the server go away, fails with whichever
  // error came first (the first error latches).
  auto closedChannel = [](Endpoint& ep) {
    auto o = open(ep);
    ep.barrier(); // both channels exist
    if (!ep.isServer()) {
      ep.barrier(); // the server has closed and checked
    }
    o->ch->close();
    auto d = makeData(gGpu, 64);
    auto fs = sendF(*o->ch, d->buffer(), 64);
    auto fr = recvF(*o->ch, d->buffer(), 64);
    Error es = waitFor(fs, "send after close");
    Error er = waitFor(fr, "recv after close");
    EXPECT_TRUE(static_cast<bool>(es));
    EXPECT_TRUE(static_cast<bool>(er));
    if (ep.isServer()) {
      EXPECT_TRUE(es.isOfType<channel::ChannelClosedError>());
      EXPECT_TRUE(er.isOfType<channel::ChannelClosedError>());
      ep.barrier();
    }
    ep.barrier();
  };
  cases.push_back({"OperationsAfterCloseFail", closedChannel, closedChannel});

  // Closing the context closes its channels.
  auto closedContext = [](Endpoint& ep) {
    auto o = open(ep);
    ep.barrier();
    o->ctx->close();
    auto d = makeData(gGpu, 64);
    auto fs = sendF(*o->ch, d->buffer(), 64);
    Error es = waitFor(fs, "send after context close");
    EXPECT_TRUE(static_cast<bool>(es));
    ep.barrier();
  };
  cases.push_back({"ContextCloseFailsOperations", closedContext, closedContext});

  // A receive that can never be matched fails once the peer has gone away.
  cases.push_back({"PeerCloseFailsPendingRecv",
                   [](Endpoint& ep) {
                     auto o = open(ep);
                     auto d = makeData(gGpu, 4096);
                     auto f = recvF(*o->ch, d->buffer(), 4096);
                     ep.barrier(); // recv posted; the client closes now
                     Error e = waitFor(f, "recv that must fail");
                     EXPECT_TRUE(static_cast<bool>(e));
                     ep.barrier();
                   },
                   [](Endpoint& ep) {
                     auto o = open(ep);
                     ep.barrier();
                     o->ch->close();
                     o.reset();
                     ep.barrier();
                   }});

  // channel/context_boilerplate.h:147-149: a context that is dropped without
  // join() cleans up after itself (the destructor joins).
  cases.push_back({"ContextIsNotJoined",
                   [](Endpoint& ep) {
                     auto ctx = makeContext();
                     auto conns = ep.openConnections(ctx->numConnectionsNeeded());
                     auto ch = ctx->createChannel(std::move(conns), channel::Endpoint::kListen);
                     auto d = makeData(gGpu, iota(256));
                     auto f = sendF(*ch, d->buffer(), 256);
                     EXPECT_OK(waitFor(f, "send"));
                     ep.barrier();
                   },
                   [](Endpoint& ep) {
                     auto ctx = makeContext();
                     auto conns = ep.openConnections(ctx->numConnectionsNeeded());
                     auto ch = ctx->createChannel(std::move(conns), channel::Endpoint::kConnect);
                     auto d = makeData(gGpu, 256);
                     auto f = recvF(*ch, d->buffer(), 256);
                     EXPECT_OK(waitFor(f, "recv"));
                     expectBytes(*d, iota(256), "received data");
                     ep.barrier();
                   }});

  return cases;
}

} // namespace

int main(int argc, char** argv) {
  Args args = parseArgs(argc, argv);
  if (!knownSuite(args.suite)) {
    std::fprintf(
        stderr, "usage: %s --suite hip_xth|hip_ipc|hip_ipc_outbox|hip_ipc_gated|hip_ipc_messages|hip_basic|hip_basic_host_ring|hip_basic_small_ring|basic|xth [--case S] [--list]\n",
        argv[0]);
    return 2;
  }
  gSuite = args.suite;
  gGpu = gSuite.rfind("hip_", 0) == 0;
  if (gSuite == "hip_ipc_outbox") {
    // The reference's algorithm (every tensor staged through the outbox), with
    // slots small enough for the sizes of this suite to span and reuse them.
    ::setenv("TP_HIP_IPC_MODE", "outbox", 1);
    ::setenv("TP_HIP_IPC_SLOT_BYTES", "1048576", 1);
    ::setenv("TP_HIP_IPC_NUM_SLOTS", "3", 1);
  }
  if (gSuite == "hip_ipc_gated") {
    // Senders whose stream is still producing announce at once; the receiver's
    // GPU waits for their word (short waits, so that the retry path runs too).
    ::setenv("TP_HIP_IPC_GATES", "1", 1);
    ::setenv("TP_HIP_IPC_GATE_WAIT_US", "200", 1);
  }
  if (gSuite == "hip_basic_host_ring") {
    // Every tensor on the host-driven routes (one launch, event and message per chunk).
    ::setenv("TP_HIP_BASIC_GPU_RING", "0", 1);
  }
  if (gSuite == "hip_basic_small_ring") {
    // Three small slots and an impatient kernel: tensors span many turns of the
    // ring, and ring kernels give up and are launched again all the time.
    ::setenv("TP_HIP_BASIC_SLOT_BYTES", "65536", 1);
    ::setenv("TP_HIP_BASIC_NUM_SLOTS", "3", 1);
    ::setenv("TP_HIP_BASIC_RING_YIELD_US", "20", 1);
  }
  if (gSuite == "hip_ipc_messages") {
    // No signal words, no copy agent: every unit acknowledged by a message.
    ::setenv("TP_HIP_IPC_SIGNALS", "0", 1);
    ::setenv("TP_HIP_IPC_AGENT", "0", 1);
  }
  std::vector<Case> cases = makeCases();
  if (args.list) {
    for (auto& c : cases) {
      std::printf("%s\n", c.name.c_str());
    }
    return 0;
  }
  const std::string addr =
      args.addr.empty() ? "tptest_" + std::to_string(::getpid()) + "_" + gSuite : args.addr;
  if (args.role == "server") {
    return runSingleRole(Role::kServer, cases, args.filter, addr, args.readyFd);
  }
  if (args.role == "client") {
    return runSingleRole(Role::kClient, cases, args.filter, addr, -1);
  }
  if (!twoProcessSuite(gSuite)) {
    return runBoth(cases, args.filter, addr);
  }
  std::vector<std::string> pass = {"--suite", gSuite};
  if (!args.filter.empty()) {
    pass.push_back("--case");
    pass.push_back(args.filter);
  }
  return orchestrate(argv[0], pass, addr);
}
