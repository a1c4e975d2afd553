// Host-only unit checks of the small building blocks under the channels; no
// GPU needed. Driven by tests/test_cpp_units.py.
//
//   unit_tests allocator <slots> <ev> <ev> ...   ev = a<k> | r<slot> | c
//       replays the events on SlotAllocator and prints "k:slot" per grant in
//       the order the grants happen (slot -1 = failed by close), so the caller
//       can compare with the golden trace (tensorpipe/common/allocator.cc:26-79).
//   unit_tests basics
//       Buffer / Device / Error / wire helpers; prints "OK" or the failures.
//   unit_tests garbage <seed> <connections>
//       opens raw transport connections to a listening context and writes
//       random bytes where a pipe's first packets belong; the context must
//       survive all of them and still serve a proper pipe afterwards.
//   unit_tests departed_peer
//       a peer writes two messages and goes away before the reader posts its
//       reads: both messages are handed over, the third read reports the end.
//   unit_tests nop_wire <vectors file>
//       the control frames an unmodified TensorPipe endpoint wrote (name, hex):
//       each must decode, carry the fields the capturing program put in, and
//       encode back to the same bytes; cut short anywhere, or with bytes
//       flipped, a frame must be refused without reading out of bounds.
//   unit_tests compat_pipe
//       two ends of the stock-protocol endpoint talk to each other over TCP.
//   unit_tests loops
//       the on-demand executor: two application threads, each inside a task of
//       one loop, defer to the other's loop at the same moment and both return
//       (no thread ever waits for a loop while it sits in a task of another);
//       a caller holding a lock that the draining thread's task wants returns
//       from defer() as well; a task queued by another thread while an
//       application thread drains is never run by that application thread and
//       still runs; tasks run exactly once, in the order they were queued; a
//       loop goes away cleanly while a helper still has it on its list.
//   unit_tests tcp
//       the TCP transport: messages of every size class both ways (empty, small,
//       many MiB: partial reads and writes), exact-length reads, a peer that
//       wrote and left, a frame written by hand with the reference's framing,
//       and a pipe with payloads and CPU tensors over it.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <functional>
#include <memory>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <future>
#include <map>
#include <mutex>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include <execinfo.h>
#include <signal.h>
#include <unistd.h>

#include <tphip.h>

#include <tensorpipe/common/buffer.h>
#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/device.h>
#include <tensorpipe/common/error.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/common/loop.h>
#include <tensorpipe/common/slot_allocator.h>
#include <tensorpipe/common/wire.h>
#include <tensorpipe/channel/error.h>
#include <sys/mman.h>

#include <tensorpipe/tensorpipe.h>
#include <tensorpipe/tensorpipe_hip.h>
#include <tensorpipe/transport/connection.h>
#include <tensorpipe/transport/listener.h>

#include <tensorpipe/transport/tcp/factory.h>

#include <arpa/inet.h>
#include <netinet/in.h>
#include <sys/socket.h>
#include <sys/un.h>
#include <poll.h>

#include <nopwire/compat_pipe.h>
#include <nopwire/nop_wire.h>

using namespace tensorpipe;

static int runAllocator(int argc, char** argv) {
  const size_t slots = std::strtoul(argv[2], nullptr, 10);
  const size_t slotSize = 64;
  std::vector<uint8_t> slab(slots * slotSize);
  SlotAllocator alloc(slab.data(), slots, slotSize);
  std::map<size_t, SlotAllocator::TSlot> held; // slot index -> grant
  for (int i = 3; i < argc; ++i) {
    const char op = argv[i][0];
    const long arg = argv[i][1] != 0 ? std::strtol(argv[i] + 1, nullptr, 10) : 0;
    if (op == 'a') {
      alloc.alloc([&, arg](const Error& e, SlotAllocator::TSlot s) {
        if (e) {
          std::printf("%ld:-1%s ", arg, e.isOfType<AllocatorClosedError>() ? "" : "?");
          return;
        }
        const size_t idx = alloc.slotIndex(s.get());
        std::printf("%ld:%zu ", arg, idx);
        held[idx] = std::move(s);
      });
    } else if (op == 'r') {
      auto it = held.find(static_cast<size_t>(arg));
      if (it == held.end()) {
        std::printf("\nslot %ld is not held\n", arg);
        return 1;
      }
      SlotAllocator::TSlot s = std::move(it->second);
      held.erase(it);
      s.reset(); // returns the slot; a waiter may be served inside this call
    } else if (op == 'c') {
      alloc.close();
    } else {
      std::printf("\nbad event %s\n", argv[i]);
      return 2;
    }
  }
  std::printf("\n");
  return 0;
}

#define CHECK(cond)                                         \
  do {                                                      \
    if (!(cond)) {                                          \
      std::printf("FAILED line %d: %s\n", __LINE__, #cond); \
      ++failed;                                             \
    }                                                       \
  } while (0)

static int runBasics() {
  int failed = 0;
  // Device: value semantics, printing, hashing (tensorpipe/common/device.h:17-64).
  Device cpu{kCpuDeviceType, 0};
  Device gpu0{kHipDeviceType, 0};
  Device gpu1{kHipDeviceType, 1};
  CHECK(cpu.toString() == "cpu:0");
  CHECK(gpu1.toString() == "cuda:1");
  CHECK(gpu0 == Device(kCudaDeviceType, 0));
  CHECK(gpu0 != gpu1);
  CHECK(std::hash<Device>{}(gpu0) == std::hash<Device>{}(Device{kHipDeviceType, 0}));
  CHECK(std::hash<Device>{}(gpu0) != std::hash<Device>{}(gpu1));

  // Buffer: type erasure over CpuBuffer / HipBuffer (tensorpipe/common/buffer.h:21-133).
  int x = 0;
  Buffer b = CpuBuffer{&x};
  CHECK(b.device() == cpu);
  CHECK(b.unwrap<CpuBuffer>().ptr == &x);
  bool threw = false;
  try {
    (void)b.unwrap<HipBuffer>();
  } catch (const std::runtime_error&) {
    threw = true;
  }
  CHECK(threw);
  Buffer copy = b;
  CHECK(copy.unwrap<CpuBuffer>().ptr == &x);
  Buffer h = HipBuffer{reinterpret_cast<void*>(0x1000), reinterpret_cast<void*>(0x2000)};
  CHECK(h.unwrap<HipBuffer>().stream == reinterpret_cast<void*>(0x2000));
  copy = h;
  CHECK(copy.unwrap<HipBuffer>().ptr == reinterpret_cast<void*>(0x1000));
  Buffer dflt;
  CHECK(dflt.unwrap<CpuBuffer>().ptr == nullptr);

  // Error: falsy when empty, what() names the origin (tensorpipe/common/error.h:38-80).
  Error ok;
  CHECK(!ok);
  CHECK(ok.what() == "success");
  Error closed = TP_CREATE_ERROR(channel::ChannelClosedError);
  CHECK(static_cast<bool>(closed));
  CHECK(closed.isOfType<channel::ChannelClosedError>());
  CHECK(!closed.isOfType<channel::ContextClosedError>());
  CHECK(closed.what().find("unit_tests.cc") != std::string::npos);
  Error sys = TP_CREATE_ERROR(SystemError, "connect", 111);
  CHECK(sys.what().find("connect") != std::string::npos);

  // Wire helpers: round trip and refusal to read past the end.
  WireWriter w;
  w.u8(7);
  w.u32(0xdeadbeef);
  w.u64(0x0123456789abcdefull);
  w.str("hello");
  w.str("");
  std::vector<uint8_t> bytes = w.bytes();
  CHECK(bytes.size() == 1 + 4 + 8 + 4 + 5 + 4);
  CHECK(bytes[1] == 0xef && bytes[4] == 0xde); // little endian
  WireReader r(bytes.data(), bytes.size());
  CHECK(r.u8() == 7);
  CHECK(r.u32() == 0xdeadbeef);
  CHECK(r.u64() == 0x0123456789abcdefull);
  CHECK(r.str() == "hello");
  std::string e = "x";
  r.str(&e);
  CHECK(e.empty());
  CHECK(r.ok() && r.atEnd());
  CHECK(r.u32() == 0 && !r.ok());
  const uint8_t lying[] = {0xff, 0xff, 0xff, 0x7f, 'a'}; // length far beyond the buffer
  WireReader bad(lying, sizeof(lying));
  CHECK(bad.str().empty() && !bad.ok());

  CHECK(kCudaDeviceType == "cuda");

  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}

// What a stream owes its reader when the writer left first: everything that
// arrived, then the end (a two-process harness whose last step is "write a
// byte, read a byte, exit" depends on exactly this).
static int runDepartedPeer() {
  int failed = 0;
  auto serverSide = transport::shm::create();
  const std::string addr = "tp_unit_departed_" + std::to_string(::getpid());
  auto listener = serverSide->listen(addr);
  std::promise<std::shared_ptr<transport::Connection>> acceptedP;
  listener->accept([&](const Error& e, std::shared_ptr<transport::Connection> c) {
    acceptedP.set_value(e ? nullptr : std::move(c));
  });
  auto clientSide = transport::shm::create();
  auto conn = clientSide->connect(addr);
  auto accepted = acceptedP.get_future().get();
  CHECK(accepted != nullptr);
  if (!accepted) {
    return 1;
  }
  const std::string first = "first message";
  const std::string second(5000, 'x');
  std::promise<void> wroteP;
  conn->write(first.data(), first.size(), [](const Error&) {});
  conn->write(second.data(), second.size(), [&](const Error&) { wroteP.set_value(); });
  wroteP.get_future().get();
  conn.reset();
  clientSide->join(); // the writer is gone, its socket closed
  clientSide.reset();
  // Let the reader's reactor see the hang-up before any read exists.
  std::this_thread::sleep_for(std::chrono::milliseconds(200));
  for (int i = 0; i < 3; ++i) {
    std::promise<std::pair<bool, std::string>> gotP;
    accepted->read([&](const Error& e, const void* ptr, size_t len) {
      gotP.set_value({static_cast<bool>(e), e ? e.what() : std::string(static_cast<const char*>(ptr), len)});
    });
    auto got = gotP.get_future().get();
    if (i == 0) {
      CHECK(!got.first && got.second == first);
    } else if (i == 1) {
      CHECK(!got.first && got.second == second);
    } else {
      CHECK(got.first && got.second.find("eof") != std::string::npos);
    }
  }
  // A connection that was closed on this side hands over nothing more.
  accepted->close();
  std::promise<bool> afterCloseP;
  accepted->read([&](const Error& e, const void*, size_t) { afterCloseP.set_value(static_cast<bool>(e)); });
  CHECK(afterCloseP.get_future().get());
  listener->close();
  serverSide->join();
  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}

// Random bytes where the first packets of a pipe belong.
static int runGarbage(int argc, char** argv) {
  const unsigned seed = static_cast<unsigned>(std::strtoul(argv[2], nullptr, 10));
  const int connections = std::atoi(argv[3]);
  std::mt19937 rng(seed);
  auto server = std::make_shared<Context>(ContextOptions().name("server"));
  server->registerTransport(1, "shm", transport::shm::create());
  server->registerChannel(1, "basic", channel::basic::create());
  const std::string addr = "tp_unit_garbage_" + std::to_string(::getpid()) + "_" + std::to_string(seed);
  auto listener = server->listen({"shm://" + addr});
  auto rawTransport = transport::shm::create();
  std::vector<std::shared_ptr<transport::Connection>> keep;
  for (int c = 0; c < connections; ++c) {
    auto conn = rawTransport->connect(addr);
    const int messages = 1 + static_cast<int>(rng() % 4);
    for (int m = 0; m < messages; ++m) {
      auto bytes = std::make_shared<std::vector<uint8_t>>(rng() % 300);
      for (auto& b : *bytes) {
        b = static_cast<uint8_t>(rng());
      }
      if (!bytes->empty() && rng() % 2 == 0) {
        (*bytes)[0] = static_cast<uint8_t>(1 + rng() % 2); // looks like a hello of either kind
      }
      conn->write(bytes->data(), bytes->size(), [bytes](const Error&) {});
    }
    if (rng() % 3 == 0) {
      conn->close();
    } else {
      keep.push_back(std::move(conn));
    }
  }
  // Pipes the garbage may have created are accepted and dropped; then a proper one.
  auto client = std::make_shared<Context>(ContextOptions().name("client"));
  client->registerTransport(1, "shm", transport::shm::create());
  client->registerChannel(1, "basic", channel::basic::create());
  auto pipe = client->connect("shm://" + addr);
  std::vector<uint8_t> data(100000);
  for (size_t i = 0; i < data.size(); ++i) {
    data[i] = static_cast<uint8_t>(i * 7);
  }
  Message msg;
  msg.metadata = "proper";
  Message::Tensor t;
  t.buffer = CpuBuffer{data.data()};
  t.length = data.size();
  msg.tensors.push_back(std::move(t));
  auto written = std::make_shared<std::promise<Error>>();
  auto fWritten = written->get_future();
  pipe->write(std::move(msg), [written](const Error& e) { written->set_value(e); });

  std::vector<uint8_t> got(data.size());
  auto done = std::make_shared<std::promise<std::string>>();
  auto fDone = done->get_future();
  auto fulfilled = std::make_shared<std::atomic<bool>>(false);
  std::function<void()> acceptNext;
  std::mutex acceptedMutex;
  std::vector<std::shared_ptr<Pipe>> accepted;
  acceptNext = [&] {
    listener->accept([&](const Error& e, std::shared_ptr<Pipe> p) {
      if (e) {
        if (!fulfilled->exchange(true)) {
          done->set_value("accept failed: " + e.what());
        }
        return; // also how the chain ends when the context closes
      }
      {
        std::lock_guard<std::mutex> lock(acceptedMutex);
        accepted.push_back(p);
      }
      p->readDescriptor([&, p](const Error& e2, Descriptor d) {
        if (e2 || d.metadata != "proper") {
          return; // one of the garbage pipes: it fails or never speaks; ignore it
        }
        Allocation a;
        Allocation::Tensor at;
        at.buffer = CpuBuffer{got.data()};
        a.tensors.push_back(std::move(at));
        p->read(std::move(a), [&](const Error& e3) {
          if (!fulfilled->exchange(true)) {
            done->set_value(e3 ? "read failed: " + e3.what() : std::string());
          }
        });
      });
      acceptNext();
    });
  };
  acceptNext();
  int rc = 0;
  if (fDone.wait_for(std::chrono::seconds(30)) != std::future_status::ready) {
    std::printf("the proper pipe did not get through\n");
    rc = 1;
  } else {
    const std::string problem = fDone.get();
    if (!problem.empty() || got != data) {
      std::printf("proper pipe: %s\n", problem.empty() ? "bytes differ" : problem.c_str());
      rc = 1;
    }
  }
  if (rc == 0 && (fWritten.wait_for(std::chrono::seconds(30)) != std::future_status::ready || fWritten.get())) {
    std::printf("the proper write did not complete\n");
    rc = 1;
  }
  // The accept chain above runs on the server's threads and uses `listener` and
  // `accepted`: the contexts are joined (no callback runs after that) before
  // either goes away.
  keep.clear();
  pipe.reset();
  client->join();
  server->join();
  accepted.clear();
  listener.reset();
  if (rc == 0) {
    std::printf("OK\n");
  }
  return rc;
}

// What a HipBuffer may wrap: device memory and pinned host memory name their
// device; plain host memory is refused with std::runtime_error, as the
// reference's driver query does (tensorpipe/common/cuda.h:141-166,
// tensorpipe/common/cuda_buffer.cc:16-28). Needs a GPU.
// mapOver: the runtime in use leaves freed ranges mapped and unreadable (the host-only stand-in
// does), so the plain memory of the last case is mapped over the freed range.
static int runPointers(bool mapOver) {
  int failed = 0;
  void* dev = nullptr;
  CHECK(tphip_malloc(0, 1 << 20, &dev) == 0);
  void* pinned = nullptr;
  void* pinnedDev = nullptr;
  CHECK(tphip_host_alloc(0, 1 << 16, &pinned, &pinnedDev) == 0);
  std::vector<uint8_t> heap(4096);
  uint8_t onStack[64];
  for (int round = 0; round < 3; ++round) { // the second and third answers come from the range table
    CHECK((HipBuffer{dev, nullptr}.getDevice() == Device{kHipDeviceType, 0}));
    CHECK((HipBuffer{static_cast<uint8_t*>(dev) + (1 << 20) - 1, nullptr}.getDevice().index == 0));
    CHECK((HipBuffer{pinned, nullptr}.getDevice().index == 0));
    for (void* bad : {static_cast<void*>(heap.data()), static_cast<void*>(onStack), static_cast<void*>(nullptr)}) {
      bool threw = false;
      try {
        (void)(HipBuffer{bad, nullptr}.getDevice());
      } catch (const std::runtime_error&) {
        threw = true;
      }
      CHECK(threw);
    }
  }
  // an address that is freed keeps no stale answer once something else lives there
  CHECK(tphip_free(0, dev) == 0);
  void* again = nullptr;
  CHECK(tphip_malloc(0, 1 << 12, &again) == 0);
  CHECK((HipBuffer{again, nullptr}.getDevice().index == 0));
  CHECK(tphip_free(0, again) == 0);
  CHECK(tphip_host_free(pinned) == 0);
  // ... and none once memory lives there that the runtime knows nothing about: the remembered
  // answer is checked again at the start of the next unit of work
  void* gone = nullptr;
  CHECK(tphip_malloc(0, 1 << 20, &gone) == 0);
  CHECK((HipBuffer{gone, nullptr}.getDevice().index == 0));
  CHECK((HipBuffer{static_cast<uint8_t*>(gone) + 4096, nullptr}.getDevice().index == 0)); // remembered
  CHECK(tphip_free(0, gone) == 0);
#ifdef MAP_FIXED_NOREPLACE
  void* plain = ::mmap(gone, 1 << 20, PROT_READ | PROT_WRITE,
                       MAP_PRIVATE | MAP_ANONYMOUS | (mapOver ? MAP_FIXED : MAP_FIXED_NOREPLACE), -1, 0);
  if (plain == gone) {
    hipPointerCheckpoint();
    bool threw = false;
    try {
      (void)(HipBuffer{static_cast<uint8_t*>(gone) + 4096, nullptr}.getDevice());
    } catch (const std::runtime_error&) {
      threw = true;
    }
    CHECK(threw);
    ::munmap(plain, 1 << 20);
  } else {
    if (plain != MAP_FAILED) {
      ::munmap(plain, 1 << 20);
    }
    std::printf("note: the freed range could not be mapped again; the stale-answer case did not run\n");
  }
#endif
  // a range that is still what it was costs one look per unit of work and keeps its answer
  void* kept = nullptr;
  CHECK(tphip_malloc(0, 1 << 16, &kept) == 0);
  for (int round = 0; round < 3; ++round) {
    hipPointerCheckpoint();
    CHECK((HipBuffer{kept, nullptr}.getDevice().index == 0));
  }
  CHECK(tphip_free(0, kept) == 0);
  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}

// A crash names its stack before the process dies.
static bool fromHex(const std::string& hex, tpnop::Bytes* out) {
  if (hex.size() % 2 != 0) {
    return false;
  }
  out->clear();
  for (size_t i = 0; i < hex.size(); i += 2) {
    unsigned v = 0;
    if (std::sscanf(hex.c_str() + i, "%2x", &v) != 1) {
      return false;
    }
    out->push_back(static_cast<uint8_t>(v));
  }
  return true;
}

// Decodes `bytes` as what `name` says it is and encodes it again.
static bool roundTrip(const std::string& name, const tpnop::Bytes& bytes, tpnop::Bytes* again, std::string* facts) {
  const uint8_t* p = bytes.data();
  const size_t n = bytes.size();
  if (name.find("spontaneous_connection") != std::string::npos || name.find("requested_connection") != std::string::npos) {
    tpnop::Packet v;
    if (!tpnop::decode(p, n, &v)) {
      return false;
    }
    *again = tpnop::encode(v);
    *facts = v.which == tpnop::Packet::kSpontaneous ? "name=" + v.spontaneous.contextName
                                                    : "token=" + std::to_string(v.requested.registrationId);
    return true;
  }
  if (name.find("brochure_answer") != std::string::npos) {
    tpnop::BrochureAnswer v;
    if (!tpnop::decode(p, n, &v)) {
      return false;
    }
    *again = tpnop::encode(v);
    *facts = "transport=" + v.transport + " domain=" + v.transportDomainDescriptor +
        " ids=" + std::to_string(v.transportRegistrationIds.size()) +
        " channels=" + std::to_string(v.channelRegistrationIds.size()) +
        " pairs=" + std::to_string(v.channelForDevicePair.size());
    if (!v.channelForDevicePair.empty()) {
      *facts += " first_pair=" + v.channelForDevicePair[0].first.first.type + "," +
          v.channelForDevicePair[0].first.second.type + "->" + v.channelForDevicePair[0].second;
    }
    return true;
  }
  if (name.find("brochure") != std::string::npos) {
    tpnop::Brochure v;
    if (!tpnop::decode(p, n, &v)) {
      return false;
    }
    *again = tpnop::encode(v);
    *facts = "transports=" + std::to_string(v.transportDomainDescriptors.size()) +
        " channels=" + std::to_string(v.channelDeviceDescriptors.size());
    if (!v.transportDomainDescriptors.empty()) {
      *facts += " first=" + v.transportDomainDescriptors[0].first + ":" + v.transportDomainDescriptors[0].second;
    }
    return true;
  }
  if (name.find("descriptor_reply") != std::string::npos) {
    tpnop::DescriptorReply v;
    if (!tpnop::decode(p, n, &v)) {
      return false;
    }
    *again = tpnop::encode(v);
    *facts = "devices=" + std::to_string(v.targetDevices.size());
    for (auto& d : v.targetDevices) {
      *facts += " " + d.type + ":" + std::to_string(d.index);
    }
    return true;
  }
  if (name.find("descriptor") != std::string::npos) {
    tpnop::Descriptor v;
    if (!tpnop::decode(p, n, &v)) {
      return false;
    }
    *again = tpnop::encode(v);
    *facts = "metadata=" + v.metadata + " payloads=";
    for (auto& pl : v.payloads) {
      *facts += std::to_string(pl.length) + "[" + pl.metadata + "]";
    }
    *facts += " tensors=";
    for (auto& t : v.tensors) {
      *facts += std::to_string(t.length) + "@" + t.sourceDevice.type + (t.hasTargetDevice ? ">" + t.targetDevice.type : ">?") +
          "[" + t.metadata + "]";
    }
    return true;
  }
  return false;
}

static int runNopWire(const char* file) {
  FILE* f = std::fopen(file, "r");
  if (f == nullptr) {
    std::perror(file);
    return 2;
  }
  int failures = 0, vectors = 0;
  char* line = nullptr;
  size_t cap = 0;
  std::mt19937 rng(99);
  while (::getline(&line, &cap, f) > 0) {
    std::string l(line);
    while (!l.empty() && (l.back() == '\n' || l.back() == '\r')) {
      l.pop_back();
    }
    if (l.empty() || l[0] == '#') {
      continue;
    }
    const size_t sp = l.find(' ');
    const std::string name = l.substr(0, sp);
    tpnop::Bytes bytes, again;
    std::string facts;
    if (sp == std::string::npos || !fromHex(l.substr(sp + 1), &bytes)) {
      std::printf("FAIL %s: not a vector line\n", name.c_str());
      ++failures;
      continue;
    }
    ++vectors;
    if (!roundTrip(name, bytes, &again, &facts)) {
      std::printf("FAIL %s: does not decode\n", name.c_str());
      ++failures;
      continue;
    }
    if (again != bytes) {
      std::printf("FAIL %s: encodes back to other bytes\n", name.c_str());
      ++failures;
    }
    std::printf("VECTOR %s %s\n", name.c_str(), facts.c_str());
    // Cut short anywhere it must be refused; with a byte changed it may decode
    // or not, but must not read out of bounds (the copies are exactly sized,
    // so a sanitizer build sees an overrun).
    for (size_t cut = 0; cut < bytes.size(); ++cut) {
      tpnop::Bytes part(bytes.begin(), bytes.begin() + cut), ignored;
      std::string ignoredFacts;
      if (roundTrip(name, part, &ignored, &ignoredFacts)) {
        std::printf("FAIL %s: decodes when cut to %zu bytes\n", name.c_str(), cut);
        ++failures;
        break;
      }
    }
    for (int k = 0; k < 200; ++k) {
      tpnop::Bytes bent(bytes), ignored;
      std::string ignoredFacts;
      bent[rng() % bent.size()] = static_cast<uint8_t>(rng());
      (void)roundTrip(name, bent, &ignored, &ignoredFacts);
    }
  }
  std::free(line);
  std::fclose(f);
  // What the writer does with values the captured frames do not hold.
  {
    tpnop::Descriptor d;
    d.metadata = std::string(300, 'm');
    d.payloads.push_back({uint64_t(1) << 40, "big"});
    d.tensors.push_back({0xffff, {"cuda", 3}, true, {"cuda", -1}, ""});
    d.tensors.push_back({0x10000, {"cpu", 200}, false, {}, "x"});
    tpnop::Descriptor back;
    const tpnop::Bytes b = tpnop::encode(d);
    if (!tpnop::decode(b.data(), b.size(), &back) || back.metadata != d.metadata || back.payloads[0].length != d.payloads[0].length ||
        back.tensors[0].targetDevice.index != -1 || back.tensors[0].length != 0xffff || back.tensors[1].sourceDevice.index != 200 ||
        back.tensors[1].hasTargetDevice || back.tensors[1].length != 0x10000) {
      std::printf("FAIL a descriptor with large and negative values does not survive a round trip\n");
      ++failures;
    }
    uint8_t header[tpnop::kFrameHeaderBytes];
    tpnop::putFrameHeader(0x0102030405060708ull, header);
    if (header[0] != 8 || header[7] != 1 || tpnop::getFrameHeader(header) != 0x0102030405060708ull) {
      std::printf("FAIL frame header\n");
      ++failures;
    }
  }
  std::printf("%s %d vectors\n", failures == 0 ? "OK" : "FAILED", vectors);
  return failures == 0 ? 0 : 1;
}

static int runCompatPipe() {
  std::string error;
  auto listener = tpnop::CompatListener::create(&error);
  if (!listener) {
    std::printf("FAIL listen: %s\n", error.c_str());
    return 1;
  }
  std::string clientError;
  auto connecting = std::async(std::launch::async, [&] {
    return tpnop::CompatPipe::connect(listener->address(), "client end", &clientError);
  });
  auto server = listener->accept("server end", &error);
  auto client = connecting.get();
  if (!server || !client) {
    std::printf("FAIL handshake: %s %s\n", error.c_str(), clientError.c_str());
    return 1;
  }
  int failures = 0;
  if (server->remoteName() != "client end") {
    std::printf("FAIL the listening end heard the name %s\n", server->remoteName().c_str());
    ++failures;
  }
  for (int round = 0; round < 4 && failures == 0; ++round) {
    tpnop::CompatMessage m, got;
    m.metadata = "round " + std::to_string(round);
    m.payloads.push_back({std::string(1000 + round, 'p'), "payload metadata"});
    m.payloads.push_back({"", ""});
    m.tensors.push_back({std::string(100000 + round, 't'), "tensor", round % 2 == 0});
    m.tensors.push_back({"", "empty", false});
    tpnop::CompatPipe& from = round % 2 == 0 ? *client : *server;
    tpnop::CompatPipe& to = round % 2 == 0 ? *server : *client;
    std::string writeError;
    auto writing = std::async(std::launch::async, [&] { return from.write(m, &writeError); });
    const bool readOk = to.read(&got, &error);
    if (!writing.get() || !readOk) {
      std::printf("FAIL round %d: %s %s\n", round, writeError.c_str(), error.c_str());
      ++failures;
    } else if (got.metadata != m.metadata || got.payloads.size() != 2 || got.payloads[0].bytes != m.payloads[0].bytes ||
               got.payloads[0].metadata != "payload metadata" || got.tensors.size() != 2 ||
               got.tensors[0].bytes != m.tensors[0].bytes || got.tensors[0].nameTarget != m.tensors[0].nameTarget ||
               !got.tensors[1].bytes.empty() || got.tensors[1].metadata != "empty") {
      std::printf("FAIL round %d: the message arrived changed\n", round);
      ++failures;
    }
  }
  std::printf("%s\n", failures == 0 ? "OK" : "FAILED");
  return failures == 0 ? 0 : 1;
}

// Messages of every size class both ways over one connection of any transport, reads
// posted before and after the writes, unsized and exact-length reads alternating; then
// an exact-length read that meets a message of another length. Returns the failures.
static int exerciseConnections(
    transport::Context& serverSide,
    transport::Context& clientSide,
    transport::Listener& listener,
    const std::string& addr) {
  int failed = 0;
  std::promise<std::shared_ptr<transport::Connection>> acceptedP;
  listener.accept([&](const Error& e, std::shared_ptr<transport::Connection> c) {
    acceptedP.set_value(e ? nullptr : std::move(c));
  });
  auto conn = clientSide.connect(addr);
  auto acceptedF = acceptedP.get_future();
  CHECK(acceptedF.wait_for(std::chrono::seconds(30)) == std::future_status::ready);
  auto accepted = acceptedF.get();
  CHECK(accepted != nullptr);
  if (!accepted) {
    return failed + 1;
  }
  (void)serverSide;
  const std::vector<size_t> sizes = {0, 1, 3, 4, 5, 4096, 65537, 1 << 20, (2u << 20) - 4, 2u << 20, (24u << 20) + 3};
  for (int direction = 0; direction < 2; ++direction) {
    auto& from = direction == 0 ? conn : accepted;
    auto& to = direction == 0 ? accepted : conn;
    std::vector<std::vector<uint8_t>> sent;
    for (size_t k = 0; k < sizes.size(); ++k) {
      std::vector<uint8_t> m(sizes[k]);
      for (size_t i = 0; i < m.size(); ++i) {
        m[i] = static_cast<uint8_t>((i * 13 + k * 7 + direction) % 251);
      }
      sent.push_back(std::move(m));
    }
    std::vector<std::future<bool>> results;
    auto postRead = [&](size_t k) {
      auto p = std::make_shared<std::promise<bool>>();
      results.push_back(p->get_future());
      const std::vector<uint8_t>* want = &sent[k];
      if (k % 2 == 0) {
        to->read([p, want](const Error& e, const void* ptr, size_t len) {
          p->set_value(!e && len == want->size() && (len == 0 || std::memcmp(ptr, want->data(), len) == 0));
        });
      } else {
        auto buf = std::make_shared<std::vector<uint8_t>>(want->size());
        to->read(buf->data(), buf->size(), [p, want, buf](const Error& e, const void*, size_t len) {
          p->set_value(!e && len == want->size() && *buf == *want);
        });
      }
    };
    for (size_t k = 0; k < sizes.size() / 2; ++k) {
      postRead(k); // these wait for their bytes
    }
    auto wroteAll = std::make_shared<std::promise<bool>>();
    auto allFine = std::make_shared<std::atomic<bool>>(true);
    for (size_t k = 0; k < sizes.size(); ++k) {
      const bool last = k + 1 == sizes.size();
      from->write(sent[k].data(), sent[k].size(), [wroteAll, allFine, last](const Error& e) {
        if (e) {
          allFine->store(false);
        }
        if (last) {
          wroteAll->set_value(allFine->load());
        }
      });
    }
    for (size_t k = sizes.size() / 2; k < sizes.size(); ++k) {
      postRead(k); // these find their bytes already there, or on their way
    }
    for (auto& r : results) {
      CHECK(r.wait_for(std::chrono::seconds(30)) == std::future_status::ready && r.get());
    }
    auto wroteF = wroteAll->get_future();
    CHECK(wroteF.wait_for(std::chrono::seconds(30)) == std::future_status::ready && wroteF.get());
  }
  // An exact-length read that meets a message of another length fails the connection.
  {
    auto other = clientSide.connect(addr);
    std::promise<std::shared_ptr<transport::Connection>> p2;
    listener.accept([&](const Error& e, std::shared_ptr<transport::Connection> c) { p2.set_value(e ? nullptr : std::move(c)); });
    auto acc2 = p2.get_future().get();
    CHECK(acc2 != nullptr);
    const std::string msg = "five!";
    std::promise<void> wroteMsg; // the bytes stay the caller's until then: the length may travel ahead of them
    other->write(msg.data(), msg.size(), [&](const Error&) { wroteMsg.set_value(); });
    char buf[4];
    std::promise<bool> failedRead;
    acc2->read(buf, sizeof(buf), [&](const Error& e, const void*, size_t) { failedRead.set_value(static_cast<bool>(e)); });
    CHECK(failedRead.get_future().get());
    wroteMsg.get_future().get();
  }
  // A peer that writes and leaves before anybody reads: the messages, then the end; a write
  // to it fails.
  {
    auto other = clientSide.connect(addr);
    std::promise<std::shared_ptr<transport::Connection>> p3;
    listener.accept([&](const Error& e, std::shared_ptr<transport::Connection> c) { p3.set_value(e ? nullptr : std::move(c)); });
    auto acc3 = p3.get_future().get();
    CHECK(acc3 != nullptr);
    const std::string one = "first", two(70000, 'z');
    std::promise<void> wrote;
    other->write(one.data(), one.size(), [](const Error&) {});
    other->write(two.data(), two.size(), [&](const Error&) { wrote.set_value(); });
    wrote.get_future().get();
    other->close();
    other.reset();
    std::this_thread::sleep_for(std::chrono::milliseconds(100));
    for (int i = 0; i < 3; ++i) {
      std::promise<std::pair<bool, std::string>> gotP;
      acc3->read([&](const Error& e, const void* ptr, size_t len) {
        gotP.set_value({static_cast<bool>(e), e ? e.what() : std::string(static_cast<const char*>(ptr), len)});
      });
      auto g = gotP.get_future().get();
      if (i == 0) {
        CHECK(!g.first && g.second == one);
      } else if (i == 1) {
        CHECK(!g.first && g.second == two);
      } else {
        CHECK(g.first && g.second.find("eof") != std::string::npos);
      }
    }
    std::promise<bool> lateWrite;
    acc3->write(one.data(), one.size(), [&](const Error& e) { lateWrite.set_value(static_cast<bool>(e)); });
    CHECK(lateWrite.get_future().get());
  }
  // Closing a listener fails its pending accept; closing a connection fails its pending read.
  {
    auto other = clientSide.connect(addr);
    std::promise<std::shared_ptr<transport::Connection>> p4;
    listener.accept([&](const Error& e, std::shared_ptr<transport::Connection> c) { p4.set_value(e ? nullptr : std::move(c)); });
    auto acc4 = p4.get_future().get();
    CHECK(acc4 != nullptr);
    std::promise<bool> pendingRead;
    acc4->read([&](const Error& e, const void*, size_t) { pendingRead.set_value(static_cast<bool>(e)); });
    acc4->close();
    CHECK(pendingRead.get_future().get());
    std::promise<bool> peersRead;
    other->read([&](const Error& e, const void*, size_t) { peersRead.set_value(static_cast<bool>(e)); });
    CHECK(peersRead.get_future().get());
  }
  return failed;
}

// The transport that speaks the reference's shm protocol, both ends this library's.
static int runShmStock() {
  int failed = 0;
  auto serverSide = transport::shm_stock::create();
  auto clientSide = transport::shm_stock::create();
  CHECK(serverSide->isViable());
  // tensorpipe/transport/shm/context_impl.cc:29-47: shm:<boot id>_<device>_<inode of the network namespace>
  const std::string d = serverSide->domainDescriptor();
  CHECK(d.rfind("shm:", 0) == 0 && std::count(d.begin(), d.end(), '_') == 2 && d == clientSide->domainDescriptor());
  CHECK(serverSide->canCommunicateWithRemote(d) && !serverSide->canCommunicateWithRemote(d + "x"));
  // a name the kernel picks, and one the caller picks
  auto anonymous = serverSide->listen("");
  CHECK(!anonymous->addr().empty());
  const std::string name = "tp_amd_unit_" + std::to_string(::getpid());
  auto listener = serverSide->listen(name);
  CHECK(listener->addr() == name);
  failed += exerciseConnections(*serverSide, *clientSide, *listener, name);
  failed += exerciseConnections(*serverSide, *serverSide, *anonymous, anonymous->addr()); // both ends on one thread
  std::promise<bool> closedAccept;
  listener->accept([&](const Error& e, std::shared_ptr<transport::Connection>) { closedAccept.set_value(static_cast<bool>(e)); });
  listener->close();
  CHECK(closedAccept.get_future().get());
  anonymous.reset();
  listener.reset();
  clientSide->join();
  serverSide->join();
  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}

// A peer of the shm transport written against the reference's protocol alone
// (tensorpipe/transport/shm/connection_impl.cc:231-291, common/shm_ringbuffer.h:23-82,
// common/ringbuffer.h:50-140), so that it can misbehave: ring headers are memory
// that both ends can write.
struct RawShmPeer {
  struct Header { // RingBufferHeader<2> on x86-64
    uint64_t dataBytes;
    uint64_t dataMask;
    uint8_t inTransaction[2];
    uint8_t pad[6];
    std::atomic<uint64_t> marker[2]; // 0: consumed, 1: produced
  };
  static_assert(sizeof(Header) == 40, "layout of the reference's ring header");

  int sock{-1};
  int mine[4]{-1, -1, -1, -1}; // reactor header/data, inbox header/data
  int theirs[4]{-1, -1, -1, -1};
  Header* theirReactor{nullptr};
  uint8_t* theirReactorData{nullptr};
  Header* theirInbox{nullptr};
  uint8_t* theirInboxData{nullptr};
  Header* myInbox{nullptr};
  uint32_t theirTokens[2]{0, 0}; // run when we wrote into their inbox / read from ours

  static int segment(size_t bytes) {
    const int fd = ::memfd_create("raw_shm_peer", MFD_CLOEXEC);
    if (fd >= 0 && ::ftruncate(fd, static_cast<off_t>(bytes)) != 0) {
      ::close(fd);
      return -1;
    }
    return fd;
  }
  static void* mapAll(int fd, size_t bytes) {
    void* p = ::mmap(nullptr, bytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    return p == MAP_FAILED ? nullptr : p;
  }
  static Header* ring(int* headerFd, int* dataFd, uint64_t saysBytes, size_t reallyBytes) {
    *headerFd = segment(sizeof(Header));
    *dataFd = segment(reallyBytes);
    auto* h = static_cast<Header*>(mapAll(*headerFd, sizeof(Header)));
    if (h != nullptr) {
      h->dataBytes = saysBytes;
      h->dataMask = saysBytes - 1;
    }
    return h;
  }

  // Connects and swaps descriptors. `inboxReallyBytes` lets the data segment
  // differ from what the header says.
  bool connect(const std::string& name, size_t inboxReallyBytes = 2u << 20) {
    sock = ::socket(AF_UNIX, SOCK_STREAM | SOCK_CLOEXEC, 0);
    sockaddr_un sun;
    std::memset(&sun, 0, sizeof(sun));
    sun.sun_family = AF_UNIX;
    std::memcpy(&sun.sun_path[1], name.data(), name.size());
    if (sock < 0 ||
        ::connect(sock, reinterpret_cast<sockaddr*>(&sun), static_cast<socklen_t>(sizeof(sun.sun_family) + 1 + name.size())) != 0) {
      return false;
    }
    Header* myReactor = ring(&mine[0], &mine[1], 4u << 20, 4u << 20);
    myInbox = ring(&mine[2], &mine[3], 2u << 20, inboxReallyBytes);
    if (myReactor == nullptr || myInbox == nullptr) {
      return false;
    }
    uint32_t tokens[2] = {0, 1};
    iovec iov{tokens, sizeof(tokens)};
    alignas(cmsghdr) char control[CMSG_SPACE(sizeof(mine))];
    std::memset(control, 0, sizeof(control));
    msghdr msg{};
    msg.msg_iov = &iov;
    msg.msg_iovlen = 1;
    msg.msg_control = control;
    msg.msg_controllen = sizeof(control);
    cmsghdr* cmsg = CMSG_FIRSTHDR(&msg);
    cmsg->cmsg_level = SOL_SOCKET;
    cmsg->cmsg_type = SCM_RIGHTS;
    cmsg->cmsg_len = CMSG_LEN(sizeof(mine));
    std::memcpy(CMSG_DATA(cmsg), mine, sizeof(mine));
    if (::sendmsg(sock, &msg, MSG_NOSIGNAL) != static_cast<ssize_t>(sizeof(tokens))) {
      return false;
    }
    // their turn
    std::memset(control, 0, sizeof(control));
    iov = iovec{theirTokens, sizeof(theirTokens)};
    msg.msg_controllen = sizeof(control);
    pollfd pfd{sock, POLLIN, 0};
    if (::poll(&pfd, 1, 10000) != 1 || ::recvmsg(sock, &msg, MSG_CMSG_CLOEXEC) != static_cast<ssize_t>(sizeof(theirTokens))) {
      return false;
    }
    cmsg = CMSG_FIRSTHDR(&msg);
    if (cmsg == nullptr || cmsg->cmsg_len != CMSG_LEN(sizeof(theirs))) {
      return false;
    }
    std::memcpy(theirs, CMSG_DATA(cmsg), sizeof(theirs));
    theirReactor = static_cast<Header*>(mapAll(theirs[0], sizeof(Header)));
    theirInbox = static_cast<Header*>(mapAll(theirs[2], sizeof(Header)));
    if (theirReactor == nullptr || theirInbox == nullptr) {
      return false;
    }
    theirReactorData = static_cast<uint8_t*>(mapAll(theirs[1], theirReactor->dataBytes));
    theirInboxData = static_cast<uint8_t*>(mapAll(theirs[3], theirInbox->dataBytes));
    return theirReactorData != nullptr && theirInboxData != nullptr;
  }

  // Appends bytes to a ring the way a well-behaved producer does.
  static void produce(Header* h, uint8_t* data, const void* src, size_t n) {
    const uint64_t head = h->marker[1].load();
    for (size_t i = 0; i < n; ++i) {
      data[(head + i) & h->dataMask] = static_cast<const uint8_t*>(src)[i];
    }
    h->marker[1].store(head + n);
  }
  void poke(uint32_t token) {
    produce(theirReactor, theirReactorData, &token, sizeof(token));
  }
  void hangUp() {
    if (sock >= 0) {
      ::close(sock);
      sock = -1;
    }
  }
  ~RawShmPeer() {
    hangUp();
    for (int fd : mine) {
      if (fd >= 0) {
        ::close(fd);
      }
    }
    for (int fd : theirs) {
      if (fd >= 0) {
        ::close(fd);
      }
    }
  }
};

// What a connection does when the other end breaks the protocol: it reports an
// error; it neither reads outside the rings nor waits for ever.
static int runShmStockHostilePeer() {
  int failed = 0;
  auto serverSide = transport::shm_stock::create();
  const std::string name = "tp_amd_unit_hostile_" + std::to_string(::getpid());
  auto listener = serverSide->listen(name);
  auto acceptOne = [&]() {
    auto p = std::make_shared<std::promise<std::shared_ptr<transport::Connection>>>();
    listener->accept([p](const Error& e, std::shared_ptr<transport::Connection> c) { p->set_value(e ? nullptr : std::move(c)); });
    return p->get_future();
  };
  auto readOutcome = [](transport::Connection& c) {
    auto p = std::make_shared<std::promise<std::string>>();
    c.read([p](const Error& e, const void* ptr, size_t len) {
      p->set_value(e ? "error: " + e.what() : std::string(static_cast<const char*>(ptr), len));
    });
    return p->get_future();
  };
  const auto patience = std::chrono::seconds(20);

  { // a well-behaved raw peer first: the helper itself speaks the protocol
    auto acceptedF = acceptOne();
    RawShmPeer peer;
    CHECK(peer.connect(name));
    auto accepted = acceptedF.get();
    CHECK(accepted != nullptr);
    auto got = readOutcome(*accepted);
    const char text[] = "hello";
    const uint32_t length = 5;
    RawShmPeer::produce(peer.theirInbox, peer.theirInboxData, &length, 4);
    RawShmPeer::produce(peer.theirInbox, peer.theirInboxData, text, 5);
    peer.poke(peer.theirTokens[0]);
    CHECK(got.wait_for(patience) == std::future_status::ready && got.get() == "hello");
  }
  { // a data segment smaller than its header says
    auto acceptedF = acceptOne();
    RawShmPeer peer;
    (void)peer.connect(name, 4096);
    auto accepted = acceptedF.get();
    CHECK(accepted != nullptr);
    auto got = readOutcome(*accepted);
    CHECK(got.wait_for(patience) == std::future_status::ready && got.get().rfind("error: ", 0) == 0);
  }
  { // more bytes announced as produced than the inbox can hold
    auto acceptedF = acceptOne();
    RawShmPeer peer;
    CHECK(peer.connect(name));
    auto accepted = acceptedF.get();
    auto got = readOutcome(*accepted);
    peer.theirInbox->marker[1].store(peer.theirInbox->marker[0].load() + (1ull << 40));
    peer.poke(peer.theirTokens[0]);
    CHECK(got.wait_for(patience) == std::future_status::ready && got.get().rfind("error: ", 0) == 0);
  }
  { // the ring's size rewritten after set-up: the size checked at set-up is what counts
    auto acceptedF = acceptOne();
    RawShmPeer peer;
    CHECK(peer.connect(name));
    auto accepted = acceptedF.get();
    auto got = readOutcome(*accepted);
    const uint32_t length = 3;
    RawShmPeer::produce(peer.theirInbox, peer.theirInboxData, &length, 4);
    RawShmPeer::produce(peer.theirInbox, peer.theirInboxData, "abc", 3);
    peer.theirInbox->dataBytes = 1ull << 40;
    peer.theirInbox->dataMask = (1ull << 40) - 1;
    peer.poke(peer.theirTokens[0]);
    CHECK(got.wait_for(patience) == std::future_status::ready && got.get() == "abc");
  }
  { // our outbox (the peer's inbox) says that more was consumed than was ever produced
    auto acceptedF = acceptOne();
    RawShmPeer peer;
    CHECK(peer.connect(name));
    auto accepted = acceptedF.get();
    peer.myInbox->marker[0].store(1ull << 40);
    auto p = std::make_shared<std::promise<bool>>();
    static const char payload[64] = {1};
    accepted->write(payload, sizeof(payload), [p](const Error& e) { p->set_value(static_cast<bool>(e)); });
    auto f = p->get_future();
    CHECK(f.wait_for(patience) == std::future_status::ready && f.get());
  }
  { // a long message announced, a few bytes of it written, then gone
    auto acceptedF = acceptOne();
    RawShmPeer peer;
    CHECK(peer.connect(name));
    auto accepted = acceptedF.get();
    auto got = readOutcome(*accepted);
    const uint32_t length = 1u << 20;
    RawShmPeer::produce(peer.theirInbox, peer.theirInboxData, &length, 4);
    RawShmPeer::produce(peer.theirInbox, peer.theirInboxData, "abc", 3);
    peer.poke(peer.theirTokens[0]);
    peer.hangUp();
    CHECK(got.wait_for(patience) == std::future_status::ready && got.get().rfind("error: ", 0) == 0);
  }
  listener.reset();
  serverSide->join();
  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}

static int runTcp() {
  int failed = 0;
  auto serverSide = transport::tcp::create();
  auto listener = serverSide->listen("127.0.0.1");
  const std::string addr = listener->addr();
  CHECK(addr.find("127.0.0.1:") == 0 && addr != "127.0.0.1:0");
  CHECK(serverSide->domainDescriptor() == "uv:*");
  std::promise<std::shared_ptr<transport::Connection>> acceptedP;
  listener->accept([&](const Error& e, std::shared_ptr<transport::Connection> c) {
    acceptedP.set_value(e ? nullptr : std::move(c));
  });
  auto clientSide = transport::tcp::create();
  auto conn = clientSide->connect(addr);
  auto accepted = acceptedP.get_future().get();
  CHECK(accepted != nullptr);
  if (!accepted) {
    return 1;
  }
  // Messages of every size class, both ways, reads posted before and after the writes.
  const std::vector<size_t> sizes = {0, 1, 7, 8, 9, 4096, 65537, 1 << 20, (24u << 20) + 3};
  for (int direction = 0; direction < 2; ++direction) {
    auto& from = direction == 0 ? conn : accepted;
    auto& to = direction == 0 ? accepted : conn;
    std::vector<std::vector<uint8_t>> sent;
    for (size_t k = 0; k < sizes.size(); ++k) {
      std::vector<uint8_t> m(sizes[k]);
      for (size_t i = 0; i < m.size(); ++i) {
        m[i] = static_cast<uint8_t>((i * 13 + k * 7 + direction) % 251);
      }
      sent.push_back(std::move(m));
    }
    std::vector<std::future<bool>> results;
    std::vector<std::shared_ptr<std::vector<uint8_t>>> exactBuffers;
    auto postRead = [&](size_t k) {
      auto p = std::make_shared<std::promise<bool>>();
      results.push_back(p->get_future());
      const std::vector<uint8_t>* want = &sent[k];
      if (k % 2 == 0) {
        to->read([p, want](const Error& e, const void* ptr, size_t len) {
          p->set_value(!e && len == want->size() && (len == 0 || std::memcmp(ptr, want->data(), len) == 0));
        });
      } else {
        auto buf = std::make_shared<std::vector<uint8_t>>(want->size());
        exactBuffers.push_back(buf);
        to->read(buf->data(), buf->size(), [p, want, buf](const Error& e, const void*, size_t len) {
          p->set_value(!e && len == want->size() && *buf == *want);
        });
      }
    };
    for (size_t k = 0; k < sizes.size() / 2; ++k) {
      postRead(k); // these wait for their bytes
    }
    std::promise<void> wroteAll;
    for (size_t k = 0; k < sizes.size(); ++k) {
      const bool last = k + 1 == sizes.size();
      from->write(sent[k].data(), sent[k].size(), [&wroteAll, last](const Error& e) {
        if (last) {
          wroteAll.set_value();
        }
        (void)e;
      });
    }
    for (size_t k = sizes.size() / 2; k < sizes.size(); ++k) {
      postRead(k); // these find their bytes already there, or on their way
    }
    for (auto& r : results) {
      CHECK(r.wait_for(std::chrono::seconds(30)) == std::future_status::ready && r.get());
    }
    wroteAll.get_future().get();
  }
  // An exact-length read that meets a message of another length fails the connection.
  {
    auto other = clientSide->connect(addr);
    std::promise<std::shared_ptr<transport::Connection>> p2;
    listener->accept([&](const Error& e, std::shared_ptr<transport::Connection> c) { p2.set_value(e ? nullptr : std::move(c)); });
    auto acc2 = p2.get_future().get();
    CHECK(acc2 != nullptr);
    const std::string msg = "five!";
    std::promise<void> wroteMsg; // the bytes stay the caller's until then: the length may travel ahead of them
    other->write(msg.data(), msg.size(), [&](const Error&) { wroteMsg.set_value(); });
    char buf[4];
    std::promise<bool> failedRead;
    acc2->read(buf, sizeof(buf), [&](const Error& e, const void*, size_t) { failedRead.set_value(static_cast<bool>(e)); });
    CHECK(failedRead.get_future().get());
    wroteMsg.get_future().get();
  }
  // A frame written by hand, the way the reference frames a stream: 8-byte little-endian length, bytes.
  {
    std::promise<std::shared_ptr<transport::Connection>> p3;
    listener->accept([&](const Error& e, std::shared_ptr<transport::Connection> c) { p3.set_value(e ? nullptr : std::move(c)); });
    const int fd = ::socket(AF_INET, SOCK_STREAM, 0);
    sockaddr_in sa{};
    sa.sin_family = AF_INET;
    sa.sin_port = htons(static_cast<uint16_t>(std::atoi(addr.c_str() + addr.rfind(':') + 1)));
    ::inet_pton(AF_INET, "127.0.0.1", &sa.sin_addr);
    CHECK(::connect(fd, reinterpret_cast<sockaddr*>(&sa), sizeof(sa)) == 0);
    auto acc3 = p3.get_future().get();
    CHECK(acc3 != nullptr);
    const uint8_t frame[8 + 3] = {3, 0, 0, 0, 0, 0, 0, 0, 'a', 'b', 'c'};
    CHECK(::write(fd, frame, 5) == 5); // in two pieces, cut inside the length
    std::promise<std::string> got;
    acc3->read([&](const Error& e, const void* ptr, size_t len) {
      got.set_value(e ? "error" : std::string(static_cast<const char*>(ptr), len));
    });
    std::this_thread::sleep_for(std::chrono::milliseconds(50));
    CHECK(::write(fd, frame + 5, sizeof(frame) - 5) == static_cast<ssize_t>(sizeof(frame) - 5));
    CHECK(got.get_future().get() == "abc");
    // and what this transport writes reads back the same way
    const std::string reply = "reply";
    acc3->write(reply.data(), reply.size(), [](const Error&) {});
    uint8_t back[8 + 5];
    size_t have = 0;
    while (have < sizeof(back)) {
      const ssize_t r = ::read(fd, back + have, sizeof(back) - have);
      if (r <= 0) {
        break;
      }
      have += static_cast<size_t>(r);
    }
    CHECK(have == sizeof(back) && back[0] == 5 && back[1] == 0 && back[7] == 0 && std::memcmp(back + 8, "reply", 5) == 0);
    // the peer writes once more and leaves before anybody reads: the message, then the end
    const uint8_t last[8 + 2] = {2, 0, 0, 0, 0, 0, 0, 0, 'o', 'k'};
    CHECK(::write(fd, last, sizeof(last)) == static_cast<ssize_t>(sizeof(last)));
    ::close(fd);
    std::this_thread::sleep_for(std::chrono::milliseconds(100));
    for (int i = 0; i < 2; ++i) {
      std::promise<std::pair<bool, std::string>> gotP;
      acc3->read([&](const Error& e, const void* ptr, size_t len) {
        gotP.set_value({static_cast<bool>(e), e ? e.what() : std::string(static_cast<const char*>(ptr), len)});
      });
      auto g = gotP.get_future().get();
      if (i == 0) {
        CHECK(!g.first && g.second == "ok");
      } else {
        CHECK(g.first && g.second.find("eof") != std::string::npos);
      }
    }
  }
  // A peer that announces half a terabyte, sends three bytes and leaves: the read ends with
  // an error, and no buffer of the announced size was ever asked for.
  // Then a peer that resets the connection while nobody reads: the reactor must not spin on
  // the hang-up (epoll keeps reporting it), and the next read learns of it.
  for (int scenario = 0; scenario < 2; ++scenario) {
    std::promise<std::shared_ptr<transport::Connection>> p4;
    listener->accept([&](const Error& e, std::shared_ptr<transport::Connection> c) { p4.set_value(e ? nullptr : std::move(c)); });
    const int fd = ::socket(AF_INET, SOCK_STREAM, 0);
    sockaddr_in sa{};
    sa.sin_family = AF_INET;
    sa.sin_port = htons(static_cast<uint16_t>(std::atoi(addr.c_str() + addr.rfind(':') + 1)));
    ::inet_pton(AF_INET, "127.0.0.1", &sa.sin_addr);
    CHECK(::connect(fd, reinterpret_cast<sockaddr*>(&sa), sizeof(sa)) == 0);
    auto acc4 = p4.get_future().get();
    CHECK(acc4 != nullptr);
    if (!acc4) {
      ::close(fd);
      continue;
    }
    if (scenario == 0) {
      const uint8_t lie[8 + 3] = {0, 0, 0, 0, 0x80, 0, 0, 0, 'x', 'y', 'z'};
      CHECK(::write(fd, lie, sizeof(lie)) == static_cast<ssize_t>(sizeof(lie)));
      ::close(fd);
    } else {
      // one message arrives first, so that the reset finds the connection set up and idle
      const uint8_t hello[8 + 2] = {2, 0, 0, 0, 0, 0, 0, 0, 'h', 'i'};
      CHECK(::write(fd, hello, sizeof(hello)) == static_cast<ssize_t>(sizeof(hello)));
      std::promise<bool> first;
      acc4->read([&](const Error& e, const void*, size_t len) { first.set_value(!e && len == 2); });
      CHECK(first.get_future().get());
      linger lg{1, 0};
      ::setsockopt(fd, SOL_SOCKET, SO_LINGER, &lg, sizeof(lg));
      ::close(fd); // sends a reset
      timespec before{}, after{};
      ::clock_gettime(CLOCK_PROCESS_CPUTIME_ID, &before);
      std::this_thread::sleep_for(std::chrono::milliseconds(400));
      ::clock_gettime(CLOCK_PROCESS_CPUTIME_ID, &after);
      const double cpuMs = (after.tv_sec - before.tv_sec) * 1e3 + (after.tv_nsec - before.tv_nsec) / 1e6;
      if (cpuMs > 200) {
        std::printf("FAIL: %.0f ms of CPU time in 400 ms of idling after a reset\n", cpuMs);
        ++failed;
      }
    }
    std::promise<bool> ended;
    acc4->read([&](const Error& e, const void*, size_t) { ended.set_value(static_cast<bool>(e)); });
    auto f = ended.get_future();
    CHECK(f.wait_for(std::chrono::seconds(20)) == std::future_status::ready && f.get());
    // a write on the dead connection fails too, it does not wait for ever
    std::promise<bool> wrote;
    const char byte = 'b';
    acc4->write(&byte, 1, [&](const Error& e) { wrote.set_value(static_cast<bool>(e)); });
    auto fw = wrote.get_future();
    CHECK(fw.wait_for(std::chrono::seconds(20)) == std::future_status::ready && fw.get());
  }
  // Closing this end fails what is pending on it.
  {
    std::promise<bool> pending;
    accepted->read([&](const Error& e, const void*, size_t) { pending.set_value(static_cast<bool>(e)); });
    accepted->close();
    CHECK(pending.get_future().get());
  }
  conn.reset();
  accepted.reset();
  listener->close();
  listener.reset();
  clientSide->join();
  serverSide->join();

  // IPv6 loopback, where the host has it.
  {
    auto v6 = transport::tcp::create();
    std::shared_ptr<transport::Listener> l6;
    try {
      l6 = v6->listen("[::1]");
    } catch (const std::exception&) {
      // no IPv6 here
    }
    if (l6) {
      CHECK(l6->addr().find("[::1]:") == 0);
      std::promise<std::shared_ptr<transport::Connection>> p6;
      l6->accept([&](const Error& e, std::shared_ptr<transport::Connection> c) { p6.set_value(e ? nullptr : std::move(c)); });
      auto c6 = v6->connect(l6->addr());
      auto a6 = p6.get_future().get();
      CHECK(a6 != nullptr);
      if (a6) {
        const std::string hello = "over v6";
        c6->write(hello.data(), hello.size(), [](const Error&) {});
        std::promise<std::string> got6;
        a6->read([&](const Error& e, const void* ptr, size_t len) {
          got6.set_value(e ? "error" : std::string(static_cast<const char*>(ptr), len));
        });
        CHECK(got6.get_future().get() == hello);
      }
      c6.reset();
      a6.reset();
      l6.reset();
    }
    v6->join();
  }

  // A pipe over it: payload and CPU tensors through the basic channel.
  {
    auto make = [](const char* name) {
      auto ctx = std::make_shared<Context>(ContextOptions().name(name));
      ctx->registerTransport(0, "uv", transport::tcp::create());
      ctx->registerChannel(0, "basic", channel::basic::create());
      return ctx;
    };
    auto server = make("tcp server");
    auto client = make("tcp client");
    auto plistener = server->listen({"uv://127.0.0.1"});
    const std::string url = plistener->url("uv");
    CHECK(url.find("uv://127.0.0.1:") == 0);
    std::promise<std::shared_ptr<Pipe>> acceptedPipe;
    plistener->accept([&](const Error& e, std::shared_ptr<Pipe> p) { acceptedPipe.set_value(e ? nullptr : std::move(p)); });
    auto cpipe = client->connect(url);
    auto spipe = acceptedPipe.get_future().get();
    CHECK(spipe != nullptr);
    if (spipe) {
      std::vector<uint8_t> tensor(3 << 20), landed;
      for (size_t i = 0; i < tensor.size(); ++i) {
        tensor[i] = static_cast<uint8_t>(i * 31 % 253);
      }
      std::string payload = "payload over tcp", payloadLanded;
      Message m;
      m.metadata = "over tcp";
      Message::Payload mp;
      mp.data = &payload[0];
      mp.length = payload.size();
      m.payloads.push_back(std::move(mp));
      Message::Tensor mt;
      mt.buffer = CpuBuffer{tensor.data()};
      mt.length = tensor.size();
      m.tensors.push_back(std::move(mt));
      std::promise<bool> wrote, readDone;
      spipe->readDescriptor([&](const Error& e, Descriptor d) {
        if (e || d.metadata != "over tcp" || d.payloads.size() != 1 || d.tensors.size() != 1) {
          readDone.set_value(false);
          return;
        }
        payloadLanded.resize(d.payloads[0].length);
        landed.resize(d.tensors[0].length);
        Allocation a;
        a.payloads.resize(1);
        a.payloads[0].data = &payloadLanded[0];
        a.tensors.resize(1);
        a.tensors[0].buffer = CpuBuffer{landed.data()};
        spipe->read(std::move(a), [&](const Error& e2) { readDone.set_value(!e2); });
      });
      cpipe->write(std::move(m), [&](const Error& e) { wrote.set_value(!e); });
      CHECK(readDone.get_future().get());
      CHECK(wrote.get_future().get());
      CHECK(payloadLanded == payload && landed == tensor);
    }
    cpipe.reset();
    spipe.reset();
    plistener.reset();
    client->join();
    server->join();
  }
  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}


// ---- on-demand loops ---------------------------------------------------------

namespace {

// Two threads meet here; returns false when the other one has not arrived
// within the time limit (the case then fails instead of hanging).
class Rendezvous {
 public:
  bool arrive(std::chrono::milliseconds limit = std::chrono::milliseconds(2000)) {
    std::unique_lock<std::mutex> lock(m_);
    const unsigned turn = turn_;
    if (++count_ == 2) {
      count_ = 0;
      ++turn_;
      cv_.notify_all();
      return true;
    }
    // wall-clock deadlines here and below: ThreadSanitizer follows pthread_cond_timedwait only
    return cv_.wait_until(lock, std::chrono::system_clock::now() + limit, [&] { return turn_ != turn; });
  }

 private:
  std::mutex m_;
  std::condition_variable cv_;
  unsigned count_{0};
  unsigned turn_{0};
};

// Ends the process when a case is stuck, naming it: a hung unit test tells
// nothing, a line and an exit code do.
class Watchdog {
 public:
  Watchdog(const char* what, int seconds) : what_(what) {
    thread_ = std::thread([this, seconds] {
      std::unique_lock<std::mutex> lock(m_);
      if (!cv_.wait_until(lock, std::chrono::system_clock::now() + std::chrono::seconds(seconds), [this] { return done_; })) {
        std::printf("TIMEOUT %s\n", what_);
        std::fflush(stdout);
        _exit(3);
      }
    });
  }
  ~Watchdog() {
    {
      std::unique_lock<std::mutex> lock(m_);
      done_ = true;
    }
    cv_.notify_all();
    thread_.join();
  }

 private:
  const char* what_;
  std::mutex m_;
  std::condition_variable cv_;
  bool done_{false};
  std::thread thread_;
};

bool waitFor(const std::function<bool()>& cond, int ms = 2000) {
  const auto until = std::chrono::steady_clock::now() + std::chrono::milliseconds(ms);
  while (!cond()) {
    if (std::chrono::steady_clock::now() > until) {
      return false;
    }
    std::this_thread::sleep_for(std::chrono::microseconds(50));
  }
  return true;
}

} // namespace

// The reference's transport suite (tensorpipe/test/transport/listener_test.cc,
// connection_test.cc, context_test.cc and shm/connection_test.cc), case by
// case, for a transport of this library: shm (own protocol), shm_stock (the
// reference's protocol) or tcp. One context per case, both ends in it, as the
// reference's ThreadPeerGroup does (tensorpipe/test/transport/transport_test.h:34-36).
namespace transport_suite {

struct Flavour {
  std::function<std::shared_ptr<transport::Context>()> make;
  std::string defaultAddr;
  size_t ringBytes; // what a connection buffers before a write has to wait (0: no such ring)
};

// A small object with libnop's face (tensorpipe/test/transport/connection_test.cc:86-93):
// four bytes of length and the characters.
struct TextHolder final : AbstractNopHolder {
  std::string text;
  size_t getSize() const override {
    return 4 + text.size();
  }
  void serialize(uint8_t* out, size_t size) const override {
    const uint32_t n = static_cast<uint32_t>(text.size());
    std::memcpy(out, &n, 4);
    std::memcpy(out + 4, text.data(), std::min(size - 4, text.size()));
  }
  bool deserialize(const uint8_t* in, size_t size) override {
    uint32_t n = 0;
    if (size < 4) {
      return false;
    }
    std::memcpy(&n, in, 4);
    if (size != 4 + static_cast<size_t>(n)) {
      return false;
    }
    text.assign(reinterpret_cast<const char*>(in + 4), n);
    return true;
  }
};

template <typename T>
bool ready(std::future<T>& f, int seconds = 30) {
  return f.wait_for(std::chrono::seconds(seconds)) == std::future_status::ready;
}

struct Pair {
  std::shared_ptr<transport::Connection> server, client;
};

static Pair connectPair(transport::Context& ctx, transport::Listener& listener) {
  auto p = std::make_shared<std::promise<std::shared_ptr<transport::Connection>>>();
  listener.accept([p](const Error& e, std::shared_ptr<transport::Connection> c) { p->set_value(e ? nullptr : std::move(c)); });
  Pair pair;
  pair.client = ctx.connect(listener.addr());
  auto f = p->get_future();
  if (ready(f)) {
    pair.server = f.get();
  }
  return pair;
}

static int run(const Flavour& flavour) {
  int failed = 0;
  // Context_Basics + Listener_Basics: the accept callback runs for a new connection.
  {
    Watchdog dog("Context_Basics", 60);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      Pair pair = connectPair(*ctx, *listener);
      CHECK(pair.server != nullptr);
    }
    ctx->join();
  }
  // Context_DomainDescriptor
  {
    Watchdog dog("Context_DomainDescriptor", 60);
    auto ctx = flavour.make();
    CHECK(!ctx->domainDescriptor().empty());
    ctx->join();
  }
  // Listener_AcceptCallbacksAreQueued / Listener_IncomingConnectionsAreQueued:
  // ten accepts and ten connections, whichever comes first; the callbacks fire
  // in the order they were given.
  for (int connectFirst = 0; connectFirst < 2; ++connectFirst) {
    Watchdog dog("Listener_*AreQueued", 60);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      std::atomic<int> accepts{0};
      std::atomic<bool> inOrder{true}, anyError{false};
      std::promise<void> done;
      std::vector<std::shared_ptr<transport::Connection>> conns, accepted(10);
      auto connectAll = [&] {
        for (int i = 0; i < 10; ++i) {
          conns.push_back(ctx->connect(listener->addr()));
        }
      };
      auto acceptAll = [&] {
        for (int i = 0; i < 10; ++i) {
          listener->accept([&, i](const Error& e, std::shared_ptr<transport::Connection> c) {
            if (e) {
              anyError = true;
            }
            if (accepts.load() != i) {
              inOrder = false;
            }
            accepted[i] = std::move(c);
            if (++accepts == 10) {
              done.set_value();
            }
          });
        }
      };
      if (connectFirst) {
        connectAll();
        acceptAll();
      } else {
        acceptAll();
        connectAll();
      }
      auto f = done.get_future();
      CHECK(ready(f));
      CHECK(inOrder.load() && !anyError.load());
    }
    ctx->join();
  }
  // Listener_CreateThenCloseAndThenGetAddress: a closed listener still says
  // where it was; an accept on it and a write towards it end, with or without
  // an error, and nothing hangs.
  {
    Watchdog dog("Listener_CreateThenCloseAndThenGetAddress", 60);
    auto ctx = flavour.make();
    auto listener = ctx->listen(flavour.defaultAddr);
    listener->close();
    const std::string addr = listener->addr();
    CHECK(!addr.empty());
    std::promise<void> acceptDone, writeDone;
    listener->accept([&](const Error&, std::shared_ptr<transport::Connection>) { acceptDone.set_value(); });
    auto conn = ctx->connect(addr);
    conn->write(nullptr, 0, [&](const Error&) { writeDone.set_value(); });
    auto fa = acceptDone.get_future();
    CHECK(ready(fa));
    conn->close(); // (a write into a ring nobody reads is allowed to wait for ever)
    auto fw = writeDone.get_future();
    CHECK(ready(fw));
    ctx->join();
  }
  // Listener_CreateAfterClosingContextAndThenGetAddress: the listener of a
  // closed context is born closed; everything asked of it ends.
  {
    Watchdog dog("Listener_CreateAfterClosingContextAndThenGetAddress", 60);
    auto ctx = flavour.make();
    ctx->close();
    auto listener = ctx->listen(flavour.defaultAddr);
    const std::string addr = listener->addr();
    std::promise<bool> acceptDone, writeDone;
    listener->accept([&](const Error& e, std::shared_ptr<transport::Connection>) { acceptDone.set_value(static_cast<bool>(e)); });
    auto conn = ctx->connect(addr);
    conn->write(nullptr, 0, [&](const Error& e) { writeDone.set_value(static_cast<bool>(e)); });
    auto fa = acceptDone.get_future();
    CHECK(ready(fa) && fa.get());
    auto fw = writeDone.get_future();
    CHECK(ready(fw) && fw.get());
    ctx->join();
  }
  // Connection_Initialization: thirteen bytes written are thirteen bytes read.
  {
    Watchdog dog("Connection_Initialization", 60);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      Pair pair = connectPair(*ctx, *listener);
      CHECK(pair.server != nullptr);
      if (pair.server) {
        char garbage[13] = {0};
        std::promise<size_t> got;
        std::promise<bool> wrote;
        pair.server->read([&](const Error& e, const void*, size_t len) { got.set_value(e ? size_t(-1) : len); });
        pair.client->write(garbage, sizeof(garbage), [&](const Error& e) { wrote.set_value(!e); });
        auto fg = got.get_future();
        auto fw = wrote.get_future();
        CHECK(ready(fg) && fg.get() == sizeof(garbage));
        CHECK(ready(fw) && fw.get());
      }
    }
    ctx->join();
  }
  // Connection_InitializationError: the server drops the connection at once;
  // each of ten reads on the client, one after the other, fails.
  {
    Watchdog dog("Connection_InitializationError", 60);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      Pair pair = connectPair(*ctx, *listener);
      CHECK(pair.server != nullptr);
      pair.server.reset();
      for (int i = 0; i < 10; ++i) {
        std::promise<bool> failedRead;
        pair.client->read([&](const Error& e, const void*, size_t) { failedRead.set_value(static_cast<bool>(e)); });
        auto f = failedRead.get_future();
        CHECK(ready(f) && f.get());
      }
    }
    ctx->join();
  }
  // Connection_NopWrite: an object written is the object read.
  {
    Watchdog dog("Connection_NopWrite", 60);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      Pair pair = connectPair(*ctx, *listener);
      CHECK(pair.server != nullptr);
      if (pair.server) {
        auto in = std::make_shared<TextHolder>();
        auto out = std::make_shared<TextHolder>();
        out->text = std::string(0x42, 'n');
        std::promise<bool> got, wrote;
        pair.server->read(*in, [&, in](const Error& e) { got.set_value(!e && in->text == std::string(0x42, 'n')); });
        pair.client->write(*out, [&, out](const Error& e) { wrote.set_value(!e); });
        auto fg = got.get_future();
        auto fw = wrote.get_future();
        CHECK(ready(fg) && fg.get());
        CHECK(ready(fw) && fw.get());
      }
    }
    ctx->join();
  }
  // Connection_QueueWritesBeforeReads: ten 16 KiB messages are all written
  // (their callbacks have fired) before the first read is posted; the reads
  // then find them in order.
  {
    Watchdog dog("Connection_QueueWritesBeforeReads", 60);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      Pair pair = connectPair(*ctx, *listener);
      CHECK(pair.server != nullptr);
      if (pair.server) {
        constexpr int kMessages = 10;
        std::vector<std::string> msg;
        for (int i = 0; i < kMessages; ++i) {
          msg.emplace_back(16 * 1024, static_cast<char>(i));
        }
        std::promise<bool> wroteAll;
        std::atomic<bool> writesFine{true};
        for (int i = 0; i < kMessages; ++i) {
          pair.server->write(msg[i].data(), msg[i].size(), [&, i](const Error& e) {
            if (e) {
              writesFine = false;
            }
            if (i == kMessages - 1) {
              wroteAll.set_value(writesFine.load());
            }
          });
        }
        auto fw = wroteAll.get_future();
        CHECK(ready(fw) && fw.get());
        std::promise<bool> readAll;
        std::atomic<bool> readsFine{true};
        for (int i = 0; i < kMessages; ++i) {
          pair.client->read([&, i](const Error& e, const void* ptr, size_t len) {
            if (e || len != msg[i].size() || std::memcmp(ptr, msg[i].data(), len) != 0) {
              readsFine = false;
            }
            if (i == kMessages - 1) {
              readAll.set_value(readsFine.load());
            }
          });
        }
        auto fr = readAll.get_future();
        CHECK(ready(fr) && fr.get());
      }
    }
    ctx->join();
  }
  // Chunking / ChunkingImplicitRead (shm/connection_test.cc:29-96): a message
  // five times the ring, into the caller's buffer and into the transport's.
  // For tcp the same sizes stand for "much more than a socket buffer".
  for (int implicit = 0; implicit < 2; ++implicit) {
    Watchdog dog("Chunking", 120);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      Pair pair = connectPair(*ctx, *listener);
      CHECK(pair.server != nullptr);
      if (pair.server) {
        const size_t bytes = 5 * (flavour.ringBytes != 0 ? flavour.ringBytes : (2u << 20));
        std::string src(bytes, 0x42);
        for (size_t i = 0; i < bytes; i += 4099) {
          src[i] = static_cast<char>(i / 4099);
        }
        std::vector<char> dst(implicit ? 0 : bytes);
        std::promise<bool> got, wrote;
        auto check = [&](const Error& e, const void* ptr, size_t len) {
          got.set_value(!e && len == bytes && (implicit || ptr == dst.data()) && std::memcmp(ptr, src.data(), bytes) == 0);
        };
        if (implicit) {
          pair.server->read(check);
        } else {
          pair.server->read(dst.data(), bytes, check);
        }
        pair.client->write(src.data(), bytes, [&](const Error& e) { wrote.set_value(!e); });
        auto fg = got.get_future();
        auto fw = wrote.get_future();
        CHECK(ready(fg, 60) && fg.get());
        CHECK(ready(fw, 60) && fw.get());
      }
    }
    ctx->join();
  }
  // QueueWrites (shm/connection_test.cc:98-141): two messages of three
  // quarters of the ring are queued before anything is read; the second
  // cannot fit until the first has been taken out.
  // NopWriteWrapAround (:152-185): the same with objects, whose bytes wrap
  // around the end of the ring.
  for (int objects = 0; objects < 2; ++objects) {
    Watchdog dog("QueueWrites / NopWriteWrapAround", 120);
    auto ctx = flavour.make();
    {
      auto listener = ctx->listen(flavour.defaultAddr);
      Pair pair = connectPair(*ctx, *listener);
      CHECK(pair.server != nullptr);
      if (pair.server) {
        const size_t bytes = 3 * (flavour.ringBytes != 0 ? flavour.ringBytes : (2u << 20)) / 4;
        std::vector<std::shared_ptr<TextHolder>> outs, ins;
        std::vector<std::string> raw;
        for (int i = 0; i < 2; ++i) {
          raw.emplace_back(bytes, static_cast<char>('B' + i));
          outs.push_back(std::make_shared<TextHolder>());
          outs.back()->text = raw.back();
          ins.push_back(std::make_shared<TextHolder>());
        }
        std::atomic<int> written{0}, readOk{0}, anyError{0};
        for (int i = 0; i < 2; ++i) {
          auto done = [&](const Error& e) {
            if (e) {
              ++anyError;
            }
            ++written;
          };
          if (objects) {
            pair.client->write(*outs[i], done);
          } else {
            pair.client->write(raw[i].data(), bytes, done);
          }
        }
        std::this_thread::sleep_for(std::chrono::milliseconds(50)); // the writes are queued, the second one stuck
        for (int i = 0; i < 2; ++i) {
          if (objects) {
            pair.server->read(*ins[i], [&, i](const Error& e) {
              if (!e && ins[i]->text == raw[i]) {
                ++readOk;
              }
            });
          } else {
            pair.server->read([&, i](const Error& e, const void* ptr, size_t len) {
              if (!e && len == bytes && std::memcmp(ptr, raw[i].data(), bytes) == 0) {
                ++readOk;
              }
            });
          }
        }
        CHECK(waitFor([&] { return readOk.load() == 2 && written.load() == 2; }, 60000));
        CHECK(anyError.load() == 0);
      }
    }
    ctx->join();
  }
  return failed;
}

} // namespace transport_suite

static int runTransportSuite(const std::string& which) {
  transport_suite::Flavour flavour;
  const std::string unique = "tp_amd_suite_" + std::to_string(::getpid());
  if (which == "shm") {
    flavour = {[] { return transport::shm::create(); }, "", 0};
  } else if (which == "shm_stock") {
    flavour = {[] { return transport::shm_stock::create(); }, "", 2u << 20};
  } else if (which == "tcp") {
    flavour = {[] { return transport::tcp::create(); }, "127.0.0.1", 0};
  } else {
    return 2;
  }
  const int failed = transport_suite::run(flavour);
  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}

static int runLoops() {
  int failed = 0;
  // 1. Thread A sits in a task of loop one and defers to loop two while thread
  // B sits in a task of loop two and defers to loop one. Neither is a thread
  // of the library. Both defer() calls must return, and both tasks must run.
  {
    Watchdog dog("crossed defers of two application threads", 5);
    OnDemandLoop one, two;
    Rendezvous inside, leaving;
    std::atomic<int> ran{0};
    bool metA = false, metB = false;
    std::thread a([&] {
      one.defer([&] {
        metA = inside.arrive();
        two.defer([&] { ++ran; });
        leaving.arrive();
      });
    });
    std::thread b([&] {
      two.defer([&] {
        metB = inside.arrive();
        one.defer([&] { ++ran; });
        leaving.arrive();
      });
    });
    a.join();
    b.join();
    CHECK(metA && metB);
    CHECK(waitFor([&] { return ran.load() == 2; }));
  }
  // 2. A caller that holds a lock while it calls defer() gets out again although
  // the thread that drains the loop is blocked, inside its own task, on that lock.
  {
    Watchdog dog("defer() with a lock held that the draining task wants", 5);
    OnDemandLoop loop;
    std::mutex userLock;
    Rendezvous drainerInside;
    std::atomic<int> ran{0};
    std::thread drainer([&] {
      loop.defer([&] {
        drainerInside.arrive();
        std::this_thread::sleep_for(std::chrono::milliseconds(20));
        std::lock_guard<std::mutex> g(userLock); // what a user's callback may do
        ++ran;
      });
    });
    std::thread caller([&] {
      std::lock_guard<std::mutex> g(userLock);
      drainerInside.arrive();
      loop.defer([&] { ++ran; }); // must come back while the drainer wants userLock
    });
    caller.join();
    drainer.join();
    CHECK(waitFor([&] { return ran.load() == 2; }));
  }
  // 3. What another thread queues while an application thread drains the loop is
  // not run on the application thread's stack (its own call is still on it),
  // and is run all the same -- whether the other thread is the library's or not,
  // inside a task of another loop or not.
  for (int variant = 0; variant < 3; ++variant) {
    Watchdog dog("a task queued beside a draining application thread", 5);
    OnDemandLoop loop, other;
    Rendezvous inside, queued;
    std::atomic<int> ran{0};
    std::thread::id ranOn;
    std::thread::id appId;
    std::thread app([&] {
      appId = std::this_thread::get_id();
      loop.defer([&] {
        inside.arrive();
        queued.arrive(std::chrono::milliseconds(300)); // a waiting library thread never gets here: fine
        std::this_thread::sleep_for(std::chrono::milliseconds(2));
      });
    });
    std::thread foreign([&] {
      thisIsLibraryThread() = (variant == 1);
      auto post = [&] {
        loop.defer([&] {
          ranOn = std::this_thread::get_id();
          ++ran;
        });
        queued.arrive(std::chrono::milliseconds(300));
      };
      inside.arrive();
      if (variant == 2) {
        other.defer(post);
      } else {
        post();
      }
    });
    app.join();
    foreign.join();
    CHECK(waitFor([&] { return ran.load() == 1; }));
    CHECK(ranOn != appId);
  }
  // 4. Many threads, two loops, tasks that hop between them: each runs once, and
  // the tasks one thread queued on one loop run in the order it queued them.
  {
    Watchdog dog("tasks from many threads over two loops", 30);
    OnDemandLoop loops[2];
    constexpr int kThreads = 6, kPerThread = 3000;
    std::atomic<int> ran{0};
    std::atomic<int> concurrent[2] = {{0}, {0}};
    std::atomic<bool> overlapped{false}, disorder{false};
    std::vector<std::vector<int>> seen(kThreads * 2);
    std::vector<std::thread> threads;
    for (int t = 0; t < kThreads; ++t) {
      threads.emplace_back([&, t] {
        thisIsLibraryThread() = (t % 3 == 0);
        for (int i = 0; i < kPerThread; ++i) {
          const int first = (t + i) & 1;
          loops[first].defer([&, t, i, first] {
            if (concurrent[first].fetch_add(1) != 0) {
              overlapped = true;
            }
            seen[t * 2 + first].push_back(i);
            concurrent[first].fetch_sub(1);
            loops[1 - first].defer([&, first] {
              if (concurrent[1 - first].fetch_add(1) != 0) {
                overlapped = true;
              }
              ++ran;
              concurrent[1 - first].fetch_sub(1);
            });
          });
        }
      });
    }
    for (auto& th : threads) {
      th.join();
    }
    CHECK(waitFor([&] { return ran.load() == kThreads * kPerThread; }, 20000));
    CHECK(!overlapped.load());
    for (auto& v : seen) {
      for (size_t k = 1; k < v.size(); ++k) {
        if (v[k] <= v[k - 1]) {
          disorder = true;
        }
      }
    }
    CHECK(!disorder.load());
  }
  // 5. A loop is destroyed right after an application thread left it with
  // another thread's task still queued.
  for (int round = 0; round < 200; ++round) {
    Watchdog dog("a loop destroyed with a helper on its way", 10);
    auto loop = std::make_unique<OnDemandLoop>();
    Rendezvous inside;
    std::atomic<int> ran{0};
    std::thread app([&] {
      loop->defer([&] {
        inside.arrive();
        std::this_thread::sleep_for(std::chrono::microseconds(100));
      });
    });
    std::thread foreign([&] {
      inside.arrive();
      loop->defer([&] { ++ran; });
    });
    app.join();
    foreign.join();
    CHECK(waitFor([&] { return ran.load() == 1; }));
    loop.reset();
  }
  // 6. The last pointer to a loop's owner is held by a task of that loop, and a
  // helper runs it: the owner, loop included, is destroyed from inside the
  // loop's own task (a context whose last holder is a callback of one of its
  // listeners). The helper must come out of it, and the loop's bookkeeping
  // must outlive the owner for as long as the helper is in it.
  for (int round = 0; round < 50; ++round) {
    Watchdog dog("a loop destroyed by one of its own tasks on a helper", 10);
    struct Owner {
      OnDemandLoop loop;
      std::atomic<int>* gone;
      ~Owner() {
        ++*gone;
      }
    };
    std::atomic<int> gone{0}, ran{0};
    auto owner = std::make_shared<Owner>();
    owner->gone = &gone;
    Owner* raw = owner.get();
    Rendezvous inside, queued;
    std::thread foreign([&, last = std::move(owner)]() mutable {
      inside.arrive();
      raw->loop.defer([&ran, last = std::move(last)] { ++ran; }); // an application thread drains: comes back at once
      queued.arrive();
    });
    raw->loop.defer([&] {
      inside.arrive();
      queued.arrive();
    });
    foreign.join();
    CHECK(waitFor([&] { return ran.load() == 1 && gone.load() == 1; }));
  }
  if (failed == 0) {
    std::printf("OK\n");
  }
  return failed == 0 ? 0 : 1;
}

static void onFatalSignal(int sig) {
  void* frames[48];
  const int n = backtrace(frames, 48);
  const char msg[] = "fatal signal, stack:\n";
  (void)!write(2, msg, sizeof(msg) - 1);
  backtrace_symbols_fd(frames, n, 2);
  signal(sig, SIG_DFL);
  raise(sig);
}

int main(int argc, char** argv) {
  signal(SIGSEGV, onFatalSignal);
  signal(SIGABRT, onFatalSignal);
  if (argc == 4 && std::strcmp(argv[1], "garbage") == 0) {
    return runGarbage(argc, argv);
  }
  if (argc >= 3 && std::strcmp(argv[1], "allocator") == 0) {
    return runAllocator(argc, argv);
  }
  if (argc == 2 && std::strcmp(argv[1], "basics") == 0) {
    return runBasics();
  }
  if (argc == 2 && std::strcmp(argv[1], "departed_peer") == 0) {
    return runDepartedPeer();
  }
  if (argc >= 2 && std::strcmp(argv[1], "pointers") == 0) {
    return runPointers(argc == 3 && std::strcmp(argv[2], "map_over") == 0);
  }
  if (argc == 3 && std::strcmp(argv[1], "nop_wire") == 0) {
    return runNopWire(argv[2]);
  }
  if (argc == 2 && std::strcmp(argv[1], "compat_pipe") == 0) {
    return runCompatPipe();
  }
  if (argc == 2 && std::strcmp(argv[1], "shm_stock") == 0) {
    return runShmStock();
  }
  if (argc == 2 && std::strcmp(argv[1], "shm_stock_hostile_peer") == 0) {
    return runShmStockHostilePeer();
  }
  if (argc == 3 && std::strcmp(argv[1], "transport_suite") == 0) {
    return runTransportSuite(argv[2]);
  }
  if (argc == 2 && std::strcmp(argv[1], "tcp") == 0) {
    return runTcp();
  }
  if (argc == 2 && std::strcmp(argv[1], "loops") == 0) {
    return runLoops();
  }
  std::fprintf(stderr, "usage: %s allocator <slots> <events...> | basics | departed_peer | pointers | garbage <seed> <n> | nop_wire <vectors> | compat_pipe | tcp | shm_stock | shm_stock_hostile_peer | transport_suite shm|shm_stock|tcp | loops\n", argv[0]);
  return 2;
}
