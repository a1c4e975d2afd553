// The wire encodings of nopwire/ against the real thing: a tpnop::CompatPipe on
// one end, an unmodified TensorPipe endpoint (the build inside PyTorch's
// libtorch_cpu.so: its Context, Pipe, uv transport and basic channel) on the
// other, in one process, talking over TCP on 127.0.0.1. Both roles (the compat
// end connects to a stock listener; a stock context connects to a compat
// listener), messages both ways with payloads, CPU tensors with and without a
// target device named by the sender, an empty tensor and metadata everywhere.
//
//   stock_wire_interop run                 prints one RESULT line per case
//   stock_wire_interop capture <file>      also writes the frames the STOCK end produced
//                                          (name, hex) -- how tests/golden/stock_wire_vectors.txt was made
//
// The same two roles once more with this library's own asynchronous pipe on the
// compat side: a context in stock wire format (ContextOptions::stockWireFormat)
// over its TCP transport registered as "uv", driven through the C harness API
// because its C++ headers share their names with the stock ones.
//
// No GPU involved.
#include <tensorpipe/tensorpipe.h> // the stock headers: listed first on the include path

#include <cstdio>
#include <unistd.h>
#include <cstring>
#include <future>
#include <map>
#include <string>
#include <vector>

#include <nopwire/compat_pipe.h>
#include <tensorpipe_c.h>

using namespace tensorpipe;

namespace {

// withShm: the stock end also holds its shm transport and prefers it. The native
// end's transport of that name does not speak the stock one's protocol and says
// so in its domain descriptor, so a pipe between the two must stay on "uv".
std::shared_ptr<Context> stockContext(const char* name, bool withShm = false) {
  auto ctx = std::make_shared<Context>(ContextOptions().name(name));
  ctx->registerTransport(0, "uv", transport::uv::create());
  if (withShm) {
    ctx->registerTransport(1, "shm", transport::shm::create());
  }
  ctx->registerChannel(0, "basic", channel::basic::create());
  return ctx;
}

std::string pattern(size_t n, int salt) {
  std::string s(n, '\0');
  for (size_t i = 0; i < n; ++i) {
    s[i] = static_cast<char>((i * 31 + (i >> 8) * 7 + static_cast<size_t>(salt) * 13) % 251);
  }
  return s;
}

// The message every case sends: two payloads (one empty), three tensors.
tpnop::CompatMessage testMessage(int salt) {
  tpnop::CompatMessage m;
  m.metadata = "message metadata " + std::to_string(salt);
  m.payloads.push_back({pattern(300, salt), "first payload"});
  m.payloads.push_back({"", ""});
  m.tensors.push_back({pattern(70001, salt + 1), "named target", true});
  m.tensors.push_back({pattern(129, salt + 2), "", false});
  m.tensors.push_back({"", "empty", true});
  return m;
}

std::string compare(const tpnop::CompatMessage& got, const tpnop::CompatMessage& want) {
  if (got.metadata != want.metadata) {
    return "metadata differs";
  }
  if (got.payloads.size() != want.payloads.size() || got.tensors.size() != want.tensors.size()) {
    return "payload or tensor count differs";
  }
  for (size_t i = 0; i < want.payloads.size(); ++i) {
    if (got.payloads[i].bytes != want.payloads[i].bytes || got.payloads[i].metadata != want.payloads[i].metadata) {
      return "payload " + std::to_string(i) + " differs";
    }
  }
  for (size_t i = 0; i < want.tensors.size(); ++i) {
    if (got.tensors[i].bytes != want.tensors[i].bytes || got.tensors[i].metadata != want.tensors[i].metadata) {
      return "tensor " + std::to_string(i) + " differs";
    }
  }
  return "";
}

// The stock end writes `m` and waits for its callback. The buffers live in `m`.
std::string stockWrite(Pipe& pipe, const tpnop::CompatMessage& m) {
  Message out;
  out.metadata = m.metadata;
  for (auto& p : m.payloads) {
    Message::Payload sp;
    sp.data = const_cast<char*>(p.bytes.data());
    sp.length = p.bytes.size();
    sp.metadata = p.metadata;
    out.payloads.push_back(std::move(sp));
  }
  for (auto& t : m.tensors) {
    Message::Tensor st;
    st.buffer = CpuBuffer{const_cast<char*>(t.bytes.data())};
    st.length = t.bytes.size();
    st.metadata = t.metadata;
    if (t.nameTarget) {
      st.targetDevice = Device{kCpuDeviceType, 0};
    }
    out.tensors.push_back(std::move(st));
  }
  auto done = std::make_shared<std::promise<std::string>>();
  pipe.write(std::move(out), [done](const Error& e) { done->set_value(e ? e.what() : std::string()); });
  auto f = done->get_future();
  if (f.wait_for(std::chrono::seconds(30)) != std::future_status::ready) {
    return "the stock write never completed";
  }
  return f.get();
}

// The stock end reads one message into `got`.
std::string stockRead(Pipe& pipe, tpnop::CompatMessage* got) {
  auto done = std::make_shared<std::promise<std::string>>();
  pipe.readDescriptor([&pipe, got, done](const Error& e, Descriptor d) {
    if (e) {
      done->set_value("readDescriptor: " + e.what());
      return;
    }
    got->metadata = d.metadata;
    got->payloads.resize(d.payloads.size());
    got->tensors.resize(d.tensors.size());
    Allocation a;
    a.payloads.resize(d.payloads.size());
    a.tensors.resize(d.tensors.size());
    for (size_t i = 0; i < d.payloads.size(); ++i) {
      got->payloads[i].metadata = d.payloads[i].metadata;
      got->payloads[i].bytes.assign(d.payloads[i].length, '\0');
      a.payloads[i].data = &got->payloads[i].bytes[0];
    }
    for (size_t i = 0; i < d.tensors.size(); ++i) {
      if (d.tensors[i].sourceDevice.type != kCpuDeviceType) {
        done->set_value("a tensor announced on " + d.tensors[i].sourceDevice.type);
        return;
      }
      got->tensors[i].metadata = d.tensors[i].metadata;
      got->tensors[i].nameTarget = d.tensors[i].targetDevice.has_value();
      got->tensors[i].bytes.assign(d.tensors[i].length, '\0');
      a.tensors[i].buffer = CpuBuffer{&got->tensors[i].bytes[0]};
    }
    pipe.read(std::move(a), [done](const Error& e2) { done->set_value(e2 ? "read: " + e2.what() : std::string()); });
  });
  auto f = done->get_future();
  if (f.wait_for(std::chrono::seconds(30)) != std::future_status::ready) {
    return "the stock read never completed";
  }
  return f.get();
}

std::map<std::string, tpnop::Bytes> captured;

// Frames the stock end produced, as the compat end read them, by kind.
void keepStockFrames(const tpnop::CompatPipe& pipe, const std::string& role) {
  size_t descriptors = 0, replies = 0;
  for (auto& f : pipe.frames()) {
    if (f.direction != 'r' || f.bytes.empty()) {
      continue;
    }
    const uint8_t first = f.bytes[0];
    if (first == 0xb8) {
      tpnop::Packet p;
      if (tpnop::decode(f.bytes.data(), f.bytes.size(), &p)) {
        captured[role + (p.which == 0 ? ".spontaneous_connection" : std::string(".requested_connection_") + f.connection)] = f.bytes;
      }
    } else if (first == 0xb9 && f.connection == 'd') {
      tpnop::Brochure b;
      tpnop::BrochureAnswer a;
      tpnop::Descriptor d;
      if (f.bytes.size() > 1 && f.bytes[1] == 2 && tpnop::decode(f.bytes.data(), f.bytes.size(), &b)) {
        captured[role + ".brochure"] = f.bytes;
      } else if (f.bytes[1] == 7 && tpnop::decode(f.bytes.data(), f.bytes.size(), &a)) {
        captured[role + ".brochure_answer"] = f.bytes;
      } else if (f.bytes[1] == 3 && tpnop::decode(f.bytes.data(), f.bytes.size(), &d)) {
        captured[role + ".descriptor_" + std::to_string(descriptors++)] = f.bytes;
      }
    } else if (first == 0xb9 && f.connection == 'r') {
      captured[role + ".descriptor_reply_" + std::to_string(replies++)] = f.bytes;
    }
  }
}

void report(const std::string& name, const std::string& problem) {
  if (problem.empty()) {
    std::printf("RESULT %s OK\n", name.c_str());
  } else {
    std::printf("RESULT %s FAIL %s\n", name.c_str(), problem.c_str());
  }
  std::fflush(stdout);
}

// Messages both ways over an established pair.
std::string exchange(tpnop::CompatPipe& compat, Pipe& stock, int salt) {
  std::string error;
  // compat -> stock
  const tpnop::CompatMessage sent = testMessage(salt);
  tpnop::CompatMessage got;
  auto reading = std::async(std::launch::async, [&] { return stockRead(stock, &got); });
  if (!compat.write(sent, &error)) {
    return "compat write: " + error;
  }
  std::string problem = reading.get();
  if (problem.empty()) {
    problem = compare(got, sent);
  }
  if (!problem.empty()) {
    return "compat -> stock: " + problem;
  }
  // stock -> compat
  const tpnop::CompatMessage back = testMessage(salt + 100);
  auto writing = std::async(std::launch::async, [&] { return stockWrite(stock, back); });
  tpnop::CompatMessage got2;
  if (!compat.read(&got2, &error)) {
    return "compat read: " + error;
  }
  problem = writing.get();
  if (problem.empty()) {
    problem = compare(got2, back);
  }
  return problem.empty() ? "" : "stock -> compat: " + problem;
}

int compatConnectsToStock() {
  auto ctx = stockContext("stock_server");
  auto listener = ctx->listen({"uv://127.0.0.1"});
  const std::string url = listener->url("uv");
  auto accepted = std::make_shared<std::promise<std::shared_ptr<Pipe>>>();
  listener->accept([accepted](const Error& e, std::shared_ptr<Pipe> p) { accepted->set_value(e ? nullptr : p); });
  std::string error;
  auto compat = tpnop::CompatPipe::connect(url.substr(std::strlen("uv://")), "compat_client", &error);
  std::string problem;
  std::shared_ptr<Pipe> stock;
  if (!compat) {
    problem = "connect: " + error;
  } else {
    auto f = accepted->get_future();
    if (f.wait_for(std::chrono::seconds(30)) != std::future_status::ready || !(stock = f.get())) {
      problem = "the stock listener did not hand out a pipe";
    }
  }
  if (problem.empty() && stock->getRemoteName() != "compat_client") {
    problem = "the stock end heard the name " + stock->getRemoteName();
  }
  for (int round = 0; round < 3 && problem.empty(); ++round) {
    problem = exchange(*compat, *stock, round);
  }
  if (compat) {
    keepStockFrames(*compat, "stock_server");
  }
  report("compat_client_with_stock_server", problem);
  stock.reset();
  compat.reset();
  listener.reset();
  ctx->join();
  return problem.empty() ? 0 : 1;
}

int stockConnectsToCompat() {
  std::string error;
  auto listener = tpnop::CompatListener::create(&error);
  if (!listener) {
    report("stock_client_with_compat_server", "listen: " + error);
    return 1;
  }
  auto ctx = stockContext("stock_client");
  auto stock = ctx->connect("uv://" + listener->address());
  auto compat = listener->accept("compat_server", &error);
  std::string problem;
  if (!compat) {
    problem = "accept: " + error;
  } else if (compat->remoteName() != "stock_client") {
    problem = "the compat end heard the name " + compat->remoteName();
  }
  for (int round = 0; round < 3 && problem.empty(); ++round) {
    problem = exchange(*compat, *stock, 10 + round);
  }
  if (compat) {
    keepStockFrames(*compat, "stock_client");
  }
  report("stock_client_with_compat_server", problem);
  stock.reset();
  compat.reset();
  ctx->join();
  return problem.empty() ? 0 : 1;
}

// ---- this library's pipe in stock wire format ---------------------------------

// Writes `m` on the native pipe and waits for the callback.
std::string nativeWrite(tpc_pipe* pipe, const tpnop::CompatMessage& m) {
  std::vector<tpc_payload> payloads;
  std::vector<tpc_tensor> tensors;
  for (auto& p : m.payloads) {
    payloads.push_back(tpc_payload{const_cast<char*>(p.bytes.data()), p.bytes.size()});
  }
  for (auto& t : m.tensors) {
    tpc_tensor ct{};
    ct.ptr = const_cast<char*>(t.bytes.data());
    ct.length = t.bytes.size();
    ct.device_type = TPC_DEVICE_CPU;
    ct.target_type = t.nameTarget ? TPC_DEVICE_CPU : TPC_NO_TARGET;
    ct.target_index = 0;
    tensors.push_back(ct);
  }
  tpc_op* op = tpc_write_async(pipe, m.metadata.c_str(), payloads.data(), static_cast<uint32_t>(payloads.size()),
                               tensors.data(), static_cast<uint32_t>(tensors.size()));
  if (op == nullptr) {
    return std::string("native write: ") + tpc_last_error();
  }
  return tpc_op_wait(op, 30000) == 0 ? "" : std::string("native write: ") + tpc_last_error();
}

// Reads one message on the native pipe (lengths and bytes; the C API does not
// hand out per-item metadata).
std::string nativeRead(tpc_pipe* pipe, tpnop::CompatMessage* got) {
  auto d = std::make_unique<tpc_descriptor>();
  if (tpc_read_descriptor(pipe, d.get(), 30000) != 0) {
    return std::string("native readDescriptor: ") + tpc_last_error();
  }
  got->metadata = d->metadata;
  got->payloads.resize(d->num_payloads);
  got->tensors.resize(d->num_tensors);
  std::vector<void*> payloadPtrs;
  std::vector<tpc_tensor> tensors;
  for (uint32_t i = 0; i < d->num_payloads; ++i) {
    got->payloads[i].bytes.assign(d->payload_lengths[i], '\0');
    payloadPtrs.push_back(&got->payloads[i].bytes[0]);
  }
  for (uint32_t i = 0; i < d->num_tensors; ++i) {
    if (d->tensor_source_type[i] != TPC_DEVICE_CPU) {
      return "a tensor announced on another device type";
    }
    got->tensors[i].bytes.assign(d->tensor_lengths[i], '\0');
    got->tensors[i].nameTarget = d->tensor_target_type[i] != TPC_NO_TARGET;
    tpc_tensor ct{};
    ct.ptr = &got->tensors[i].bytes[0];
    ct.length = d->tensor_lengths[i];
    ct.device_type = TPC_DEVICE_CPU;
    ct.target_type = TPC_NO_TARGET;
    tensors.push_back(ct);
  }
  tpc_op* op = tpc_read_async(pipe, payloadPtrs.data(), d->num_payloads, tensors.data(), d->num_tensors);
  if (op == nullptr) {
    return std::string("native read: ") + tpc_last_error();
  }
  return tpc_op_wait(op, 30000) == 0 ? "" : std::string("native read: ") + tpc_last_error();
}

std::string compareBytes(const tpnop::CompatMessage& got, const tpnop::CompatMessage& want, bool itemMetadata) {
  if (got.metadata != want.metadata || got.payloads.size() != want.payloads.size() ||
      got.tensors.size() != want.tensors.size()) {
    return "metadata or counts differ";
  }
  for (size_t i = 0; i < want.payloads.size(); ++i) {
    if (got.payloads[i].bytes != want.payloads[i].bytes ||
        (itemMetadata && got.payloads[i].metadata != want.payloads[i].metadata)) {
      return "payload " + std::to_string(i) + " differs";
    }
  }
  for (size_t i = 0; i < want.tensors.size(); ++i) {
    if (got.tensors[i].bytes != want.tensors[i].bytes || got.tensors[i].nameTarget != want.tensors[i].nameTarget ||
        (itemMetadata && got.tensors[i].metadata != want.tensors[i].metadata)) {
      return "tensor " + std::to_string(i) + " differs";
    }
  }
  return "";
}

// The C API sends no per-item metadata: the message without it.
tpnop::CompatMessage plain(tpnop::CompatMessage m) {
  for (auto& p : m.payloads) {
    p.metadata.clear();
  }
  for (auto& t : m.tensors) {
    t.metadata.clear();
  }
  return m;
}

std::string nativeExchange(tpc_pipe* native, Pipe& stock, int salt) {
  for (int round = 0; round < 3; ++round) {
    // native -> stock
    const tpnop::CompatMessage sent = plain(testMessage(salt + round));
    tpnop::CompatMessage got;
    auto reading = std::async(std::launch::async, [&] { return stockRead(stock, &got); });
    std::string problem = nativeWrite(native, sent);
    const std::string r = reading.get();
    if (problem.empty()) {
      problem = r.empty() ? compareBytes(got, sent, true) : r;
    }
    if (!problem.empty()) {
      return "native -> stock: " + problem;
    }
    // stock -> native
    const tpnop::CompatMessage back = testMessage(salt + round + 50);
    tpnop::CompatMessage got2;
    auto writing = std::async(std::launch::async, [&] { return stockWrite(stock, back); });
    problem = nativeRead(native, &got2);
    const std::string w = writing.get();
    if (problem.empty()) {
      problem = w.empty() ? compareBytes(got2, back, false) : w;
    }
    if (!problem.empty()) {
      return "stock -> native: " + problem;
    }
  }
  return "";
}

std::string runsOn(tpc_pipe* pipe, const std::string& expected) {
  char transport[64] = {0};
  if (tpc_pipe_transport(pipe, transport, sizeof(transport)) != 0 || std::string(transport) != expected) {
    return std::string("the native end runs on transport \"") + transport + "\", not on " + expected;
  }
  return "";
}

// What the native end holds beside uv: nothing, this library's own shm transport
// (another protocol under the same name: the pipe must stay on uv), or the
// transport that speaks the stock shm protocol (the pipe must move there, in
// both roles: tensorpipe/core/pipe_impl.cc:987-1042,1108-1125).
enum class NativeShm { kNone, kOwnProtocol, kStockProtocol };

const char* nativeTransports(NativeShm shm) {
  return shm == NativeShm::kNone ? "uv:0" : shm == NativeShm::kOwnProtocol ? "uv:0,shm:1" : "uv:0,shm_stock:1";
}
std::string caseSuffix(NativeShm shm) {
  return shm == NativeShm::kNone ? "" : shm == NativeShm::kOwnProtocol ? "_both_hold_shm" : "_moves_to_shm";
}

int nativeConnectsToStock(NativeShm shm) {
  const bool withShm = shm != NativeShm::kNone;
  auto ctx = stockContext("stock_server", withShm);
  auto listener = withShm ? ctx->listen({"uv://127.0.0.1", "shm://stock_wire_interop_" + std::to_string(::getpid())})
                          : ctx->listen({"uv://127.0.0.1"});
  auto accepted = std::make_shared<std::promise<std::shared_ptr<Pipe>>>();
  listener->accept([accepted](const Error& e, std::shared_ptr<Pipe> p) { accepted->set_value(e ? nullptr : p); });
  tpc_context* native = tpc_context_create_ex("native_client", nativeTransports(shm), "basic:0", 1);
  tpc_pipe* pipe = native != nullptr ? tpc_connect(native, listener->url("uv").c_str()) : nullptr;
  std::string problem;
  std::shared_ptr<Pipe> stock;
  if (pipe == nullptr) {
    problem = std::string("native connect: ") + tpc_last_error();
  } else {
    auto f = accepted->get_future();
    if (f.wait_for(std::chrono::seconds(30)) != std::future_status::ready || !(stock = f.get())) {
      problem = "the stock listener did not hand out a pipe";
    }
  }
  if (problem.empty() && stock->getRemoteName() != "native_client") {
    problem = "the stock end heard the name " + stock->getRemoteName();
  }
  if (problem.empty()) {
    problem = nativeExchange(pipe, *stock, 200);
  }
  if (problem.empty()) {
    problem = runsOn(pipe, shm == NativeShm::kStockProtocol ? "shm" : "uv");
  }
  report("native_client_with_stock_server" + caseSuffix(shm), problem);
  stock.reset();
  if (pipe != nullptr) {
    tpc_pipe_destroy(pipe);
  }
  if (native != nullptr) {
    tpc_context_destroy(native);
  }
  listener.reset();
  ctx->join();
  return problem.empty() ? 0 : 1;
}

int stockConnectsToNative(NativeShm shm) {
  const bool withShm = shm != NativeShm::kNone;
  const std::string caseName = "stock_client_with_native_server" + caseSuffix(shm);
  tpc_context* native = tpc_context_create_ex("native_server", nativeTransports(shm), "basic:0", 1);
  tpc_listener* listener =
      native != nullptr ? tpc_listen(native, withShm ? "uv://127.0.0.1,shm://" : "uv://127.0.0.1") : nullptr;
  char url[256] = {0};
  std::string problem;
  if (listener == nullptr || tpc_listener_url(listener, "uv", url, sizeof(url)) != 0) {
    problem = std::string("native listen: ") + tpc_last_error();
    report(caseName, problem);
    return 1;
  }
  auto ctx = stockContext("stock_client", withShm);
  auto stock = ctx->connect(url);
  tpc_pipe* pipe = tpc_accept(listener, 30000);
  char name[256] = {0};
  if (pipe == nullptr) {
    problem = std::string("native accept: ") + tpc_last_error();
  } else if (tpc_pipe_remote_name(pipe, name, sizeof(name)) != 0 || std::string(name) != "stock_client") {
    problem = std::string("the native end heard the name ") + name;
  }
  if (problem.empty()) {
    problem = nativeExchange(pipe, *stock, 300);
  }
  if (problem.empty()) {
    problem = runsOn(pipe, shm == NativeShm::kStockProtocol ? "shm" : "uv");
  }
  report(caseName, problem);
  stock.reset();
  if (pipe != nullptr) {
    tpc_pipe_destroy(pipe);
  }
  tpc_listener_destroy(listener);
  tpc_context_destroy(native);
  ctx->join();
  return problem.empty() ? 0 : 1;
}

} // namespace

int main(int argc, char** argv) {
  if (argc < 2 || (std::strcmp(argv[1], "run") != 0 && std::strcmp(argv[1], "capture") != 0) ||
      (std::strcmp(argv[1], "capture") == 0 && argc != 3)) {
    std::fprintf(stderr, "usage: %s run | capture <file>\n", argv[0]);
    return 2;
  }
  int rc = compatConnectsToStock();
  rc |= stockConnectsToCompat();
  rc |= nativeConnectsToStock(NativeShm::kNone);
  rc |= stockConnectsToNative(NativeShm::kNone);
  rc |= nativeConnectsToStock(NativeShm::kOwnProtocol);
  rc |= stockConnectsToNative(NativeShm::kOwnProtocol);
  rc |= nativeConnectsToStock(NativeShm::kStockProtocol);
  rc |= stockConnectsToNative(NativeShm::kStockProtocol);
  if (std::strcmp(argv[1], "capture") == 0 && rc == 0) {
    FILE* f = std::fopen(argv[2], "w");
    if (f == nullptr) {
      std::perror(argv[2]);
      return 3;
    }
    std::fprintf(f, "# Control frames written by an unmodified TensorPipe endpoint (the build inside PyTorch's\n");
    std::fprintf(f, "# libtorch_cpu.so), as read off the TCP connections by tests/cpp/stock_wire_interop.cc capture\n# (tests/golden/make_stock_wire_vectors.sh runs it):\n");
    std::fprintf(f, "# <who wrote it>.<what> <hex>. Ports and registration tokens are those of the capturing run.\n");
    for (auto& kv : captured) {
      std::fprintf(f, "%s ", kv.first.c_str());
      for (uint8_t b : kv.second) {
        std::fprintf(f, "%02x", b);
      }
      std::fprintf(f, "\n");
    }
    std::fclose(f);
  }
  return rc;
}
