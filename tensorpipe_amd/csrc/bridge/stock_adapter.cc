// See stock_adapter.h. The two interfaces a stock TensorPipe build does not
// ship headers for are declared here with the members, in the order, of
// tensorpipe/transport/connection.h:21-69 and tensorpipe/channel/channel.h:52-72,
// which is what fixes their virtual tables.
#include <bridge/stock_adapter.h>

#include <atomic>
#include <functional>
#include <unordered_map>
#include <vector>

#include <tensorpipe/common/buffer.h>
#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/error.h>

#include <bridge/bridge.h>

#ifdef TPAMD_BRIDGE_HOST_HAS_CHANNEL_HEADERS
#include <tensorpipe/channel/channel.h>
#include <tensorpipe/transport/connection.h>
#else
// A host that installs channel/context.h without these two abstract classes
// (PyTorch does): their declaration, virtual functions in the order of
// tensorpipe/transport/connection.h:21-69 and tensorpipe/channel/channel.h:52-72.
namespace tensorpipe {

class AbstractNopHolder; // only ever named, in two members this adapter does not call

namespace transport {
class Connection {
 public:
  using read_callback_fn = std::function<void(const Error& error, const void* ptr, size_t length)>;
  virtual void read(read_callback_fn fn) = 0;
  virtual void read(void* ptr, size_t length, read_callback_fn fn) = 0;
  using write_callback_fn = std::function<void(const Error& error)>;
  virtual void write(const void* ptr, size_t length, write_callback_fn fn) = 0;
  using read_nop_callback_fn = std::function<void(const Error& error)>;
  virtual void read(AbstractNopHolder& object, read_nop_callback_fn fn) = 0;
  virtual void write(const AbstractNopHolder& object, write_callback_fn fn) = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual ~Connection() = default;
};
} // namespace transport

namespace channel {
using TSendCallback = std::function<void(const Error&)>;
using TRecvCallback = std::function<void(const Error&)>;
class Channel {
 public:
  virtual void send(Buffer buffer, size_t length, TSendCallback callback) = 0;
  virtual void recv(Buffer buffer, size_t length, TRecvCallback callback) = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual ~Channel() = default;
};
} // namespace channel

} // namespace tensorpipe
#endif

namespace tensorpipe_amd_bridge {

namespace {

namespace tp = ::tensorpipe;

class ChannelError final : public tp::BaseError {
 public:
  explicit ChannelError(std::string what) : what_(std::move(what)) {}
  std::string what() const override {
    return what_;
  }

 private:
  std::string what_;
};

tp::Error toError(const std::string& text) {
  if (text.empty()) {
    return tp::Error();
  }
  return tp::Error(std::make_shared<ChannelError>(text), __FILE__, __LINE__);
}

std::string toText(const tp::Error& error) {
  return error ? error.what() : std::string();
}

// The host's connection behind the neutral interface.
class ConnectionFace final : public tpbridge::Connection {
 public:
  explicit ConnectionFace(std::shared_ptr<tp::transport::Connection> inner) : inner_(std::move(inner)) {}
  void read(tpbridge::ReadFn fn) override {
    inner_->read([fn{std::move(fn)}](const tp::Error& e, const void* p, size_t n) { fn(toText(e), p, n); });
  }
  void read(void* ptr, size_t length, tpbridge::ReadFn fn) override {
    inner_->read(ptr, length, [fn{std::move(fn)}](const tp::Error& e, const void* p, size_t n) {
      fn(toText(e), p, n);
    });
  }
  void write(const void* ptr, size_t length, tpbridge::DoneFn fn) override {
    inner_->write(ptr, length, [fn{std::move(fn)}](const tp::Error& e) { fn(toText(e)); });
  }
  void setId(std::string id) override {
    inner_->setId(std::move(id));
  }
  void close() override {
    inner_->close();
  }

 private:
  std::shared_ptr<tp::transport::Connection> inner_;
};

// GPU buffers handed over so far: all, and per channel kind.
std::atomic<unsigned long long> gpuOperations{0};
constexpr const char* kChannelNames[] = {"hip_xth", "hip_ipc", "hip_basic"};
std::atomic<unsigned long long> gpuOperationsOf[3];

int channelKind(const std::string& name) {
  for (int k = 0; k < 3; ++k) {
    if (name == kChannelNames[k]) {
      return k;
    }
  }
  return -1;
}

tpbridge::BufferRef toRef(const tp::Buffer& buffer, int kind) {
  tpbridge::BufferRef ref;
  if (buffer.device().type == tp::kCpuDeviceType) {
    ref.ptr = buffer.unwrap<tp::CpuBuffer>().ptr;
    return ref;
  }
  const HipBuffer& hb = buffer.unwrap<HipBuffer>(); // throws on any other kind, as Buffer::unwrap does
  gpuOperations.fetch_add(1, std::memory_order_relaxed);
  if (kind >= 0) {
    gpuOperationsOf[kind].fetch_add(1, std::memory_order_relaxed);
  }
  ref.onGpu = true;
  ref.ptr = hb.ptr;
  ref.stream = hb.stream;
  return ref;
}

class ChannelAdapter final : public tp::channel::Channel {
 public:
  ChannelAdapter(std::shared_ptr<tpbridge::Channel> impl, int kind) : impl_(std::move(impl)), kind_(kind) {}
  void send(tp::Buffer buffer, size_t length, tp::channel::TSendCallback callback) override {
    impl_->send(toRef(buffer, kind_), length, [callback{std::move(callback)}](const std::string& e) {
      callback(toError(e));
    });
  }
  void recv(tp::Buffer buffer, size_t length, tp::channel::TRecvCallback callback) override {
    impl_->recv(toRef(buffer, kind_), length, [callback{std::move(callback)}](const std::string& e) {
      callback(toError(e));
    });
  }
  void setId(std::string id) override {
    impl_->setId(std::move(id));
  }
  void close() override {
    impl_->close();
  }

 private:
  std::shared_ptr<tpbridge::Channel> impl_;
  const int kind_;
};

class ContextAdapter final : public tp::channel::Context {
 public:
  ContextAdapter(std::shared_ptr<tpbridge::Context> impl, int kind) : impl_(std::move(impl)), kind_(kind) {
    for (auto& d : impl_->deviceDescriptors()) {
      descriptors_[tp::Device{d.deviceType, d.deviceIndex}] = d.descriptor;
    }
  }
  bool isViable() const override {
    return impl_->isViable();
  }
  size_t numConnectionsNeeded() const override {
    return impl_->numConnectionsNeeded();
  }
  const std::unordered_map<tp::Device, std::string>& deviceDescriptors() const override {
    return descriptors_;
  }
  bool canCommunicateWithRemote(const std::string& local, const std::string& remote) const override {
    return impl_->canCommunicateWithRemote(local, remote);
  }
  std::shared_ptr<tp::channel::Channel> createChannel(
      std::vector<std::shared_ptr<tp::transport::Connection>> connections,
      tp::channel::Endpoint endpoint) override {
    std::vector<std::shared_ptr<tpbridge::Connection>> faces;
    for (auto& c : connections) {
      faces.push_back(std::make_shared<ConnectionFace>(std::move(c)));
    }
    return std::make_shared<ChannelAdapter>(
        impl_->createChannel(std::move(faces), endpoint == tp::channel::Endpoint::kListen), kind_);
  }
  void setId(std::string id) override {
    impl_->setId(std::move(id));
  }
  void close() override {
    impl_->close();
  }
  void join() override {
    impl_->join();
  }

 private:
  std::shared_ptr<tpbridge::Context> impl_;
  const int kind_;
  std::unordered_map<tp::Device, std::string> descriptors_;
};

} // namespace

unsigned long long gpuOperationsServed() {
  return gpuOperations.load(std::memory_order_relaxed);
}

unsigned long long gpuOperationsServedBy(const std::string& channelName) {
  const int kind = channelKind(channelName);
  return kind < 0 ? 0 : gpuOperationsOf[kind].load(std::memory_order_relaxed);
}

std::shared_ptr<::tensorpipe::channel::Context> createChannelContext(const std::string& channelName) {
  auto impl = tpbridge::createContext(channelName);
  if (!impl) {
    return nullptr;
  }
  return std::make_shared<ContextAdapter>(std::move(impl), channelKind(channelName));
}

} // namespace tensorpipe_amd_bridge
