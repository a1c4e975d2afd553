// This library's side of tpbridge (see bridge.h): its channel contexts behind
// the neutral interfaces, the host's connections in front of them.
#include <bridge/bridge.h>

#include <tensorpipe/channel/basic/factory.h>
#include <tensorpipe/channel/channel.h>
#include <tensorpipe/channel/context.h>
#include <tensorpipe/channel/hip_basic/factory.h>
#include <tensorpipe/channel/hip_ipc/factory.h>
#include <tensorpipe/channel/hip_xth/factory.h>
#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/error.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/transport/connection.h>

namespace tpbridge {

namespace {

namespace tp = ::tensorpipe;

// An error that came across the bridge as text.
class ForeignError final : public tp::BaseError {
 public:
  explicit ForeignError(std::string what) : what_(std::move(what)) {}
  std::string what() const override {
    return what_;
  }

 private:
  std::string what_;
};

tp::Error toError(const std::string& text) {
  if (text.empty()) {
    return tp::Error::kSuccess;
  }
  return TP_CREATE_ERROR(ForeignError, text);
}

std::string toText(const tp::Error& error) {
  return error ? error.what() : std::string();
}

// The host's connection as this library's channels expect one.
class HostConnection final : public tp::transport::Connection {
 public:
  explicit HostConnection(std::shared_ptr<tpbridge::Connection> inner) : inner_(std::move(inner)) {}
  void read(read_callback_fn fn) override {
    inner_->read([fn{std::move(fn)}](const std::string& e, const void* p, size_t n) { fn(toError(e), p, n); });
  }
  void read(void* ptr, size_t length, read_callback_fn fn) override {
    inner_->read(ptr, length, [fn{std::move(fn)}](const std::string& e, const void* p, size_t n) {
      fn(toError(e), p, n);
    });
  }
  void write(const void* ptr, size_t length, write_callback_fn fn) override {
    inner_->write(ptr, length, [fn{std::move(fn)}](const std::string& e) { fn(toError(e)); });
  }
  void read(tp::AbstractNopHolder& object, read_nop_callback_fn fn) override {
    inner_->read([&object, fn{std::move(fn)}](const std::string& e, const void* p, size_t n) {
      if (e.empty() && !object.deserialize(static_cast<const uint8_t*>(p), n)) {
        fn(toError("a message of " + std::to_string(n) + " bytes did not parse"));
        return;
      }
      fn(toError(e));
    });
  }
  void write(const tp::AbstractNopHolder& object, write_callback_fn fn) override {
    auto bytes = std::make_shared<std::vector<uint8_t>>(object.getSize());
    object.serialize(bytes->data(), bytes->size());
    inner_->write(bytes->data(), bytes->size(), [bytes, fn{std::move(fn)}](const std::string& e) { fn(toError(e)); });
  }
  void setId(std::string id) override {
    inner_->setId(std::move(id));
  }
  void close() override {
    inner_->close();
  }

 private:
  std::shared_ptr<tpbridge::Connection> inner_;
};

tp::Buffer toBuffer(const BufferRef& b) {
  if (b.onGpu) {
    return tp::HipBuffer{b.ptr, b.stream};
  }
  return tp::CpuBuffer{b.ptr};
}

class ChannelFace final : public Channel {
 public:
  explicit ChannelFace(std::shared_ptr<tp::channel::Channel> impl) : impl_(std::move(impl)) {}
  void send(BufferRef buffer, size_t length, DoneFn fn) override {
    impl_->send(toBuffer(buffer), length, [fn{std::move(fn)}](const tp::Error& e) { fn(toText(e)); });
  }
  void recv(BufferRef buffer, size_t length, DoneFn fn) override {
    impl_->recv(toBuffer(buffer), length, [fn{std::move(fn)}](const tp::Error& e) { fn(toText(e)); });
  }
  void setId(std::string id) override {
    impl_->setId(std::move(id));
  }
  void close() override {
    impl_->close();
  }

 private:
  std::shared_ptr<tp::channel::Channel> impl_;
};

class ContextFace final : public Context {
 public:
  explicit ContextFace(std::shared_ptr<tp::channel::Context> impl) : impl_(std::move(impl)) {}
  bool isViable() const override {
    return impl_->isViable();
  }
  size_t numConnectionsNeeded() const override {
    return impl_->numConnectionsNeeded();
  }
  std::vector<DeviceDescriptor> deviceDescriptors() const override {
    std::vector<DeviceDescriptor> out;
    for (const auto& kv : impl_->deviceDescriptors()) {
      out.push_back(DeviceDescriptor{kv.first.type, kv.first.index, kv.second});
    }
    return out;
  }
  bool canCommunicateWithRemote(const std::string& local, const std::string& remote) const override {
    return impl_->canCommunicateWithRemote(local, remote);
  }
  std::shared_ptr<Channel> createChannel(
      std::vector<std::shared_ptr<Connection>> connections, bool listenSide) override {
    std::vector<std::shared_ptr<tp::transport::Connection>> mine;
    for (auto& c : connections) {
      mine.push_back(std::make_shared<HostConnection>(std::move(c)));
    }
    return std::make_shared<ChannelFace>(impl_->createChannel(
        std::move(mine), listenSide ? tp::channel::Endpoint::kListen : tp::channel::Endpoint::kConnect));
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
  std::shared_ptr<tp::channel::Context> impl_;
};

} // namespace

std::shared_ptr<Context> createContext(const std::string& channelName) {
  std::shared_ptr<tp::channel::Context> impl;
  if (channelName == "hip_xth") {
    impl = tp::channel::hip_xth::create();
  } else if (channelName == "hip_ipc") {
    impl = tp::channel::hip_ipc::create();
  } else if (channelName == "hip_basic") {
    impl = tp::channel::hip_basic::create(tp::channel::basic::create());
  } else {
    return nullptr;
  }
  return std::make_shared<ContextFace>(std::move(impl));
}

} // namespace tpbridge
