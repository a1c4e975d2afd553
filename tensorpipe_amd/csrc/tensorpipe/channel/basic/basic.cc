// basic: a CPU tensor is written to / read from the channel's single
// connection as one message. Behaviour of
// tensorpipe/channel/basic/channel_impl.cc:85-97 (write) and :152-169 (read).

#include <tensorpipe/channel/basic/factory.h>

#include <deque>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/common/cpu_buffer.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace basic {

namespace {

class ChannelImpl final : public ChannelImplBase {
 public:
  ChannelImpl(
      std::shared_ptr<ContextCore> ctx,
      std::string id,
      std::shared_ptr<transport::Connection> connection)
      : ChannelImplBase(std::move(ctx), std::move(id)), connection_(std::move(connection)) {}

 protected:
  void sendFromLoop(uint64_t seq, Buffer buffer, size_t length, TSendCallback cb) override {
    if (length == 0) {
      cb(error_);
      return;
    }
    auto op = std::make_shared<Op>(Op{seq, std::move(cb)});
    pending_.insert(op);
    TP_VLOG(6) << "Channel " << id_ << " is writing payload (#" << seq << ")";
    connection_->write(buffer.unwrap<CpuBuffer>().ptr, length, onWritten([this, op] {
      finish(op);
    }));
  }

  void recvFromLoop(uint64_t seq, Buffer buffer, size_t length, TRecvCallback cb) override {
    if (length == 0) {
      cb(error_);
      return;
    }
    auto op = std::make_shared<Op>(Op{seq, std::move(cb)});
    pending_.insert(op);
    TP_VLOG(6) << "Channel " << id_ << " is reading payload (#" << seq << ")";
    connection_->read(buffer.unwrap<CpuBuffer>().ptr, length, onRead([this, op] { finish(op); }));
  }

  void handleError() override {
    connection_->close();
    // The connection fails every queued read/write in order, which runs
    // finish() for each pending op with error_ set.
  }

 private:
  struct Op {
    uint64_t seq;
    std::function<void(const Error&)> cb;
  };

  void finish(const std::shared_ptr<Op>& op) {
    if (pending_.erase(op) == 0) {
      return;
    }
    TP_VLOG(6) << "Channel " << id_ << " done with payload (#" << op->seq << ")";
    auto cb = std::move(op->cb);
    cb(error_);
  }

  std::shared_ptr<transport::Connection> connection_;
  std::unordered_set<std::shared_ptr<Op>> pending_;
};

class ContextImpl final : public Context {
 public:
  ContextImpl() : core_(std::make_shared<ContextCore>()) {
    // One descriptor for the only CPU device; every process accepts it
    // (tensorpipe/channel/basic/context_impl.cc:22).
    descriptors_[Device{kCpuDeviceType, 0}] = "any";
  }
  ~ContextImpl() override {
    core_->join();
  }
  bool isViable() const override {
    return true;
  }
  size_t numConnectionsNeeded() const override {
    return 1;
  }
  const std::unordered_map<Device, std::string>& deviceDescriptors() const override {
    return descriptors_;
  }
  bool canCommunicateWithRemote(const std::string& local, const std::string& remote)
      const override {
    return local == remote;
  }
  std::shared_ptr<Channel> createChannel(
      std::vector<std::shared_ptr<transport::Connection>> connections,
      Endpoint /*endpoint*/) override {
    TP_THROW_ASSERT_IF(connections.size() != 1);
    auto impl = std::make_shared<ChannelImpl>(
        core_, core_->nextChannelId(), std::move(connections[0]));
    impl->init();
    return std::make_shared<ChannelHandle<ChannelImpl>>(std::move(impl));
  }
  void setId(std::string id) override {
    core_->setId(std::move(id));
  }
  void close() override {
    core_->close();
  }
  void join() override {
    core_->join();
  }

 private:
  std::shared_ptr<ContextCore> core_;
  std::unordered_map<Device, std::string> descriptors_;
};

} // namespace

std::shared_ptr<Context> create() {
  return std::make_shared<ContextImpl>();
}

} // namespace basic
} // namespace channel
TP_AMD_NAMESPACE_END
