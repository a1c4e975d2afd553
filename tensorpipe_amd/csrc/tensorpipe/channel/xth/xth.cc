// xth: CPU tensors between two endpoints of one process. The sender writes
// {pointer, length}; the receiver memcpy's on the context's copy thread and
// acknowledges. Behaviour of tensorpipe/channel/xth/channel_impl.cc:30-33 and
// context_impl.cc:105-123; kept as the CPU counterpart of hip_xth for the
// baseline figures.

#include <tensorpipe/channel/xth/factory.h>

#include <cstring>
#include <deque>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/channel/hip_common.h>
#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/wire.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace xth {

namespace {

class XthCore final : public ContextCore {
 public:
  ThreadLoop copier{"tp_xth_copy"};
  void joinImpl() override {
    copier.join();
  }
};

class ChannelImpl final : public ChannelImplBase {
 public:
  ChannelImpl(
      std::shared_ptr<XthCore> ctx,
      std::string id,
      std::shared_ptr<transport::Connection> descriptorConnection,
      std::shared_ptr<transport::Connection> completionConnection)
      : ChannelImplBase(ctx, std::move(id)),
        xctx_(std::move(ctx)),
        descriptorConnection_(std::move(descriptorConnection)),
        completionConnection_(std::move(completionConnection)) {}

 protected:
  struct Op {
    uint64_t seq;
    void* ptr;
    size_t length;
    std::function<void(const Error&)> cb;
    bool done{false};
    bool copying{false}; // handed to the copier thread, which still writes to ptr
  };

  void sendFromLoop(uint64_t seq, Buffer buffer, size_t length, TSendCallback cb) override {
    if (length == 0) {
      cb(error_);
      return;
    }
    auto op = std::make_shared<Op>(Op{seq, buffer.unwrap<CpuBuffer>().ptr, length, std::move(cb)});
    ops_.push_back(op);
    WireWriter w;
    w.u64(reinterpret_cast<uint64_t>(op->ptr));
    w.u64(length);
    TP_VLOG(6) << "Channel " << id_ << " is writing descriptor (#" << seq << ")";
    writeMessage(*descriptorConnection_, std::move(w.bytes()));
    completionConnection_->read(nullptr, 0, onRead([this, op] {
      TP_VLOG(6) << "Channel " << id_ << " done reading completion (#" << op->seq << ")";
      finish(op);
    }));
  }

  void recvFromLoop(uint64_t seq, Buffer buffer, size_t length, TRecvCallback cb) override {
    if (length == 0) {
      cb(error_);
      return;
    }
    auto op = std::make_shared<Op>(Op{seq, buffer.unwrap<CpuBuffer>().ptr, length, std::move(cb)});
    ops_.push_back(op);
    TP_VLOG(6) << "Channel " << id_ << " is reading descriptor (#" << seq << ")";
    descriptorConnection_->read(onReadMessage([this, op](std::vector<uint8_t> bytes) {
      TP_VLOG(6) << "Channel " << id_ << " done reading descriptor (#" << op->seq << ")";
      if (error_) {
        finish(op);
        return;
      }
      WireReader r(bytes.data(), bytes.size());
      const void* src = reinterpret_cast<const void*>(r.u64());
      const uint64_t len = r.u64();
      if (!r.ok() || len != op->length) {
        setError(TP_CREATE_ERROR(
            ShortReadError, static_cast<ssize_t>(op->length), static_cast<ssize_t>(len)));
        return;
      }
      auto self = shared_from_this();
      op->copying = true;
      xctx_->copier.defer([this, self, op, src] {
        std::memcpy(op->ptr, src, op->length);
        ctx_->defer([this, self, op] {
          TP_VLOG(6) << "Channel " << id_ << " done copying payload (#" << op->seq << ")";
          op->copying = false;
          finish(op);
          if (!error_) {
            completionConnection_->write(nullptr, 0, onWritten([] {}));
          }
        });
      });
    }));
  }

  void handleError() override {
    descriptorConnection_->close();
    completionConnection_->close();
    // A receive that the copier thread is working on keeps its buffer until
    // the copy has ended; the copier's completion finishes it.
    auto ops = std::move(ops_);
    ops_.clear();
    for (auto& op : ops) {
      if (!op->copying) {
        finish(op);
      }
    }
  }

 private:
  void finish(const std::shared_ptr<Op>& op) {
    if (op->done) {
      return;
    }
    op->done = true;
    for (auto it = ops_.begin(); it != ops_.end(); ++it) {
      if (*it == op) {
        ops_.erase(it);
        break;
      }
    }
    auto cb = std::move(op->cb);
    cb(error_);
  }

  std::shared_ptr<XthCore> xctx_;
  std::shared_ptr<transport::Connection> descriptorConnection_;
  std::shared_ptr<transport::Connection> completionConnection_;
  std::deque<std::shared_ptr<Op>> ops_;
};

class ContextImpl final : public Context {
 public:
  ContextImpl() : core_(std::make_shared<XthCore>()) {
    descriptors_[Device{kCpuDeviceType, 0}] = processIdentity();
  }
  ~ContextImpl() override {
    core_->join();
  }
  bool isViable() const override {
    return true;
  }
  size_t numConnectionsNeeded() const override {
    return 2;
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
    TP_THROW_ASSERT_IF(connections.size() != 2);
    auto impl = std::make_shared<ChannelImpl>(
        core_, core_->nextChannelId(), std::move(connections[0]), std::move(connections[1]));
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
  std::shared_ptr<XthCore> core_;
  std::unordered_map<Device, std::string> descriptors_;
};

} // namespace

std::shared_ptr<Context> create() {
  return std::make_shared<ContextImpl>();
}

} // namespace xth
} // namespace channel
TP_AMD_NAMESPACE_END
