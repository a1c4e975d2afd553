// hip_xth: GPU-to-GPU channel between two pipe endpoints of ONE process.
//
// Sender: records a start event on the stream(s) of the source buffers and
// ships raw {event, stream, device, src pointer, length} words over the
// descriptor connection -- they are valid in the receiver because it is the
// same address space. Receiver: makes its stream wait for the start event(s),
// enqueues ONE batched copy kernel for all tensors of the message, records a
// stop event, makes the sender's stream(s) wait for it, fires the recv
// callback (copy enqueued, not finished: consumers order on their stream) and
// acknowledges with an empty message, upon which the send callback fires.
//
// Same protocol and stream semantics as
// tensorpipe/channel/cuda_xth/channel_impl.cc:40-77,96-315; what differs is
// that a whole message travels in one descriptor and one kernel launch
// instead of one cudaMemcpyAsync and three event operations per tensor, and
// that events come from a pool instead of being created per operation.

#include <tensorpipe/channel/hip_xth/factory.h>

#include <deque>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/channel/hip_common.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/common/wire.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_xth {

namespace {

class XthContextCore final : public ContextCore {
 public:
  HipEventPool events;
};

struct StreamRef {
  void* stream;
  int device;
  bool operator==(const StreamRef& o) const {
    return stream == o.stream && device == o.device;
  }
};

class ChannelImpl final : public ChannelImplBase {
 public:
  ChannelImpl(
      std::shared_ptr<XthContextCore> ctx,
      std::string id,
      std::shared_ptr<transport::Connection> descriptorConnection,
      std::shared_ptr<transport::Connection> completionConnection)
      : ChannelImplBase(ctx, std::move(id)),
        xctx_(std::move(ctx)),
        descriptorConnection_(std::move(descriptorConnection)),
        completionConnection_(std::move(completionConnection)) {}

  void sendBatch(std::vector<BatchEntry> entries, TSendCallback callback) {
    auto self = std::static_pointer_cast<ChannelImpl>(shared_from_this());
    ctx_->defer([self, entries{std::move(entries)}, callback{std::move(callback)}]() mutable {
      const uint64_t seq = self->nextSend_++;
      if (self->error_) {
        callback(self->error_);
        return;
      }
      self->sendEntries(seq, std::move(entries), std::move(callback));
    });
  }

  void recvBatch(std::vector<BatchEntry> entries, TRecvCallback callback) {
    auto self = std::static_pointer_cast<ChannelImpl>(shared_from_this());
    ctx_->defer([self, entries{std::move(entries)}, callback{std::move(callback)}]() mutable {
      const uint64_t seq = self->nextRecv_++;
      if (self->error_) {
        callback(self->error_);
        return;
      }
      self->recvEntries(seq, std::move(entries), std::move(callback));
    });
  }

 protected:
  void sendFromLoop(uint64_t seq, Buffer buffer, size_t length, TSendCallback cb) override {
    std::vector<BatchEntry> entries;
    entries.push_back({std::move(buffer), length});
    sendEntries(seq, std::move(entries), std::move(cb));
  }

  void recvFromLoop(uint64_t seq, Buffer buffer, size_t length, TRecvCallback cb) override {
    std::vector<BatchEntry> entries;
    entries.push_back({std::move(buffer), length});
    recvEntries(seq, std::move(entries), std::move(cb));
  }

  void handleError() override {
    descriptorConnection_->close();
    completionConnection_->close();
    // Every pending callback fires now, in order, with the error.
    auto sends = std::move(sendOps_);
    sendOps_.clear();
    for (auto& op : sends) {
      finishSend(op);
    }
    auto recvs = std::move(recvOps_);
    recvOps_.clear();
    for (auto& op : recvs) {
      finishRecv(op);
    }
  }

 private:
  struct SendOp {
    uint64_t seq;
    TSendCallback cb;
    std::vector<std::unique_ptr<HipEvent>> startEvents;
    bool done{false};
  };

  struct RecvOp {
    uint64_t seq;
    TRecvCallback cb;
    std::vector<BatchEntry> entries; // non-empty ones only
    bool done{false};
  };

  void sendEntries(uint64_t seq, std::vector<BatchEntry> entries, TSendCallback cb) {
    // Zero-length tensors complete at once and put nothing on the wire
    // (tensorpipe/channel/cuda_xth/channel_impl.cc:122-126).
    std::vector<BatchEntry> live;
    for (auto& e : entries) {
      if (e.length > 0) {
        live.push_back(std::move(e));
      }
    }
    if (live.empty()) {
      cb(error_);
      return;
    }
    auto op = std::make_shared<SendOp>();
    op->seq = seq;
    op->cb = std::move(cb);

    std::vector<StreamRef> streams;
    WireWriter body;
    try {
      for (auto& e : live) {
        const HipBuffer& hb = e.buffer.unwrap<HipBuffer>();
        StreamRef ref{hb.stream, hipDeviceForPointer(hb.ptr)};
        TP_THROW_ASSERT_IF(ref.device < 0);
        bool known = false;
        for (auto& s : streams) {
          known |= s == ref;
        }
        if (!known) {
          streams.push_back(ref);
        }
        body.u64(reinterpret_cast<uint64_t>(hb.ptr));
        body.u64(e.length);
      }
      for (auto& s : streams) {
        auto ev = xctx_->events.get(s.device);
        ev->record(s.stream);
        op->startEvents.push_back(std::move(ev));
      }
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " send failed: " << ex.what();
      op->cb(TP_CREATE_ERROR(HipError, "hip_xth send", TPHIP_ERR_INVALID_ARG));
      setError(TP_CREATE_ERROR(HipError, "hip_xth send", TPHIP_ERR_INVALID_ARG));
      return;
    }

    WireWriter w;
    w.u32(static_cast<uint32_t>(live.size()));
    w.u32(static_cast<uint32_t>(streams.size()));
    for (size_t i = 0; i < streams.size(); ++i) {
      w.u64(reinterpret_cast<uint64_t>(op->startEvents[i]->raw()));
      w.u64(reinterpret_cast<uint64_t>(streams[i].stream));
      w.u32(static_cast<uint32_t>(streams[i].device));
    }
    w.raw(body.bytes().data(), body.bytes().size());

    sendOps_.push_back(op);
    TP_VLOG(6) << "Channel " << id_ << " is writing descriptor (#" << seq << ")";
    writeMessage(*descriptorConnection_, std::move(w.bytes()));
    TP_VLOG(6) << "Channel " << id_ << " is reading completion (#" << seq << ")";
    completionConnection_->read(nullptr, 0, onRead([this, op] {
      TP_VLOG(6) << "Channel " << id_ << " done reading completion (#" << op->seq << ")";
      removeSend(op);
      finishSend(op);
    }));
  }

  void recvEntries(uint64_t seq, std::vector<BatchEntry> entries, TRecvCallback cb) {
    auto op = std::make_shared<RecvOp>();
    op->seq = seq;
    op->cb = std::move(cb);
    for (auto& e : entries) {
      if (e.length > 0) {
        op->entries.push_back(std::move(e));
      }
    }
    if (op->entries.empty()) {
      op->cb(error_);
      return;
    }
    recvOps_.push_back(op);
    TP_VLOG(6) << "Channel " << id_ << " is reading descriptor (#" << seq << ")";
    descriptorConnection_->read(onReadMessage([this, op](std::vector<uint8_t> bytes) {
      TP_VLOG(6) << "Channel " << id_ << " done reading descriptor (#" << op->seq << ")";
      if (!error_) {
        copyFromDescriptor(op, bytes);
      }
      removeRecv(op);
      finishRecv(op);
      if (!error_) {
        TP_VLOG(6) << "Channel " << id_ << " is writing completion (#" << op->seq << ")";
        completionConnection_->write(nullptr, 0, onWritten([] {}));
      }
    }));
  }

  // Wait for the sender's start events, copy everything with one launch per
  // (device, stream) of the destination buffers (normally one in total), and
  // make the sender's streams wait for the copy.
  void copyFromDescriptor(const std::shared_ptr<RecvOp>& op, const std::vector<uint8_t>& bytes) {
    WireReader r(bytes.data(), bytes.size());
    const uint32_t n = r.u32();
    const uint32_t nStreams = r.u32();
    struct SrcStream {
      void* event;
      void* stream;
      int device;
    };
    std::vector<SrcStream> srcStreams;
    for (uint32_t i = 0; i < nStreams && r.ok(); ++i) {
      SrcStream s;
      s.event = reinterpret_cast<void*>(r.u64());
      s.stream = reinterpret_cast<void*>(r.u64());
      s.device = static_cast<int>(r.u32());
      srcStreams.push_back(s);
    }
    if (!r.ok() || n != op->entries.size()) {
      setError(TP_CREATE_ERROR(ShortReadError, static_cast<ssize_t>(op->entries.size()), n));
      return;
    }
    struct Group {
      StreamRef dst;
      std::vector<tphip_copy_desc> table;
    };
    std::vector<Group> groups;
    try {
      for (uint32_t i = 0; i < n; ++i) {
        const void* src = reinterpret_cast<const void*>(r.u64());
        const uint64_t len = r.u64();
        if (!r.ok() || len != op->entries[i].length) {
          setError(TP_CREATE_ERROR(
              ShortReadError, static_cast<ssize_t>(op->entries[i].length), static_cast<ssize_t>(len)));
          return;
        }
        const HipBuffer& hb = op->entries[i].buffer.unwrap<HipBuffer>();
        StreamRef ref{hb.stream, hipDeviceForPointer(hb.ptr)};
        TP_THROW_ASSERT_IF(ref.device < 0);
        Group* g = nullptr;
        for (auto& cand : groups) {
          if (cand.dst == ref) {
            g = &cand;
          }
        }
        if (g == nullptr) {
          groups.push_back(Group{ref, {}});
          g = &groups.back();
        }
        g->table.push_back(tphip_copy_desc{src, hb.ptr, len});
      }
      for (auto& g : groups) {
        for (auto& s : srcStreams) {
          TP_HIP_CHECK(tphip_stream_wait_event(g.dst.device, g.dst.stream, s.event));
        }
        TP_VLOG(6) << "Channel " << id_ << " is copying payload (#" << op->seq << ")";
        hipBatchedCopy(g.dst.device, g.dst.stream, g.table);
        auto stop = xctx_->events.get(g.dst.device);
        stop->record(g.dst.stream);
        for (auto& s : srcStreams) {
          stop->wait(s.stream, s.device);
        }
        // The waits above captured the record; the event can be reused.
        xctx_->events.put(std::move(stop));
      }
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " copy failed: " << ex.what();
      setError(TP_CREATE_ERROR(HipError, "hip_xth copy", TPHIP_ERR_INVALID_ARG));
    }
  }

  void removeSend(const std::shared_ptr<SendOp>& op) {
    for (auto it = sendOps_.begin(); it != sendOps_.end(); ++it) {
      if (*it == op) {
        sendOps_.erase(it);
        return;
      }
    }
  }

  void removeRecv(const std::shared_ptr<RecvOp>& op) {
    for (auto it = recvOps_.begin(); it != recvOps_.end(); ++it) {
      if (*it == op) {
        recvOps_.erase(it);
        return;
      }
    }
  }

  void finishSend(const std::shared_ptr<SendOp>& op) {
    if (op->done) {
      return;
    }
    op->done = true;
    for (auto& ev : op->startEvents) {
      xctx_->events.put(std::move(ev));
    }
    op->startEvents.clear();
    auto cb = std::move(op->cb);
    cb(error_);
  }

  void finishRecv(const std::shared_ptr<RecvOp>& op) {
    if (op->done) {
      return;
    }
    op->done = true;
    auto cb = std::move(op->cb);
    cb(error_);
  }

  std::shared_ptr<XthContextCore> xctx_;
  std::shared_ptr<transport::Connection> descriptorConnection_;
  std::shared_ptr<transport::Connection> completionConnection_;
  std::deque<std::shared_ptr<SendOp>> sendOps_;
  std::deque<std::shared_ptr<RecvOp>> recvOps_;
};

class XthChannel final : public ChannelHandle<ChannelImpl>, public BatchedChannel {
 public:
  using ChannelHandle<ChannelImpl>::ChannelHandle;
  void sendBatch(std::vector<BatchEntry> entries, TSendCallback callback) override {
    if (!impl_) {
      callback(TP_CREATE_ERROR(ContextNotViableError));
      return;
    }
    impl_->sendBatch(std::move(entries), std::move(callback));
  }
  void recvBatch(std::vector<BatchEntry> entries, TRecvCallback callback) override {
    if (!impl_) {
      callback(TP_CREATE_ERROR(ContextNotViableError));
      return;
    }
    impl_->recvBatch(std::move(entries), std::move(callback));
  }
};

class ContextImpl final : public Context {
 public:
  ContextImpl() {
    const int n = hipDeviceCountNoThrow();
    if (n <= 0) {
      return; // not viable: no GPU or no runtime
    }
    core_ = std::make_shared<XthContextCore>();
    // Every device gets the process identity as descriptor: two endpoints can
    // talk iff they are the same process.
    for (int i = 0; i < n; ++i) {
      descriptors_[Device{kHipDeviceType, i}] = processIdentity();
    }
  }
  ~ContextImpl() override {
    join();
  }
  bool isViable() const override {
    return core_ != nullptr;
  }
  size_t numConnectionsNeeded() const override {
    return 2; // descriptors one way, completions the other
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
    if (!core_) {
      return std::make_shared<XthChannel>(nullptr);
    }
    TP_THROW_ASSERT_IF(connections.size() != 2);
    auto impl = std::make_shared<ChannelImpl>(
        core_, core_->nextChannelId(), std::move(connections[0]), std::move(connections[1]));
    impl->init();
    return std::make_shared<XthChannel>(std::move(impl));
  }
  void setId(std::string id) override {
    if (core_) {
      core_->setId(std::move(id));
    }
  }
  void close() override {
    if (core_) {
      core_->close();
    }
  }
  void join() override {
    if (core_) {
      core_->join();
    }
  }

 private:
  std::shared_ptr<XthContextCore> core_;
  std::unordered_map<Device, std::string> descriptors_;
};

} // namespace

std::shared_ptr<Context> create() {
  return std::make_shared<ContextImpl>();
}

} // namespace hip_xth
} // namespace channel
TP_AMD_NAMESPACE_END
