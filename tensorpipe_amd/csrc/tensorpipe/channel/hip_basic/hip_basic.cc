// hip_basic: host-staged GPU channel that wraps a CPU channel.
//
// A tensor is cut into chunks of at most one staging slot. Sender, per chunk:
// take a slot of the pinned send ring, copy GPU -> slot with the batched copy
// kernel on the caller's stream (the kernel stores straight into host-mapped
// pinned memory), and when that copy has completed hand the slot to the inner
// CPU channel. Receiver, per chunk: take a slot of the pinned receive ring,
// let the inner CPU channel fill it, copy slot -> GPU on the caller's stream,
// free the slot when that copy has completed. CPU-resident buffers skip the
// staging hop on their side, so the channel also carries CPU<->GPU transfers.
//
// Follows tensorpipe/channel/cuda_basic/channel_impl.cc:84-229 (send) and
// :335-506 (recv), context_impl.cc:27-154, constants.h:22-24, with these
// differences: copies are kernel launches instead of cudaMemcpyAsync,
// completion is detected by polling an event instead of a stream callback,
// and the "ready to send" notification is replaced by a one-time exchange of
// the chunk size (both sides know every tensor's length, so the receiver can
// post its inner recvs without being told).
//
// Callbacks: send fires once the last chunk has left the GPU (source
// reusable); recv fires once the last host-to-device copy has been enqueued.

#include <tensorpipe/channel/hip_basic/factory.h>

#include <algorithm>
#include <deque>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/channel/hip_common.h>
#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/common/slot_allocator.h>
#include <tensorpipe/common/wire.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_basic {

namespace {

// Defaults as tensorpipe/channel/cuda_basic/constants.h:22-24 (16 x 1 MiB per
// ring); TP_HIP_BASIC_SLOT_BYTES and TP_HIP_BASIC_NUM_SLOTS override them.
// Both are read when a context is created.
size_t slotBytesFromEnv() {
  const char* e = std::getenv("TP_HIP_BASIC_SLOT_BYTES");
  size_t b = e != nullptr ? std::strtoull(e, nullptr, 10) : (1u << 20);
  return b < 4096 ? size_t(4096) : b;
}

size_t numSlotsFromEnv() {
  const char* e = std::getenv("TP_HIP_BASIC_NUM_SLOTS");
  size_t n = e != nullptr ? std::strtoull(e, nullptr, 10) : 16;
  return n < 1 ? size_t(1) : n;
}

struct PinnedRing {
  PinnedRing(int device, size_t slots, size_t bytes)
      : slab(device, slots * bytes), allocator(slab.host(), slots, bytes) {}
  HipPinnedSlab slab;
  SlotAllocator allocator;
  // Address kernels use for a host pointer inside the slab.
  void* devAddress(const uint8_t* host) const {
    return slab.dev() + (host - slab.host());
  }
};

class BasicContextCore final : public ContextCore {
 public:
  HipEventPool events;
  HipEventPoller poller;
  const size_t slotBytes{slotBytesFromEnv()};
  const size_t numSlots{numSlotsFromEnv()};

  // Rings are created on first use (loop only), as the reference allocates its
  // pinned buffers lazily (tensorpipe/channel/cuda_basic/context_impl.cc:134-154).
  PinnedRing& sendRing() {
    if (!sendRing_) {
      sendRing_ = std::make_unique<PinnedRing>(0, numSlots, slotBytes);
    }
    return *sendRing_;
  }
  PinnedRing& recvRing() {
    if (!recvRing_) {
      recvRing_ = std::make_unique<PinnedRing>(0, numSlots, slotBytes);
    }
    return *recvRing_;
  }
  void closeRings() {
    if (sendRing_) {
      sendRing_->allocator.close();
    }
    if (recvRing_) {
      recvRing_->allocator.close();
    }
  }
  void joinImpl() override {
    poller.join();
  }

 private:
  std::unique_ptr<PinnedRing> sendRing_;
  std::unique_ptr<PinnedRing> recvRing_;
};

class ChannelImpl final : public ChannelImplBase {
 public:
  ChannelImpl(
      std::shared_ptr<BasicContextCore> ctx,
      std::string id,
      std::shared_ptr<transport::Connection> controlConnection,
      std::shared_ptr<Channel> cpuChannel)
      : ChannelImplBase(ctx, std::move(id)),
        bctx_(std::move(ctx)),
        controlConnection_(std::move(controlConnection)),
        cpuChannel_(std::move(cpuChannel)) {}

 protected:
  void initFromLoop() override {
    // Agree on the chunk size: both sides announce theirs, the smaller wins.
    WireWriter w;
    w.u64(bctx_->slotBytes);
    writeMessage(*controlConnection_, std::move(w.bytes()));
    controlConnection_->read(onReadMessage([this](std::vector<uint8_t> bytes) {
      if (error_) {
        return;
      }
      WireReader r(bytes.data(), bytes.size());
      const uint64_t remote = r.u64();
      if (!r.ok() || remote == 0) {
        setError(TP_CREATE_ERROR(ShortReadError, 8, static_cast<ssize_t>(bytes.size())));
        return;
      }
      chunkBytes_ = std::min<uint64_t>(remote, bctx_->slotBytes);
      auto deferred = std::move(deferred_);
      deferred_.clear();
      for (auto& fn : deferred) {
        fn();
      }
    }));
  }

  void sendFromLoop(uint64_t seq, Buffer buffer, size_t length, TSendCallback cb) override {
    if (length == 0) {
      cb(error_); // tensorpipe/channel/cuda_basic/channel_impl.cc:78-81
      return;
    }
    auto op = std::make_shared<Op>();
    op->seq = seq;
    op->cb = std::move(cb);
    op->buffer = std::move(buffer);
    op->length = length;
    ops_.push_back(op);
    whenReady([this, op] { startSend(op); });
  }

  void recvFromLoop(uint64_t seq, Buffer buffer, size_t length, TRecvCallback cb) override {
    if (length == 0) {
      cb(error_);
      return;
    }
    auto op = std::make_shared<Op>();
    op->seq = seq;
    op->cb = std::move(cb);
    op->buffer = std::move(buffer);
    op->length = length;
    ops_.push_back(op);
    whenReady([this, op] { startRecv(op); });
  }

  void handleError() override {
    controlConnection_->close();
    cpuChannel_->close();
    if (ctx_->closed()) {
      bctx_->closeRings();
    }
    deferred_.clear();
    sendQueue_.clear();
    recvQueue_.clear();
    auto ops = std::move(ops_);
    ops_.clear();
    for (auto& op : ops) {
      finish(op);
    }
  }

 private:
  struct Op {
    uint64_t seq;
    std::function<void(const Error&)> cb;
    Buffer buffer;
    size_t length{0};
    size_t pending{0};
    bool done{false};
  };

  // One chunk waiting for its turn on the inner channel: inner sends must be
  // issued in chunk order even if device-to-host copies finish out of order.
  struct SendChunk {
    void* hostPtr{nullptr};
    size_t length{0};
    SlotAllocator::TSlot slot;
    bool ready{false};
    std::shared_ptr<Op> op;
  };

  struct RecvChunk {
    void* hostPtr{nullptr};
    size_t length{0};
    size_t offset{0};
    SlotAllocator::TSlot slot;
    bool ready{false};
    std::shared_ptr<Op> op;
  };

  void whenReady(std::function<void()> fn) {
    if (chunkBytes_ != 0) {
      fn();
    } else {
      deferred_.push_back(std::move(fn));
    }
  }

  static bool isCpu(const Buffer& b) {
    return b.device().type == kCpuDeviceType;
  }

  // ---- send -----------------------------------------------------------------

  void startSend(const std::shared_ptr<Op>& op) {
    if (error_) {
      return;
    }
    const size_t chunks = (op->length + chunkBytes_ - 1) / chunkBytes_;
    op->pending = chunks; // chunks whose source bytes are still needed
    for (size_t k = 0; k < chunks; ++k) {
      const size_t offset = k * chunkBytes_;
      const size_t len = std::min<size_t>(op->length - offset, chunkBytes_);
      auto chunk = std::make_shared<SendChunk>();
      chunk->length = len;
      chunk->op = op;
      sendQueue_.push_back(chunk);
      if (isCpu(op->buffer)) {
        // Host source: no staging (tensorpipe/channel/cuda_basic/channel_impl.cc:138-145).
        chunk->hostPtr = static_cast<uint8_t*>(op->buffer.unwrap<CpuBuffer>().ptr) + offset;
        chunk->ready = true;
        continue;
      }
      const HipBuffer hb = op->buffer.unwrap<HipBuffer>();
      auto self = shared_from_this();
      PinnedRing& ring = bctx_->sendRing();
      ring.allocator.alloc([this, self, chunk, hb, offset, len, &ring](
                               const Error& error, SlotAllocator::TSlot slot) {
        if (error) {
          setError(error);
          return;
        }
        if (error_) {
          return;
        }
        chunk->slot = std::move(slot);
        chunk->hostPtr = chunk->slot.get();
        const int device = hipDeviceForPointer(hb.ptr);
        int rc = tphip_copy(
            device,
            ring.devAddress(chunk->slot.get()),
            static_cast<const uint8_t*>(hb.ptr) + offset,
            len,
            hb.stream);
        if (rc != 0) {
          setError(TP_CREATE_ERROR(HipError, "tphip_copy", rc));
          return;
        }
        auto ev = bctx_->events.get(device);
        ev->record(hb.stream);
        watch(std::move(ev), [this, chunk] {
          chunk->ready = true;
          flushSends();
        });
      });
    }
    flushSends();
  }

  void flushSends() {
    while (!sendQueue_.empty() && sendQueue_.front()->ready && !error_) {
      auto chunk = sendQueue_.front();
      sendQueue_.pop_front();
      auto self = shared_from_this();
      const bool staged = static_cast<bool>(chunk->slot);
      if (staged) {
        // The bytes now live in the pinned slot: the source is free.
        sourceDone(chunk->op);
      }
      cpuChannel_->send(
          CpuBuffer{chunk->hostPtr}, chunk->length, [this, self, chunk, staged](const Error& error) {
            ctx_->defer([this, self, chunk, staged, error] {
              setError(error);
              chunk->slot.reset(); // returns the slot to the ring
              if (!staged) {
                sourceDone(chunk->op);
              }
            });
          });
    }
  }

  void sourceDone(const std::shared_ptr<Op>& op) {
    if (op->done || --op->pending > 0) {
      return;
    }
    remove(op);
    finish(op);
  }

  // ---- recv -----------------------------------------------------------------

  void startRecv(const std::shared_ptr<Op>& op) {
    if (error_) {
      return;
    }
    const size_t chunks = (op->length + chunkBytes_ - 1) / chunkBytes_;
    op->pending = chunks; // chunks not yet landed (CPU) / not yet enqueued (GPU)
    for (size_t k = 0; k < chunks; ++k) {
      const size_t offset = k * chunkBytes_;
      const size_t len = std::min<size_t>(op->length - offset, chunkBytes_);
      auto chunk = std::make_shared<RecvChunk>();
      chunk->length = len;
      chunk->offset = offset;
      chunk->op = op;
      recvQueue_.push_back(chunk);
      if (isCpu(op->buffer)) {
        chunk->hostPtr = static_cast<uint8_t*>(op->buffer.unwrap<CpuBuffer>().ptr) + offset;
        chunk->ready = true;
        continue;
      }
      auto self = shared_from_this();
      bctx_->recvRing().allocator.alloc(
          [this, self, chunk](const Error& error, SlotAllocator::TSlot slot) {
            if (error) {
              setError(error);
              return;
            }
            if (error_) {
              return;
            }
            chunk->slot = std::move(slot);
            chunk->hostPtr = chunk->slot.get();
            chunk->ready = true;
            flushRecvPosts();
          });
    }
    flushRecvPosts();
  }

  // Inner recvs are posted strictly in chunk order (the inner channel pairs
  // sends and recvs by position), each as soon as its landing area exists.
  void flushRecvPosts() {
    while (!recvQueue_.empty() && recvQueue_.front()->ready && !error_) {
      auto chunk = recvQueue_.front();
      recvQueue_.pop_front();
      postInnerRecv(chunk->hostPtr, chunk->length, [this, chunk] {
        if (!chunk->slot) {
          chunkLanded(chunk->op); // host target: the bytes are where they belong
          return;
        }
        const HipBuffer hb = chunk->op->buffer.unwrap<HipBuffer>();
        PinnedRing& ring = bctx_->recvRing();
        const int device = hipDeviceForPointer(hb.ptr);
        int rc = tphip_copy(
            device,
            static_cast<uint8_t*>(hb.ptr) + chunk->offset,
            ring.devAddress(chunk->slot.get()),
            chunk->length,
            hb.stream);
        if (rc != 0) {
          setError(TP_CREATE_ERROR(HipError, "tphip_copy", rc));
          return;
        }
        auto ev = bctx_->events.get(device);
        ev->record(hb.stream);
        // The slot goes back to the ring when the copy has read it.
        watch(std::move(ev), [chunk] { chunk->slot.reset(); });
        chunkLanded(chunk->op);
      });
    }
  }

  template <typename F>
  void postInnerRecv(void* host, size_t len, F fn) {
    auto self = shared_from_this();
    cpuChannel_->recv(CpuBuffer{host}, len, [this, self, fn{std::move(fn)}](const Error& error) mutable {
      ctx_->defer([this, self, fn{std::move(fn)}, error]() mutable {
        setError(error);
        if (!error_) {
          fn();
        }
      });
    });
  }

  void chunkLanded(const std::shared_ptr<Op>& op) {
    if (op->done || --op->pending > 0) {
      return;
    }
    remove(op);
    finish(op);
  }

  // ---- helpers ----------------------------------------------------------------

  template <typename F>
  void watch(std::unique_ptr<HipEvent> ev, F fn) {
    auto self = shared_from_this();
    bctx_->poller.watch(
        std::move(ev), &bctx_->events, [this, self, fn{std::move(fn)}](const Error& error) mutable {
          ctx_->defer([this, self, fn{std::move(fn)}, error]() mutable {
            setError(error);
            fn(); // also on error: releases what the closure holds
          });
        });
  }

  void remove(const std::shared_ptr<Op>& op) {
    for (auto it = ops_.begin(); it != ops_.end(); ++it) {
      if (*it == op) {
        ops_.erase(it);
        return;
      }
    }
  }

  void finish(const std::shared_ptr<Op>& op) {
    if (op->done) {
      return;
    }
    op->done = true;
    auto cb = std::move(op->cb);
    cb(error_);
  }

  std::shared_ptr<BasicContextCore> bctx_;
  std::shared_ptr<transport::Connection> controlConnection_;
  std::shared_ptr<Channel> cpuChannel_;
  uint64_t chunkBytes_{0};
  std::vector<std::function<void()>> deferred_;
  std::deque<std::shared_ptr<Op>> ops_;
  std::deque<std::shared_ptr<SendChunk>> sendQueue_;
  std::deque<std::shared_ptr<RecvChunk>> recvQueue_;
};

class ContextImpl final : public Context {
 public:
  explicit ContextImpl(std::shared_ptr<Context> cpuContext) : cpuContext_(std::move(cpuContext)) {
    if (!cpuContext_->isViable()) {
      return;
    }
    const int n = hipDeviceCountNoThrow();
    if (n <= 0) {
      return;
    }
    const auto& inner = cpuContext_->deviceDescriptors();
    auto it = inner.find(Device{kCpuDeviceType, 0});
    if (it == inner.end()) {
      return;
    }
    // "<device type>|<inner descriptor>" for the CPU and for every GPU
    // (tensorpipe/channel/cuda_basic/context_impl.cc:27-93).
    descriptors_[Device{kCpuDeviceType, 0}] = kCpuDeviceType + "|" + it->second;
    for (int i = 0; i < n; ++i) {
      descriptors_[Device{kHipDeviceType, i}] = kHipDeviceType + "|" + it->second;
    }
    core_ = std::make_shared<BasicContextCore>();
  }
  ~ContextImpl() override {
    join();
  }
  bool isViable() const override {
    return core_ != nullptr;
  }
  size_t numConnectionsNeeded() const override {
    // One of our own plus whatever the wrapped channel wants
    // (tensorpipe/channel/cuda_basic/context_impl.cc:95-99).
    return 1 + cpuContext_->numConnectionsNeeded();
  }
  const std::unordered_map<Device, std::string>& deviceDescriptors() const override {
    return descriptors_;
  }
  // CPU-to-CPU is refused (a plain CPU channel should carry that); otherwise
  // the wrapped channel decides (tensorpipe/channel/cuda_basic/context_impl.cc:111-132).
  bool canCommunicateWithRemote(const std::string& local, const std::string& remote)
      const override {
    auto a = local.find('|');
    auto b = remote.find('|');
    if (a == std::string::npos || b == std::string::npos) {
      return false;
    }
    const std::string lt = local.substr(0, a), rt = remote.substr(0, b);
    if (lt == kCpuDeviceType && rt == kCpuDeviceType) {
      return false;
    }
    return cpuContext_->canCommunicateWithRemote(local.substr(a + 1), remote.substr(b + 1));
  }
  std::shared_ptr<Channel> createChannel(
      std::vector<std::shared_ptr<transport::Connection>> connections,
      Endpoint endpoint) override {
    if (!core_) {
      return std::make_shared<ChannelHandle<ChannelImpl>>(nullptr);
    }
    TP_THROW_ASSERT_IF(connections.size() != numConnectionsNeeded());
    // The last connection is ours, the others go to the wrapped channel
    // (tensorpipe/channel/cuda_basic/context_impl.cc:101-109).
    auto control = std::move(connections.back());
    connections.pop_back();
    auto cpuChannel = cpuContext_->createChannel(std::move(connections), endpoint);
    auto impl = std::make_shared<ChannelImpl>(
        core_, core_->nextChannelId(), std::move(control), std::move(cpuChannel));
    impl->init();
    return std::make_shared<ChannelHandle<ChannelImpl>>(std::move(impl));
  }
  void setId(std::string id) override {
    cpuContext_->setId(id + ".cpu");
    if (core_) {
      core_->setId(std::move(id));
    }
  }
  void close() override {
    if (core_) {
      core_->close();
    }
    cpuContext_->close();
  }
  void join() override {
    if (core_) {
      core_->join();
    }
    cpuContext_->join();
  }

 private:
  std::shared_ptr<Context> cpuContext_;
  std::shared_ptr<BasicContextCore> core_;
  std::unordered_map<Device, std::string> descriptors_;
};

} // namespace

std::shared_ptr<Context> create(std::shared_ptr<Context> cpuContext) {
  return std::make_shared<ContextImpl>(std::move(cpuContext));
}

} // namespace hip_basic
} // namespace channel
TP_AMD_NAMESPACE_END
