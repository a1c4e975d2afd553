// hip_basic: host-staged GPU channel that wraps a CPU channel.
//
// A tensor is cut into chunks of at most one staging slot and every chunk
// bounces through pinned host memory. Two routes, chosen per tensor by the
// sender and announced on the channel's control connection:
//
//  ring   (GPU source, both endpoints on one machine) The sender's pinned send
//         ring is exported once with a HIP IPC memory handle and mapped by the
//         receiver's GPU. Per chunk the sender's copy kernel stores GPU -> ring
//         slot and, once that has completed, a {slot, length} notification
//         goes over the control connection; the receiver's copy kernel then
//         loads ring slot -> GPU straight from the sender's pinned memory and
//         acknowledges the slot. The bytes cross the host link twice and are
//         never touched by a CPU; the two directions overlap, which is what
//         lets the path approach the PCIe rate.
//  stream (GPU source of more than one chunk, peer on this machine) The ring
//         route with the GPUs driving the ring themselves: the channel has a
//         pinned ring of its own, one kernel per tensor on the sender's GPU
//         pushes chunk after chunk into it and one kernel on the receiver's GPU
//         pulls them out, the two kept apart by a pair of counters beside the
//         slots (tphip_ring_push / tphip_ring_pull). Per tensor one route
//         message goes out and one "pulling" message comes back; no launch, no
//         polled event and no control message per chunk. The kernels run on
//         streams of the channel's own, never on the caller's: a kernel that
//         waits for the peer's progress there would hold the caller's later
//         work behind it. They give up after a bounded wait and are launched
//         again, so no kernel relies on another one running at the same time.
//  inner  (CPU source, or the ring could not be shared) What the reference
//         does for every chunk (tensorpipe/channel/cuda_basic/channel_impl.cc
//         :84-229 send, :335-506 recv): GPU -> pinned slot, the wrapped CPU
//         channel moves the slot to a pinned slot of the receiver, pinned
//         slot -> GPU. CPU-resident buffers skip the staging on their side,
//         so the channel also carries CPU<->GPU transfers.
//
// Geometry defaults follow tensorpipe/channel/cuda_basic/constants.h:22-24
// (16 slots of 1 MiB per ring); TP_HIP_BASIC_SLOT_BYTES and
// TP_HIP_BASIC_NUM_SLOTS override them per context. Copies are launches of the
// batched copy kernel instead of cudaMemcpyAsync, completion is detected by
// polling an event instead of a stream callback, and the reference's
// per-chunk "ready to send" message is replaced by a hello exchange (chunk
// size, ring handle) plus one route message per tensor.
//
// Callbacks: send fires once the last chunk has left the GPU (source
// reusable); recv fires once the last host-to-device copy has been enqueued
// (GPU target) or the last byte has landed (CPU target, and every target on
// the stream route, whose copies are not on the caller's stream).

#include <tensorpipe/channel/hip_basic/factory.h>

#include <algorithm>
#include <cstring>
#include <deque>
#include <map>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/channel/hip_common.h>
#include <tensorpipe/common/cpu_buffer.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/common/slot_allocator.h>
#include <tensorpipe/common/stage_timer.h>
#include <tensorpipe/common/wire.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_basic {

namespace {

// Both are read when a context is created.
size_t slotBytesFromEnv() {
  const char* e = std::getenv("TP_HIP_BASIC_SLOT_BYTES");
  size_t b = e != nullptr ? std::strtoull(e, nullptr, 10) : (1u << 20);
  b = b < 4096 ? size_t(4096) : b;
  return b > (size_t(1) << 30) ? (size_t(1) << 30) : b; // see numSlots below
}

size_t numSlotsFromEnv() {
  const char* e = std::getenv("TP_HIP_BASIC_NUM_SLOTS");
  size_t n = e != nullptr ? std::strtoull(e, nullptr, 10) : 16;
  return n < 1 ? size_t(1) : (n > 4096 ? size_t(4096) : n);
}

bool ringSharingDisabled() {
  const char* e = std::getenv("TP_HIP_BASIC_NO_SHARED_RING");
  return e != nullptr && e[0] == '1';
}

// TP_HIP_BASIC_GPU_RING=0 keeps every tensor on the host-driven routes.
bool gpuRingDisabled() {
  const char* e = std::getenv("TP_HIP_BASIC_GPU_RING");
  return e != nullptr && e[0] == '0';
}

// How long a ring kernel watches a counter that does not move before it leaves
// (and is launched again): long enough for the peer's kernel to be launched
// and start, short enough that a kernel whose peer cannot run meanwhile (two
// streams on one hardware queue) does not hold the GPU for long.
uint32_t ringYieldUs() {
  static const uint32_t v = [] {
    const char* e = std::getenv("TP_HIP_BASIC_RING_YIELD_US");
    const long us = e != nullptr ? std::atol(e) : 500;
    return static_cast<uint32_t>(us < 1 ? 1 : us);
  }();
  return v;
}

// The kernels of the stream route hand the ring over in pieces smaller than a
// slot: the pulling kernel can only start on a piece once all of it is there,
// and each workgroup moves whole pieces by itself, so the ring should hold a
// few dozen of them. A thirty-second of the ring, between 128 and 512 KiB
// (measured, 256 MiB through 4 slots, GB/s with 1 MiB / 4 MiB slots: pieces of
// 64 KiB 34.4 / 22.7, 128 KiB 38.7 / 21.2, 256 KiB 37.9 / 33.1, 512 KiB
// 35.7 / 45.1, 1 MiB 32.3 / 35.7; the host-driven route: 29.4 / 35.1).
// TP_HIP_BASIC_RING_PIECE_BYTES overrides the target.
size_t ringPieceBytes(size_t slotBytes, size_t numSlots) {
  static const size_t forced = [] {
    const char* e = std::getenv("TP_HIP_BASIC_RING_PIECE_BYTES");
    return e != nullptr ? std::strtoull(e, nullptr, 10) : size_t(0);
  }();
  size_t wanted = forced;
  if (wanted == 0) {
    wanted = slotBytes * numSlots / 32;
    wanted = std::min<size_t>(std::max<size_t>(wanted, size_t(128) << 10), size_t(512) << 10);
  }
  wanted = std::max<size_t>(wanted, 4096);
  size_t piece = slotBytes;
  while (piece > wanted && piece % 2 == 0 && (piece / 2) % 16 == 0) {
    piece /= 2;
  }
  return piece;
}

// Head of a stream ring's slab: the two counters the kernels of both sides
// share, then words of the owner's own.
constexpr size_t kRingHeaderBytes = 4096;
constexpr size_t kRingProducedAt = 0;
constexpr size_t kRingConsumedAt = 64;
constexpr size_t kRingStatusAt = 128;
constexpr size_t kRingAbortAt = 192;

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
  // A ring is mapped by the peer: the whole of it stays below 2 GiB (larger
  // mappings in a second process have been seen never to return).
  const size_t numSlots{std::max<size_t>(
      1, std::min<size_t>(numSlotsFromEnv(), ((size_t(2) << 30) - 1) / slotBytesFromEnv()))};
  const bool shareRing{!ringSharingDisabled()};

  // Loop only. The send ring exists from the first channel on (its handle is
  // part of the hello); the receive ring is created on first use, as the
  // reference allocates its pinned buffers lazily
  // (tensorpipe/channel/cuda_basic/context_impl.cc:134-154).
  PinnedRing& sendRing() {
    if (!sendRing_) {
      sendRing_ = std::make_unique<PinnedRing>(0, numSlots, slotBytes);
      if (shareRing &&
          tphip_ipc_mem_export(0, sendRing_->slab.host(), sendRingHandle_.data()) == 0) {
        sendRingExported_ = true;
      }
    }
    return *sendRing_;
  }
  bool sendRingExported() {
    sendRing();
    return sendRingExported_;
  }
  const HandleBytes& sendRingHandle() const {
    return sendRingHandle_;
  }
  PinnedRing& recvRing() {
    if (!recvRing_) {
      recvRing_ = std::make_unique<PinnedRing>(0, numSlots, slotBytes);
    }
    return *recvRing_;
  }
  // Stream for copies that belong to no caller stream (ring -> local pinned
  // slot on behalf of a CPU target).
  void* internalStream() {
    if (internalStream_ == nullptr) {
      TP_HIP_CHECK(tphip_stream_create(0, &internalStream_));
    }
    return internalStream_;
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
  HandleBytes sendRingHandle_{};

 public:
  // Names the send ring towards peers that map it.
  const uint64_t sendRingId{nextExportId()};

 private:
  bool sendRingExported_{false};
  void* internalStream_{nullptr};
};

enum MsgKind : uint8_t {
  kHello = 1,    // chunk size, slots, identities, ring handle
  kHelloAck = 2, // whether the peer's ring could be mapped
  kRoute = 3,    // start of a tensor: route and length
  kNotify = 4,   // ring route: chunk staged in {slot}
  kAck = 5,      // ring route: slot consumed
  kPulling = 6,  // stream route: the receiver's kernel for the next tensor has been launched
  kStaged = 7,   // inner route: {count} more chunks are on their way through the inner channel
};

enum Route : uint8_t { kRouteInner = 0, kRouteRing = 1, kRouteStream = 2 };

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

  // Every copy out of the peer's ring is followed by an event whose watcher
  // keeps this object alive, so nothing reads the mapping any more.
  ~ChannelImpl() override {
    if (remoteRing_ != nullptr) {
      HipIpcImports::get().release(0, remoteRingPeer_, remoteRingId_);
    }
    if (streamIn_.ring != nullptr) {
      HipIpcImports::get().release(0, remoteRingPeer_, streamIn_.ringId);
    }
    for (void* stream : {streamOut_.stream, streamIn_.stream}) {
      if (stream != nullptr) {
        tphip_stream_destroy(0, stream);
      }
    }
  }

 protected:
  void initFromLoop() override {
    WireWriter w;
    w.u8(kHello);
    w.u64(bctx_->slotBytes);
    w.u64(bctx_->numSlots);
    w.str(bootIdentity());
    w.str(processIdentity());
    bool exported = false;
    try {
      exported = bctx_->sendRingExported();
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " cannot create its send ring: " << ex.what();
      setError(TP_CREATE_ERROR(HipError, "tphip_host_alloc", TPHIP_ERR_INVALID_ARG));
      return;
    }
    w.u8(exported ? 1 : 0);
    if (exported) {
      w.u64(bctx_->sendRingId);
      w.raw(bctx_->sendRingHandle().data(), TPHIP_IPC_HANDLE_BYTES);
      w.u64(reinterpret_cast<uint64_t>(bctx_->sendRing().slab.host()));
      w.u64(bctx_->sendRing().slab.size());
    }
    writeMessage(*controlConnection_, std::move(w.bytes()));
    readControl();
  }

  void sendFromLoop(uint64_t seq, Buffer buffer, size_t length, TSendCallback cb) override {
    hipPointerCheckpoint(); // the caller's buffers: believed for this call only
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
    hipPointerCheckpoint(); // the caller's buffers: believed for this call only
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
    recvOps_.push_back(op);
    whenReady([this] { advanceRecvs(); });
  }

  void handleError() override {
    // Ring kernels that wait for the peer leave at their next look.
    if (streamOut_.slab) {
      __atomic_store_n(hostWord(streamOut_.slab->host(), kRingAbortAt), uint64_t(1), __ATOMIC_RELEASE);
    }
    if (streamIn_.own) {
      __atomic_store_n(hostWord(streamIn_.own->host(), kRingAbortAt), uint64_t(1), __ATOMIC_RELEASE);
    }
    streamOut_.jobs.clear();
    streamIn_.jobs.clear();
    controlConnection_->close();
    cpuChannel_->close();
    if (ctx_->closed()) {
      bctx_->closeRings();
    }
    deferred_.clear();
    sendQueue_.clear();
    recvPostQueue_.clear();
    innerAwaited_.clear();
    recvOps_.clear();
    inbox_.clear();
    slotsInFlight_.clear();
    stagePending_.clear();
    ringPending_.clear();
    auto ops = std::move(ops_);
    ops_.clear();
    for (auto& op : ops) {
      if (!op->kernelBusy) {
        finish(op);
      }
    }
  }

 private:
  struct Op {
    uint64_t seq;
    std::function<void(const Error&)> cb;
    Buffer buffer;
    size_t length{0};
    size_t pending{0};
    // recv side
    bool routed{false};
    uint8_t route{kRouteInner};
    size_t received{0}; // bytes of this tensor already handled (ring route)
    bool done{false};
    // A ring kernel is reading or writing the buffer: on error the callback,
    // which hands the buffer back, waits until that kernel has ended.
    bool kernelBusy{false};
  };

  // A chunk waiting for its turn: inner sends / control notifications must go
  // out in chunk order even if device-to-host copies finish out of order.
  struct SendChunk {
    void* hostPtr{nullptr};
    size_t length{0};
    SlotAllocator::TSlot slot;
    bool ready{false};
    bool ring{false};
    bool isRoute{false}; // not a chunk: the tensor's route message
    bool stream{false};  // ... of a tensor on the stream route: the push kernel follows it
    std::shared_ptr<Op> op;
  };

  // One tensor on the stream route, either side.
  struct RingJob {
    std::shared_ptr<Op> op;
    uint64_t index{0};    // among the channel's stream-route tensors of this direction
    uint64_t firstSeq{0}; // ring sequence number of its first chunk
    uint64_t chunks{0};
    uint64_t done{0};     // chunks complete
    bool launchedOnce{false};
    bool waitsForPeer{false}; // sender: gave up once before the receiver said it was pulling
  };

  // Sending end of the channel's own ring.
  struct StreamOut {
    std::unique_ptr<HipPinnedSlab> slab; // header page, then the slots
    std::unique_ptr<HipDeviceSlab> scratch;
    HandleBytes handle{};
    uint64_t id{0};
    bool announced{false};
    void* stream{nullptr};
    uint64_t pieceBytes{0}; // what the kernels call a slot
    uint32_t numPieces{0};
    uint64_t nextSeq{0};
    uint64_t nextIndex{0};
    uint64_t pullingSeen{0}; // kPulling messages so far
    std::deque<std::shared_ptr<RingJob>> jobs;
    bool running{false};
  };

  // Receiving end: the peer's ring as mapped here, and a page of this side's own.
  struct StreamIn {
    uint8_t* ring{nullptr};
    uint64_t ringId{0};
    uint64_t slotBytes{0};
    uint32_t numSlots{0};
    std::unique_ptr<HipPinnedSlab> own; // status and abort words
    std::unique_ptr<HipDeviceSlab> scratch;
    std::unique_ptr<HipPinnedSlab> bounce; // landing area for CPU targets, one ring's worth
    void* stream{nullptr};
    uint64_t nextSeq{0};
    uint64_t nextIndex{0};
    std::deque<std::shared_ptr<RingJob>> jobs;
    bool running{false};
  };

  static uint64_t* hostWord(uint8_t* base, size_t at) {
    return reinterpret_cast<uint64_t*>(base + at);
  }

  struct RecvChunk {
    void* hostPtr{nullptr};
    size_t length{0};
    size_t offset{0};
    SlotAllocator::TSlot slot;
    bool ready{false};
    std::shared_ptr<Op> op;
  };

  // A staging copy (GPU -> ring slot) waiting to be launched.
  struct StageItem {
    std::shared_ptr<SendChunk> chunk;
    tphip_copy_desc desc;
    void* stream;
    int device;
  };

  // A ring-route copy (peer's ring slot -> GPU) waiting to be launched.
  struct RingItem {
    std::shared_ptr<Op> op;
    uint32_t slot;
    tphip_copy_desc desc;
    void* stream;
    int device;
  };

  // A control message for the receive side, kept until a recv op consumes it.
  struct Incoming {
    uint8_t kind;
    uint8_t route;
    uint32_t slot;
    uint64_t length;
    // stream route, first tensor: where the sender's ring is
    bool announce{false};
    uint64_t ringId{0};
    HandleBytes handle{};
    uint64_t ringBase{0};
    uint64_t ringSize{0};
    uint64_t slotBytes{0};
    uint32_t numSlots{0};
  };

  void whenReady(std::function<void()> fn) {
    if (ready_) {
      fn();
    } else {
      deferred_.push_back(std::move(fn));
    }
  }

  static bool isCpu(const Buffer& b) {
    return b.device().type == kCpuDeviceType;
  }

  // ---- control connection -----------------------------------------------------

  void readControl() {
    controlConnection_->read(onReadMessage([this](std::vector<uint8_t> bytes) {
      if (error_) {
        return;
      }
      onControl(bytes);
      if (!error_) {
        readControl();
      }
    }));
  }

  void onControl(const std::vector<uint8_t>& bytes) {
    WireReader r(bytes.data(), bytes.size());
    const uint8_t kind = r.u8();
    if (kind == kHello) {
      const uint64_t remoteSlot = r.u64();
      const uint64_t remoteSlots = r.u64();
      const std::string boot = r.str();
      const std::string process = r.str();
      const bool hasHandle = r.u8() != 0;
      if (!r.ok() || remoteSlot == 0) {
        failProtocol();
        return;
      }
      chunkBytes_ = std::min<uint64_t>(remoteSlot, bctx_->slotBytes);
      remoteSlotBytes_ = remoteSlot;
      remoteNumSlots_ = remoteSlots;
      bool mapped = false;
      if (hasHandle) {
        const uint64_t ringId = r.u64();
        HandleBytes h;
        r.raw(h.data(), h.size());
        const uint64_t ringBase = r.u64();
        const uint64_t ringSize = r.u64();
        // Map the peer's send ring if it lives on this machine in another
        // process; otherwise its chunks come through the inner channel.
        // (a ring smaller than the geometry it was announced with is not mapped)
        if (r.ok() && bctx_->shareRing && boot == bootIdentity() && process != processIdentity() &&
            remoteSlots != 0 && remoteSlot <= ringSize / remoteSlots) {
          void* ptr = nullptr;
          if (HipIpcImports::get().acquire(0, process, ringId, h, ringBase, ringSize, &ptr) == 0) {
            remoteRingPeer_ = process;
            remoteRingId_ = ringId;
            remoteRing_ = static_cast<uint8_t*>(ptr);
            mapped = true;
          }
        }
      }
      WireWriter w;
      w.u8(kHelloAck);
      w.u8(mapped ? 1 : 0);
      writeMessage(*controlConnection_, std::move(w.bytes()));
      gotHello_ = true;
    } else if (kind == kHelloAck) {
      peerMappedOurRing_ = r.u8() != 0;
      gotHelloAck_ = true;
    } else if (kind == kAck) {
      TP_MARK("basic: acknowledgement arrived");
      const uint32_t count = r.u32();
      for (uint32_t i = 0; i < count; ++i) {
        const uint32_t slot = r.u32();
        auto it = slotsInFlight_.find(slot);
        if (!r.ok() || it == slotsInFlight_.end()) {
          failProtocol();
          return;
        }
        TP_VLOG(7) << "Channel " << id_ << " got ack for slot " << slot;
        slotsInFlight_.erase(it); // drops the slot back into the ring
      }
    } else if (kind == kRoute) {
      Incoming in{};
      in.kind = kind;
      in.route = r.u8();
      in.length = r.u64();
      if (in.route == kRouteStream) {
        in.announce = r.u8() != 0;
        if (in.announce) {
          in.ringId = r.u64();
          r.raw(in.handle.data(), in.handle.size());
          in.ringBase = r.u64();
          in.ringSize = r.u64();
          in.slotBytes = r.u64();
          in.numSlots = r.u32();
        }
      }
      if (!r.ok()) {
        failProtocol();
        return;
      }
      inbox_.push_back(in);
      advanceRecvs();
    } else if (kind == kPulling) {
      ++streamOut_.pullingSeen;
      pumpStreamOut();
    } else if (kind == kStaged) {
      const uint32_t count = r.u32();
      if (!r.ok() || count == 0) {
        failProtocol();
        return;
      }
      innerChunksOnTheirWay_ += count;
      admitInnerChunks();
    } else if (kind == kNotify) {
      const uint32_t count = r.u32();
      for (uint32_t i = 0; i < count; ++i) {
        Incoming in{};
        in.kind = kind;
        in.slot = r.u32();
        in.length = r.u64();
        if (!r.ok()) {
          failProtocol();
          return;
        }
        inbox_.push_back(in);
      }
      advanceRecvs();
    } else {
      failProtocol();
      return;
    }
    if (!ready_ && gotHello_ && gotHelloAck_) {
      ready_ = true;
      TP_VLOG(5) << "Channel " << id_ << " ready: chunk " << chunkBytes_ << " B, ring route "
                 << (peerMappedOurRing_ ? "on" : "off") << " for sends, "
                 << (remoteRing_ != nullptr ? "on" : "off") << " for recvs";
      auto deferred = std::move(deferred_);
      deferred_.clear();
      for (auto& fn : deferred) {
        fn();
      }
    }
  }

  void failProtocol() {
    setError(TP_CREATE_ERROR(ShortReadError, -1, -1));
  }

  // ---- send -------------------------------------------------------------------

  void startSend(const std::shared_ptr<Op>& op) {
    if (error_) {
      return;
    }
    const bool cpuSource = isCpu(op->buffer);
    const bool ring = !cpuSource && peerMappedOurRing_;
    // (a ring that the runtime's copy engine is asked to fill cannot be driven by kernels)
    if (ring && op->length > chunkBytes_ && !gpuRingDisabled() && engine() == Engine::kKernel &&
        streamOutReady()) {
      startStreamSend(op);
      return;
    }
    {
      // The route message takes its place in the queue: it must reach the peer
      // after the last notification of the previous tensor.
      auto marker = std::make_shared<SendChunk>();
      marker->isRoute = true;
      marker->ring = ring;
      marker->length = op->length;
      marker->ready = true;
      sendQueue_.push_back(marker);
    }
    const size_t chunks = (op->length + chunkBytes_ - 1) / chunkBytes_;
    op->pending = chunks; // chunks whose source bytes are still needed
    for (size_t k = 0; k < chunks; ++k) {
      const size_t offset = k * chunkBytes_;
      const size_t len = std::min<size_t>(op->length - offset, chunkBytes_);
      auto chunk = std::make_shared<SendChunk>();
      chunk->length = len;
      chunk->op = op;
      chunk->ring = ring;
      sendQueue_.push_back(chunk);
      if (cpuSource) {
        // Host source: no staging (tensorpipe/channel/cuda_basic/channel_impl.cc:138-145).
        chunk->hostPtr = static_cast<uint8_t*>(op->buffer.unwrap<CpuBuffer>().ptr) + offset;
        chunk->ready = true;
        continue;
      }
      const HipBuffer hb = op->buffer.unwrap<HipBuffer>();
      auto self = shared_from_this();
      PinnedRing& sring = bctx_->sendRing();
      sring.allocator.alloc([this, self, chunk, hb, offset, len, &sring](
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
        TP_VLOG(7) << "Channel " << id_ << " stages " << len << " B at offset " << offset;
        // Launched together with every other chunk that gets its slot in this
        // turn of the loop: one kernel and one event for all of them.
        stagePending_.push_back(StageItem{
            chunk,
            tphip_copy_desc{
                static_cast<const uint8_t*>(hb.ptr) + offset,
                sring.devAddress(chunk->slot.get()),
                len},
            hb.stream,
            hipDeviceForPointer(hb.ptr)});
        scheduleLaunches();
      });
    }
    flushSends();
  }

  // Copies queued during one turn of the loop are launched together at its
  // end: a burst of freed slots or of notifications costs one kernel launch
  // and one event per stream instead of one per chunk.
  void scheduleLaunches() {
    if (launchScheduled_) {
      return;
    }
    launchScheduled_ = true;
    auto self = shared_from_this();
    ctx_->defer([this, self] {
      launchScheduled_ = false;
      if (error_) {
        stagePending_.clear();
        ringPending_.clear();
        return;
      }
      launchStaging();
      launchRingCopies();
    });
  }

  void launchStaging() {
    while (!stagePending_.empty()) {
      // One launch per (device, stream); normally there is only one.
      void* stream = stagePending_.front().stream;
      const int device = stagePending_.front().device;
      std::vector<tphip_copy_desc> table;
      std::vector<std::shared_ptr<SendChunk>> chunks;
      const size_t cap = batchCap(bctx_->numSlots, bctx_->slotBytes);
      for (auto it = stagePending_.begin(); it != stagePending_.end() && table.size() < cap;) {
        if (it->stream == stream && it->device == device) {
          table.push_back(it->desc);
          chunks.push_back(std::move(it->chunk));
          it = stagePending_.erase(it);
        } else {
          ++it;
        }
      }
      auto ev = bctx_->events.get(device, stream);
      if (!launchHostLinkCopy(device, stream, table, /*towardsHost=*/true, *ev)) {
        return;
      }
      TP_MARK("basic: chunk staged towards the host (launched)");
      watch(std::move(ev), [this, chunks{std::move(chunks)}] {
        TP_MARK("basic: staging seen finished");
        for (auto& c : chunks) {
          c->ready = true;
        }
        flushSends();
      });
    }
  }

  // Chunks per launch. One launch for the whole ring would put the two ends in
  // lock step (the sender stages all slots, then idles while the receiver
  // drains all of them); a quarter of the ring per launch keeps both ends busy
  // on different slots. Measured, 256 MiB each way: 4 x 1 MiB slots 29 GB/s with
  // one slot per launch against 22 with two and 20 with four; 16 x 1 MiB 29.5
  // with four per launch against 28.5 with one; 4 MiB slots are best alone (36).
  static size_t batchCap(size_t numSlots, size_t slotBytes) {
    static const long forced = [] {
      const char* e = std::getenv("TP_HIP_BASIC_BATCH_CAP");
      return e != nullptr ? std::atol(e) : 0L;
    }();
    if (forced > 0) {
      return static_cast<size_t>(forced);
    }
    if (slotBytes >= (2u << 20)) {
      return 1; // a slot this large amortises its launch by itself
    }
    return std::max<size_t>(1, numSlots / 4);
  }

  // A copy with one end in pinned host memory: the host link saturates with
  // about 32 workgroups, more only add contention (50 vs 42 GB/s reading
  // alone; with the other direction busy 64 workgroups lose 1-5 GB/s).
  // TP_HIP_BASIC_ENGINE chooses who moves the bytes, for comparison: "kernel"
  // (default: the copy kernel in both directions), "sdma" (the runtime's
  // hipMemcpyAsync in both) or "mixed" (kernel towards the host, the runtime's
  // copy from it).
  enum class Engine { kKernel, kSdma, kMixed };
  static Engine engine() {
    static const Engine chosen = [] {
      const char* e = std::getenv("TP_HIP_BASIC_ENGINE");
      if (e != nullptr && std::strcmp(e, "sdma") == 0) {
        return Engine::kSdma;
      }
      if (e != nullptr && std::strcmp(e, "mixed") == 0) {
        return Engine::kMixed;
      }
      return Engine::kKernel;
    }();
    return chosen;
  }

  // `done` ends up behind the copy on `stream`.
  bool launchHostLinkCopy(
      int device,
      void* stream,
      const std::vector<tphip_copy_desc>& table,
      bool towardsHost,
      HipEvent& done) {
    const Engine how = engine();
    try {
      if (how == Engine::kSdma || (how == Engine::kMixed && !towardsHost)) {
        for (const auto& d : table) {
          TP_HIP_CHECK(tphip_memcpy_async(device, d.dst, d.src, d.bytes, stream));
        }
        done.record(stream);
        return true;
      }
      static const long forcedBlocks = [] {
        const char* e = std::getenv("TP_HIP_BASIC_BLOCKS");
        return e != nullptr ? std::atol(e) : 0L;
      }();
      const uint32_t blocks = forcedBlocks > 0 ? static_cast<uint32_t>(forcedBlocks) : 32;
      // a marker behind the kernel: signalling from the kernel gains nothing measurable per chunk
      hipBatchedCopy(device, stream, table, done, /*signalOnKernel=*/false, blocks, 3);
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " host-link copy failed: " << ex.what();
      setError(TP_CREATE_ERROR(HipError, "hip_basic copy", TPHIP_ERR_INVALID_ARG));
      return false;
    }
    return true;
  }

  void flushSends() {
    std::vector<std::pair<uint32_t, uint64_t>> notifies;
    auto flushNotifies = [&] {
      if (notifies.empty()) {
        return;
      }
      WireWriter w;
      w.u8(kNotify);
      w.u32(static_cast<uint32_t>(notifies.size()));
      for (auto& n : notifies) {
        w.u32(n.first);
        w.u64(n.second);
      }
      writeMessage(*controlConnection_, std::move(w.bytes()));
      TP_MARK("basic: notification written");
      notifies.clear();
    };
    while (!sendQueue_.empty() && sendQueue_.front()->ready && !error_) {
      auto chunk = sendQueue_.front();
      sendQueue_.pop_front();
      if (chunk->isRoute && chunk->stream) {
        flushNotifies();
        routeStreamTensor(chunk->op);
        continue;
      }
      if (chunk->isRoute) {
        flushNotifies();
        WireWriter w;
        w.u8(kRoute);
        w.u8(chunk->ring ? kRouteRing : kRouteInner);
        w.u64(chunk->length);
        writeMessage(*controlConnection_, std::move(w.bytes()));
        continue;
      }
      if (chunk->ring) {
        // The bytes sit in our pinned ring, which the peer's GPU has mapped:
        // tell it where; the slot comes back with the ack.
        const uint32_t slotIdx =
            static_cast<uint32_t>(bctx_->sendRing().allocator.slotIndex(chunk->slot.get()));
        slotsInFlight_[slotIdx] = std::move(chunk->slot);
        TP_VLOG(7) << "Channel " << id_ << " notifies slot " << slotIdx << " (" << chunk->length
                   << " B)";
        notifies.emplace_back(slotIdx, chunk->length);
        sourceDone(chunk->op);
        continue;
      }
      flushNotifies();
      auto self = shared_from_this();
      const bool staged = static_cast<bool>(chunk->slot);
      if (staged) {
        sourceDone(chunk->op); // the bytes now live in the pinned slot
      }
      ++stagedToAnnounce_;
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
    flushNotifies();
    if (stagedToAnnounce_ > 0 && !error_) {
      // The receiver takes a landing slot for a chunk only once the chunk is on
      // its way (tensorpipe/channel/cuda_basic/channel_impl.cc:152-166,413-441:
      // ready-to-send first, the receive buffer after it). A receiver that took
      // its slots when the recv was posted would hold them while waiting for
      // sends that may themselves be waiting, for send slots held by another
      // channel of this context whose receiver finds no landing slot: with two
      // channels sharing the contexts' rings that is a deadlock.
      WireWriter w;
      w.u8(kStaged);
      w.u32(stagedToAnnounce_);
      stagedToAnnounce_ = 0;
      writeMessage(*controlConnection_, std::move(w.bytes()));
    }
  }

  void sourceDone(const std::shared_ptr<Op>& op) {
    if (op->done || --op->pending > 0) {
      return;
    }
    remove(op);
    finish(op);
  }

  // ---- recv -------------------------------------------------------------------

  // Feed control messages to the recv ops, strictly in order.
  void advanceRecvs() {
    while (ready_ && !error_ && !recvOps_.empty() && !inbox_.empty()) {
      auto op = recvOps_.front();
      const Incoming in = inbox_.front();
      if (!op->routed) {
        if (in.kind != kRoute || in.length != op->length) {
          failProtocol();
          return;
        }
        inbox_.pop_front();
        op->routed = true;
        op->route = in.route;
        const size_t chunks = (op->length + chunkBytes_ - 1) / chunkBytes_;
        op->pending = chunks; // chunks not yet landed (CPU) / enqueued (GPU)
        if (op->route == kRouteStream) {
          recvOps_.pop_front();
          if (!startStreamRecv(op, in)) {
            return;
          }
        } else if (op->route == kRouteInner) {
          recvOps_.pop_front();
          startInnerRecv(op);
        } else if (remoteRing_ == nullptr) {
          failProtocol();
          return;
        }
        continue;
      }
      // Ring route: one notification per chunk.
      if (in.kind != kNotify) {
        failProtocol();
        return;
      }
      inbox_.pop_front();
      const size_t offset = op->received;
      const size_t expect = std::min<size_t>(op->length - offset, chunkBytes_);
      if (in.length != expect || in.slot >= remoteNumSlots_) {
        failProtocol();
        return;
      }
      op->received += in.length;
      if (op->received == op->length) {
        recvOps_.pop_front();
      }
      ringChunkArrived(op, in.slot, offset, in.length);
    }
  }

  void ringChunkArrived(const std::shared_ptr<Op>& op, uint32_t slot, size_t offset, size_t len) {
    const uint8_t* remote = remoteRing_ + static_cast<size_t>(slot) * remoteSlotBytes_;
    TP_VLOG(7) << "Channel " << id_ << " got notification for slot " << slot << " (" << len
               << " B)";
    TP_MARK("basic: notification arrived");
    if (!isCpu(op->buffer)) {
      const HipBuffer hb = op->buffer.unwrap<HipBuffer>();
      ringPending_.push_back(RingItem{
          op,
          slot,
          tphip_copy_desc{remote, static_cast<uint8_t*>(hb.ptr) + offset, len},
          hb.stream,
          hipDeviceForPointer(hb.ptr)});
      scheduleLaunches();
      return;
    }
    // CPU target: the mapping of the peer's ring is only addressable by the
    // GPU, so the GPU moves the chunk into a local pinned slot first.
    auto self = shared_from_this();
    PinnedRing& rring = bctx_->recvRing();
    rring.allocator.alloc([this, self, op, remote, slot, offset, len, &rring](
                              const Error& error, SlotAllocator::TSlot local) {
      if (error) {
        setError(error);
        return;
      }
      if (error_) {
        return;
      }
      void* stream = nullptr;
      try {
        stream = bctx_->internalStream();
      } catch (const std::exception&) {
        setError(TP_CREATE_ERROR(HipError, "tphip_stream_create", TPHIP_ERR_INVALID_ARG));
        return;
      }
      auto ev = bctx_->events.get(0, stream);
      if (!launchHostLinkCopy(
              0,
              stream,
              {tphip_copy_desc{remote, rring.devAddress(local.get()), len}},
              /*towardsHost=*/true,
              *ev)) {
        return;
      }
      watch(std::move(ev), [this, op, slot, offset, len, local] {
        if (error_) {
          return;
        }
        ackSlot(slot);
        std::memcpy(
            static_cast<uint8_t*>(op->buffer.unwrap<CpuBuffer>().ptr) + offset, local.get(), len);
        chunkLanded(op);
      });
    });
  }

  void launchRingCopies() {
    while (!ringPending_.empty()) {
      void* stream = ringPending_.front().stream;
      const int device = ringPending_.front().device;
      std::vector<tphip_copy_desc> table;
      std::vector<uint32_t> slots;
      std::vector<std::shared_ptr<Op>> ops;
      const size_t cap = batchCap(remoteNumSlots_, remoteSlotBytes_);
      for (auto it = ringPending_.begin(); it != ringPending_.end() && table.size() < cap;) {
        if (it->stream == stream && it->device == device) {
          table.push_back(it->desc);
          slots.push_back(it->slot);
          ops.push_back(std::move(it->op));
          it = ringPending_.erase(it);
        } else {
          ++it;
        }
      }
      auto ev = bctx_->events.get(device, stream);
      if (!launchHostLinkCopy(device, stream, table, /*towardsHost=*/false, *ev)) {
        return;
      }
      TP_MARK("basic: chunk copied from the ring (launched)");
      // The slots go back to the sender when the copy has read them.
      watch(std::move(ev), [this, slots{std::move(slots)}] {
        TP_MARK("basic: ring copy seen finished");
        ackSlots(slots);
      });
      for (auto& op : ops) {
        chunkLanded(op); // enqueued on the caller's stream
      }
    }
  }

  void ackSlot(uint32_t slot) {
    ackSlots(std::vector<uint32_t>{slot});
  }

  void ackSlots(const std::vector<uint32_t>& slots) {
    if (error_) {
      return;
    }
    WireWriter w;
    w.u8(kAck);
    w.u32(static_cast<uint32_t>(slots.size()));
    for (uint32_t slot : slots) {
      TP_VLOG(7) << "Channel " << id_ << " acks slot " << slot;
      w.u32(slot);
    }
    writeMessage(*controlConnection_, std::move(w.bytes()));
    TP_MARK("basic: acknowledgement written");
  }

  void startInnerRecv(const std::shared_ptr<Op>& op) {
    const size_t chunks = (op->length + chunkBytes_ - 1) / chunkBytes_;
    for (size_t k = 0; k < chunks; ++k) {
      const size_t offset = k * chunkBytes_;
      const size_t len = std::min<size_t>(op->length - offset, chunkBytes_);
      auto chunk = std::make_shared<RecvChunk>();
      chunk->length = len;
      chunk->offset = offset;
      chunk->op = op;
      innerAwaited_.push_back(std::move(chunk));
    }
    admitInnerChunks();
  }

  // A chunk gets its landing area, and its inner recv, once the sender has said
  // that it is on its way (kStaged), in chunk order.
  void admitInnerChunks() {
    while (innerChunksOnTheirWay_ > 0 && !innerAwaited_.empty() && !error_) {
      --innerChunksOnTheirWay_;
      auto chunk = innerAwaited_.front();
      innerAwaited_.pop_front();
      recvPostQueue_.push_back(chunk);
      if (isCpu(chunk->op->buffer)) {
        chunk->hostPtr = static_cast<uint8_t*>(chunk->op->buffer.unwrap<CpuBuffer>().ptr) + chunk->offset;
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
    while (!recvPostQueue_.empty() && recvPostQueue_.front()->ready && !error_) {
      auto chunk = recvPostQueue_.front();
      recvPostQueue_.pop_front();
      auto self = shared_from_this();
      cpuChannel_->recv(
          CpuBuffer{chunk->hostPtr}, chunk->length, [this, self, chunk](const Error& error) {
            ctx_->defer([this, self, chunk, error] {
              setError(error);
              if (!error_) {
                innerChunkArrived(chunk);
              }
            });
          });
    }
  }

  void innerChunkArrived(const std::shared_ptr<RecvChunk>& chunk) {
    if (!chunk->slot) {
      chunkLanded(chunk->op); // host target: the bytes are where they belong
      return;
    }
    const HipBuffer hb = chunk->op->buffer.unwrap<HipBuffer>();
    PinnedRing& rring = bctx_->recvRing();
    const int device = hipDeviceForPointer(hb.ptr);
    auto ev = bctx_->events.get(device, hb.stream);
    if (!launchHostLinkCopy(
            device,
            hb.stream,
            {tphip_copy_desc{
                rring.devAddress(chunk->slot.get()),
                static_cast<uint8_t*>(hb.ptr) + chunk->offset,
                chunk->length}},
            /*towardsHost=*/false,
            *ev)) {
      return;
    }
    // The slot goes back to the ring when the copy has read it.
    watch(std::move(ev), [chunk] { chunk->slot.reset(); });
    chunkLanded(chunk->op);
  }

  void chunkLanded(const std::shared_ptr<Op>& op) {
    if (op->done || --op->pending > 0) {
      return;
    }
    remove(op);
    finish(op);
  }


  // ---- stream route: the GPUs drive the channel's own ring -------------------------

  // Creates this channel's ring on first use. False: stay on the other routes.
  bool streamOutReady() {
    StreamOut& so = streamOut_;
    if (so.slab) {
      return true;
    }
    if (streamOutFailed_) {
      return false;
    }
    try {
      auto slab = std::make_unique<HipPinnedSlab>(0, kRingHeaderBytes + bctx_->numSlots * bctx_->slotBytes);
      std::memset(slab->host(), 0, kRingHeaderBytes);
      HandleBytes handle{};
      TP_HIP_CHECK(tphip_ipc_mem_export(0, slab->host(), handle.data()));
      const uint64_t pieceBytes = ringPieceBytes(bctx_->slotBytes, bctx_->numSlots);
      const uint32_t numPieces = static_cast<uint32_t>(bctx_->numSlots * (bctx_->slotBytes / pieceBytes));
      auto scratch = std::make_unique<HipDeviceSlab>(0, tphip_ring_scratch_bytes(numPieces));
      void* stream = nullptr;
      TP_HIP_CHECK(tphip_stream_create(0, &stream));
      TP_HIP_CHECK(tphip_fill(0, scratch->ptr(), 0, scratch->size(), stream));
      TP_HIP_CHECK(tphip_stream_sync(0, stream));
      so.slab = std::move(slab);
      so.scratch = std::move(scratch);
      so.handle = handle;
      so.id = nextExportId();
      so.stream = stream;
      so.pieceBytes = pieceBytes;
      so.numPieces = numPieces;
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " cannot set up its own ring: " << ex.what();
      streamOutFailed_ = true;
      return false;
    }
    return true;
  }

  // The tensor keeps its place among the channel's sends: its route message
  // goes out in order, once everything queued on the source's stream has run
  // (a pull kernel of the peer then never waits for the caller's own work).
  void startStreamSend(const std::shared_ptr<Op>& op) {
    auto marker = std::make_shared<SendChunk>();
    marker->isRoute = true;
    marker->stream = true;
    marker->ring = true;
    marker->length = op->length;
    marker->op = op;
    op->pending = 1;
    sendQueue_.push_back(marker);
    const HipBuffer hb = op->buffer.unwrap<HipBuffer>();
    const int device = hipDeviceForPointer(hb.ptr);
    try {
      auto ev = bctx_->events.get(device, hb.stream);
      ev->record(hb.stream);
      watch(std::move(ev), [this, marker] {
        marker->ready = true;
        flushSends();
      });
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " cannot order a send behind its stream: " << ex.what();
      setError(TP_CREATE_ERROR(HipError, "hip_basic stream route", TPHIP_ERR_INVALID_ARG));
    }
  }

  // From flushSends(), in the tensor's turn.
  void routeStreamTensor(const std::shared_ptr<Op>& op) {
    StreamOut& so = streamOut_;
    auto job = std::make_shared<RingJob>();
    job->op = op;
    job->index = so.nextIndex++;
    job->firstSeq = so.nextSeq;
    job->chunks = (op->length + so.pieceBytes - 1) / so.pieceBytes;
    so.nextSeq += job->chunks;
    WireWriter w;
    w.u8(kRoute);
    w.u8(kRouteStream);
    w.u64(op->length);
    w.u8(so.announced ? 0 : 1);
    if (!so.announced) {
      so.announced = true;
      w.u64(so.id);
      w.raw(so.handle.data(), so.handle.size());
      w.u64(reinterpret_cast<uint64_t>(so.slab->host()));
      w.u64(so.slab->size());
      w.u64(so.pieceBytes);
      w.u32(so.numPieces);
    }
    writeMessage(*controlConnection_, std::move(w.bytes()));
    TP_MARK("basic: stream route announced");
    so.jobs.push_back(std::move(job));
    pumpStreamOut();
  }

  // One push kernel at a time, for the oldest tensor that still has chunks to push.
  void pumpStreamOut() {
    StreamOut& so = streamOut_;
    if (so.running || so.jobs.empty() || error_) {
      return;
    }
    auto job = so.jobs.front();
    if (job->waitsForPeer && so.pullingSeen <= job->index) {
      return; // the ring is full and nobody pulls yet: kPulling launches the next one
    }
    const HipBuffer hb = job->op->buffer.unwrap<HipBuffer>();
    const uint64_t offset = job->done * so.pieceBytes;
    tphip_ring_end end{};
    end.slots = so.slab->dev() + kRingHeaderBytes;
    end.slot_bytes = so.pieceBytes;
    end.num_slots = so.numPieces;
    end.produced = so.slab->dev() + kRingProducedAt;
    end.consumed = so.slab->dev() + kRingConsumedAt;
    end.scratch = so.scratch->ptr();
    end.status = so.slab->dev() + kRingStatusAt;
    end.abort = so.slab->dev() + kRingAbortAt;
    try {
      auto ev = bctx_->events.get(0, so.stream);
      TP_HIP_CHECK(tphip_ring_push(
          0, &end, static_cast<const uint8_t*>(hb.ptr) + offset, job->op->length - offset,
          job->firstSeq + job->done, ringYieldUs(), 0, so.stream, ev->raw()));
      so.running = true;
      job->launchedOnce = true;
      job->op->kernelBusy = true;
      TP_MARK("basic: push kernel launched");
      watch(std::move(ev), [this, job] { onPushEnded(job); });
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " push kernel failed: " << ex.what();
      setError(TP_CREATE_ERROR(HipError, "tphip_ring_push", TPHIP_ERR_INVALID_ARG));
    }
  }

  void onPushEnded(const std::shared_ptr<RingJob>& job) {
    StreamOut& so = streamOut_;
    so.running = false;
    job->op->kernelBusy = false;
    if (error_) {
      finish(job->op);
      return;
    }
    const uint64_t status = __atomic_load_n(hostWord(so.slab->host(), kRingStatusAt), __ATOMIC_ACQUIRE);
    const uint64_t seq = status & ~TPHIP_RING_YIELDED;
    if (seq < job->firstSeq + job->done || seq > job->firstSeq + job->chunks) {
      failProtocol();
      return;
    }
    job->done = seq - job->firstSeq;
    TP_MARK("basic: push kernel ended");
    if (job->done == job->chunks) {
      so.jobs.pop_front();
      sourceDone(job->op); // every byte is in the ring: the source is the caller's again
    } else if (so.pullingSeen <= job->index) {
      job->waitsForPeer = true;
    }
    pumpStreamOut();
  }

  // The receiving side of a tensor on the stream route. False: the channel failed.
  bool startStreamRecv(const std::shared_ptr<Op>& op, const Incoming& in) {
    StreamIn& si = streamIn_;
    if (in.announce) {
      // (same conditions as for the context's ring in the hello)
      void* ptr = nullptr;
      if (si.ring != nullptr || remoteRing_ == nullptr || in.numSlots == 0 || in.slotBytes == 0 ||
          in.slotBytes % 16 != 0 || in.ringSize < kRingHeaderBytes ||
          in.slotBytes > (in.ringSize - kRingHeaderBytes) / in.numSlots ||
          HipIpcImports::get().acquire(
              0, remoteRingPeer_, in.ringId, in.handle, in.ringBase, in.ringSize, &ptr) != 0) {
        failProtocol();
        return false;
      }
      si.ring = static_cast<uint8_t*>(ptr);
      si.ringId = in.ringId;
      si.slotBytes = in.slotBytes;
      si.numSlots = in.numSlots;
      try {
        si.own = std::make_unique<HipPinnedSlab>(0, kRingHeaderBytes);
        std::memset(si.own->host(), 0, kRingHeaderBytes);
        si.scratch = std::make_unique<HipDeviceSlab>(0, tphip_ring_scratch_bytes(si.numSlots));
        TP_HIP_CHECK(tphip_stream_create(0, &si.stream));
        TP_HIP_CHECK(tphip_fill(0, si.scratch->ptr(), 0, si.scratch->size(), si.stream));
        TP_HIP_CHECK(tphip_stream_sync(0, si.stream));
      } catch (const std::exception& ex) {
        TP_LOG_WARNING() << "Channel " << id_ << " cannot set up its end of the peer's ring: " << ex.what();
        setError(TP_CREATE_ERROR(HipError, "hip_basic stream route", TPHIP_ERR_INVALID_ARG));
        return false;
      }
    } else if (si.ring == nullptr) {
      failProtocol();
      return false;
    }
    auto job = std::make_shared<RingJob>();
    job->op = op;
    job->index = si.nextIndex++;
    job->firstSeq = si.nextSeq;
    job->chunks = (op->length + si.slotBytes - 1) / si.slotBytes;
    si.nextSeq += job->chunks;
    op->pending = 1;
    si.jobs.push_back(std::move(job));
    pumpStreamIn();
    return !error_;
  }

  // One pull kernel at a time, for the oldest tensor that still has chunks in the ring.
  void pumpStreamIn() {
    StreamIn& si = streamIn_;
    if (si.running || si.jobs.empty() || error_) {
      return;
    }
    auto job = si.jobs.front();
    const uint64_t offset = job->done * si.slotBytes;
    uint64_t bytes = job->op->length - offset;
    uint8_t* target = nullptr;
    const bool toCpu = isCpu(job->op->buffer);
    tphip_ring_end end{};
    end.slots = si.ring + kRingHeaderBytes;
    end.slot_bytes = si.slotBytes;
    end.num_slots = si.numSlots;
    end.produced = si.ring + kRingProducedAt;
    end.consumed = si.ring + kRingConsumedAt;
    try {
      if (toCpu) {
        // The GPU cannot write the caller's memory: a ring's worth at a time
        // lands in pinned memory of the channel's and is copied on from there.
        if (!si.bounce) {
          si.bounce = std::make_unique<HipPinnedSlab>(0, si.numSlots * si.slotBytes);
        }
        bytes = std::min<uint64_t>(bytes, si.numSlots * si.slotBytes);
        target = si.bounce->dev();
      } else {
        const HipBuffer hb = job->op->buffer.unwrap<HipBuffer>();
        target = static_cast<uint8_t*>(hb.ptr) + offset;
        if (!job->launchedOnce) {
          // The kernel may touch the target once everything the receiver had
          // queued on the buffer's stream before recv() is done.
          const int device = hipDeviceForPointer(hb.ptr);
          auto ready = bctx_->events.get(device, hb.stream);
          ready->record(hb.stream);
          ready->wait(si.stream, 0);
          bctx_->events.put(std::move(ready)); // the wait captured the record
        }
      }
      end.scratch = si.scratch->ptr();
      end.status = si.own->dev() + kRingStatusAt;
      end.abort = si.own->dev() + kRingAbortAt;
      auto ev = bctx_->events.get(0, si.stream);
      TP_HIP_CHECK(tphip_ring_pull(
          0, &end, target, bytes, job->firstSeq + job->done, ringYieldUs(), 0, si.stream, ev->raw()));
      si.running = true;
      job->op->kernelBusy = true;
      TP_MARK("basic: pull kernel launched");
      if (!job->launchedOnce) {
        job->launchedOnce = true;
        WireWriter w;
        w.u8(kPulling);
        writeMessage(*controlConnection_, std::move(w.bytes()));
      }
      watch(std::move(ev), [this, job, toCpu] { onPullEnded(job, toCpu); });
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " pull kernel failed: " << ex.what();
      setError(TP_CREATE_ERROR(HipError, "tphip_ring_pull", TPHIP_ERR_INVALID_ARG));
    }
  }

  void onPullEnded(const std::shared_ptr<RingJob>& job, bool toCpu) {
    StreamIn& si = streamIn_;
    si.running = false;
    job->op->kernelBusy = false;
    if (error_) {
      finish(job->op);
      return;
    }
    const uint64_t status = __atomic_load_n(hostWord(si.own->host(), kRingStatusAt), __ATOMIC_ACQUIRE);
    const uint64_t seq = status & ~TPHIP_RING_YIELDED;
    if (seq < job->firstSeq + job->done || seq > job->firstSeq + job->chunks) {
      failProtocol();
      return;
    }
    const uint64_t before = job->done;
    job->done = seq - job->firstSeq;
    TP_MARK("basic: pull kernel ended");
    if (toCpu && job->done > before) {
      const uint64_t from = before * si.slotBytes;
      const uint64_t to = std::min<uint64_t>(job->done * si.slotBytes, job->op->length);
      std::memcpy(
          static_cast<uint8_t*>(job->op->buffer.unwrap<CpuBuffer>().ptr) + from, si.bounce->host(), to - from);
    }
    if (job->done == job->chunks) {
      si.jobs.pop_front();
      chunkLanded(job->op);
    }
    pumpStreamIn();
  }

  // ---- helpers ------------------------------------------------------------------

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
  bool gotHello_{false};
  bool gotHelloAck_{false};
  bool ready_{false};
  uint64_t chunkBytes_{0};
  uint64_t remoteSlotBytes_{0};
  uint64_t remoteNumSlots_{0};
  uint8_t* remoteRing_{nullptr};  // peer's send ring as mapped by our GPU
  std::string remoteRingPeer_;    // who exported it, and under which identifier
  uint64_t remoteRingId_{0};
  bool peerMappedOurRing_{false}; // peer can read our send ring
  std::vector<std::function<void()>> deferred_;
  std::deque<std::shared_ptr<Op>> ops_;
  std::deque<std::shared_ptr<Op>> recvOps_; // not yet fully routed / notified
  std::deque<Incoming> inbox_;
  std::deque<std::shared_ptr<SendChunk>> sendQueue_;
  std::deque<std::shared_ptr<RecvChunk>> recvPostQueue_;
  std::deque<std::shared_ptr<RecvChunk>> innerAwaited_; // inner-route chunks the sender has not announced yet
  uint32_t innerChunksOnTheirWay_{0}; // announced by the sender (kStaged), not yet matched with a chunk
  uint32_t stagedToAnnounce_{0}; // inner sends started since the last kStaged message
  std::map<uint32_t, SlotAllocator::TSlot> slotsInFlight_;
  std::vector<StageItem> stagePending_;
  std::vector<RingItem> ringPending_;
  bool launchScheduled_{false};
  StreamOut streamOut_;
  StreamIn streamIn_;
  bool streamOutFailed_{false};
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
