// hip_ipc: GPU-to-GPU channel between two processes of one machine.
//
// Two data paths, chosen per tensor by the sender:
//
//  direct  The sender exports the allocation that contains the tensor
//          (hipIpcGetMemHandle on its base, cached per allocation) and sends
//          {export id, handle, address range} of every allocation a message
//          touches, then {allocation, offset, length} per tensor. The receiver
//          maps the allocation (cached) and its batched copy kernel reads the
//          sender's memory directly: one read and one write per payload byte,
//          all tensors of a message in one launch. Because every message
//          carries the handles it needs, the receiver may drop a mapping
//          whenever no copy reads from it: it keeps the most recently used
//          ones up to TP_HIP_IPC_MAX_MAPPED_BYTES (a mapping keeps the memory
//          alive after the sender has freed it).
//  outbox  What the reference does for every transfer
//          (tensorpipe/channel/cuda_ipc/channel_impl.cc:107-136,238-252,
//          431-467, context_impl.cc:173-195,341-418): the tensor is cut into
//          chunks of at most one slot, each chunk is copied into a slot of a
//          per-device staging slab that was exported once, the receiver copies
//          slot -> target and its reply frees the slot. Two reads and two
//          writes per byte. Used when an allocation cannot be exported, or
//          for everything when TP_HIP_IPC_MODE=outbox.
//
// Synchronisation between the two processes. Exporting a HIP event to another
// process fails on the deployment this was built for, so the inter-process
// events of the reference (tensorpipe/channel/cuda_ipc/channel_impl.cc:238-252,
// 453-463) are replaced by signal words: every channel end owns a few 64-bit
// words in a pinned host page of its context, exported once; the peer maps the
// page for its GPU (a peer's CPUs cannot reach a mapped page, only the owner's
// can). For a unit small enough for the receiver's copy agent, the receiving
// GPU raises acks[unit % 64] in the SENDER's page once the copy has finished
// -- the agent does it as part of the command -- and the sender's host watches
// that word of its own page: no reply message, no event polled for it. Other
// units, and ends that have no page (TP_HIP_IPC_SIGNALS=0, or the export
// failed), are acknowledged with a message on the reply connection; each unit
// says which of the two its sender expects.
//
// A tensor whose producing work is still running on the sender's stream is
// announced at once all the same: the sender raises ready[k % 64] of its page
// in stream order behind that work (tphip_stream_signal) and names the word in
// the unit; the receiver launches its copy gated on the word
// (tphip_batched_copy_gated), so the copy starts on the GPU the moment the
// bytes are there instead of an event poll, a message and a launch later. The
// gate's wait is bounded and the launch repeated if it ran out, so no kernel
// ever waits for good on something queued behind it; the recv callback of such
// a unit fires when its copy has finished. This is switched on with
// TP_HIP_IPC_GATES=1; by default, and without words on both ends, the sender
// polls an event behind the producing work before it announces (see
// gatesEnabled for the measurement behind that default).
//
// Small tensors whose source and destination streams have nothing pending are
// copied by the context's resident copy agent (tphip_agent_*): no launch, the
// bytes land about 3 us after the descriptor arrived. Everything else is one
// batched copy launch on the caller's stream per unit.
//
// The recv callback fires when the copy has been enqueued on the caller's
// stream (as in the reference), or, for a copy the agent does, when the bytes
// have landed; callbacks fire in the order of the recv calls. The send
// callback fires when the source may be reused: after the receiver's
// acknowledgement (direct) or after the last chunk has been staged (outbox).

#include <tensorpipe/channel/hip_ipc/factory.h>

#include <algorithm>
#include <array>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <mutex>
#include <set>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/channel/hip_common.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/common/slot_allocator.h>
#include <tensorpipe/common/stage_timer.h>
#include <tensorpipe/common/wire.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_ipc {

namespace {

// Staging geometry of the outbox path. The reference uses 4 slots of 8 MiB
// (tensorpipe/channel/cuda_ipc/constants.h:22-24); every chunk costs two host
// round trips here (there are no cross-process events to let the GPU order the
// two copies), so the defaults are larger -- 8 slots of 32 MiB, 256 MiB of a
// 288 GB device, allocated when the path is first used -- and both are
// settable per context (TP_HIP_IPC_SLOT_BYTES, TP_HIP_IPC_NUM_SLOTS). The
// sender's geometry travels with the first chunk it announces.
constexpr size_t kDefaultSlotBytes = 32u << 20;
constexpr size_t kDefaultNumSlots = 8;
constexpr size_t kMaxNumSlots = 1024;

size_t envSize(const char* name, size_t fallback) {
  const char* e = std::getenv(name);
  if (e == nullptr || *e == 0) {
    return fallback;
  }
  const unsigned long long v = std::strtoull(e, nullptr, 10);
  return v > 0 ? static_cast<size_t>(v) : fallback;
}

// Read when a context is created, so that one process can host contexts of
// both kinds.
bool outboxForcedByEnv() {
  const char* e = std::getenv("TP_HIP_IPC_MODE");
  return e != nullptr && std::string(e) == "outbox";
}

// Allocations of this size or more are not exported but staged through the
// outbox: mapping an allocation of 2 GiB or more in another process has been
// seen never to return on the deployment this was built for. Settable per
// context (TP_HIP_IPC_MAX_EXPORT_BYTES) where larger mappings are known to work.
constexpr size_t kDefaultMaxExportBytes = size_t(2) << 30;

// Allocations smaller than this are staged through the outbox as well. The
// runtime carves small device allocations out of 2 MiB blocks, and the handle
// of one such allocation stops working when ANOTHER exported allocation of the
// same block is freed before the peer has opened it ("IPC Attach: Invalid IPC
// handle", seen for allocations of 100 KB and 1 MiB, not for 2 MiB - 4 KiB and
// more, nor for pinned host memory): a sender that frees tensors as their
// sends complete would break the sends behind them. Allocators of frameworks
// hand out tensors inside segments of 2 MiB and more, which are exported as
// before. TP_HIP_IPC_MIN_EXPORT_BYTES overrides.
constexpr size_t kDefaultMinExportBytes = size_t(2) << 20;

// Peer allocations a channel keeps mapped: least recently used ones go once
// their sizes add up to more than this, or there are more than this many.
constexpr size_t kDefaultMaxMappedBytes = size_t(64) << 30;
constexpr size_t kMaxMappedAllocations = 1024;

// Staged tensors of at least this many chunks use the copy kernels' own
// completion signals.
constexpr size_t kChunksForKernelSignals = 4;

// Allocations this process has exported, keyed by base address. Process-wide:
// a handle describes an allocation, not a context.
struct ExportedAllocation {
  uint64_t id;
  HandleBytes handle;
  uint64_t base;
  size_t size;
  uint64_t bufferId;
};

class ExportRegistry {
 public:
  static ExportRegistry& get() {
    static ExportRegistry* r = new ExportRegistry();
    return *r;
  }

  // Returns false if the allocation containing ptr cannot be exported.
  bool lookup(
      int device,
      const void* ptr,
      size_t minExportBytes,
      size_t maxExportBytes,
      ExportedAllocation* out,
      uint64_t* offset) {
    // Common case first: ptr falls inside an allocation exported before. One
    // runtime query (the allocation's identifier) confirms that the address
    // range still belongs to that allocation.
    {
      uint64_t bufferId = 0;
      const bool haveId = tphip_mem_buffer_id(ptr, &bufferId) == 0 && bufferId != 0;
      std::lock_guard<std::mutex> lock(mutex_);
      auto it = exports_.upper_bound(const_cast<void*>(ptr));
      if (haveId && it != exports_.begin()) {
        --it;
        const uint8_t* base = static_cast<const uint8_t*>(it->first);
        const uint8_t* p = static_cast<const uint8_t*>(ptr);
        if (p < base + it->second.size && it->second.bufferId == bufferId &&
            it->second.size < maxExportBytes && it->second.size >= minExportBytes) {
          *out = it->second;
          *offset = static_cast<uint64_t>(p - base);
          return true;
        }
      }
    }
    void* base = nullptr;
    size_t size = 0;
    if (tphip_mem_base(ptr, &base, &size) != 0 || base == nullptr || size >= maxExportBytes ||
        size < minExportBytes) {
      return false;
    }
    uint64_t bufferId = 0;
    tphip_mem_buffer_id(base, &bufferId);
    *offset = static_cast<uint64_t>(
        static_cast<const uint8_t*>(ptr) - static_cast<const uint8_t*>(base));
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = exports_.find(base);
    if (bufferId != 0 && it != exports_.end() && it->second.size == size &&
        it->second.bufferId == bufferId) {
      *out = it->second;
      return true;
    }
    // New allocation, or the address was freed and handed out again -- or the
    // runtime cannot tell the two apart (no identifier): then every send
    // exports afresh under a new identifier and nothing is remembered, rather
    // than risk the peer reading a stale mapping of freed memory.
    ExportedAllocation e;
    if (tphip_ipc_mem_export(device, base, e.handle.data()) != 0) {
      return false;
    }
    e.id = nextExportId();
    e.base = reinterpret_cast<uint64_t>(base);
    e.size = size;
    e.bufferId = bufferId;
    TP_VLOG(5) << "IPC exports: #" << e.id << " is " << base << " + " << size << " (allocation " << bufferId << ")";
    *out = e;
    if (bufferId != 0) {
      exports_[base] = e;
      forgetFreedAllocations();
    }
    return true;
  }

 private:
  // Entries of allocations that no longer exist are dropped now and then (each
  // time the table has doubled), so that a process that keeps allocating and
  // freeing does not grow it for ever. Called with the mutex held.
  void forgetFreedAllocations() {
    if (exports_.size() < purgeAt_) {
      return;
    }
    for (auto it = exports_.begin(); it != exports_.end();) {
      uint64_t now = 0;
      if (tphip_mem_buffer_id(it->first, &now) != 0 || now != it->second.bufferId) {
        it = exports_.erase(it);
      } else {
        ++it;
      }
    }
    purgeAt_ = std::max<size_t>(1024, 2 * exports_.size());
  }

  std::mutex mutex_;
  size_t purgeAt_{1024};
  std::map<void*, ExportedAllocation> exports_;
};

// Per-device staging slab of the outbox path, created on first use.
struct Outbox {
  Outbox(int device, size_t slotBytes, size_t numSlots)
      // (never below the size at which the runtime gives an allocation a block of its own)
      : slab(device, std::max(slotBytes * numSlots, kDefaultMinExportBytes)),
        allocator(slab.ptr(), numSlots, slotBytes) {
    TP_HIP_CHECK(tphip_ipc_mem_export(device, slab.ptr(), handle.data()));
  }
  HipDeviceSlab slab;
  HandleBytes handle;
  SlotAllocator allocator;
  const uint64_t id{nextExportId()};
};

// Signal words of one channel end (see the top of the file), all about the
// units this end SENDS. Read and written by the owner's CPUs and by the GPU
// on behalf of either process.
constexpr size_t kWordSlots = 64;
struct ChannelWords {
  uint64_t acks[kWordSlots]; // acks[u % 64] == ackValue(generation, u): the peer has copied unit u (raised by the peer's copy)
  uint64_t ready[kWordSlots]; // ready[k % 64] >= the value named in the k-th gated unit: its sources are ready (raised by the owner's stream)
  uint64_t expired[kWordSlots]; // this end's own gated copies report here that they gave up waiting
};
constexpr size_t kChannelsPerSlab = 256;

// Pinned page holding the words of up to kChannelsPerSlab channel ends of a
// context, exported once.
class SignalSlab {
 public:
  explicit SignalSlab(int device)
      : slab_(device, sizeof(ChannelWords) * kChannelsPerSlab), device_(device) {
    std::memset(slab_.host(), 0, slab_.size());
    TP_HIP_CHECK(tphip_ipc_mem_export(device, slab_.host(), handle_.data()));
    for (uint32_t i = 0; i < kChannelsPerSlab; ++i) {
      free_.push_back(kChannelsPerSlab - 1 - i);
    }
  }
  // The index of a free set of words, or -1. `generation` tells this use of
  // the words from earlier ones: a copy of a channel that is gone may still
  // raise a word after the words have gone to the next channel, and must not
  // be taken for the acknowledgement that one waits for.
  int acquire(uint32_t* generation) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (free_.empty()) {
      return -1;
    }
    const uint32_t i = free_.back();
    free_.pop_back();
    nextGeneration_ = nextGeneration_ % 0xffffu + 1; // 1..65535
    *generation = nextGeneration_;
    return static_cast<int>(i);
  }
  void release(int index) {
    std::lock_guard<std::mutex> lock(mutex_);
    std::memset(hostWords(index), 0, sizeof(ChannelWords));
    free_.push_back(static_cast<uint32_t>(index));
  }
  ChannelWords* hostWords(int index) const {
    return reinterpret_cast<ChannelWords*>(slab_.host()) + index;
  }
  ChannelWords* devWords(int index) const {
    return reinterpret_cast<ChannelWords*>(slab_.dev()) + index;
  }
  const HandleBytes& handle() const {
    return handle_;
  }
  uint64_t id() const {
    return id_;
  }
  uint64_t base() const {
    return reinterpret_cast<uint64_t>(slab_.host());
  }
  uint64_t size() const {
    return slab_.size();
  }
  int device() const {
    return device_;
  }

 private:
  HipPinnedSlab slab_;
  int device_;
  HandleBytes handle_;
  const uint64_t id_{nextExportId()};
  std::mutex mutex_;
  std::vector<uint32_t> free_;
  uint32_t nextGeneration_{0};
};

// What acks[unit % 64] reads once the peer has copied `unit`: the unit's
// number (+1, so that zeroed words mean nothing) under the generation of the
// words' current user. Fits the 48 bits a copy agent command carries.
uint64_t ackValue(uint32_t generation, uint64_t unitSeq) {
  return (static_cast<uint64_t>(generation & 0xffffu) << 32) | ((unitSeq + 1) & 0xffffffffu);
}

bool envFlag(const char* name, bool fallback) {
  const char* e = std::getenv(name);
  return e == nullptr || *e == 0 ? fallback : std::atoi(e) != 0;
}

class IpcContextCore final : public ContextCore {
 public:
  HipEventPool events;
  HipEventPoller poller;
  // Signal words for the channels of this context; null when switched off
  // (TP_HIP_IPC_SIGNALS=0) or when pinned memory cannot be exported here.
  std::unique_ptr<SignalSlab> signals;
  // What the gates of this context's channels wait for: ever growing, so that
  // a word raised late for a channel that is gone opens nobody else's gate.
  std::atomic<uint64_t> nextGateValue{0};
  // Tensors of a unit adding up to at most this many bytes go to the copy
  // agent when their streams are idle (TP_HIP_IPC_AGENT=0 switches it off,
  // TP_HIP_IPC_AGENT_MAX_BYTES moves the limit).
  const bool agentEnabled{envFlag("TP_HIP_IPC_AGENT", true)};
  const size_t agentMaxBytes{envSize("TP_HIP_IPC_AGENT_MAX_BYTES", 128 * 1024)};
  // How long the thread that posted a copy to the agent looks for its end
  // itself before leaving that to the poller thread (TP_HIP_IPC_AGENT_SPIN_US).
  const long agentSpinUs{static_cast<long>(envSize("TP_HIP_IPC_AGENT_SPIN_US", 8))};
  // A channel with nothing else in flight looks for the acknowledgement of a
  // small unit itself for this long after writing it, before leaving it to
  // the poller thread: it comes about 5 us later, and whatever the send
  // callback starts then runs on the thread that has the pipe's state in its
  // caches (TP_HIP_IPC_ACK_SPIN_US; 1 switches it off).
  const long ackSpinUs{static_cast<long>(envSize("TP_HIP_IPC_ACK_SPIN_US", 8))};
  // Gated copies are there, tested and switched off: TP_HIP_IPC_GATES=1 lets a
  // sender whose stream is still producing announce at once and the receiver's
  // GPU wait for its word. Measured against the host hand-off (event polled,
  // then announced) in the ping-pong it is no faster on this stack -- the
  // signal kernel behind the producer and the gate kernel ahead of the copy
  // each cost a kernel-to-kernel gap of 3-4 us, which is what the host path
  // costs too: 1 MiB 45.0 against 41.3 us per round trip, 64 MiB 76.0 against
  // 74.9. A gate gives up after TP_HIP_IPC_GATE_WAIT_US (doubling up to 64
  // times that on every further try).
  const bool gatesEnabled{envFlag("TP_HIP_IPC_GATES", false)};
  const uint32_t gateWaitUs{static_cast<uint32_t>(envSize("TP_HIP_IPC_GATE_WAIT_US", 2000))};

  IpcContextCore() {
    if (envFlag("TP_HIP_IPC_SIGNALS", true)) {
      try {
        signals = std::make_unique<SignalSlab>(0);
      } catch (const std::exception& ex) {
        TP_LOG_WARNING() << "hip_ipc: no signal words (" << ex.what()
                         << "); acknowledging with messages";
      }
    }
  }

  // Loop only. The agent of `device`, created on first use; null if it cannot be.
  void* agent(int device) {
    if (!agentEnabled) {
      return nullptr;
    }
    if (device >= static_cast<int>(agents_.size())) {
      agents_.resize(device + 1, nullptr);
    }
    if (agents_[device] == nullptr && !agentFailed_) {
      if (tphip_agent_create(device, &agents_[device]) != 0) {
        agents_[device] = nullptr;
        agentFailed_ = true;
      }
    }
    return agents_[device];
  }

  StreamIdleProbe idleProbe; // loop only
  StreamMarkers markers;
  const bool forceOutbox{outboxForcedByEnv()};
  const size_t minExportBytes{envSize("TP_HIP_IPC_MIN_EXPORT_BYTES", kDefaultMinExportBytes)};
  const size_t maxExportBytes{envSize("TP_HIP_IPC_MAX_EXPORT_BYTES", kDefaultMaxExportBytes)};
  const size_t maxMappedBytes{envSize("TP_HIP_IPC_MAX_MAPPED_BYTES", kDefaultMaxMappedBytes)};
  // 16-byte multiples keep every slot vector-aligned.
  const size_t slotBytes{
      (std::min<size_t>(envSize("TP_HIP_IPC_SLOT_BYTES", kDefaultSlotBytes), size_t(1) << 30) + 15) / 16 *
      16};
  // The slab is mapped by the peer: the whole of it stays below 2 GiB, like
  // everything else this channel lets a peer map.
  const size_t numSlots{std::max<size_t>(
      1,
      std::min(
          std::min(envSize("TP_HIP_IPC_NUM_SLOTS", kDefaultNumSlots), kMaxNumSlots),
          ((size_t(2) << 30) - 1) / slotBytes))};

  // Loop only.
  Outbox& outbox(int device) {
    if (device >= static_cast<int>(outboxes_.size())) {
      outboxes_.resize(device + 1);
    }
    if (!outboxes_[device]) {
      outboxes_[device] = std::make_unique<Outbox>(device, slotBytes, numSlots);
    }
    return *outboxes_[device];
  }

  void closeAllocators() {
    for (auto& o : outboxes_) {
      if (o) {
        o->allocator.close();
      }
    }
  }

  void joinImpl() override {
    poller.join(); // nothing asks the agents about tickets any more
    for (void*& a : agents_) {
      if (a != nullptr) {
        tphip_agent_destroy(a);
        a = nullptr;
      }
    }
  }

 private:
  std::vector<std::unique_ptr<Outbox>> outboxes_;
  std::vector<void*> agents_;
  bool agentFailed_{false};
};

enum MsgKind : uint8_t { kDirect = 1, kChunk = 2, kHello = 3 };

class ChannelImpl final : public ChannelImplBase {
 public:
  ChannelImpl(
      std::shared_ptr<IpcContextCore> ctx,
      std::string id,
      std::shared_ptr<transport::Connection> descriptorConnection,
      std::shared_ptr<transport::Connection> replyConnection)
      : ChannelImplBase(ctx, std::move(id)),
        ictx_(std::move(ctx)),
        descriptorConnection_(std::move(descriptorConnection)),
        replyConnection_(std::move(replyConnection)) {}

  // Every copy out of a mapped peer allocation is followed by an event or an
  // agent ticket whose watcher keeps this object alive, so nothing reads the
  // mappings any more.
  ~ChannelImpl() override {
    for (auto& i : imports_) {
      HipIpcImports::get().release(i.device, i.peer, i.id);
    }
    for (auto& kv : remoteAllocations_) {
      HipIpcImports::get().release(kv.second.device, peerIdentity_, kv.first);
    }
    if (wordsIndex_ >= 0) {
      ictx_->signals->release(wordsIndex_);
    }
  }

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
  // Both ends open with a hello: who they are and where their signal words
  // live. It is the first message on the descriptor connection each way, so
  // it is always there before the first unit.
  void initFromLoop() override {
    if (ictx_->signals) {
      wordsIndex_ = ictx_->signals->acquire(&wordsGeneration_);
    }
    WireWriter w;
    w.u8(kHello);
    w.str(processIdentity());
    w.u8(wordsIndex_ >= 0 ? 1 : 0);
    if (wordsIndex_ >= 0) {
      const SignalSlab& slab = *ictx_->signals;
      w.u64(slab.id());
      w.raw(slab.handle().data(), slab.handle().size());
      w.u64(slab.base());
      w.u64(slab.size());
      w.u32(static_cast<uint32_t>(wordsIndex_ * sizeof(ChannelWords)));
      w.u32(wordsGeneration_);
    }
    // what this end's copy agent takes in one unit (0: it has none)
    w.u64(ictx_->agentEnabled ? ictx_->agentMaxBytes : 0);
    writeMessage(*descriptorConnection_, std::move(w.bytes()));
    helloPending_ = true;
    descriptorConnection_->read(onReadMessage([this](std::vector<uint8_t> bytes) {
      helloPending_ = false;
      if (error_) {
        return;
      }
      onHello(bytes);
      pumpUnits();
    }));
  }

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
    cancel_->store(true, std::memory_order_release); // watchers of acknowledgement words give up
    if (wordsIndex_ >= 0) {
      // Copies of the peer that wait for a word of ours need not wait it out.
      ChannelWords* mine = ictx_->signals->hostWords(wordsIndex_);
      for (size_t k = 0; k < kWordSlots; ++k) {
        __atomic_store_n(&mine->ready[k], ~uint64_t(0), __ATOMIC_RELEASE);
      }
    }
    descriptorConnection_->close();
    replyConnection_->close();
    // Slot requests still queued fail with AllocatorClosedError, as in
    // tensorpipe/channel/cuda_ipc/context_impl.cc:420-426; only when the whole
    // context goes down, since the allocator is shared by its channels.
    if (ctx_->closed()) {
      ictx_->closeAllocators();
    }
    auto sends = std::move(sendOps_);
    sendOps_.clear();
    for (auto& op : sends) {
      finishSend(op);
    }
    auto recvs = std::move(recvOps_);
    recvOps_.clear();
    for (auto& op : recvs) {
      // A buffer the agent is still writing is handed back when it has finished.
      if (op->landing == 0) {
        finishRecv(op);
      }
    }
    wireQueue_.clear();
    replyQueue_.clear();
    pendingAcks_.clear(); // their watchers give up (cancel_); the send ops were finished above
  }

 private:
  struct StreamRef {
    void* stream;
    int device;
    bool operator==(const StreamRef& o) const {
      return stream == o.stream && device == o.device;
    }
  };

  // A unit that goes on the descriptor connection: a whole direct batch or one
  // staged chunk. Units are written strictly in creation order. Every unit
  // starts with {kind u8, acknowledgement mode u8, unit number u64}; the last
  // two are filled in when the unit is written.
  struct WireUnit {
    std::vector<uint8_t> bytes;
    bool ready{false};
    // Direct units: bytes and tensors in all, for the sender's guess whether
    // the peer's copy agent will take the unit (0 tensors: a staged chunk).
    uint64_t totalBytes{0};
    uint32_t tensors{0};
    std::function<void()> onReply; // runs when the unit has been acknowledged
  };
  static constexpr size_t kUnitHeaderBytes = 10;
  static constexpr uint32_t kAgentMaxTensors = 16;
  enum AckMode : uint8_t { kAckByMessage = 0, kAckByWord = 1 };

  static void unitHeader(WireWriter& w, MsgKind kind) {
    w.u8(kind);
    w.u8(kAckByMessage);
    w.u64(0);
  }

  struct SendOp {
    uint64_t seq;
    TSendCallback cb;
    size_t pending{0}; // things that must happen before the callback
    bool done{false};
  };

  struct RecvOp {
    uint64_t seq;
    TRecvCallback cb;
    std::vector<BatchEntry> entries;
    size_t unitsExpected{0};
    size_t unitsSeen{0};
    bool allSeen{false}; // every unit of the op has arrived and its copy is enqueued or posted
    size_t landing{0}; // units handed to the copy agent whose bytes have not landed yet
    bool done{false};
  };

  // A reply owed to the peer; replies are written in the order the units
  // arrived, each once the copy it acknowledges has finished.
  struct ReplyUnit {
    bool ready{false};
  };

  size_t numChunks(size_t length) const {
    return (length + ictx_->slotBytes - 1) / ictx_->slotBytes;
  }

  void onHello(const std::vector<uint8_t>& bytes) {
    WireReader r(bytes.data(), bytes.size());
    if (r.u8() != kHello) {
      failProtocol();
      return;
    }
    peerIdentity_ = r.str();
    const bool hasWords = r.u8() != 0;
    if (!r.ok() || peerIdentity_.empty()) {
      failProtocol();
      return;
    }
    if (!hasWords) {
      peerAgentMaxBytes_ = r.u64();
      if (!r.ok()) {
        failProtocol();
      }
      return;
    }
    const uint64_t id = r.u64();
    HandleBytes h;
    r.raw(h.data(), h.size());
    const uint64_t base = r.u64();
    const uint64_t size = r.u64();
    const uint32_t offset = r.u32();
    peerWordsGeneration_ = r.u32();
    peerAgentMaxBytes_ = r.u64();
    peerGates_ = true; // an end with words of its own can run gated copies
    if (!r.ok() || size < sizeof(ChannelWords) || offset > size - sizeof(ChannelWords) ||
        offset % alignof(ChannelWords) != 0) {
      failProtocol();
      return;
    }
    void* mapped = nullptr;
    const int rc = HipIpcImports::get().acquire(0, peerIdentity_, id, h, base, size, &mapped);
    if (rc != 0) {
      setError(TP_CREATE_ERROR(HipError, "tphip_ipc_mem_open (signal words)", rc));
      return;
    }
    imports_.push_back(Import{0, peerIdentity_, id});
    peerWords_ = reinterpret_cast<ChannelWords*>(static_cast<uint8_t*>(mapped) + offset);
  }

  // ---- send -----------------------------------------------------------------

  void sendEntries(uint64_t seq, std::vector<BatchEntry> entries, TSendCallback cb) {
    hipPointerCheckpoint(); // the caller's buffers: believed for this call only
    std::vector<BatchEntry> live;
    for (auto& e : entries) {
      if (e.length > 0) {
        live.push_back(std::move(e));
      }
    }
    if (live.empty()) {
      cb(error_); // zero length: tensorpipe/channel/cuda_ipc/channel_impl.cc:112-115
      return;
    }
    TP_MARK("ipc: send");
    reapAcks();
    auto op = std::make_shared<SendOp>();
    op->seq = seq;
    op->cb = std::move(cb);
    sendOps_.push_back(op);
    op->pending = 1; // guard until everything below has been issued

    try {
      // Split the batch: exportable tensors travel together in one direct unit,
      // the others go through the outbox chunk by chunk. Both endpoints derive
      // the unit sequence from the descriptors, so no negotiation is needed.
      struct DirectItem {
        ExportedAllocation alloc;
        uint64_t offset;
        uint64_t length;
        uint32_t index;
      };
      std::vector<DirectItem> direct;
      std::vector<uint32_t> staged;
      std::vector<StreamRef> directStreams;
      for (uint32_t i = 0; i < live.size(); ++i) {
        const HipBuffer& hb = live[i].buffer.unwrap<HipBuffer>();
        const int device = hipDeviceForPointer(hb.ptr);
        TP_THROW_ASSERT_IF(device < 0);
        DirectItem item;
        if (!ictx_->forceOutbox && ExportRegistry::get().lookup(
                device, hb.ptr, ictx_->minExportBytes, ictx_->maxExportBytes, &item.alloc, &item.offset)) {
          item.length = live[i].length;
          item.index = i;
          direct.push_back(item);
          StreamRef ref{hb.stream, device};
          bool known = false;
          for (auto& s : directStreams) {
            known |= s == ref;
          }
          if (!known) {
            directStreams.push_back(ref);
          }
        } else {
          staged.push_back(i);
        }
      }

      TP_MARK("ipc: sources looked up");
      if (!direct.empty()) {
        // The distinct allocations of the unit, then the tensors by reference.
        std::vector<const ExportedAllocation*> allocs;
        std::vector<uint32_t> allocOf(direct.size());
        for (size_t k = 0; k < direct.size(); ++k) {
          uint32_t a = 0;
          while (a < allocs.size() && allocs[a]->id != direct[k].alloc.id) {
            ++a;
          }
          if (a == allocs.size()) {
            allocs.push_back(&direct[k].alloc);
          }
          allocOf[k] = a;
        }
        WireWriter w;
        w.reserve(64 + 96 * allocs.size() + 24 * direct.size());
        unitHeader(w, kDirect);
        // gate: {used u8, word u32, value u64}, filled in below if one is used
        const size_t gateAt = w.bytes().size();
        uint32_t gateSlot = 0;
        uint64_t gateValue = 0;
        w.u8(0);
        w.u32(0);
        w.u64(0);
        w.u32(static_cast<uint32_t>(allocs.size()));
        for (const ExportedAllocation* a : allocs) {
          w.u64(a->id);
          w.raw(a->handle.data(), a->handle.size());
          w.u64(a->base);
          w.u64(a->size);
        }
        w.u32(static_cast<uint32_t>(direct.size()));
        for (size_t k = 0; k < direct.size(); ++k) {
          w.u32(direct[k].index);
          w.u32(allocOf[k]);
          w.u64(direct[k].offset);
          w.u64(direct[k].length);
        }
        auto unit = std::make_shared<WireUnit>();
        unit->bytes = std::move(w.bytes());
        unit->tensors = static_cast<uint32_t>(direct.size());
        for (auto& d : direct) {
          unit->totalBytes += d.length;
        }
        // The source may be reused once the receiver has copied it.
        ++op->pending;
        unit->onReply = [this, op] { sendStepDone(op); };
        wireQueue_.push_back(unit);
        // Announce once the producing work on every source stream is done.
        // Streams with nothing pending need no event at all.
        std::vector<StreamRef> busy;
        for (auto& s : directStreams) {
          if (!ictx_->idleProbe.idle(s.device, s.stream)) {
            busy.push_back(s);
          }
        }
        TP_MARK("ipc: source streams probed");
        if (busy.size() == 1 && wordsIndex_ >= 0 && peerGates_ && ictx_->gatesEnabled) {
          // One stream still producing: its last kernel is followed by a word
          // the receiver's copy waits for on the GPU.
          // Values grow over the whole context, so a word raised late for a
          // channel that is gone can never open a gate of the words' next user.
          gateSlot = static_cast<uint32_t>(nextGate_++ % kWordSlots);
          gateValue = ictx_->nextGateValue.fetch_add(1, std::memory_order_relaxed) + 1;
          TP_HIP_CHECK(tphip_stream_signal(
              busy[0].device,
              busy[0].stream,
              &ictx_->signals->devWords(wordsIndex_)->ready[gateSlot],
              gateValue));
          // a marker, so that the runtime knows when the stream has drained
          auto marker = ictx_->events.get(busy[0].device, busy[0].stream);
          marker->record(busy[0].stream);
          ictx_->events.put(std::move(marker));
          unit->bytes[gateAt] = 1;
          std::memcpy(unit->bytes.data() + gateAt + 1, &gateSlot, sizeof(gateSlot));
          std::memcpy(unit->bytes.data() + gateAt + 5, &gateValue, sizeof(gateValue));
          busy.clear();
        }
        if (busy.empty()) {
          unit->ready = true;
          flushWire();
        }
        auto remaining = std::make_shared<size_t>(busy.size());
        for (auto& s : busy) {
          auto ev = ictx_->events.get(s.device, s.stream);
          ev->record(s.stream);
          watch(std::move(ev), [this, unit, remaining] {
            if (--*remaining == 0) {
              unit->ready = true;
              flushWire();
            }
          });
        }
      }

      for (uint32_t i : staged) {
        const HipBuffer& hb = live[i].buffer.unwrap<HipBuffer>();
        const int device = hipDeviceForPointer(hb.ptr);
        const size_t chunks = numChunks(live[i].length);
        for (size_t k = 0; k < chunks; ++k) {
          const size_t offset = k * ictx_->slotBytes;
          const size_t len = std::min(live[i].length - offset, ictx_->slotBytes);
          auto unit = std::make_shared<WireUnit>();
          wireQueue_.push_back(unit);
          ++op->pending; // staged copy of this chunk finished
          stageChunk(op, unit, device, hb, i, offset, len, live[i].length);
        }
      }
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " send failed: " << ex.what();
      setError(TP_CREATE_ERROR(HipError, "hip_ipc send", TPHIP_ERR_INVALID_ARG));
      return;
    }
    sendStepDone(op); // drop the guard
  }

  // Outbox path, one chunk: wait for a slot, copy source -> slot on the
  // caller's stream, announce the slot when the copy is done, free the slot
  // when the receiver has acknowledged it.
  void stageChunk(
      const std::shared_ptr<SendOp>& op,
      const std::shared_ptr<WireUnit>& unit,
      int device,
      HipBuffer hb,
      uint32_t index,
      size_t offset,
      size_t len,
      size_t tensorLength) {
    Outbox& outbox = ictx_->outbox(device);
    auto self = shared_from_this();
    outbox.allocator.alloc([this, self, op, unit, device, hb, index, offset, len, tensorLength, &outbox](
                               const Error& error, SlotAllocator::TSlot slot) {
      if (error) {
        setError(error);
        return;
      }
      if (error_) {
        return;
      }
      const size_t slotIdx = outbox.allocator.slotIndex(slot.get());
      std::unique_ptr<HipEvent> ev;
      bool onKernel = false;
      try {
        ev = ictx_->events.get(device, hb.stream);
        // The chunks of a long tensor queue up on the caller's stream several
        // deep: the kernels' own completion signals then, and no marker between
        // two of them (1 GiB: 1.4 instead of 1.2 TB/s). A short tensor is better
        // off with a marker polled at once (64 MiB: 125 against 140 us).
        onKernel = hipBatchedCopy(
            device,
            hb.stream,
            {tphip_copy_desc{static_cast<const uint8_t*>(hb.ptr) + offset, slot.get(), len}},
            *ev,
            /*signalOnKernel=*/numChunks(tensorLength) >= kChunksForKernelSignals);
      } catch (const std::exception& ex) {
        TP_LOG_WARNING() << "Channel " << id_ << " staging failed: " << ex.what();
        setError(TP_CREATE_ERROR(HipError, "hip_ipc staging", TPHIP_ERR_INVALID_ARG));
        return;
      }
      WireWriter w;
      unitHeader(w, kChunk);
      w.u32(index);
      w.u32(static_cast<uint32_t>(device));
      const bool announce = !outboxAnnounced_[device];
      outboxAnnounced_[device] = true;
      w.u8(announce ? 1 : 0);
      if (announce) {
        w.str(processIdentity());
        w.u64(outbox.id);
        w.u64(ictx_->slotBytes);
        w.u32(static_cast<uint32_t>(ictx_->numSlots));
        w.raw(outbox.handle.data(), outbox.handle.size());
        w.u64(reinterpret_cast<uint64_t>(outbox.slab.ptr()));
        w.u64(outbox.slab.size());
      }
      w.u32(static_cast<uint32_t>(slotIdx));
      w.u64(offset);
      w.u64(len);
      unit->bytes = std::move(w.bytes());
      unit->onReply = [slot]() mutable { slot.reset(); }; // the acknowledgement frees the slot
      watchCopy(std::move(ev), device, hb.stream, onKernel, [this, op, unit] {
        unit->ready = true;
        flushWire();
        sendStepDone(op); // this chunk no longer needs the source
      });
    });
  }

  void sendStepDone(const std::shared_ptr<SendOp>& op) {
    if (op->done || --op->pending > 0) {
      return;
    }
    removeSend(op);
    finishSend(op);
  }

  // Write every unit at the head of the queue whose data is ready, and start
  // waiting for its acknowledgement: this end's acks word for the unit when
  // the peer's copy agent is likely to take it (small enough; the word not
  // still owed to an older unit), a message on the reply connection
  // otherwise.
  void flushWire() {
    while (!wireQueue_.empty() && wireQueue_.front()->ready && !error_) {
      auto unit = wireQueue_.front();
      wireQueue_.pop_front();
      const uint64_t seq = nextUnitOut_++;
      const size_t slot = seq % kWordSlots;
      const bool byWord = wordsIndex_ >= 0 && unit->tensors > 0 &&
          unit->tensors <= kAgentMaxTensors && unit->totalBytes <= peerAgentMaxBytes_ &&
          !ackSlotBusy_[slot];
      unit->bytes[1] = byWord ? kAckByWord : kAckByMessage;
      std::memcpy(unit->bytes.data() + 2, &seq, sizeof(seq));
      TP_VLOG(6) << "Channel " << id_ << " is writing descriptor #" << seq;
      writeMessage(*descriptorConnection_, std::move(unit->bytes));
      TP_MARK("ipc: unit written");
      auto acknowledged = [this, unit] {
        if (!error_ && unit->onReply) {
          unit->onReply();
        }
        unit->onReply = nullptr;
      };
      if (byWord) {
        ackSlotBusy_[slot] = true;
        auto ack = std::make_shared<PendingAck>();
        ack->word = &ictx_->signals->hostWords(wordsIndex_)->acks[slot];
        ack->value = ackValue(wordsGeneration_, seq);
        ack->slot = slot;
        ack->done = acknowledged;
        pendingAcks_.push_back(ack);
        // The poller thread watches the word; whoever runs on the loop for
        // this channel meanwhile looks at it in passing (reapAcks).
        auto cancel = cancel_;
        auto self = shared_from_this();
        ictx_->poller.watchCondition(
            [ack, cancel](bool* done) {
              *done = ack->reaped.load(std::memory_order_acquire) ||
                  cancel->load(std::memory_order_acquire) ||
                  __atomic_load_n(ack->word, __ATOMIC_ACQUIRE) == ack->value;
              return 0;
            },
            [this, self, ack](const Error& error) {
              if (ack->reaped.load(std::memory_order_acquire)) {
                return; // the loop got there first
              }
              TP_MARK("ipc: ack word seen");
              ctx_->defer([this, self, ack, error] {
                setError(error);
                reap(ack);
              });
            });
      } else {
        replyConnection_->read(nullptr, 0, onRead(acknowledged));
      }
    }
    // Alone on the channel: wait for the word right here for a moment.
    if (!error_ && pendingAcks_.size() == 1 && sendOps_.size() == 1 && recvOps_.empty() &&
        wireQueue_.empty() && ictx_->ackSpinUs > 1) {
      auto ack = pendingAcks_.front();
      const auto giveUp = std::chrono::steady_clock::now() + std::chrono::microseconds(ictx_->ackSpinUs);
      do {
        if (__atomic_load_n(ack->word, __ATOMIC_ACQUIRE) == ack->value) {
          TP_MARK("ipc: ack word seen (inline)");
          reap(ack);
          break;
        }
      } while (std::chrono::steady_clock::now() < giveUp);
    }
  }

  // An acknowledgement word this end waits for. Loop only, except `reaped`.
  struct PendingAck {
    const uint64_t* word{nullptr};
    uint64_t value{0};
    size_t slot{0};
    std::function<void()> done;
    std::atomic<bool> reaped{false};
  };

  void reap(const std::shared_ptr<PendingAck>& ack) {
    if (ack->reaped.exchange(true)) {
      return;
    }
    for (auto it = pendingAcks_.begin(); it != pendingAcks_.end(); ++it) {
      if (*it == ack) {
        pendingAcks_.erase(it);
        break;
      }
    }
    ackSlotBusy_[ack->slot] = false;
    ack->done();
    flushWire(); // a unit may have been waiting for this word to come free
  }

  // Whoever runs on the loop on behalf of this channel looks at the words it
  // is waiting for while it is there.
  void reapAcks() {
    for (size_t i = 0; i < pendingAcks_.size();) {
      auto ack = pendingAcks_[i];
      if (__atomic_load_n(ack->word, __ATOMIC_ACQUIRE) == ack->value) {
        TP_MARK("ipc: ack word reaped in passing");
        reap(ack); // erases it
      } else {
        ++i;
      }
    }
  }

  // ---- recv -----------------------------------------------------------------

  void recvEntries(uint64_t seq, std::vector<BatchEntry> entries, TRecvCallback cb) {
    hipPointerCheckpoint(); // the caller's buffers: believed for this call only
    TP_MARK("ipc: recv");
    reapAcks();
    auto op = std::make_shared<RecvOp>();
    op->seq = seq;
    op->cb = std::move(cb);
    for (auto& e : entries) {
      if (e.length > 0) {
        op->entries.push_back(std::move(e));
      }
    }
    if (op->entries.empty()) {
      op->allSeen = true; // nothing travels; the callback keeps its place in the order
    }
    recvOps_.push_back(op);
    flushRecvCallbacks();
    pumpUnits();
  }

  // One reader per channel. The transport serves reads in the order they were
  // posted, and how many units an op takes is only known as they arrive (a
  // direct unit says how many tensors it covers, a staged tensor takes one
  // unit per chunk): a read posted for a later op while an earlier one still
  // expects units would be handed that earlier op's next unit. So a single
  // read is outstanding at any time and every unit goes to the oldest op that
  // is still missing some, as the reference gates its descriptor reads per
  // operation in sequence
  // (tensorpipe/channel/cuda_ipc/channel_impl.cc:319-347,349-399).
  std::shared_ptr<RecvOp> opAwaitingUnits() const {
    for (auto& op : recvOps_) {
      if (!op->allSeen) {
        return op;
      }
    }
    return nullptr;
  }

  void pumpUnits() {
    if (unitReadPosted_ || helloPending_ || error_ || opAwaitingUnits() == nullptr) {
      return;
    }
    unitReadPosted_ = true;
    descriptorConnection_->read(onReadMessage([this](std::vector<uint8_t> bytes) {
      unitReadPosted_ = false;
      if (error_) {
        return;
      }
      auto op = opAwaitingUnits();
      if (op == nullptr) {
        return;
      }
      onUnit(op, bytes);
      pumpUnits();
    }));
  }

  // What has to happen once the copies of a received unit have finished.
  struct UnitCompletion {
    std::shared_ptr<ReplyUnit> reply; // owed when the peer waits for a message
    bool byWord{false};
    uint64_t unitSeq{0};
    std::vector<uint64_t> inUse; // peer allocations the copies read from
  };

  void unitCopiesFinished(const UnitCompletion& c) {
    for (uint64_t id : c.inUse) {
      auto it = remoteAllocations_.find(id);
      if (it != remoteAllocations_.end() && it->second.inFlight > 0) {
        --it->second.inFlight;
      }
    }
    dropLeastRecentlyUsedMappings();
    if (c.reply) { // a unit acknowledged by word had its word raised by the GPU behind the copy
      c.reply->ready = true;
      flushReplies();
    }
  }

  void onUnit(const std::shared_ptr<RecvOp>& op, const std::vector<uint8_t>& bytes) {
    TP_MARK("ipc: unit arrived");
    reapAcks();
    WireReader r(bytes.data(), bytes.size());
    const uint8_t kind = r.u8();
    const uint8_t ackMode = r.u8();
    const uint64_t unitSeq = r.u64();
    TP_VLOG(6) << "Channel " << id_ << " got descriptor #" << unitSeq << " of kind " << int(kind)
               << " (recv #" << op->seq << ")";
    if (!r.ok() || unitSeq != nextUnitIn_ || ackMode > kAckByWord ||
        (ackMode == kAckByWord && peerWords_ == nullptr)) {
      failProtocol();
      return;
    }
    ++nextUnitIn_;
    UnitCompletion completion;
    completion.byWord = ackMode == kAckByWord;
    completion.unitSeq = unitSeq;
    if (!completion.byWord) {
      completion.reply = std::make_shared<ReplyUnit>();
      replyQueue_.push_back(completion.reply);
    }
    std::vector<std::unique_ptr<HipEvent>> launched; // one event per copy launch
    std::vector<StreamRef> launchedOn;
    bool chunkOnKernel = false; // a staged chunk whose event is the kernel's own signal
    StreamRef chunkStream{nullptr, 0};
    bool viaAgent = false;
    bool gatedLaunched = false;
    uint64_t agentTicket = 0;
    void* agent = nullptr;
    try {
      if (kind == kDirect) {
        const bool gated = r.u8() != 0;
        const uint32_t gateSlot = r.u32();
        const uint64_t gateValue = r.u64();
        if (gated && (peerWords_ == nullptr || wordsIndex_ < 0 || gateSlot >= kWordSlots)) {
          failProtocol();
          return;
        }
        const uint32_t nAllocs = r.u32();
        // every allocation takes 88 bytes on the wire
        if (!r.ok() || peerIdentity_.empty() || nAllocs > r.remaining() / 88) {
          failProtocol();
          return;
        }
        struct Announced {
          uint64_t id;
          HandleBytes handle;
          uint64_t base;
          uint64_t size;
        };
        std::vector<Announced> announced(nAllocs);
        for (auto& a : announced) {
          a.id = r.u64();
          r.raw(a.handle.data(), a.handle.size());
          a.base = r.u64();
          a.size = r.u64();
        }
        const uint32_t n = r.u32();
        if (!r.ok() || n == 0 || n > r.remaining() / 24) {
          failProtocol();
          return;
        }
        struct Group {
          StreamRef dst;
          std::vector<tphip_copy_desc> table;
        };
        std::vector<Group> groups;
        std::vector<RemoteAllocation*> mappedOf(nAllocs, nullptr);
        uint64_t totalBytes = 0;
        for (uint32_t k = 0; k < n; ++k) {
          const uint32_t index = r.u32();
          const uint32_t allocIdx = r.u32();
          const uint64_t offset = r.u64();
          const uint64_t length = r.u64();
          if (!r.ok() || index >= op->entries.size() || allocIdx >= nAllocs) {
            failProtocol();
            return;
          }
          const HipBuffer& hb = op->entries[index].buffer.unwrap<HipBuffer>();
          const int device = hipDeviceForPointer(hb.ptr);
          TP_THROW_ASSERT_IF(device < 0);
          const Announced& a = announced[allocIdx];
          if (mappedOf[allocIdx] == nullptr) {
            auto it = remoteAllocations_.find(a.id);
            if (it == remoteAllocations_.end()) {
              void* mapped = nullptr;
              int rc = HipIpcImports::get().acquire(
                  device, peerIdentity_, a.id, a.handle, a.base, a.size, &mapped);
              if (rc != 0) {
                setError(TP_CREATE_ERROR(HipError, "tphip_ipc_mem_open", rc));
                return;
              }
              // What the runtime says about the mapping bounds the ranges the
              // peer may name; what the peer said about its size does not.
              uint64_t realSize = a.size;
              void* realBase = nullptr;
              size_t queried = 0;
              if (tphip_mem_base(mapped, &realBase, &queried) == 0 && realBase == mapped && queried > 0) {
                realSize = std::min<uint64_t>(realSize, queried);
              }
              it = remoteAllocations_.emplace(a.id, RemoteAllocation{mapped, realSize, a.size, device, 0, 0}).first;
              mappedBytes_ += a.size;
            } else if (it->second.announcedSize != a.size) {
              failProtocol(); // one identifier, one allocation
              return;
            }
            it->second.lastUse = ++useCounter_;
            mappedOf[allocIdx] = &it->second;
          }
          // The range must lie inside the mapped allocation: the copy kernel
          // would fault on anything else.
          const uint64_t limit = mappedOf[allocIdx]->size;
          if (length != op->entries[index].length || offset > limit || length > limit - offset) {
            failProtocol();
            return;
          }
          StreamRef ref{hb.stream, device};
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
          g->table.push_back(tphip_copy_desc{
              static_cast<const uint8_t*>(mappedOf[allocIdx]->ptr) + offset, hb.ptr, length});
          totalBytes += length;
          ++op->unitsSeen;
        }
        TP_MARK("ipc: unit parsed and mapped");
        // From here until the copies have finished the mappings must stay.
        for (uint32_t a = 0; a < nAllocs; ++a) {
          if (mappedOf[a] != nullptr) {
            ++mappedOf[a]->inFlight;
            completion.inUse.push_back(announced[a].id);
          }
        }
        // Small and nothing pending on the streams the bytes go to: the copy
        // agent, no launch. (The sender announced the unit only once its
        // sources were ready.)
        if (gated) {
          // Launched now, started by the GPU when the sender's word is there.
          auto pending = std::make_shared<GatedUnit>();
          pending->completion = completion;
          pending->op = op;
          pending->word = &peerWords_->ready[gateSlot];
          pending->value = gateValue;
          pending->waitUs = ictx_->gateWaitUs;
          for (auto& g : groups) {
            pending->groups.push_back(GatedGroup{g.dst, std::move(g.table), 0});
          }
          pending->remaining = pending->groups.size();
          ++op->landing;
          gatedLaunched = true;
          for (size_t k = 0; k < pending->groups.size(); ++k) {
            try {
              launchGated(pending, k);
            } catch (const std::exception& ex) {
              TP_LOG_WARNING() << "Channel " << id_ << " gated copy failed: " << ex.what();
              setError(TP_CREATE_ERROR(HipError, "hip_ipc gated copy", TPHIP_ERR_INVALID_ARG));
              for (size_t j = k; j < pending->groups.size(); ++j) {
                gatedGroupFinished(pending); // this one and those never launched
              }
              break;
            }
          }
          if (error_) {
            return;
          }
        } else if (ictx_->agentEnabled && totalBytes <= ictx_->agentMaxBytes && n <= kAgentMaxTensors) {
          const int device = groups.front().dst.device;
          bool quiet = true;
          for (auto& g : groups) {
            quiet = quiet && g.dst.device == device && ictx_->idleProbe.idle(g.dst.device, g.dst.stream);
          }
          TP_MARK("ipc: destination streams probed");
          agent = quiet ? ictx_->agent(device) : nullptr;
          if (agent != nullptr) {
            std::vector<tphip_copy_desc> all;
            for (auto& g : groups) {
              all.insert(all.end(), g.table.begin(), g.table.end());
            }
            void* notify = completion.byWord ? &peerWords_->acks[unitSeq % kWordSlots] : nullptr;
            const int rc = tphip_agent_submit(
                agent, all.data(), static_cast<uint32_t>(all.size()), notify,
                ackValue(peerWordsGeneration_, unitSeq), &agentTicket);
            viaAgent = rc == 0; // a full ring or an address it cannot carry: launch as usual
            TP_MARK("ipc: posted to the agent");
          }
        }
        if (!viaAgent && !gatedLaunched) {
          for (auto& g : groups) {
            auto ev = ictx_->events.get(g.dst.device, g.dst.stream);
            hipBatchedCopy(g.dst.device, g.dst.stream, g.table, *ev, /*signalOnKernel=*/false);
            launched.push_back(std::move(ev));
            launchedOn.push_back(g.dst);
          }
          if (completion.byWord) {
            // The sender watches its word: raise it from the GPU behind the
            // copies, on the first stream once it has waited for the others.
            for (size_t k = 1; k < launched.size(); ++k) {
              launched[k]->wait(launchedOn[0].stream, launchedOn[0].device);
            }
            TP_HIP_CHECK(tphip_stream_signal(
                launchedOn[0].device,
                launchedOn[0].stream,
                &peerWords_->acks[unitSeq % kWordSlots],
                ackValue(peerWordsGeneration_, unitSeq)));
          }
        }
        op->unitsExpected += n;
      } else if (kind == kChunk) {
        const uint32_t index = r.u32();
        const int srcDevice = static_cast<int>(r.u32());
        const bool announce = r.u8() != 0;
        if (!r.ok() || index >= op->entries.size()) {
          failProtocol();
          return;
        }
        const HipBuffer& hb = op->entries[index].buffer.unwrap<HipBuffer>();
        const int device = hipDeviceForPointer(hb.ptr);
        TP_THROW_ASSERT_IF(device < 0);
        if (announce) {
          const std::string peer = r.str();
          const uint64_t outboxId = r.u64();
          const uint64_t remoteSlotBytes = r.u64();
          const uint32_t remoteNumSlots = r.u32();
          HandleBytes h;
          r.raw(h.data(), h.size());
          const uint64_t remoteBase = r.u64();
          const uint64_t remoteSize = r.u64();
          if (!r.ok() || remoteOutboxes_.count(srcDevice) != 0 || remoteSlotBytes == 0 ||
              remoteNumSlots == 0 || remoteNumSlots > kMaxNumSlots ||
              remoteSlotBytes > remoteSize / remoteNumSlots) {
            failProtocol();
            return;
          }
          void* mapped = nullptr;
          int rc = HipIpcImports::get().acquire(
              device, peer, outboxId, h, remoteBase, remoteSize, &mapped);
          if (rc != 0) {
            setError(TP_CREATE_ERROR(HipError, "tphip_ipc_mem_open", rc));
            return;
          }
          imports_.push_back(Import{device, peer, outboxId});
          // The slots must fit what was really mapped.
          void* realBase = nullptr;
          size_t queried = 0;
          if (tphip_mem_base(mapped, &realBase, &queried) == 0 && realBase == mapped && queried > 0 &&
              remoteSlotBytes > queried / remoteNumSlots) {
            failProtocol();
            return;
          }
          remoteOutboxes_[srcDevice] = RemoteOutbox{mapped, remoteSlotBytes, remoteNumSlots};
        }
        const uint32_t slotIdx = r.u32();
        const uint64_t offset = r.u64();
        const uint64_t len = r.u64();
        auto it = remoteOutboxes_.find(srcDevice);
        const uint64_t tensorLength = op->entries[index].length;
        if (!r.ok() || it == remoteOutboxes_.end() || slotIdx >= it->second.numSlots ||
            len > it->second.slotBytes || offset > tensorLength || len > tensorLength - offset) {
          failProtocol();
          return;
        }
        auto ev = ictx_->events.get(device, hb.stream);
        chunkOnKernel = hipBatchedCopy(
            device,
            hb.stream,
            {tphip_copy_desc{
                static_cast<const uint8_t*>(it->second.ptr) + slotIdx * it->second.slotBytes,
                static_cast<uint8_t*>(hb.ptr) + offset,
                len}},
            *ev,
            /*signalOnKernel=*/(tensorLength + it->second.slotBytes - 1) / it->second.slotBytes >=
                kChunksForKernelSignals);
        chunkStream = StreamRef{hb.stream, device};
        launched.push_back(std::move(ev));
        launchedOn.push_back(chunkStream);
        // A staged tensor counts as seen when its last chunk arrived.
        if (offset + len == tensorLength) {
          ++op->unitsSeen;
        }
        if (offset == 0) {
          ++op->unitsExpected;
        }
      } else {
        failProtocol();
        return;
      }
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " recv failed: " << ex.what();
      // Copies already enqueued for this unit read the peer's memory; they are
      // followed by no watcher now, so wait for them here before the error
      // lets the mappings go.
      for (auto& s : launchedOn) {
        tphip_stream_sync(s.device, s.stream);
      }
      setError(TP_CREATE_ERROR(HipError, "hip_ipc recv", TPHIP_ERR_INVALID_ARG));
      return;
    }

    TP_VLOG(6) << "Channel " << id_ << " enqueued the copies (recv #" << op->seq << ")";
    if (viaAgent) {
      // The agent lands a small copy about 3 us after it was posted: less than
      // handing the wait to the poller thread and coming back costs. Look for
      // it right here for a few microseconds first.
      const auto giveUp = std::chrono::steady_clock::now() + std::chrono::microseconds(ictx_->agentSpinUs);
      bool landed = false;
      do {
        int d = 0;
        if (tphip_agent_done(agent, agentTicket, &d) != 0) {
          break;
        }
        landed = d != 0;
      } while (!landed && std::chrono::steady_clock::now() < giveUp);
      if (landed) {
        TP_MARK("ipc: agent done seen (inline)");
        viaAgent = false;
        unitCopiesFinished(completion);
      }
    }
    if (viaAgent) {
      // The recv callback waits for the bytes: nothing on the caller's stream
      // orders later work behind the agent's copy.
      ++op->landing;
      auto self = shared_from_this();
      ictx_->poller.watchCondition(
          [agent, agentTicket](bool* done) {
            int d = 0;
            const int rc = tphip_agent_done(agent, agentTicket, &d);
            *done = d != 0;
            return rc;
          },
          [this, self, op, completion](const Error& error) {
            TP_MARK("ipc: agent done seen");
            ctx_->defer([this, self, op, completion, error] {
              setError(error);
              unitCopiesFinished(completion);
              --op->landing;
              if (error_) {
                if (op->landing == 0) {
                  finishRecv(op); // held back by handleError until now
                }
              } else {
                flushRecvCallbacks();
              }
            });
          });
    } else if (!gatedLaunched) {
      // Acknowledge once the copies of this unit have finished.
      auto remaining = std::make_shared<size_t>(launched.size());
      for (auto& ev : launched) {
        watchCopy(std::move(ev), chunkStream.device, chunkStream.stream, chunkOnKernel, [this, remaining, completion] {
          if (--*remaining == 0) {
            unitCopiesFinished(completion);
          }
        });
      }
    }

    if (op->unitsSeen == op->entries.size()) {
      // Every copy of the op is enqueued (or posted to the agent).
      op->allSeen = true;
      flushRecvCallbacks();
    }
  }

  // A received unit whose copies wait for the sender's word on the GPU.
  struct GatedGroup {
    StreamRef dst;
    std::vector<tphip_copy_desc> table;
    uint32_t expiredSlot;
  };
  struct GatedUnit {
    UnitCompletion completion;
    std::shared_ptr<RecvOp> op;
    const uint64_t* word{nullptr};
    uint64_t value{0};
    uint32_t waitUs{0};
    std::vector<GatedGroup> groups;
    size_t remaining{0};
    bool acked{false};
  };

  // Launch (again) the copies of group k behind the gate and look at how they
  // ended once they have.
  void launchGated(const std::shared_ptr<GatedUnit>& u, size_t k) {
    GatedGroup& g = u->groups[k];
    g.expiredSlot = static_cast<uint32_t>(nextExpired_++ % kWordSlots);
    ChannelWords* mine = ictx_->signals->hostWords(wordsIndex_);
    __atomic_store_n(&mine->expired[g.expiredSlot], uint64_t(0), __ATOMIC_RELEASE);
    auto ev = ictx_->events.get(g.dst.device, g.dst.stream);
    TP_HIP_CHECK(tphip_batched_copy_gated(
        g.dst.device,
        g.table.data(),
        static_cast<uint32_t>(g.table.size()),
        g.dst.stream,
        ev->raw(),
        u->word,
        u->value,
        u->waitUs,
        &ictx_->signals->devWords(wordsIndex_)->expired[g.expiredSlot]));
    auto self = shared_from_this();
    ictx_->poller.watch(std::move(ev), &ictx_->events, [this, self, u, k](const Error& error) {
      ctx_->defer([this, self, u, k, error] {
        setError(error);
        const ChannelWords* words = ictx_->signals->hostWords(wordsIndex_);
        const bool gaveUp =
            __atomic_load_n(&words->expired[u->groups[k].expiredSlot], __ATOMIC_ACQUIRE) != 0;
        if (gaveUp && !error_) {
          // The producer is not done yet: wait again, longer.
          u->waitUs = std::min<uint32_t>(u->waitUs * 2, ictx_->gateWaitUs * 64);
          try {
            launchGated(u, k);
            return;
          } catch (const std::exception& ex) {
            TP_LOG_WARNING() << "Channel " << id_ << " gated copy failed: " << ex.what();
            setError(TP_CREATE_ERROR(HipError, "hip_ipc gated copy", TPHIP_ERR_INVALID_ARG));
          }
        }
        gatedGroupFinished(u);
      });
    });
  }

  // One group of a gated unit will not be launched again; the last one
  // acknowledges the unit and lets the recv callback go.
  void gatedGroupFinished(const std::shared_ptr<GatedUnit>& u) {
    if (--u->remaining > 0) {
      return;
    }
    if (!error_ && u->completion.byWord) {
      // the sender watches its word: raise it from the GPU, behind the copies
      const StreamRef& first = u->groups[0].dst;
      tphip_stream_signal(
          first.device,
          first.stream,
          &peerWords_->acks[u->completion.unitSeq % kWordSlots],
          ackValue(peerWordsGeneration_, u->completion.unitSeq));
    }
    unitCopiesFinished(u->completion);
    --u->op->landing;
    if (error_) {
      if (u->op->landing == 0) {
        finishRecv(u->op);
      }
    } else {
      flushRecvCallbacks();
    }
  }

  // Recv callbacks fire in the order of the recv calls: an op whose copies are
  // all enqueued waits for an older one whose bytes the agent has yet to land.
  void flushRecvCallbacks() {
    while (!recvOps_.empty() && recvOps_.front()->allSeen && recvOps_.front()->landing == 0) {
      auto op = recvOps_.front();
      recvOps_.pop_front();
      finishRecv(op);
    }
  }

  // Mappings nobody reads from go, oldest use first, while this channel holds
  // more than it may. (On an error the watchers still run and the destructor
  // releases what is left.)
  void dropLeastRecentlyUsedMappings() {
    while (mappedBytes_ > ictx_->maxMappedBytes || remoteAllocations_.size() > kMaxMappedAllocations) {
      auto victim = remoteAllocations_.end();
      for (auto it = remoteAllocations_.begin(); it != remoteAllocations_.end(); ++it) {
        if (it->second.inFlight == 0 &&
            (victim == remoteAllocations_.end() || it->second.lastUse < victim->second.lastUse)) {
          victim = it;
        }
      }
      if (victim == remoteAllocations_.end()) {
        return; // everything mapped is being read
      }
      TP_VLOG(5) << "Channel " << id_ << " drops its mapping of peer allocation #" << victim->first;
      HipIpcImports::get().release(victim->second.device, peerIdentity_, victim->first);
      mappedBytes_ -= victim->second.announcedSize;
      remoteAllocations_.erase(victim);
    }
  }

  void flushReplies() {
    while (!replyQueue_.empty() && replyQueue_.front()->ready && !error_) {
      replyQueue_.pop_front();
      TP_VLOG(6) << "Channel " << id_ << " is writing a reply";
      replyConnection_->write(nullptr, 0, onWritten([] {}));
    }
  }

  void failProtocol() {
    setError(TP_CREATE_ERROR(ShortReadError, -1, -1));
  }

  // ---- helpers ----------------------------------------------------------------

  // For the event behind a copy just launched on (device, stream): when it is
  // the kernel's own completion signal, the marker behind it is StreamMarkers'
  // business.
  template <typename F>
  void watchCopy(std::unique_ptr<HipEvent> ev, int device, void* stream, bool onKernel, F fn) {
    StreamMarkers::Launch launch;
    if (onKernel) {
      launch = ictx_->markers.launched(device, stream, ictx_->events);
    }
    auto self = shared_from_this();
    ictx_->poller.watch(
        std::move(ev),
        &ictx_->events,
        [this, self, device, stream, onKernel, launch, fn{std::move(fn)}](const Error& error) mutable {
          if (onKernel) {
            ictx_->markers.finished(device, stream, launch, ictx_->events);
          }
          ctx_->defer([this, self, fn{std::move(fn)}, error]() mutable {
            setError(error);
            if (!error_) {
              fn();
            }
          });
        });
  }

  // Run fn on the context loop once the event has completed.
  template <typename F>
  void watch(std::unique_ptr<HipEvent> ev, F fn) {
    auto self = shared_from_this();
    ictx_->poller.watch(
        std::move(ev), &ictx_->events, [this, self, fn{std::move(fn)}](const Error& error) mutable {
          ctx_->defer([this, self, fn{std::move(fn)}, error]() mutable {
            setError(error);
            if (!error_) {
              fn();
            }
          });
        });
  }

  void removeSend(const std::shared_ptr<SendOp>& op) {
    for (auto it = sendOps_.begin(); it != sendOps_.end(); ++it) {
      if (*it == op) {
        sendOps_.erase(it);
        return;
      }
    }
  }

  void finishSend(const std::shared_ptr<SendOp>& op) {
    if (op->done) {
      return;
    }
    op->done = true;
    auto cb = std::move(op->cb);
    cb(error_);
  }

  void finishRecv(const std::shared_ptr<RecvOp>& op) {
    if (op->done) {
      return;
    }
    op->done = true;
    auto cb = std::move(op->cb);
    TP_MARK("ipc: recv callback");
    cb(error_);
  }

  std::shared_ptr<IpcContextCore> ictx_;
  std::shared_ptr<transport::Connection> descriptorConnection_;
  std::shared_ptr<transport::Connection> replyConnection_;
  std::deque<std::shared_ptr<SendOp>> sendOps_;
  std::deque<std::shared_ptr<RecvOp>> recvOps_; // oldest first; callbacks fire from the front
  bool unitReadPosted_{false};
  bool helloPending_{false};
  std::deque<std::shared_ptr<WireUnit>> wireQueue_;
  std::deque<std::shared_ptr<ReplyUnit>> replyQueue_;
  std::map<int, bool> outboxAnnounced_;
  // Signal words: this end's slot in the context's page, and the peer's words
  // as mapped here for the GPU (null until its hello has arrived, or when it
  // has none).
  int wordsIndex_{-1};
  ChannelWords* peerWords_{nullptr}; // a device address: kernels only, never this process's CPUs
  uint64_t peerAgentMaxBytes_{0};
  bool peerGates_{false};
  uint32_t wordsGeneration_{0}; // of this end's words, told to the peer in the hello
  uint32_t peerWordsGeneration_{0};
  uint64_t nextGate_{0};
  uint64_t nextExpired_{0};
  uint64_t nextUnitOut_{0};
  uint64_t nextUnitIn_{0};
  std::array<bool, kWordSlots> ackSlotBusy_{};
  std::deque<std::shared_ptr<PendingAck>> pendingAcks_;
  std::shared_ptr<std::atomic<bool>> cancel_{std::make_shared<std::atomic<bool>>(false)};
  // Peer allocations this channel keeps mapped (direct route), by export id.
  struct RemoteAllocation {
    void* ptr;
    uint64_t size; // what a range inside it is checked against
    uint64_t announcedSize;
    int device;
    uint64_t lastUse;
    uint32_t inFlight; // units whose copies may still read from it
  };
  std::map<uint64_t, RemoteAllocation> remoteAllocations_;
  std::string peerIdentity_; // the peer's processIdentity(), from its hello
  uint64_t mappedBytes_{0};
  uint64_t useCounter_{0};
  struct RemoteOutbox {
    void* ptr;
    uint64_t slotBytes;
    uint32_t numSlots;
  };
  std::map<int, RemoteOutbox> remoteOutboxes_;
  // The peer's slabs (outboxes, signal page) this channel holds in the
  // process-wide import table.
  struct Import {
    int device;
    std::string peer;
    uint64_t id;
  };
  std::vector<Import> imports_;
};

class IpcChannel final : public ChannelHandle<ChannelImpl>, public BatchedChannel {
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

// Device descriptor "<boot id>|<process identity>|<device uuid>"
// (cf. DeviceDescriptor{bootId, pid, deviceUuid},
// tensorpipe/channel/cuda_ipc/context_impl.cc:108-113).
struct ParsedDescriptor {
  std::string boot;
  std::string process;
  std::string uuid;
};

bool parseDescriptor(const std::string& s, ParsedDescriptor* out) {
  auto a = s.find('|');
  auto b = a == std::string::npos ? a : s.find('|', a + 1);
  if (b == std::string::npos) {
    return false;
  }
  out->boot = s.substr(0, a);
  out->process = s.substr(a + 1, b - a - 1);
  out->uuid = s.substr(b + 1);
  return true;
}

class ContextImpl final : public Context {
 public:
  ContextImpl() {
    const int n = hipDeviceCountNoThrow();
    if (n <= 0) {
      return;
    }
    for (int i = 0; i < n; ++i) {
      char uuid[TPHIP_UUID_STRLEN + 1];
      if (tphip_device_uuid(i, uuid) != 0) {
        return;
      }
      descriptors_[Device{kHipDeviceType, i}] =
          bootIdentity() + "|" + processIdentity() + "|" + uuid;
    }
    core_ = std::make_shared<IpcContextCore>();
  }
  ~ContextImpl() override {
    join();
  }
  bool isViable() const override {
    return core_ != nullptr;
  }
  size_t numConnectionsNeeded() const override {
    return 2; // descriptors one way, replies the other
  }
  const std::unordered_map<Device, std::string>& deviceDescriptors() const override {
    return descriptors_;
  }
  // Same machine boot, different process
  // (tensorpipe/channel/cuda_ipc/context_impl.cc:310-335; the peer-to-peer
  // matrix check of the reference has no counterpart on a one-GPU machine:
  // a device can always reach itself).
  bool canCommunicateWithRemote(const std::string& local, const std::string& remote)
      const override {
    ParsedDescriptor l, r;
    if (!parseDescriptor(local, &l) || !parseDescriptor(remote, &r)) {
      return false;
    }
    if (l.boot != r.boot || l.process == r.process) {
      return false;
    }
    return l.uuid == r.uuid;
  }
  std::shared_ptr<Channel> createChannel(
      std::vector<std::shared_ptr<transport::Connection>> connections,
      Endpoint /*endpoint*/) override {
    if (!core_) {
      return std::make_shared<IpcChannel>(nullptr);
    }
    TP_THROW_ASSERT_IF(connections.size() != 2);
    auto impl = std::make_shared<ChannelImpl>(
        core_, core_->nextChannelId(), std::move(connections[0]), std::move(connections[1]));
    impl->init();
    return std::make_shared<IpcChannel>(std::move(impl));
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
  std::shared_ptr<IpcContextCore> core_;
  std::unordered_map<Device, std::string> descriptors_;
};

} // namespace

std::shared_ptr<Context> create() {
  return std::make_shared<ContextImpl>();
}

} // namespace hip_ipc
} // namespace channel
TP_AMD_NAMESPACE_END
