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
// Synchronisation between the two processes goes through the host: the sender
// announces a tensor (or chunk) once a HIP event recorded behind the producing
// work has completed, and the receiver replies once an event recorded behind
// its copy has completed. Inter-process HIP events would let both sides skip
// the host, as the reference does with CUDA IPC events, but exporting an event
// fails on the deployment this was built for, so they are not used.
//
// The recv callback fires when the copy has been enqueued on the caller's
// stream (as in the reference); the send callback fires when the source may be
// reused: after the receiver's reply (direct) or after the last chunk has been
// staged (outbox).

#include <tensorpipe/channel/hip_ipc/factory.h>

#include <algorithm>
#include <array>
#include <cstdlib>
#include <deque>
#include <map>
#include <mutex>
#include <set>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/channel/hip_common.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/common/slot_allocator.h>
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
            it->second.size < maxExportBytes) {
          *out = it->second;
          *offset = static_cast<uint64_t>(p - base);
          return true;
        }
      }
    }
    void* base = nullptr;
    size_t size = 0;
    if (tphip_mem_base(ptr, &base, &size) != 0 || base == nullptr || size >= maxExportBytes) {
      return false;
    }
    uint64_t bufferId = 0;
    tphip_mem_buffer_id(base, &bufferId);
    *offset = static_cast<uint64_t>(
        static_cast<const uint8_t*>(ptr) - static_cast<const uint8_t*>(base));
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = exports_.find(base);
    if (it != exports_.end() && it->second.size == size && it->second.bufferId == bufferId) {
      *out = it->second;
      return true;
    }
    // New allocation, or the address was freed and handed out again.
    ExportedAllocation e;
    if (tphip_ipc_mem_export(device, base, e.handle.data()) != 0) {
      return false;
    }
    e.id = nextExportId();
    e.base = reinterpret_cast<uint64_t>(base);
    e.size = size;
    e.bufferId = bufferId;
    exports_[base] = e;
    *out = e;
    forgetFreedAllocations();
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
      : slab(device, slotBytes * numSlots), allocator(slab.ptr(), numSlots, slotBytes) {
    TP_HIP_CHECK(tphip_ipc_mem_export(device, slab.ptr(), handle.data()));
  }
  HipDeviceSlab slab;
  HandleBytes handle;
  SlotAllocator allocator;
  const uint64_t id{nextExportId()};
};

class IpcContextCore final : public ContextCore {
 public:
  HipEventPool events;
  HipEventPoller poller;
  StreamIdleProbe idleProbe; // loop only
  StreamMarkers markers;
  const bool forceOutbox{outboxForcedByEnv()};
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
    poller.join();
  }

 private:
  std::vector<std::unique_ptr<Outbox>> outboxes_;
};

enum MsgKind : uint8_t { kDirect = 1, kChunk = 2 };

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

  // Every copy out of a mapped peer allocation is followed by an event whose
  // watcher keeps this object alive, so nothing reads the mappings any more.
  ~ChannelImpl() override {
    for (auto& i : imports_) {
      HipIpcImports::get().release(i.device, i.peer, i.id);
    }
    for (auto& kv : remoteAllocations_) {
      HipIpcImports::get().release(kv.second.device, peerIdentity_, kv.first);
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
      finishRecv(op);
    }
    wireQueue_.clear();
    replyQueue_.clear();
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
  // staged chunk. Units are written strictly in creation order.
  struct WireUnit {
    std::vector<uint8_t> bytes;
    bool ready{false};
    std::function<void()> onReply; // runs when the matching reply arrives
  };

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

  // ---- send -----------------------------------------------------------------

  void sendEntries(uint64_t seq, std::vector<BatchEntry> entries, TSendCallback cb) {
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
                device, hb.ptr, ictx_->maxExportBytes, &item.alloc, &item.offset)) {
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
        w.u8(kDirect);
        w.u8(identitySent_ ? 0 : 1);
        if (!identitySent_) {
          w.str(processIdentity());
          identitySent_ = true;
        }
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
        if (busy.empty()) {
          unit->ready = true;
          flushWire();
        }
        auto remaining = std::make_shared<size_t>(busy.size());
        for (auto& s : busy) {
          auto ev = ictx_->events.get(s.device);
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
  // when the receiver has replied.
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
        ev = ictx_->events.get(device);
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
      w.u8(kChunk);
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
      unit->onReply = [slot]() mutable { slot.reset(); }; // reply frees the slot
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

  // Write every unit at the head of the queue whose data is ready, and post
  // the read for its reply.
  void flushWire() {
    while (!wireQueue_.empty() && wireQueue_.front()->ready && !error_) {
      auto unit = wireQueue_.front();
      wireQueue_.pop_front();
      TP_VLOG(6) << "Channel " << id_ << " is writing a descriptor";
      writeMessage(*descriptorConnection_, std::move(unit->bytes));
      replyConnection_->read(nullptr, 0, onRead([this, unit] {
        if (!error_ && unit->onReply) {
          unit->onReply();
        }
        unit->onReply = nullptr;
      }));
    }
  }

  // ---- recv -----------------------------------------------------------------

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
  void pumpUnits() {
    if (unitReadPosted_ || recvOps_.empty() || error_) {
      return;
    }
    unitReadPosted_ = true;
    descriptorConnection_->read(onReadMessage([this](std::vector<uint8_t> bytes) {
      unitReadPosted_ = false;
      if (error_ || recvOps_.empty()) {
        return;
      }
      auto op = recvOps_.front();
      onUnit(op, bytes);
      pumpUnits();
    }));
  }

  void onUnit(const std::shared_ptr<RecvOp>& op, const std::vector<uint8_t>& bytes) {
    WireReader r(bytes.data(), bytes.size());
    const uint8_t kind = r.u8();
    TP_VLOG(6) << "Channel " << id_ << " got a descriptor of kind " << int(kind) << " (#"
               << op->seq << ")";
    auto reply = std::make_shared<ReplyUnit>();
    replyQueue_.push_back(reply);
    std::vector<std::unique_ptr<HipEvent>> launched; // one event per copy launch
    std::vector<uint64_t> inUse; // peer allocations the copies of this unit read from
    bool chunkOnKernel = false; // a staged chunk whose event is the kernel's own signal
    StreamRef chunkStream{nullptr, 0};
    try {
      if (kind == kDirect) {
        if (r.u8() != 0) {
          peerIdentity_ = r.str();
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
          // The range must lie inside the allocation the peer announced: the
          // copy kernel would fault on anything else.
          if (length != op->entries[index].length || offset > a.size || length > a.size - offset) {
            failProtocol();
            return;
          }
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
              it = remoteAllocations_.emplace(a.id, RemoteAllocation{mapped, a.size, device, 0, 0}).first;
              mappedBytes_ += a.size;
            } else if (it->second.size != a.size) {
              failProtocol(); // one identifier, one allocation
              return;
            }
            it->second.lastUse = ++useCounter_;
            mappedOf[allocIdx] = &it->second;
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
          ++op->unitsSeen;
        }
        // From here until the copies have finished the mappings must stay.
        for (uint32_t a = 0; a < nAllocs; ++a) {
          if (mappedOf[a] != nullptr) {
            ++mappedOf[a]->inFlight;
            inUse.push_back(announced[a].id);
          }
        }
        for (auto& g : groups) {
          auto ev = ictx_->events.get(g.dst.device);
          hipBatchedCopy(g.dst.device, g.dst.stream, g.table, *ev, /*signalOnKernel=*/false);
          launched.push_back(std::move(ev));
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
          remoteOutboxes_[srcDevice] = RemoteOutbox{mapped, remoteSlotBytes, remoteNumSlots};
          imports_.push_back(Import{device, peer, outboxId});
        }
        const uint32_t slotIdx = r.u32();
        const uint64_t offset = r.u64();
        const uint64_t len = r.u64();
        auto it = remoteOutboxes_.find(srcDevice);
        if (!r.ok() || it == remoteOutboxes_.end() || slotIdx >= it->second.numSlots ||
            len > it->second.slotBytes || offset + len > op->entries[index].length) {
          failProtocol();
          return;
        }
        auto ev = ictx_->events.get(device);
        chunkOnKernel = hipBatchedCopy(
            device,
            hb.stream,
            {tphip_copy_desc{
                static_cast<const uint8_t*>(it->second.ptr) + slotIdx * it->second.slotBytes,
                static_cast<uint8_t*>(hb.ptr) + offset,
                len}},
            *ev,
            /*signalOnKernel=*/(op->entries[index].length + it->second.slotBytes - 1) /
                    it->second.slotBytes >=
                kChunksForKernelSignals);
        chunkStream = StreamRef{hb.stream, device};
        launched.push_back(std::move(ev));
        // A staged tensor counts as seen when its last chunk arrived.
        if (offset + len == op->entries[index].length) {
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
      setError(TP_CREATE_ERROR(HipError, "hip_ipc recv", TPHIP_ERR_INVALID_ARG));
      return;
    }

    TP_VLOG(6) << "Channel " << id_ << " enqueued the copies (#" << op->seq << ")";
    // Reply once the copies of this unit have finished.
    auto remaining = std::make_shared<size_t>(launched.size());
    for (auto& ev : launched) {
      watchCopy(std::move(ev), chunkStream.device, chunkStream.stream, chunkOnKernel, [this, reply, remaining, inUse] {
        if (--*remaining == 0) {
          for (uint64_t id : inUse) {
            auto it = remoteAllocations_.find(id);
            if (it != remoteAllocations_.end() && it->second.inFlight > 0) {
              --it->second.inFlight;
            }
          }
          dropLeastRecentlyUsedMappings();
          reply->ready = true;
          flushReplies();
        }
      });
    }

    if (op->unitsSeen == op->entries.size()) {
      // Every copy of the op is enqueued: that is what the recv callback means.
      removeRecv(op);
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
      mappedBytes_ -= victim->second.size;
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

  std::shared_ptr<IpcContextCore> ictx_;
  std::shared_ptr<transport::Connection> descriptorConnection_;
  std::shared_ptr<transport::Connection> replyConnection_;
  std::deque<std::shared_ptr<SendOp>> sendOps_;
  std::deque<std::shared_ptr<RecvOp>> recvOps_; // oldest first; the front one takes the next unit
  bool unitReadPosted_{false};
  std::deque<std::shared_ptr<WireUnit>> wireQueue_;
  std::deque<std::shared_ptr<ReplyUnit>> replyQueue_;
  bool identitySent_{false};
  std::map<int, bool> outboxAnnounced_;
  // Peer allocations this channel keeps mapped (direct route), by export id.
  struct RemoteAllocation {
    void* ptr;
    uint64_t size;
    int device;
    uint64_t lastUse;
    uint32_t inFlight; // units whose copies may still read from it
  };
  std::map<uint64_t, RemoteAllocation> remoteAllocations_;
  std::string peerIdentity_; // the peer's processIdentity(), from its first direct unit
  uint64_t mappedBytes_{0};
  uint64_t useCounter_{0};
  struct RemoteOutbox {
    void* ptr;
    uint64_t slotBytes;
    uint32_t numSlots;
  };
  std::map<int, RemoteOutbox> remoteOutboxes_;
  // The peer's outboxes this channel holds in the process-wide import table.
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
