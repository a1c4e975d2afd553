// hip_xth: GPU-to-GPU channel between two pipe endpoints of ONE process.
//
// Sender: ships raw {stream, device, src pointer, length} words over the
// descriptor connection -- they are valid in the receiver because it is the
// same address space -- and waits for an empty completion message.
// Receiver: enqueues ONE batched copy kernel for all tensors of the message
// ON THE SENDER'S STREAM, which orders the copy after the work that produced
// the source and before anything the sender enqueues later (it may overwrite
// the source as soon as its send callback has fired), without a single
// cross-stream dependency. A destination stream that still has work pending is
// made a dependency of the copy (event + stream wait); an idle one costs one
// query. A poller thread watches an event recorded behind the copy; when it
// has completed the recv callback fires and the completion message goes out.
// Receives that become ready while a copy of the channel is still running
// share the next launch (launchReady below): a caller that moves a message
// tensor by tensor still gets few launches.
//
// The wire protocol of tensorpipe/channel/cuda_xth/channel_impl.cc:30-36,
// 96-315 (descriptor one way, completion back), with a completion that counts
// the receives it stands for instead of being empty. Differences, all for
// latency: a whole message travels in one descriptor and one kernel launch
// instead of one cudaMemcpyAsync per tensor; there are no start/stop events
// and no stream waits on the common path (a stream wait costs 12-19 us of host
// time on MI355X with ROCm 7, an event query about one); and the recv
// callback fires when the copy has FINISHED rather than when it was enqueued
// (cuda_xth/channel_impl.cc:66-77), which is the stronger guarantee and is
// required because the copy does not run on the receiver's stream.

#include <tensorpipe/channel/hip_xth/factory.h>

#include <deque>

#include <mutex>
#include <unordered_map>

#include <tensorpipe/channel/channel_base.h>
#include <tensorpipe/channel/hip_common.h>
#include <tensorpipe/common/hip_buffer.h>
#include <tensorpipe/common/stage_timer.h>
#include <tensorpipe/common/wire.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_xth {

namespace {

class XthContextCore final : public ContextCore {
 public:
  HipEventPool events;
  HipEventPoller poller;
  StreamIdleProbe idleProbe; // loop only
  StreamMarkers markers;
  void joinImpl() override {
    poller.join();
  }
};

struct StreamRef {
  void* stream;
  int device;
  bool operator==(const StreamRef& o) const {
    return stream == o.stream && device == o.device;
  }
};

// Where the tensors of one send come from. Both ends of this channel live in
// one process, so the sender does not spell the list out on the connection: it
// parks it here and sends its ticket, the receiver takes it out (for the 256
// tensors of a many-tensor message that is 16 bytes on the wire instead of
// 7 KiB, and no encoding or decoding on either side). A ticket that is not
// here any more -- the sender failed and took its list back -- is an error, not
// a dangling pointer.
struct SourceList {
  struct Item {
    StreamRef src;
    const void* ptr;
    uint64_t length;
  };
  std::vector<Item> items;
};

class SourceLists {
 public:
  static SourceLists& get() {
    static SourceLists* lists = new SourceLists();
    return *lists;
  }
  uint64_t park(std::unique_ptr<SourceList> list) {
    std::lock_guard<std::mutex> lock(mutex_);
    const uint64_t ticket = next_++;
    parked_[ticket] = std::move(list);
    return ticket;
  }
  std::unique_ptr<SourceList> take(uint64_t ticket) {
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = parked_.find(ticket);
    if (it == parked_.end()) {
      return nullptr;
    }
    auto list = std::move(it->second);
    parked_.erase(it);
    return list;
  }

 private:
  std::mutex mutex_;
  uint64_t next_{1};
  std::unordered_map<uint64_t, std::unique_ptr<SourceList>> parked_;
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
    // Every pending callback fires now, in order, with the error -- except for
    // receives whose copy is already running: that kernel sits on the sender's
    // stream and keeps writing into the receive buffer, so its callback waits
    // for the event behind the copy (the watcher finishes the op).
    auto sends = std::move(sendOps_);
    sendOps_.clear();
    for (auto& op : sends) {
      SourceLists::get().take(op->ticket); // if the receiver has not come for it, nobody will
      finishSend(op);
    }
    toLaunch_.clear();
    toLaunchBytes_ = 0;
    decodedInQueue_ = 0;
    auto recvs = std::move(recvOps_);
    recvOps_.clear();
    for (auto& op : recvs) {
      if (op->copiesInFlight == 0) {
        finishRecv(op);
      }
    }
  }

 private:
  struct SendOp {
    uint64_t seq;
    TSendCallback cb;
    uint64_t ticket{0}; // of the source list parked for the receiver
    bool done{false};
  };

  struct RecvOp {
    uint64_t seq;
    TRecvCallback cb;
    std::vector<BatchEntry> entries; // non-empty ones only
    // From the descriptor: where each entry comes from, which streams are involved.
    struct Piece {
      StreamRef src;
      StreamRef dst;
      tphip_copy_desc copy;
    };
    std::vector<Piece> pieces;
    uint64_t bytes{0};
    size_t copiesInFlight{0};
    bool copied{false}; // every copy of the op has completed
    bool done{false};
  };

  void sendEntries(uint64_t seq, std::vector<BatchEntry> entries, TSendCallback cb) {
    hipPointerCheckpoint(); // the caller's buffers: believed for this call only
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
    TP_MARK("xth: send");
    auto op = std::make_shared<SendOp>();
    op->seq = seq;
    op->cb = std::move(cb);
    TP_VLOG(9) << "Channel " << id_ << " is encoding descriptor (#" << seq << ")";

    // On the wire: how many tensors, and the ticket of their list.
    StageScope timer(Stage::kXthEncode);
    auto list = std::make_unique<SourceList>();
    list->items.reserve(live.size());
    try {
      for (auto& e : live) {
        const HipBuffer& hb = e.buffer.unwrap<HipBuffer>();
        const int device = hipDeviceForPointer(hb.ptr);
        TP_THROW_ASSERT_IF(device < 0);
        list->items.push_back(SourceList::Item{StreamRef{hb.stream, device}, hb.ptr, e.length});
      }
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " send failed: " << ex.what();
      op->cb(TP_CREATE_ERROR(HipError, "hip_xth send", TPHIP_ERR_INVALID_ARG));
      setError(TP_CREATE_ERROR(HipError, "hip_xth send", TPHIP_ERR_INVALID_ARG));
      return;
    }
    WireWriter w;
    w.u32(static_cast<uint32_t>(live.size()));
    op->ticket = SourceLists::get().park(std::move(list));
    w.u64(op->ticket);

    sendOps_.push_back(op);
    TP_VLOG(6) << "Channel " << id_ << " is writing descriptor (#" << seq << ")";
    writeMessage(*descriptorConnection_, std::move(w.bytes()));
    TP_MARK("xth: descriptor written");
    armCompletionRead();
  }

  // One read is kept posted while sends are out. A completion message names
  // how many of them, oldest first, the receiver has copied: receives that
  // shared a launch are reported together.
  void armCompletionRead() {
    if (completionReadArmed_ || sendOps_.empty() || error_) {
      return;
    }
    completionReadArmed_ = true;
    TP_VLOG(6) << "Channel " << id_ << " is reading a completion";
    completionConnection_->read(&completedSends_, sizeof(completedSends_), onRead([this] {
      completionReadArmed_ = false;
      if (error_) {
        return;
      }
      TP_MARK("xth: completion arrived (send callback)");
      if (completedSends_ == 0 || completedSends_ > sendOps_.size()) {
        setError(TP_CREATE_ERROR(ShortReadError, static_cast<ssize_t>(sendOps_.size()), completedSends_));
        return;
      }
      for (uint32_t k = 0; k < completedSends_ && !sendOps_.empty(); ++k) {
        auto op = sendOps_.front();
        sendOps_.pop_front();
        TP_VLOG(6) << "Channel " << id_ << " done reading completion (#" << op->seq << ")";
        finishSend(op);
      }
      armCompletionRead();
    }));
  }

  void recvEntries(uint64_t seq, std::vector<BatchEntry> entries, TRecvCallback cb) {
    hipPointerCheckpoint(); // the caller's buffers: believed for this call only
    TP_MARK("xth: recv");
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
        TP_MARK("xth: descriptor arrived");
        copyFromDescriptor(op, bytes);
      }
    }));
  }

  // Reads where the op's tensors come from, then launches -- at once, or
  // together with the ops behind it (see launchReady).
  void copyFromDescriptor(const std::shared_ptr<RecvOp>& op, const std::vector<uint8_t>& bytes) {
    WireReader r(bytes.data(), bytes.size());
    const uint32_t n = r.u32();
    const uint64_t ticket = r.u64();
    if (!r.ok() || n != op->entries.size()) {
      setError(TP_CREATE_ERROR(ShortReadError, static_cast<ssize_t>(op->entries.size()), n));
      return;
    }
    {
      StageScope decodeTimer(Stage::kXthDecode);
      auto list = SourceLists::get().take(ticket);
      if (!list || list->items.size() != n) {
        // the sender is gone, or this is not a descriptor of this library's
        setError(TP_CREATE_ERROR(ShortReadError, static_cast<ssize_t>(n), list ? static_cast<ssize_t>(list->items.size()) : -1));
        return;
      }
      try {
        op->pieces.reserve(n);
        for (uint32_t i = 0; i < n; ++i) {
          const SourceList::Item& item = list->items[i];
          if (item.length != op->entries[i].length) {
            setError(TP_CREATE_ERROR(
                ShortReadError, static_cast<ssize_t>(op->entries[i].length), static_cast<ssize_t>(item.length)));
            return;
          }
          const HipBuffer& hb = op->entries[i].buffer.unwrap<HipBuffer>();
          StreamRef dstRef{hb.stream, hipDeviceForPointer(hb.ptr)};
          TP_THROW_ASSERT_IF(dstRef.device < 0);
          op->pieces.push_back(RecvOp::Piece{item.src, dstRef, tphip_copy_desc{item.ptr, hb.ptr, item.length}});
          op->bytes += item.length;
        }
      } catch (const std::exception& ex) {
        TP_LOG_WARNING() << "Channel " << id_ << " copy failed: " << ex.what();
        setError(TP_CREATE_ERROR(HipError, "hip_xth copy", TPHIP_ERR_INVALID_ARG));
        return;
      }
    }
    TP_MARK("xth: descriptor decoded");
    ++decodedInQueue_;
    toLaunch_.push_back(op);
    toLaunchBytes_ += op->bytes;
    launchReady(/*copyFinished=*/false);
  }

  // Launches the ops whose descriptors are in, all of them in one kernel per
  // source stream. A caller that hands over a message tensor by tensor (a
  // stock pipe does: one send and one recv per tensor) would otherwise pay one
  // launch, one event and one poll per tensor, 4-5 us of host time each, for
  // copies that take the GPU a microsecond. So while a copy of this channel is
  // still running and more receives are posted than descriptors have come in,
  // small ops wait and ride together on the next launch, which goes out when
  // the running copy ends, when every posted receive has its descriptor, or
  // when enough has gathered. Nothing waits while the GPU has none of this
  // channel's work, and large copies never wait: for them the launch is
  // noise, and queueing them behind the running one keeps the GPU fed.
  void launchReady(bool copyFinished) {
    if (toLaunch_.empty() || error_) {
      return;
    }
    const bool moreComing = recvOps_.size() > decodedInQueue_;
    if (!copyFinished && launchesInFlight_ > 0 && moreComing && toLaunchBytes_ < kGatherBytes &&
        toLaunch_.size() < kGatherOps) {
      return;
    }
    struct Group {
      StreamRef src;
      std::vector<StreamRef> dstStreams;
      std::vector<tphip_copy_desc> table;
      std::vector<std::shared_ptr<RecvOp>> ops;
    };
    std::vector<Group> groups;
    auto ops = std::move(toLaunch_);
    toLaunch_.clear();
    toLaunchBytes_ = 0;
    size_t pieces = 0;
    for (auto& op : ops) {
      pieces += op->pieces.size();
    }
    for (auto& op : ops) {
      for (auto& piece : op->pieces) {
        Group* g = nullptr;
        for (auto& cand : groups) {
          if (cand.src == piece.src) {
            g = &cand;
          }
        }
        if (g == nullptr) {
          groups.push_back(Group{piece.src, {}, {}, {}});
          g = &groups.back();
          g->table.reserve(pieces); // normally the only group
        }
        bool known = false;
        for (auto& d : g->dstStreams) {
          known |= d == piece.dst;
        }
        if (!known && !(piece.dst == piece.src)) {
          g->dstStreams.push_back(piece.dst);
        }
        g->table.push_back(piece.copy);
        if (g->ops.empty() || g->ops.back() != op) {
          g->ops.push_back(op);
        }
      }
      op->pieces.clear();
    }
    try {
      for (auto& g : groups) {
        StageScope launchTimer(Stage::kXthLaunch);
        // The copy may only touch a destination once everything the receiver
        // enqueued before recv() on that buffer's stream is done.
        for (auto& d : g.dstStreams) {
          if (!xctx_->idleProbe.idle(d.device, d.stream)) {
            auto ev = xctx_->events.get(d.device, d.stream);
            ev->record(d.stream);
            ev->wait(g.src.stream, g.src.device);
            xctx_->events.put(std::move(ev)); // the wait captured the record
          }
        }
        TP_VLOG(6) << "Channel " << id_ << " is copying payload (#" << g.ops.front()->seq << " to #"
                   << g.ops.back()->seq << ")";
        TP_MARK("xth: destination streams checked");
        auto done = xctx_->events.get(g.src.device, g.src.stream);
        const bool onKernel =
            hipBatchedCopy(g.src.device, g.src.stream, g.table, *done, /*signalOnKernel=*/true);
        TP_MARK("xth: kernel launch call returned");
        StreamMarkers::Launch launch;
        if (onKernel) {
          launch = xctx_->markers.launched(g.src.device, g.src.stream, xctx_->events);
        }
        TP_MARK("xth: copy launched");
        auto self = shared_from_this();
        // Counted per launch: if a later launch fails, the error path still
        // waits for exactly the copies that are running.
        for (auto& op : g.ops) {
          ++op->copiesInFlight;
        }
        ++launchesInFlight_;
        const StreamRef src = g.src;
        xctx_->poller.watch(
            std::move(done), &xctx_->events,
            [this, self, carried{std::move(g.ops)}, src, onKernel, launch](const Error& error) {
              TP_MARK("xth: copy seen finished");
              if (onKernel) {
                // before anybody hears of the completion: the stream is still the sender's to keep
                xctx_->markers.finished(src.device, src.stream, launch, xctx_->events);
              }
              ctx_->defer([this, self, carried, error] {
                setError(error);
                --launchesInFlight_;
                for (auto& op : carried) {
                  if (--op->copiesInFlight > 0) {
                    continue;
                  }
                  if (error_) {
                    finishRecv(op); // no longer in recvOps_: the error path left it to us
                    continue;
                  }
                  TP_VLOG(6) << "Channel " << id_ << " done copying payload (#" << op->seq << ")";
                  op->copied = true;
                }
                if (!error_) {
                  TP_MARK("xth: recv callback due");
                  launchReady(/*copyFinished=*/true); // what gathered meanwhile goes first: the GPU is idle
                  flushRecvs();
                }
              });
            });
      }
    } catch (const std::exception& ex) {
      TP_LOG_WARNING() << "Channel " << id_ << " copy failed: " << ex.what();
      // A copy may have been launched without an event behind it: wait for the
      // source streams before the receive buffers are handed back.
      for (auto& g : groups) {
        tphip_stream_sync(g.src.device, g.src.stream);
      }
      setError(TP_CREATE_ERROR(HipError, "hip_xth copy", TPHIP_ERR_INVALID_ARG));
    }
  }

  // Completions go out in the order the descriptors came in (the sender pairs
  // them by position), each once its copies have finished.
  void flushRecvs() {
    uint32_t finished = 0;
    while (!recvOps_.empty() && recvOps_.front()->copied && !error_) {
      auto op = recvOps_.front();
      recvOps_.pop_front();
      --decodedInQueue_;
      // The receiver's callback first, the completion after it: the sender's
      // callback then is the last one of a transfer and runs on the sender's own
      // loop, where a caller that chains its next write from the callbacks
      // wants to be (the other order saves the sender a microsecond and costs
      // such a caller ten: its next write starts on a foreign thread).
      finishRecv(op);
      ++finished;
    }
    if (finished > 0 && !error_) {
      TP_VLOG(6) << "Channel " << id_ << " is writing the completion of " << finished << " receive(s)";
      WireWriter w;
      w.u32(finished);
      writeMessage(*completionConnection_, std::move(w.bytes()));
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

  std::shared_ptr<XthContextCore> xctx_;
  std::shared_ptr<transport::Connection> descriptorConnection_;
  std::shared_ptr<transport::Connection> completionConnection_;
  std::deque<std::shared_ptr<SendOp>> sendOps_;
  std::deque<std::shared_ptr<RecvOp>> recvOps_;
  // Decoded, not yet launched (a run at the tail of the decoded part of recvOps_).
  std::vector<std::shared_ptr<RecvOp>> toLaunch_;
  uint64_t toLaunchBytes_{0};
  size_t launchesInFlight_{0};
  bool completionReadArmed_{false};
  uint32_t completedSends_{0}; // the posted completion read lands here
  size_t decodedInQueue_{0}; // members of recvOps_ whose descriptor has come in (they sit at its front)
  static constexpr uint64_t kGatherBytes = 8u << 20;
  static constexpr size_t kGatherOps = 256;
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
