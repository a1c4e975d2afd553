// Shared machinery of this library's channel implementations: one on-demand
// loop per channel context that serialises all of its channels, the error
// latch, enroll/unenroll for close(), and wrappers that bring transport
// callbacks onto that loop. Plays the part of
// tensorpipe/channel/{context,channel}_impl_boilerplate.h with plain base
// classes instead of CRTP.
#pragma once

#include <atomic>
#include <cstring>
#include <future>
#include <memory>
#include <string>
#include <unordered_set>
#include <vector>

#include <tensorpipe/channel/channel.h>
#include <tensorpipe/channel/context.h>
#include <tensorpipe/channel/error.h>
#include <tensorpipe/common/loop.h>
#include <tensorpipe/transport/connection.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {

class ChannelImplBase;

// State shared by a context object and all channels it created.
class ContextCore : public std::enable_shared_from_this<ContextCore> {
 public:
  virtual ~ContextCore() = default;

  void defer(TTask fn) {
    loop_.defer(std::move(fn));
  }
  bool inLoop() const {
    return loop_.inLoop();
  }
  bool closed() const {
    return closed_.load();
  }
  const std::string& id() const {
    return id_;
  }
  void setId(std::string id) {
    auto self = shared_from_this();
    defer([self, id{std::move(id)}]() mutable { self->id_ = std::move(id); });
  }
  std::string nextChannelId() {
    return id_ + ".c" + std::to_string(channelCounter_.fetch_add(1));
  }

  void enroll(std::shared_ptr<ChannelImplBase> ch) {
    channels_.insert(std::move(ch));
  }
  void unenroll(const std::shared_ptr<ChannelImplBase>& ch) {
    channels_.erase(ch);
  }

  void close();
  // Subclasses with threads or device resources stop/release them here;
  // called once, after close, from join().
  virtual void joinImpl() {}
  // close() only queues the closing on the loop, and a queued task may be run
  // later by another thread: the closing must have happened before joinImpl()
  // stops the threads that in-flight operations still need, so a second task
  // is queued behind it and awaited, as
  // tensorpipe/channel/context_impl_boilerplate.h:242-264 does.
  void join() {
    close();
    if (!joined_.exchange(true)) {
      if (!inLoop()) {
        auto closed = std::make_shared<std::promise<void>>();
        auto done = closed->get_future();
        defer([closed] { closed->set_value(); });
        done.wait();
      }
      joinImpl();
    }
  }

 private:
  OnDemandLoop loop_;
  std::atomic<bool> closed_{false};
  std::atomic<bool> joined_{false};
  std::atomic<uint64_t> channelCounter_{0};
  std::string id_{"N/A"};
  std::unordered_set<std::shared_ptr<ChannelImplBase>> channels_;
};

class ChannelImplBase : public std::enable_shared_from_this<ChannelImplBase> {
 public:
  ChannelImplBase(std::shared_ptr<ContextCore> ctx, std::string id)
      : ctx_(std::move(ctx)), id_(std::move(id)) {}
  virtual ~ChannelImplBase() = default;

  void init() {
    auto self = shared_from_this();
    ctx_->defer([self] {
      if (self->ctx_->closed()) {
        self->setError(TP_CREATE_ERROR(ContextClosedError));
        return;
      }
      self->ctx_->enroll(self);
      self->initFromLoop();
    });
  }

  void send(Buffer buffer, size_t length, TSendCallback callback) {
    auto self = shared_from_this();
    ctx_->defer([self, buffer, length, callback{std::move(callback)}]() mutable {
      const uint64_t seq = self->nextSend_++;
      TP_VLOG(4) << "Channel " << self->id_ << " received a send request (#" << seq << ")";
      if (self->error_) {
        callback(self->error_);
        return;
      }
      self->sendFromLoop(seq, std::move(buffer), length, std::move(callback));
    });
  }

  void recv(Buffer buffer, size_t length, TRecvCallback callback) {
    auto self = shared_from_this();
    ctx_->defer([self, buffer, length, callback{std::move(callback)}]() mutable {
      const uint64_t seq = self->nextRecv_++;
      TP_VLOG(4) << "Channel " << self->id_ << " received a recv request (#" << seq << ")";
      if (self->error_) {
        callback(self->error_);
        return;
      }
      self->recvFromLoop(seq, std::move(buffer), length, std::move(callback));
    });
  }

  void setId(std::string id) {
    auto self = shared_from_this();
    ctx_->defer([self, id{std::move(id)}]() mutable { self->id_ = std::move(id); });
  }

  void close() {
    auto self = shared_from_this();
    ctx_->defer([self] { self->setError(TP_CREATE_ERROR(ChannelClosedError)); });
  }

  // Loop only. First error wins and triggers handleError() once.
  void setError(Error error) {
    if (error_ || !error) {
      return;
    }
    error_ = std::move(error);
    TP_VLOG(5) << "Channel " << id_ << " is handling error " << error_.what();
    handleError();
    ctx_->unenroll(shared_from_this());
  }

 protected:
  virtual void initFromLoop() {}
  virtual void sendFromLoop(uint64_t seq, Buffer buffer, size_t length, TSendCallback cb) = 0;
  virtual void recvFromLoop(uint64_t seq, Buffer buffer, size_t length, TRecvCallback cb) = 0;
  // Must flush every pending callback with error_ and close the connections.
  virtual void handleError() = 0;

  // Wrap a loop-side handler into a transport write callback: hops onto the
  // context loop, latches the error first, then runs the handler regardless
  // (the handler looks at error_), like tensorpipe/common/callback.h:137-148.
  template <typename F>
  transport::Connection::write_callback_fn onWritten(F fn) {
    auto self = shared_from_this();
    return [self, fn{std::move(fn)}](const Error& error) mutable {
      self->ctx_->defer([self, fn{std::move(fn)}, error]() mutable {
        self->setError(error);
        fn();
      });
    };
  }

  // For reads into caller-provided memory (ptr stays valid).
  template <typename F>
  transport::Connection::read_callback_fn onRead(F fn) {
    auto self = shared_from_this();
    return [self, fn{std::move(fn)}](const Error& error, const void*, size_t) mutable {
      self->ctx_->defer([self, fn{std::move(fn)}, error]() mutable {
        self->setError(error);
        fn();
      });
    };
  }

  // For reads into a connection-owned buffer: the bytes are copied out before
  // leaving the transport's thread.
  template <typename F>
  transport::Connection::read_callback_fn onReadMessage(F fn) {
    auto self = shared_from_this();
    return [self, fn{std::move(fn)}](const Error& error, const void* ptr, size_t len) mutable {
      std::vector<uint8_t> bytes;
      if (!error && len > 0) {
        bytes.assign(static_cast<const uint8_t*>(ptr), static_cast<const uint8_t*>(ptr) + len);
      }
      self->ctx_->defer([self, fn{std::move(fn)}, error, bytes{std::move(bytes)}]() mutable {
        self->setError(error);
        fn(std::move(bytes));
      });
    };
  }

  // Write a small control message whose bytes are kept alive until written.
  void writeMessage(transport::Connection& conn, std::vector<uint8_t> bytes) {
    auto holder = std::make_shared<std::vector<uint8_t>>(std::move(bytes));
    conn.write(holder->data(), holder->size(), onWritten([holder] {}));
  }

  const std::shared_ptr<ContextCore> ctx_;
  std::string id_;
  Error error_;
  uint64_t nextSend_{0};
  uint64_t nextRecv_{0};
};

inline void ContextCore::close() {
  if (closed_.exchange(true)) {
    return;
  }
  auto self = shared_from_this();
  defer([self] {
    TP_VLOG(4) << "Channel context " << self->id_ << " is closing";
    auto channels = self->channels_;
    for (auto& ch : channels) {
      ch->setError(TP_CREATE_ERROR(ContextClosedError));
    }
  });
}

// Public channel handle: forwards to the impl, closes it when dropped
// (tensorpipe/channel/channel_boilerplate.h:86-140). A null impl means the
// context was not viable: every op fails with ContextNotViableError.
template <typename TImpl>
class ChannelHandle : public Channel {
 public:
  explicit ChannelHandle(std::shared_ptr<TImpl> impl) : impl_(std::move(impl)) {}
  ~ChannelHandle() override {
    if (impl_) {
      impl_->close();
    }
  }
  void send(Buffer buffer, size_t length, TSendCallback callback) override {
    if (!impl_) {
      callback(TP_CREATE_ERROR(ContextNotViableError));
      return;
    }
    impl_->send(std::move(buffer), length, std::move(callback));
  }
  void recv(Buffer buffer, size_t length, TRecvCallback callback) override {
    if (!impl_) {
      callback(TP_CREATE_ERROR(ContextNotViableError));
      return;
    }
    impl_->recv(std::move(buffer), length, std::move(callback));
  }
  void setId(std::string id) override {
    if (impl_) {
      impl_->setId(std::move(id));
    }
  }
  void close() override {
    if (impl_) {
      impl_->close();
    }
  }

 protected:
  std::shared_ptr<TImpl> impl_;
};

} // namespace channel
TP_AMD_NAMESPACE_END
