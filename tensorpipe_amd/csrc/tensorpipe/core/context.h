// tensorpipe::Context, same public surface as tensorpipe/core/context.h:26-94.
#pragma once

#include <memory>
#include <string>
#include <utility>
#include <vector>

#include <tensorpipe/channel/context.h>
#include <tensorpipe/transport/context.h>

TP_AMD_NAMESPACE_BEGIN

class ContextImpl;
class Listener;
class Pipe;

class ContextOptions {
 public:
  ContextOptions&& name(std::string name) && {
    name_ = std::move(name);
    return std::move(*this);
  }

  // Not in the reference: the pipes of this context put the reference's own
  // encodings on the wire (the libnop forms of tensorpipe/core/nop_types.h:26-80,
  // descriptor replies on a connection of their own as in
  // tensorpipe/core/pipe_impl.cc:262-345,987-1157) instead of this library's, so
  // that the peer may be an unmodified TensorPipe. Both ends of a pipe must
  // agree on the format. TP_STOCK_WIRE=1 in the environment switches it on
  // for every context.
  ContextOptions&& stockWireFormat(bool on = true) && {
    stockWire_ = on ? 1 : 0;
    return std::move(*this);
  }

 private:
  std::string name_;
  int stockWire_{-1}; // -1: as the environment says
  friend ContextImpl;
};

class PipeOptions {
 public:
  PipeOptions&& remoteName(std::string remoteName) && {
    remoteName_ = std::move(remoteName);
    return std::move(*this);
  }

 private:
  std::string remoteName_;
  friend ContextImpl;
};

class Context final {
 public:
  explicit Context(ContextOptions opts = ContextOptions());

  void registerTransport(
      int64_t priority,
      std::string transport,
      std::shared_ptr<transport::Context> context);

  void registerChannel(
      int64_t priority,
      std::string channel,
      std::shared_ptr<channel::Context> context);

  std::shared_ptr<Listener> listen(const std::vector<std::string>& urls);

  std::shared_ptr<Pipe> connect(const std::string& url, PipeOptions opts = PipeOptions());

  void close();
  void join();

  ~Context();

 private:
  const std::shared_ptr<ContextImpl> impl_;
};

TP_AMD_NAMESPACE_END
