// tensorpipe::Pipe, same public surface as tensorpipe/core/pipe.h:40-96.
#pragma once

#include <functional>
#include <memory>
#include <string>

#include <tensorpipe/common/error.h>
#include <tensorpipe/core/message.h>

TP_AMD_NAMESPACE_BEGIN

class ContextImpl;
class ListenerImpl;
class PipeImpl;

class Pipe final {
  struct ConstructorToken {};

 public:
  Pipe(ConstructorToken token, std::shared_ptr<PipeImpl> impl);

  using read_descriptor_callback_fn = std::function<void(const Error&, Descriptor)>;
  void readDescriptor(read_descriptor_callback_fn fn);

  using read_callback_fn = std::function<void(const Error&)>;
  void read(Allocation allocation, read_callback_fn fn);

  using write_callback_fn = std::function<void(const Error&)>;
  void write(Message message, write_callback_fn fn);

  const std::string& getRemoteName();

  // Not in the reference: the name of the transport the pipe's own connections
  // run on once the handshake is over (it may differ from the one the pipe was
  // opened on, tensorpipe/core/pipe_impl.cc:1108-1125); empty until then. Waits
  // for the pipe's loop: not to be called from one of its callbacks.
  std::string transportInUse();

  void close();

  ~Pipe();

 private:
  const std::shared_ptr<PipeImpl> impl_;
  friend ContextImpl;
  friend ListenerImpl;
};

TP_AMD_NAMESPACE_END
