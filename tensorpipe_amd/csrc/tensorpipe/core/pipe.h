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

  void close();

  ~Pipe();

 private:
  const std::shared_ptr<PipeImpl> impl_;
  friend ContextImpl;
  friend ListenerImpl;
};

TP_AMD_NAMESPACE_END
