#pragma once

#include <functional>
#include <memory>
#include <string>

#include <tensorpipe/common/error.h>
#include <tensorpipe/transport/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace transport {

// tensorpipe/transport/listener.h:20-44
class Listener {
 public:
  using accept_callback_fn =
      std::function<void(const Error& error, std::shared_ptr<Connection> connection)>;
  virtual void accept(accept_callback_fn fn) = 0;
  virtual std::string addr() const = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual ~Listener() = default;
};

} // namespace transport
TP_AMD_NAMESPACE_END
