// tensorpipe::Listener, same public surface as tensorpipe/core/listener.h:35-94.
#pragma once

#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include <tensorpipe/common/error.h>

TP_AMD_NAMESPACE_BEGIN

class ContextImpl;
class ListenerImpl;
class Pipe;

class Listener final {
  struct ConstructorToken {};

 public:
  Listener(ConstructorToken token, std::shared_ptr<ListenerImpl> impl);

  using accept_callback_fn = std::function<void(const Error&, std::shared_ptr<Pipe>)>;
  void accept(accept_callback_fn fn);

  const std::map<std::string, std::string>& addresses() const;
  const std::string& address(const std::string& transport) const;
  std::string url(const std::string& transport) const;

  void close();

  ~Listener();

 private:
  const std::shared_ptr<ListenerImpl> impl_;
  friend ContextImpl;
};

TP_AMD_NAMESPACE_END
