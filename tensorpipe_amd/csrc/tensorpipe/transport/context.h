#pragma once

#include <memory>
#include <string>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN
namespace transport {

class Connection;
class Listener;

// Same virtual surface as tensorpipe/transport/context.h:20-75.
class Context {
 public:
  virtual std::shared_ptr<Connection> connect(std::string addr) = 0;
  virtual std::shared_ptr<Listener> listen(std::string addr) = 0;
  virtual bool isViable() const = 0;
  virtual const std::string& domainDescriptor() const = 0;
  virtual bool canCommunicateWithRemote(const std::string& remoteDomainDescriptor) const {
    return domainDescriptor() == remoteDomainDescriptor;
  }
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual void join() = 0;
  virtual ~Context() = default;
};

} // namespace transport
TP_AMD_NAMESPACE_END
