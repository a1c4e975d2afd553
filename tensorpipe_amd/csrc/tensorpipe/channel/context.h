#pragma once

#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include <tensorpipe/common/buffer.h>
#include <tensorpipe/transport/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {

enum class Endpoint : bool { kConnect, kListen };

class Channel;

// Plugin surface of a channel type; same virtuals, in the same order, as
// tensorpipe/channel/context.h:32-105.
class Context {
 public:
  virtual bool isViable() const = 0;
  virtual size_t numConnectionsNeeded() const = 0;
  virtual const std::unordered_map<Device, std::string>& deviceDescriptors() const = 0;
  virtual bool canCommunicateWithRemote(
      const std::string& localDeviceDescriptor,
      const std::string& remoteDeviceDescriptor) const = 0;
  virtual std::shared_ptr<Channel> createChannel(
      std::vector<std::shared_ptr<transport::Connection>>,
      Endpoint) = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual void join() = 0;
  virtual ~Context() = default;
};

} // namespace channel
TP_AMD_NAMESPACE_END
