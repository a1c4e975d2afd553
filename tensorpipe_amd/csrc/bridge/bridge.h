// A neutral face of this library's channels for hosting them inside another
// TensorPipe build -- the stock one that PyTorch carries in libtorch_cpu.so --
// without either header set seeing the other: both declare namespace
// tensorpipe, and this library's inline namespace keeps the symbols apart but
// not the names in one translation unit. Nothing here names a tensorpipe type
// of either side: strings, plain pointers, std::function.
//
//   host side (compiled against the host's tensorpipe headers)
//       tpbridge::Connection over the host's transport::Connection   --+
//       the host's channel::Context / Channel over tpbridge::Context  <-+-- this header
//   this side (bridge_amd.cc, part of libtensorpipe_amd.so)
//       tpbridge::Context over hip_xth / hip_ipc / hip_basic
//
// Interfaces followed on the host's side: tensorpipe/channel/context.h:32-105,
// tensorpipe/channel/channel.h:52-72, tensorpipe/transport/connection.h:21-69.
#pragma once

#include <cstddef>
#include <functional>
#include <memory>
#include <string>
#include <vector>

namespace tpbridge {

// An empty string means success; anything else is the error's text.
using ReadFn = std::function<void(const std::string& error, const void* ptr, size_t length)>;
using DoneFn = std::function<void(const std::string& error)>;

// One control connection handed to createChannel, implemented by the host.
class Connection {
 public:
  virtual void read(ReadFn fn) = 0; // next whole message, in the connection's own memory
  virtual void read(void* ptr, size_t length, ReadFn fn) = 0;
  virtual void write(const void* ptr, size_t length, DoneFn fn) = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual ~Connection() = default;
};

// What a tensor buffer boils down to on either side.
struct BufferRef {
  bool onGpu{false};
  void* ptr{nullptr};
  void* stream{nullptr}; // hipStream_t; unused for host memory
};

class Channel {
 public:
  virtual void send(BufferRef buffer, size_t length, DoneFn fn) = 0;
  virtual void recv(BufferRef buffer, size_t length, DoneFn fn) = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual ~Channel() = default;
};

struct DeviceDescriptor {
  std::string deviceType; // "cpu" or "cuda" (what PyTorch on ROCm calls a GPU)
  int deviceIndex{0};
  std::string descriptor;
};

class Context {
 public:
  virtual bool isViable() const = 0;
  virtual size_t numConnectionsNeeded() const = 0;
  virtual std::vector<DeviceDescriptor> deviceDescriptors() const = 0;
  virtual bool canCommunicateWithRemote(const std::string& local, const std::string& remote) const = 0;
  virtual std::shared_ptr<Channel> createChannel(
      std::vector<std::shared_ptr<Connection>> connections, bool listenSide) = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual void join() = 0;
  virtual ~Context() = default;
};

// "hip_xth", "hip_ipc" or "hip_basic" (which wraps this library's own basic CPU
// channel); null for any other name.
std::shared_ptr<Context> createContext(const std::string& channelName);

} // namespace tpbridge
