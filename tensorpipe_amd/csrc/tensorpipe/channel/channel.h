#pragma once

#include <functional>
#include <string>
#include <vector>

#include <tensorpipe/channel/context.h>
#include <tensorpipe/common/buffer.h>
#include <tensorpipe/common/error.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {

using TSendCallback = std::function<void(const Error&)>;
using TRecvCallback = std::function<void(const Error&)>;

// tensorpipe/channel/channel.h:52-72
class Channel {
 public:
  virtual void send(Buffer buffer, size_t length, TSendCallback callback) = 0;
  virtual void recv(Buffer buffer, size_t length, TRecvCallback callback) = 0;
  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual ~Channel() = default;
};

// Optional extension (no counterpart in the reference): a channel that can
// move all tensors of one message as one unit implements this as well. A
// caller that knows the message boundary (this library's Pipe does) finds it
// with dynamic_cast and hands over the whole message; the callback fires once
// for the batch. Both endpoints must use batches with the same number of
// entries and the same lengths, in the same order, as they must for
// individual send/recv calls.
struct BatchEntry {
  Buffer buffer;
  size_t length{0};
};

class BatchedChannel {
 public:
  virtual void sendBatch(std::vector<BatchEntry> entries, TSendCallback callback) = 0;
  virtual void recvBatch(std::vector<BatchEntry> entries, TRecvCallback callback) = 0;
  virtual ~BatchedChannel() = default;
};

} // namespace channel
TP_AMD_NAMESPACE_END
