#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <string>

#include <tensorpipe/common/error.h>
#include <tensorpipe/transport/context.h>

TP_AMD_NAMESPACE_BEGIN

// Object that can turn itself into bytes and back. Occupies the place of the
// reference's nop holder in the Connection interface; the encoding is this
// library's own (see common/wire.h), not libnop's.
class AbstractNopHolder {
 public:
  virtual size_t getSize() const = 0;
  virtual void serialize(uint8_t* out, size_t size) const = 0;
  virtual bool deserialize(const uint8_t* in, size_t size) = 0;
  virtual ~AbstractNopHolder() = default;
};

namespace transport {

// Message-oriented, ordered, reliable byte pipe between two endpoints.
// Virtual functions in the order of tensorpipe/transport/connection.h:21-69.
class Connection {
 public:
  using read_callback_fn = std::function<void(const Error& error, const void* ptr, size_t length)>;

  // Read the next message into a buffer owned by the connection, valid only
  // during the callback.
  virtual void read(read_callback_fn fn) = 0;
  // Read the next message, which must be exactly `length` bytes, into `ptr`.
  virtual void read(void* ptr, size_t length, read_callback_fn fn) = 0;

  using write_callback_fn = std::function<void(const Error& error)>;
  // `ptr` must stay valid until the callback fires.
  virtual void write(const void* ptr, size_t length, write_callback_fn fn) = 0;

  using read_nop_callback_fn = std::function<void(const Error& error)>;
  virtual void read(AbstractNopHolder& object, read_nop_callback_fn fn) = 0;
  virtual void write(const AbstractNopHolder& object, write_callback_fn fn) = 0;

  virtual void setId(std::string id) = 0;
  virtual void close() = 0;
  virtual ~Connection() = default;
};

} // namespace transport
TP_AMD_NAMESPACE_END
