#pragma once

#include <memory>

#include <tensorpipe/transport/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace transport {
namespace tcp {

// TCP transport whose bytes on the wire are those of the reference's uv
// transport (tensorpipe/transport/uv/*, common/stream_read_write_ops.h:30-65,
// 146-188): every message is its length as a 64-bit little-endian word followed
// by the bytes, nothing else. Register it under the name "uv" to be matched
// with stock peers (its domain descriptor is the one theirs announce).
// Addresses are "a.b.c.d:port" or "[v6 address]:port"; listening on port 0, or
// on a bare address, takes a free port.
std::shared_ptr<Context> create();

} // namespace tcp
} // namespace transport
TP_AMD_NAMESPACE_END
