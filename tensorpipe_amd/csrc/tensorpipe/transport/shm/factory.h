#pragma once

#include <memory>

#include <tensorpipe/transport/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace transport {
namespace shm {

// Same-host transport: one shared-memory byte ring per direction, connection
// set-up over an abstract Unix socket. cf. tensorpipe/transport/shm/factory.h.
std::shared_ptr<Context> create();

} // namespace shm
} // namespace transport
TP_AMD_NAMESPACE_END
