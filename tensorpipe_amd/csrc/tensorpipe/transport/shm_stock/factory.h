// Shared-memory transport that speaks the protocol of the reference's shm
// transport (tensorpipe/transport/shm/*), so that the peer may be an
// unmodified TensorPipe on the same host. Register it under the name "shm" in
// a context that uses the stock wire format.
#pragma once

#include <memory>

#include <tensorpipe/transport/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace transport {
namespace shm_stock {

// cf. tensorpipe/transport/shm/factory.h:19
std::shared_ptr<Context> create();

} // namespace shm_stock
} // namespace transport
TP_AMD_NAMESPACE_END
