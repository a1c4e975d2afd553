#pragma once

#include <memory>

#include <tensorpipe/channel/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_ipc {

// Cross-process, same-machine GPU channel on HIP IPC memory handles
// (cf. tensorpipe/channel/cuda_ipc/factory.h).
std::shared_ptr<Context> create();

} // namespace hip_ipc
} // namespace channel
TP_AMD_NAMESPACE_END
