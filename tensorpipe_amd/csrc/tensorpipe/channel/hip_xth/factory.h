#pragma once

#include <memory>

#include <tensorpipe/channel/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_xth {

// Same-process GPU-to-GPU channel (cf. tensorpipe/channel/cuda_xth/factory.h:19).
std::shared_ptr<Context> create();

} // namespace hip_xth
} // namespace channel
TP_AMD_NAMESPACE_END
