#pragma once

#include <memory>

#include <tensorpipe/channel/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace hip_basic {

// Host-staged GPU channel wrapping a CPU channel
// (cf. tensorpipe/channel/cuda_basic/factory.h:19).
std::shared_ptr<Context> create(std::shared_ptr<Context> cpuContext);

} // namespace hip_basic
} // namespace channel
TP_AMD_NAMESPACE_END
