#pragma once

#include <memory>

#include <tensorpipe/channel/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace basic {

// CPU channel that ships tensor bytes over its control connection
// (tensorpipe/channel/basic/factory.h).
std::shared_ptr<Context> create();

} // namespace basic
} // namespace channel
TP_AMD_NAMESPACE_END
