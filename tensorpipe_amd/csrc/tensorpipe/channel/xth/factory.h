#pragma once

#include <memory>

#include <tensorpipe/channel/context.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {
namespace xth {

// Same-process CPU channel: the source pointer travels over the connection
// and a copy thread does the memcpy (tensorpipe/channel/xth/factory.h).
std::shared_ptr<Context> create();

} // namespace xth
} // namespace channel
TP_AMD_NAMESPACE_END
