#pragma once

#include <string>

#include <tensorpipe/common/error.h>

TP_AMD_NAMESPACE_BEGIN
namespace channel {

// tensorpipe/channel/error.h:18-37
class ContextClosedError final : public BaseError {
 public:
  std::string what() const override {
    return "context closed";
  }
};

class ChannelClosedError final : public BaseError {
 public:
  std::string what() const override {
    return "channel closed";
  }
};

class ContextNotViableError final : public BaseError {
 public:
  std::string what() const override {
    return "context not viable";
  }
};

} // namespace channel
TP_AMD_NAMESPACE_END
