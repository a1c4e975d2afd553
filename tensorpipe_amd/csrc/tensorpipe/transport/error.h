#pragma once

#include <string>

#include <tensorpipe/common/error.h>

TP_AMD_NAMESPACE_BEGIN
namespace transport {

// tensorpipe/transport/error.h:18-44
class ContextClosedError final : public BaseError {
 public:
  std::string what() const override {
    return "context closed";
  }
};

class ListenerClosedError final : public BaseError {
 public:
  std::string what() const override {
    return "listener closed";
  }
};

class ConnectionClosedError final : public BaseError {
 public:
  std::string what() const override {
    return "connection closed";
  }
};

class ContextNotViableError final : public BaseError {
 public:
  std::string what() const override {
    return "context not viable";
  }
};

} // namespace transport
TP_AMD_NAMESPACE_END
