#pragma once

#include <string>

#include <tensorpipe/common/error.h>

TP_AMD_NAMESPACE_BEGIN

// tensorpipe/core/error.h:17-46
class LogicError final : public BaseError {
 public:
  explicit LogicError(std::string reason) : reason_(std::move(reason)) {}
  std::string what() const override {
    return "logic error: " + reason_;
  }

 private:
  const std::string reason_;
};

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

class PipeClosedError final : public BaseError {
 public:
  std::string what() const override {
    return "pipe closed";
  }
};

TP_AMD_NAMESPACE_END
