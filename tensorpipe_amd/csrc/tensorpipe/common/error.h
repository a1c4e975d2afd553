// Error value type: falsy means success, copyable, keeps the dynamic type of
// the underlying cause. Same surface as tensorpipe/common/error.h:38-127.
#pragma once

#include <memory>
#include <string>

#include <sys/types.h>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

class BaseError {
 public:
  virtual ~BaseError() = default;
  virtual std::string what() const = 0;
};

class Error final {
 public:
  static const Error kSuccess;

  Error() {}
  Error(std::shared_ptr<BaseError> error, std::string file, int line)
      : error_(std::move(error)), file_(std::move(file)), line_(line) {}

  operator bool() const {
    return static_cast<bool>(error_);
  }

  template <typename T>
  std::shared_ptr<T> castToType() const {
    return std::dynamic_pointer_cast<T>(error_);
  }

  template <typename T>
  bool isOfType() const {
    return castToType<T>() != nullptr;
  }

  // Explanatory string followed by the place the error was created.
  std::string what() const;

 private:
  std::shared_ptr<BaseError> error_;
  std::string file_;
  int line_{-1};
};

class SystemError final : public BaseError {
 public:
  SystemError(const char* syscall, int error) : syscall_(syscall), error_(error) {}
  std::string what() const override;
  int errorCode() const {
    return error_;
  }

 private:
  const char* syscall_;
  const int error_;
};

class ShortReadError final : public BaseError {
 public:
  ShortReadError(ssize_t expected, ssize_t actual) : expected_(expected), actual_(actual) {}
  std::string what() const override;

 private:
  const ssize_t expected_;
  const ssize_t actual_;
};

class ShortWriteError final : public BaseError {
 public:
  ShortWriteError(ssize_t expected, ssize_t actual) : expected_(expected), actual_(actual) {}
  std::string what() const override;

 private:
  const ssize_t expected_;
  const ssize_t actual_;
};

class EOFError final : public BaseError {
 public:
  std::string what() const override;
};

// A failed call into the HIP C ABI (code as returned by libtphip).
class HipError final : public BaseError {
 public:
  HipError(const char* call, int code) : call_(call), code_(code) {}
  std::string what() const override;
  int code() const {
    return code_;
  }

 private:
  const char* call_;
  const int code_;
};

TP_AMD_NAMESPACE_END

#define TP_CREATE_ERROR(typ, ...) \
  (::tensorpipe::Error(std::make_shared<typ>(__VA_ARGS__), ::tensorpipe::tpTrimFilename(__FILE__), __LINE__))
