// Message / Descriptor / Allocation, field for field as
// tensorpipe/core/message.h:27-102.
#pragma once

#include <cstddef>
#include <string>
#include <vector>

#include <tensorpipe/common/buffer.h>
#include <tensorpipe/common/optional.h>

TP_AMD_NAMESPACE_BEGIN

class Message final {
 public:
  std::string metadata;

  struct Payload {
    void* data{nullptr};
    size_t length{0};
    std::string metadata;
  };
  // Travel over the pipe's primary connection.
  std::vector<Payload> payloads;

  struct Tensor {
    tensorpipe::Buffer buffer;
    size_t length{0};
    // Device the receiver must allocate on; unset = receiver's choice.
    optional<Device> targetDevice;
    std::string metadata;
  };
  // Offered to the channels.
  std::vector<Tensor> tensors;
};

class Descriptor final {
 public:
  std::string metadata;

  struct Payload {
    size_t length{0};
    std::string metadata;
  };
  std::vector<Payload> payloads;

  struct Tensor {
    size_t length{0};
    Device sourceDevice;
    optional<Device> targetDevice;
    std::string metadata;
  };
  std::vector<Tensor> tensors;
};

class Allocation final {
 public:
  struct Payload {
    void* data{nullptr};
  };
  std::vector<Payload> payloads;

  struct Tensor {
    tensorpipe::Buffer buffer;
  };
  std::vector<Tensor> tensors;
};

TP_AMD_NAMESPACE_END
