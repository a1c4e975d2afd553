// Device{type, index} and its hashes, as tensorpipe/common/device.h:17-64.
#pragma once

#include <string>
#include <utility>

#include <tensorpipe/common/defs.h>

TP_AMD_NAMESPACE_BEGIN

const std::string kCpuDeviceType{"cpu"};
// PyTorch on ROCm names its GPUs "cuda"; a HipBuffer reports this type so that
// callers keyed on the reference's kCudaDeviceType keep working.
const std::string kCudaDeviceType{"cuda"};
const std::string kHipDeviceType{kCudaDeviceType};

struct Device {
  std::string type;
  int index{0};

  Device() {}
  Device(std::string type, int index) : type(std::move(type)), index(index) {}

  std::string toString() const {
    return type + ":" + std::to_string(index);
  }

  bool operator==(const Device& other) const {
    return type == other.type && index == other.index;
  }
  bool operator!=(const Device& other) const {
    return !(*this == other);
  }
};

TP_AMD_NAMESPACE_END

namespace std {

template <>
struct hash<::tensorpipe::Device> {
  size_t operator()(const ::tensorpipe::Device& device) const noexcept {
    return std::hash<std::string>{}(device.toString());
  }
};

template <>
struct hash<std::pair<::tensorpipe::Device, ::tensorpipe::Device>> {
  size_t operator()(
      const std::pair<::tensorpipe::Device, ::tensorpipe::Device>& p) const noexcept {
    size_t h1 = std::hash<::tensorpipe::Device>{}(p.first);
    size_t h2 = std::hash<::tensorpipe::Device>{}(p.second);
    return h1 ^ (h2 << 1);
  }
};

} // namespace std
