#pragma once

#include <cstdint>

#include <tensorpipe/common/device.h>

TP_AMD_NAMESPACE_BEGIN

// tensorpipe/common/cpu_buffer.h:15-21
struct CpuBuffer {
  void* ptr{nullptr};

  Device getDevice() const {
    return Device{kCpuDeviceType, 0};
  }
  // See Buffer::deviceKey().
  uint32_t getDeviceKey() const {
    return 1u << 16;
  }
};

TP_AMD_NAMESPACE_END
