#pragma once

#include <cstdint>

#include <tensorpipe/common/device.h>

TP_AMD_NAMESPACE_BEGIN

// Opaque stand-in for hipStream_t so that this header needs no HIP include;
// the value is passed unchanged to the HIP C ABI.
using HipStreamHandle = void*;

// Mirrors CudaBuffer{ptr, stream}, tensorpipe/common/cuda_buffer.h:17-22.
// The stream is the one the caller's producer/consumer work is ordered on.
struct HipBuffer {
  void* ptr{nullptr};
  HipStreamHandle stream{nullptr};

  // Device that owns `ptr` (tensorpipe/common/cuda_buffer.cc:16-28).
  Device getDevice() const;
  // See Buffer::deviceKey(); throws like getDevice() for memory no GPU owns.
  uint32_t getDeviceKey() const;
};

// Start of a unit of work on the calling thread (see common/hip_api.h): what
// getDevice() remembers about address ranges is checked once before its next use.
void hipPointerCheckpoint();

TP_AMD_NAMESPACE_END
