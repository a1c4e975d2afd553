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

// The same for a stretch of code: one mark when the outermost scope of the thread
// opens, and none from hipPointerCheckpoint() calls further down the stack while it
// is open (a pipe that handles a message opens one; the channels it calls into
// from there do not mark again).
class HipPointerScope {
 public:
  HipPointerScope();
  ~HipPointerScope();
  HipPointerScope(const HipPointerScope&) = delete;
  HipPointerScope& operator=(const HipPointerScope&) = delete;
};

TP_AMD_NAMESPACE_END
