// The host's side of tpbridge for a stock TensorPipe (the build PyTorch ships
// in libtorch_cpu.so): this library's channels as a tensorpipe::channel::Context
// that Context::registerChannel takes, exactly as the reference registers its
// CUDA channels (tensorpipe/core/context.h:67-70,
// tensorpipe/test/core/pipe_test.h:300-316). Compile this file's .cc against
// the HOST's tensorpipe headers, never against this library's.
//
// A GPU tensor travels in a message as a tensorpipe::Buffer that wraps the
// HipBuffer below -- the counterpart of CudaBuffer (tensorpipe/common/cuda_buffer.h:17-22);
// its device type is "cuda", what PyTorch on ROCm calls a GPU.
#pragma once

#include <memory>
#include <string>

#include <tensorpipe/channel/context.h>
#include <tensorpipe/common/device.h>

namespace tensorpipe_amd_bridge {

struct HipBuffer {
  void* ptr{nullptr};
  void* stream{nullptr}; // hipStream_t
  int deviceIndex{0};
  ::tensorpipe::Device getDevice() const {
    return ::tensorpipe::Device{"cuda", deviceIndex};
  }
};

// GPU buffers this process has handed to this library's channels through the
// adapter so far (sends plus receives): lets a test prove which channel a
// tensor travelled on.
unsigned long long gpuOperationsServed();
// The same count for one kind of channel ("hip_xth", "hip_ipc", "hip_basic").
unsigned long long gpuOperationsServedBy(const std::string& channelName);

// channelName: "hip_xth", "hip_ipc" or "hip_basic".
std::shared_ptr<::tensorpipe::channel::Context> createChannelContext(const std::string& channelName);

} // namespace tensorpipe_amd_bridge
