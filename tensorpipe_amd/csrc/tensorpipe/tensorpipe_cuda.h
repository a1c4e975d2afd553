// Source-level names of the reference's GPU side (tensorpipe/tensorpipe_cuda.h,
// tensorpipe/common/cuda_buffer.h:17-22, tensorpipe/channel/cuda_{xth,ipc,basic}/factory.h)
// for code written against it: including this header instead of the
// reference's makes CudaBuffer, kCudaDeviceType and channel::cuda_*::create()
// resolve to the HIP channels of this library. Nothing else is implied: there
// is no CUDA runtime here, and a stream is a hipStream_t.
#pragma once

#include <tensorpipe/tensorpipe_hip.h>

#define TENSORPIPE_HAS_CUDA_IPC_CHANNEL 1

TP_AMD_NAMESPACE_BEGIN

using CudaBuffer = HipBuffer;

namespace channel {
namespace cuda_xth {
inline std::shared_ptr<Context> create() {
  return hip_xth::create();
}
} // namespace cuda_xth
namespace cuda_ipc {
inline std::shared_ptr<Context> create() {
  return hip_ipc::create();
}
} // namespace cuda_ipc
namespace cuda_basic {
inline std::shared_ptr<Context> create(std::shared_ptr<Context> cpuContext) {
  return hip_basic::create(std::move(cpuContext));
}
} // namespace cuda_basic
} // namespace channel

TP_AMD_NAMESPACE_END
