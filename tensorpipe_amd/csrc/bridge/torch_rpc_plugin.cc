// A loadable module that gives the TensorPipe RPC agent of a PyTorch-ROCm
// build what its CUDA builds get from torch/csrc/distributed/rpc/tensorpipe_cuda.cpp
// and a ROCm build lacks: channels that move GPU tensors, and the converter
// between an at::Tensor's storage and the buffer a channel takes.
//
//   torch.ops.load_library(".../libtensorpipe_amd_torch_rpc.so")   # before rpc.init_rpc
//
// What is registered, through the agent's public registries
// (torch/csrc/distributed/rpc/tensorpipe_agent.h, tensorpipe_utils.h):
//   TensorPipeChannelRegistry   hip_xth, hip_ipc, hip_basic -- this library's
//                               channels behind the host's channel::Context
//                               (bridge/stock_adapter.h), ranked among
//                               themselves the way the reference's agent ranks
//                               cuda_xth, cuda_ipc and cuda_basic
//   device type converter CUDA  (a GPU is "cuda" to PyTorch on ROCm)
//                               storage + stream  -> HipBuffer on the way out,
//                               caching-allocator block + stream -> HipBuffer
//                               on the way in
// Compiled against the HOST's TensorPipe headers (the ones PyTorch installs),
// never against this library's.
#include <memory>

#include <ATen/hip/impl/HIPCachingAllocatorMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/util/Registry.h>
#include <tensorpipe/tensorpipe.h>
#include <torch/csrc/distributed/rpc/tensorpipe_agent.h>
#include <torch/csrc/distributed/rpc/tensorpipe_utils.h>

#include <bridge/stock_adapter.h>

namespace tensorpipe_amd_bridge {
namespace {

namespace rpc = ::torch::distributed::rpc;
using GpuStream = ::c10::hip::HIPStreamMasqueradingAsCUDA;

class GpuTensorConverter final : public rpc::TensorpipeDeviceTypeConverter {
 public:
  std::optional<std::vector<char>> prepareTensorForSending(
      const c10::Storage& storage,
      const std::vector<c10::Stream>& streams,
      tensorpipe::Message& message) const override {
    const GpuStream stream(rpc::getStreamForDevice(streams, storage.device()));
    // The channel reads the block on this stream after the caller has let go
    // of the tensor: the allocator must not hand the block out again before
    // that stream has passed the read.
    c10::hip::HIPCachingAllocatorMasqueradingAsCUDA::recordStreamMasqueradingAsCUDA(storage.data_ptr(), stream);
    tensorpipe::Message::Tensor tensor;
    tensor.buffer = HipBuffer{storage.mutable_data(), stream.stream(), static_cast<int>(storage.device().index())};
    tensor.length = storage.nbytes();
    message.tensors.push_back(std::move(tensor));
    return std::nullopt; // nothing was copied aside
  }

  at::DataPtr allocateTensorForReceiving(
      c10::DeviceIndex deviceIndex,
      size_t length,
      const std::vector<c10::Stream>& streams,
      tensorpipe::Allocation& allocation) const override {
    const c10::Device device(c10::kCUDA, deviceIndex);
    const c10::Stream& generic = rpc::getStreamForDevice(streams, device);
    const GpuStream stream(generic);
    // Allocated with that stream current, the block belongs to it: what the
    // agent later runs on the stream is ordered after the channel's copy.
    c10::hip::HIPStreamGuardMasqueradingAsCUDA guard(generic);
    at::DataPtr block = c10::hip::HIPCachingAllocatorMasqueradingAsCUDA::get()->allocate(length);
    tensorpipe::Allocation::Tensor tensor;
    tensor.buffer = HipBuffer{block.get(), stream.stream(), static_cast<int>(deviceIndex)};
    allocation.tensors.push_back(std::move(tensor));
    return block;
  }
};

// Same-process before cross-process before staged through the host, the order
// in which PyTorch's CUDA builds rank cuda_xth, cuda_ipc and cuda_basic. The
// agent's CPU channels only serve CPU pairs, so the two groups never compete.
std::unique_ptr<rpc::ChannelRegistration> makeChannel(const char* name, int64_t priority) {
  return std::make_unique<rpc::ChannelRegistration>(rpc::ChannelRegistration{createChannelContext(name), priority});
}
std::unique_ptr<rpc::ChannelRegistration> makeHipXth() {
  return makeChannel("hip_xth", 400);
}
std::unique_ptr<rpc::ChannelRegistration> makeHipIpc() {
  return makeChannel("hip_ipc", 300);
}
std::unique_ptr<rpc::ChannelRegistration> makeHipBasic() {
  return makeChannel("hip_basic", 0);
}

// A build that already converts GPU tensors (one with the reference's CUDA
// channels compiled in) wraps them in its own buffer type, which these
// channels do not take. Its converter is left in place and the module reports
// the conflict through tensorpipe_amd_torch_rpc_status(): an exception out of
// a static initialiser would end the process inside dlopen.
bool converterConflict = false;
struct ConverterRegistration {
  ConverterRegistration() {
    if (rpc::getDeviceTypeConverter(c10::DeviceType::CUDA) != nullptr) {
      converterConflict = true;
      return;
    }
    static rpc::TensorpipeDeviceTypeConverterRegistrar registrar(c10::DeviceType::CUDA, new GpuTensorConverter());
  }
};
const ConverterRegistration converterRegistration;

} // namespace
} // namespace tensorpipe_amd_bridge

// (the registration macro pastes the registry's name into identifiers, so it is
// used from inside the registry's own namespace)
namespace torch::distributed::rpc {
C10_REGISTER_CREATOR(TensorPipeChannelRegistry, hip_xth, ::tensorpipe_amd_bridge::makeHipXth)
C10_REGISTER_CREATOR(TensorPipeChannelRegistry, hip_ipc, ::tensorpipe_amd_bridge::makeHipIpc)
C10_REGISTER_CREATOR(TensorPipeChannelRegistry, hip_basic, ::tensorpipe_amd_bridge::makeHipBasic)
} // namespace torch::distributed::rpc

// 0: channels and converter registered. 1: this PyTorch already had a converter
// for GPU tensors; the module must not be used with it.
extern "C" int tensorpipe_amd_torch_rpc_status() {
  return tensorpipe_amd_bridge::converterConflict ? 1 : 0;
}

// For a caller that wants proof of the route taken: GPU buffers handed to
// this library's channels by this process so far.
extern "C" unsigned long long tensorpipe_amd_torch_rpc_gpu_operations() {
  return tensorpipe_amd_bridge::gpuOperationsServed();
}
// The same for one kind of channel: "hip_xth", "hip_ipc" or "hip_basic".
extern "C" unsigned long long tensorpipe_amd_torch_rpc_gpu_operations_of(const char* channelName) {
  return channelName == nullptr ? 0 : tensorpipe_amd_bridge::gpuOperationsServedBy(channelName);
}
