"""torch.distributed.rpc with GPU tensors on ROCm.

PyTorch's TensorPipe RPC agent gets its GPU channels (cuda_xth, cuda_ipc, cuda_basic) and its
GPU tensor converter from a source file that ROCm builds leave out, so on ROCm the agent refuses
device maps' tensors. `load()` loads a module that registers this library's hip_xth, hip_ipc and
hip_basic channels and a converter with the agent's public registries
(csrc/bridge/torch_rpc_plugin.cc); after it, `rpc.init_rpc` with a device map moves GPU tensors:

    import tensorpipe_amd.torch_rpc as tp_rpc
    tp_rpc.load()
    opts = rpc.TensorPipeRpcBackendOptions()
    opts.set_device_map("worker1", {0: 0})
    rpc.init_rpc("worker0", rank=0, world_size=2, rpc_backend_options=opts)
    y = rpc.rpc_sync("worker1", torch.add, args=(x_on_gpu, 1))

No fallback: where the module was not built, `load()` raises.
"""
import ctypes
import os

_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libtensorpipe_amd_torch_rpc.so")
_loaded = None

CHANNELS = ("hip_xth", "hip_ipc", "hip_basic")


def library_path():
    return _LIB


def load():
    """Registers the channels and the converter with this process's RPC agent registries. Call it
    before rpc.init_rpc, in every process of the group."""
    global _loaded
    if _loaded is None:
        if not os.path.exists(_LIB):
            raise RuntimeError(
                f"{_LIB} is not built (python -m tensorpipe_amd.build; needs PyTorch's RPC agent headers)")
        import torch

        torch.ops.load_library(_LIB)
        lib = ctypes.CDLL(_LIB)
        if lib.tensorpipe_amd_torch_rpc_status() != 0:
            raise RuntimeError(
                "this PyTorch already has a TensorPipe converter for GPU tensors (a build with its own GPU "
                "channels); the hip_* channels are meant for builds without one")
        _loaded = lib
        _loaded.tensorpipe_amd_torch_rpc_gpu_operations.restype = ctypes.c_ulonglong
        _loaded.tensorpipe_amd_torch_rpc_gpu_operations_of.restype = ctypes.c_ulonglong
        _loaded.tensorpipe_amd_torch_rpc_gpu_operations_of.argtypes = [ctypes.c_char_p]
    return _loaded


def gpu_operations():
    """GPU buffers this process has handed to the hip_* channels so far (sends plus receives):
    proof of the route a tensor took."""
    return int(load().tensorpipe_amd_torch_rpc_gpu_operations())


def gpu_operations_by_channel():
    """The same count per kind of channel, e.g. {"hip_xth": 4, "hip_ipc": 120, "hip_basic": 0}."""
    lib = load()
    return {name: int(lib.tensorpipe_amd_torch_rpc_gpu_operations_of(name.encode())) for name in CHANNELS}
