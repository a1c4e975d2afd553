"""One rank of the torch.distributed.rpc measurement of bench.py (leg "torch_rpc"):

    python bench_rpc_peer.py <rank> <rendezvous file> [all|staged]

Two processes on the one GPU, PyTorch's own TensorPipe agent, this library's channels registered
with it (tensorpipe_amd.torch_rpc). Rank 0 times rpc_sync(echo) round trips -- the tensor goes to
the other process and comes back -- and prints one JSON line. "all" (every channel registered):
GPU tensors to the other process (hip_ipc carries them), GPU tensors to rank 0 itself through
the agent's pipe to itself (hip_xth), and CPU tensors of the same sizes on the agent's stock
channels. "staged": the agent's channel list cut to hip_basic + basic, GPU tensors to the other
process through pinned host memory."""
import json
import sys
import time

import torch
import torch.distributed.rpc as rpc

from tensorpipe_amd import torch_rpc as tp_rpc


def echo(t):
    return t


def main():
    rank, rendezvous = int(sys.argv[1]), sys.argv[2]
    mode = sys.argv[3] if len(sys.argv) > 3 else "all"
    tp_rpc.load()
    kwargs = {"_channels": ["hip_basic", "basic"]} if mode == "staged" else {}
    opts = rpc.TensorPipeRpcBackendOptions(num_worker_threads=8, rpc_timeout=120,
                                           init_method="file://" + rendezvous, **kwargs)
    for peer in (0, 1):
        opts.set_device_map(f"w{peer}", {0: 0})
    rpc.init_rpc(f"w{rank}", rank=rank, world_size=2, rpc_backend_options=opts)
    out = {}
    if rank == 0:
        g = torch.Generator(device="cpu")
        g.manual_seed(5)
        if mode == "staged":
            runs = (("gpu_tensors_hip_basic", "cuda:0", "w1"),)
        else:
            runs = (("gpu_tensors_hip_ipc", "cuda:0", "w1"), ("gpu_tensors_hip_xth_to_self", "cuda:0", "w0"),
                    ("cpu_tensors_stock_channels", "cpu", "w1"))
        for name, device, callee in runs:
            before = tp_rpc.gpu_operations_by_channel()
            legs = {}
            for nbytes, iters in ((4096, 300), (1 << 20, 200), (64 << 20, 30)):
                x = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g).to(device)
                for _ in range(30):
                    y = rpc.rpc_sync(callee, echo, args=(x,))
                times = []
                for _ in range(iters):
                    t0 = time.perf_counter()
                    y = rpc.rpc_sync(callee, echo, args=(x,))
                    if device != "cpu":
                        torch.cuda.current_stream().synchronize()  # the result is usable on this stream
                    times.append(time.perf_counter() - t0)
                times.sort()
                p50 = times[len(times) // 2]
                legs[str(nbytes)] = {
                    "rtt_p50_us": p50 * 1e6,
                    "payload_GBps": 2 * nbytes / p50 / 1e9,
                    "byte_exact": bool(torch.equal(x, y)),
                    "iters": iters,
                }
            after = tp_rpc.gpu_operations_by_channel()
            legs["gpu_buffers_by_channel"] = {k: after[k] - before.get(k, 0) for k in after}
            out[name] = legs
        if mode != "staged":
            out["gpu_tensors_hip_channels"] = out["gpu_tensors_hip_ipc"]  # the name this row had before
        out["gpu_buffers_by_channel"] = tp_rpc.gpu_operations_by_channel()
    rpc.shutdown()
    if rank == 0:
        print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
