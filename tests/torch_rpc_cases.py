"""One rank of a two-process torch.distributed.rpc group whose GPU tensors travel on this
library's channels (tensorpipe_amd.torch_rpc). Started by tests/test_torch_rpc.py and tests/test_zy_torch_rpc_gpu.py, once per rank:

    python tests/torch_rpc_cases.py <rank> <rendezvous file> <mode>

mode: "cpu"    no device map, CPU tensors only (the module loaded must not disturb the agent)
      "gpu"    device maps 0 -> 0 both ways and to oneself; all three channels registered
      "staged" as "gpu" with the agent's channel list cut to hip_basic + basic
      "gpu3"   three processes on the one GPU, device maps between all of them: calls to both
               peers and a call that the first peer relays to the second
      "peer_dies" / "cpu_peer_dies"   rank 1 ends abruptly inside a call that brought it a (GPU)
               tensor while more calls with tensors are on their way: rank 0's calls must fail,
               none may hang

Rank 0 drives the cases and prints "RESULT <case> OK|FAIL ..." lines; both ranks print how many GPU
buffers went through the hip_* channels. What the reference's agent tests for its CUDA channels
(PyTorch's torch/testing/_internal/distributed/rpc/rpc_test.py: device maps, tensors in arguments and
results, many calls in flight, RRefs) is the model for the cases.
"""
import ctypes
import faulthandler
import os
import sys
import threading

import torch
import torch.distributed.rpc as rpc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import tensorpipe_amd.torch_rpc as tp_rpc  # noqa: E402


def seeded(nbytes, seed, device):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    t = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g)
    return t.to(device)


# ---- functions the other rank runs
def echo(t):
    return t


def echo_many(ts):
    return list(reversed(ts))


def devices_of(ts):
    return [str(t.device) for t in ts]


def add_one(t):
    return t + 1


def make_on_gpu(nbytes, seed):
    return seeded(nbytes, seed, "cuda:0")


def relay(name, t):
    # the tensor goes on to a third process, comes back changed, and returns to the first
    return rpc.rpc_sync(name, add_one, args=(t,))


def leave_abruptly(t):
    os._exit(3)


def checksum(t):
    # computed where the tensor arrived, on the stream the agent made current
    return int(t.to(torch.int64).sum().item())


def main():
    rank, rendezvous, mode = int(sys.argv[1]), sys.argv[2], sys.argv[3]
    # A rank that is still here after this long says where every thread stands and ends, so that
    # the test reports what was reached instead of running into the runner's own time limit.
    limit = int(os.environ.get("TP_RPC_CASES_LIMIT_S", "90"))

    def stalled():
        print(f"RESULT stalled FAIL rank {rank} was still running after {limit} s", flush=True)
        faulthandler.dump_traceback(all_threads=True)
        sys.stderr.flush()
        # exit() rather than _exit(): the library prints its timeline of recent events
        # (TP_TIMELINE) when the process ends in the ordinary way
        ctypes.CDLL(None).exit(3)

    watchdog = threading.Timer(limit, stalled)
    watchdog.daemon = True
    watchdog.start()
    faulthandler.dump_traceback_later(limit + 20, exit=True)  # should the ordinary exit not get through
    gpu = mode in ("gpu", "staged", "peer_dies", "gpu3")
    world = 3 if mode == "gpu3" else 2
    tp_rpc.load()
    # the ranks meet through a file: no port that somebody else might take in between
    kwargs = {"init_method": "file://" + rendezvous}
    if mode == "staged":
        kwargs["_channels"] = ["hip_basic", "basic"]
    opts = rpc.TensorPipeRpcBackendOptions(num_worker_threads=8, rpc_timeout=90, **kwargs)
    if gpu:
        for peer in range(world):
            opts.set_device_map(f"w{peer}", {0: 0})
    rpc.init_rpc(f"w{rank}", rank=rank, world_size=world, rpc_backend_options=opts)
    failures = 0

    def result(name, ok, note=""):
        nonlocal failures
        failures += 0 if ok else 1
        print(f"RESULT {name} {'OK' if ok else 'FAIL'} {note}", flush=True)

    if mode == "gpu3":
        if rank == 0:
            dev = "cuda:0"
            xs = [seeded((1 << 20) + 17 * i, 400 + i, dev) for i in range(6)]
            futs = [rpc.rpc_async(f"w{1 + i % 2}", echo, args=(x,)) for i, x in enumerate(xs)]
            result("both_peers", all(torch.equal(x, f.wait()) for x, f in zip(xs, futs)))
            x = seeded((2 << 20) + 3, 41, dev)
            y = rpc.rpc_sync("w1", relay, args=("w2", x))
            result("relayed", str(y.device) == dev and torch.equal(y, x + 1))
            by = tp_rpc.gpu_operations_by_channel()
            result("channel_chosen", by["hip_ipc"] >= 14 and by["hip_basic"] == 0, str(by))
        rpc.shutdown()
        print(f"RANK {rank} gpu_buffers_through_hip_channels {tp_rpc.gpu_operations()} {tp_rpc.gpu_operations_by_channel()}",
              flush=True)
        if rank == 0:
            print("RESULT route OK" if tp_rpc.gpu_operations() else "RESULT route FAIL", flush=True)
        sys.exit(1 if failures else 0)
    if mode.endswith("peer_dies"):
        if rank == 0:
            dev = "cuda:0" if gpu else "cpu"
            x = seeded(3 << 20, 21, dev)
            ok = rpc.rpc_sync("w1", checksum, args=(x,)) == int(x.to(torch.int64).sum().item())
            result("before", ok)
            futs = [rpc.rpc_async("w1", leave_abruptly if i == 2 else echo, args=(seeded((1 << 20) + i, 30 + i, dev),))
                    for i in range(8)]
            failed = 0
            for f in futs:
                try:
                    f.wait()
                except RuntimeError:
                    failed += 1
            # the calls behind the fatal one fail; those ahead of it may have been answered
            result("calls_fail_instead_of_hanging", failed >= 6, f"{failed} of 8 failed")
            print("RESULT route OK", flush=True)
            sys.stdout.flush()
            try:
                rpc.shutdown(graceful=False)
            finally:
                os._exit(1 if failures else 0)
        else:
            import time

            time.sleep(60)  # ended from inside leave_abruptly long before
            os._exit(4)
    if rank == 0:
        dev = "cuda:0" if gpu else "cpu"
        # a tensor there and back, sizes from nothing to 64 MiB, odd ones among them
        # (An empty tensor only travels as a CPU tensor: PyTorch's unpickler does not ask for the
        # storage of a tensor without elements and rebuilds it on the CPU, which the agent then
        # rejects for a GPU target -- in CUDA builds with the reference's channels just the same.)
        for nbytes in (0, 1, 4097, (1 << 20) + 3, 64 << 20):
            x = seeded(nbytes, 100 + nbytes % 97, dev if nbytes else "cpu")
            y = rpc.rpc_sync("w1", echo, args=(x,))
            result(f"echo_{nbytes}", y.device == x.device and y.shape == x.shape and torch.equal(x, y))
        # arithmetic on the other side
        x = torch.arange(1 << 18, dtype=torch.float32, device=dev)
        y = rpc.rpc_sync("w1", add_one, args=(x,))
        result("add_one", str(y.device) == dev and torch.equal(y, x + 1))
        # what arrives is what was sent, checked where it arrived
        x = seeded((3 << 20) + 5, 7, dev)
        result("checksum_at_callee", rpc.rpc_sync("w1", checksum, args=(x,)) == int(x.to(torch.int64).sum().item()))
        # several tensors of one message, GPU and CPU mixed
        xs = [seeded(n, 200 + i, dev if i % 3 and n else "cpu")
              for i, n in enumerate((5, 70000, 0, 1 << 20, 33, 4096, 999999, 2 << 20))]
        where = rpc.rpc_sync("w1", devices_of, args=(xs,))
        result("mixed_devices_arrive_in_place", where == [str(t.device) for t in xs], str(where))
        ys = rpc.rpc_sync("w1", echo_many, args=(xs,))
        ok = len(ys) == len(xs) and all(
            str(y.device) == str(x.device) and torch.equal(x, y) for x, y in zip(reversed(xs), ys))
        result("mixed_echo", ok)
        # many calls in flight
        xs = [seeded(100000 + 4099 * i, 300 + i, dev) for i in range(24)]
        futs = [rpc.rpc_async("w1", echo, args=(x,)) for x in xs]
        ok = all(torch.equal(x, f.wait()) for x, f in zip(xs, futs))
        result("in_flight_24", ok)
        # a view into a larger storage
        big = seeded(1 << 20, 9, dev)
        part = big[12345:54321]
        y = rpc.rpc_sync("w1", echo, args=(part,))
        result("view", torch.equal(part, y))
        if gpu:
            # made on the other side's GPU, fetched through an RRef
            rref = rpc.remote("w1", make_on_gpu, args=(777777, 11))
            y = rref.to_here()
            result("rref_to_here", str(y.device) == "cuda:0" and torch.equal(y.cpu(), seeded(777777, 11, "cpu")))
            before = tp_rpc.gpu_operations()
            # to oneself: same process, the agent's pipe to itself
            x = seeded((1 << 20) + 1, 13, dev)
            y = rpc.rpc_sync("w0", echo, args=(x,))
            result("to_self", str(y.device) == dev and torch.equal(x, y))
            result("to_self_used_the_channels", tp_rpc.gpu_operations() >= before + 4,
                   f"{tp_rpc.gpu_operations() - before} GPU buffers")
            # which channel carried what: same process -> hip_xth, the other process -> hip_ipc,
            # unless the agent was only given hip_basic
            by = tp_rpc.gpu_operations_by_channel()
            if mode == "staged":
                ok = by["hip_basic"] > 50 and by["hip_xth"] == 0 and by["hip_ipc"] == 0
            else:
                ok = by["hip_xth"] >= 4 and by["hip_ipc"] > 50 and by["hip_basic"] == 0
            result("channel_chosen", ok, str(by))
        # the other rank calls back while this one is calling it
        fut = rpc.rpc_async("w1", call_back_to, args=("w0", 65536 + 7, dev))
        result("callee_calls_back", fut.wait())
    rpc.shutdown()
    print(f"RANK {rank} gpu_buffers_through_hip_channels {tp_rpc.gpu_operations()} {tp_rpc.gpu_operations_by_channel()}",
          flush=True)
    if gpu and tp_rpc.gpu_operations() == 0:
        failures += 1
        print("RESULT route FAIL no GPU buffer went through the hip channels", flush=True)
    elif rank == 0:
        print("RESULT route OK", flush=True)
    sys.exit(1 if failures else 0)


def call_back_to(name, nbytes, dev):
    x = seeded(nbytes, 17, dev)
    y = rpc.rpc_sync(name, echo, args=(x,))
    return bool(str(y.device) == dev and torch.equal(y, x))


if __name__ == "__main__":
    main()
