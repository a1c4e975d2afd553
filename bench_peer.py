"""Echo side of the two-process benchmark configurations.

    python bench_peer.py URL CHANNELS

Connects to URL, then serves commands that arrive as the metadata (JSON) of
tensor-less messages: {"op": "pingpong", "sizes": [...], "device": "gpu"|"cpu",
"warmup": W, "iters": K} allocates buffers, answers "ready" and runs the native
echo loop; {"op": "connect", "count": N} opens N more pipes to the same URL;
{"op": "pingpong_multi", ...} runs one echo loop per pipe side by side, each
with buffers and a stream of its own; {"op": "quit"} ends the process."""
import json
import sys


def die_with_parent():
    """The kernel ends this process when the process that started it has gone, however that
    went: no echo side is ever left behind by a benchmark that crashed or was killed."""
    import ctypes
    import os
    import signal

    PR_SET_PDEATHSIG = 1
    ctypes.CDLL(None, use_errno=True).prctl(PR_SET_PDEATHSIG, signal.SIGKILL, 0, 0, 0)
    if os.getppid() == 1:  # the parent went before the request was in
        os._exit(0)


def main(url, channels):
    die_with_parent()
    import numpy as np
    import torch

    from tensorpipe_amd import pipe as tp

    # the transport is the one the URL names ("uv" is this library's TCP transport)
    import os

    # (the starter names the transport where the URL's scheme does not: "shm_stock" listens on shm://)
    transport = os.environ.get("TP_BENCH_PEER_TRANSPORT") or url.split("://", 1)[0]
    ctx = tp.Context("bench_peer", transports=transport + ":0", channels=channels)
    p = ctx.connect(url)
    extra = []
    multi_bufs = multi_streams = bufs = tensors = None  # kept from one pingpong_multi to the next of the same size
    while True:
        d = p.read_descriptor(timeout_ms=600000)
        p.read([], []).wait()
        cmd = json.loads(d.metadata.decode())
        if cmd["op"] == "quit":
            break
        if cmd["op"] == "connect":
            extra += [ctx.connect(url) for _ in range(cmd["count"])]
            p.write([], metadata="connected").wait()
            continue
        if cmd["op"] == "pingpong_multi":
            import threading

            pipes = [p] + extra
            n = cmd["sizes"][0]
            if multi_bufs is None or multi_bufs[0].numel() != n or len(multi_bufs) != len(pipes):
                multi_bufs = bufs = tensors = None  # the previous size's buffers go before the next size's come
                multi_bufs = [torch.zeros(n, dtype=torch.uint8, device="cuda") for _ in pipes]
                multi_streams = [torch.cuda.Stream() for _ in pipes]
            bufs, streams = multi_bufs, multi_streams
            tensors = [[tp.make_tensor(b, nbytes=n, stream=s, target=(tp.HIP, 0))] for b, s in zip(bufs, streams)]
            torch.cuda.synchronize()
            p.write([], metadata="ready").wait()
            threads = [threading.Thread(target=tp.bench_pingpong, args=(q, False, t, t),
                                        kwargs={"warmup": cmd["warmup"], "iters": cmd["iters"]})
                       for q, t in zip(pipes, tensors)]
            for t in threads:
                t.start()
            for t in threads:
                t.join()
            continue
        if cmd["op"] == "pingpong":
            bufs, tensors = [], []
            for n in cmd["sizes"]:
                if cmd["device"] == "gpu":
                    b = torch.zeros(max(n, 1), dtype=torch.uint8, device="cuda")
                    tensors.append(tp.make_tensor(b, nbytes=n, target=(tp.HIP, 0)))
                else:
                    b = np.zeros(max(n, 1), np.uint8)
                    tensors.append(tp.make_tensor(b, nbytes=n, target=(tp.CPU, 0)))
                bufs.append(b)
            payload = np.zeros(cmd.get("payload", 0), np.uint8)
            payloads = [payload] if payload.size else []
            if cmd["device"] == "gpu":
                torch.cuda.synchronize()
            p.write([], metadata="ready").wait()
            tp.bench_pingpong(p, False, tensors, tensors, payloads=payloads,
                              recv_payloads=payloads, warmup=cmd["warmup"], iters=cmd["iters"])
    for q in extra:
        q.destroy()
    p.destroy()
    ctx.destroy()


if __name__ == "__main__":
    main(sys.argv[1], sys.argv[2])
