"""Echo peer for the two-process channel tests: connects to the given URL and
echoes every message back until it sees metadata "quit". The metadata of each
message says where the peer allocates: "gpu", "cpu", or "gpu,cpu,..." per tensor.
Run as a spawned child process (never forked: the parent may hold a GPU)."""
import os
import sys
import traceback


def echo_peer(url, channels, env, ready, errors):
    try:
        os.environ.update(env)
        root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
        if root not in sys.path:
            sys.path.insert(0, root)
        import numpy as np
        import torch

        from tensorpipe_amd import pipe as tp

        ctx = tp.Context("peer", channels=channels)
        p = ctx.connect(url)
        ready.set()
        while True:
            d = p.read_descriptor(timeout_ms=60000)
            meta = d.metadata.decode()
            if meta == "quit":
                break
            if meta == "die":
                os._exit(3)  # the process vanishes with the message half read
            places = meta.split(",") if meta else []
            bufs, tensors = [], []
            for i in range(d.num_tensors):
                n = int(d.tensor_lengths[i])
                place = places[i] if i < len(places) else (places[-1] if places else "gpu")
                if place == "cpu":
                    b = np.full(n, 0xEE, np.uint8)
                else:
                    b = torch.full((max(n, 1),), 0xEE, dtype=torch.uint8, device="cuda")
                bufs.append(b)
                tensors.append(tp.make_tensor(b, nbytes=n))
            pbufs = [np.zeros(int(d.payload_lengths[i]), np.uint8) for i in range(d.num_payloads)]
            p.read(tensors, pbufs).wait(60000)
            # Echo from the same buffers on the same stream: ordered after the receive.
            out = [tp.make_tensor(b, nbytes=t.length) for b, t in zip(bufs, tensors)]
            p.write(out, payloads=pbufs, metadata=meta).wait(60000)
        p.destroy()
        ctx.destroy()
    except Exception:
        errors.put(traceback.format_exc())
        ready.set()
