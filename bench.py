#!/usr/bin/env python3
"""Benchmark of the HIP device channels on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The headline line is the same-process device-to-device configuration (configs[1] of the
benchmark definition): hip_xth channel, one 64 MiB uint8 tensor, two connected pipes in one
process, K write/read steps after W warm-up steps, received bytes compared with the sent
ones. One step = Pipe::write + Pipe::readDescriptor + Pipe::read of one message
and a synchronisation of the receive stream. `value` is payload bytes delivered
per second with the tensors already resident in HBM.

The other configurations (cross-process IPC size sweep and 4 KiB round trip,
host-staged 256 MiB with the copy kernel and with hipMemcpyAsync, 256-tensor RPC-style
message), the headline's tensor with four transfers in flight and with a source that is
not in the Infinity Cache, the host link's ceilings and the CPU baseline are reported
under "extra" / "cpu_baseline" of the same JSON line; each runs in a process of its own
(`--leg`), and one that fails is reported in its place without taking the line with it.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

TRAFFIC_PROFILE = "profiles/single_copy_kernel_d2d_64MiB_pmc_fetch_write.txt"
HBM_PEAK_GBPS = 8000.0
PCIE_PEAK_GBPS = 63.0
MIB = 1 << 20


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def profiled(fn, max_launches):
    """Run fn() with per-launch device timing of the copy kernels switched on."""
    import ctypes

    from tensorpipe_amd import _native

    lib = _native.tphip()
    _native.check(lib.tphip_profile_start(0, max_launches), "profile_start")
    out = fn()
    n, ms, nbytes = ctypes.c_uint32(), ctypes.c_double(), ctypes.c_uint64()
    _native.check(lib.tphip_profile_stop(0, ctypes.byref(n), ctypes.byref(ms), ctypes.byref(nbytes)),
                  "profile_stop")
    return out, n.value, ms.value, nbytes.value


def traffic_from_profile(path, kernel):
    """HBM-side bytes per launch of `kernel` from a committed rocprofv3 --pmc summary under
    profiles/: average FETCH_SIZE and WRITE_SIZE per dispatch (KiB), each times the calibration
    factor the summary's header states for it. None when the file or the rows are not there."""
    import re

    try:
        text = open(os.path.join(ROOT, path)).read()
    except OSError:
        return None
    factors, values = {}, {}
    for line in text.splitlines():
        m = re.match(r"#\s*(FETCH_SIZE|WRITE_SIZE):.*", line)
        if m:
            current = m.group(1)
        f = re.search(r"-> factor ([0-9.]+)", line)
        if f and line.startswith("#") and "current" in locals():
            factors[current] = float(f.group(1))
        cols = line.split()
        if kernel in line and not line.startswith("#") and len(cols) >= 5 and cols[-5] in ("FETCH_SIZE", "WRITE_SIZE"):
            values[cols[-5]] = float(cols[-3])
    if set(values) != {"FETCH_SIZE", "WRITE_SIZE"} or set(factors) != {"FETCH_SIZE", "WRITE_SIZE"}:
        return None
    kib = values["FETCH_SIZE"] * factors["FETCH_SIZE"] + values["WRITE_SIZE"] * factors["WRITE_SIZE"]
    return int(kib * 1024)


def make_pair(channels):
    from tensorpipe_amd import pipe as tp

    server = tp.Context("bench_server", channels=channels)
    client = tp.Context("bench_client", channels=channels)
    listener = server.listen()
    cpipe = client.connect(listener.url())
    spipe = listener.accept()
    return cpipe, spipe, listener, client, server


def destroy(objs):
    for o in objs:
        o.destroy()


def bench_d2d(steps, warmup):
    """configs[1]: hip_xth, 1 x 64 MiB uint8, same process."""
    import torch

    from tensorpipe_amd import datagen, hip
    from tensorpipe_amd import pipe as tp

    nbytes = 64 * MIB
    host = datagen.uniform_u8(datagen.SEED_BASE + 2, nbytes)
    src = torch.from_numpy(host).cuda()
    dst = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    objs = make_pair("basic:0,hip_xth:10")
    cpipe, spipe = objs[0], objs[1]
    send_stream, recv_stream = torch.cuda.Stream(), torch.cuda.Stream()
    st = [tp.make_tensor(src, stream=send_stream, target=(tp.HIP, 0))]
    rt = [tp.make_tensor(dst, stream=recv_stream)]
    torch.cuda.synchronize()

    # warm-up steps, then a full compare of the first transfer
    tp.bench_transfer(cpipe, spipe, st, rt, warmup=0, iters=max(warmup, 1))
    assert torch.equal(src, dst), "received bytes differ from sent bytes"
    dst.zero_()
    torch.cuda.synchronize()

    # Timed region: K steps, nothing instrumented.
    per_us, total_s = tp.bench_transfer(cpipe, spipe, st, rt, warmup=0, iters=steps)
    torch.cuda.synchronize()
    assert torch.equal(src, dst), "received bytes differ from sent bytes after the timed loop"

    # The same K steps once more with every copy launch bracketed by the kernel's own
    # start/stop events (the instrumented launch path costs host time, so it is kept out
    # of the timed region above; the kernel and its arguments are identical).
    dst.zero_()
    torch.cuda.synchronize()
    (prof_per_us, prof_total_s), launches, kernel_ms, kernel_bytes = profiled(
        lambda: tp.bench_transfer(cpipe, spipe, st, rt, warmup=0, iters=steps), steps + 8)
    torch.cuda.synchronize()
    assert torch.equal(src, dst), "received bytes differ from sent bytes after the profiled loop"
    assert launches == steps and kernel_bytes == steps * nbytes, (launches, kernel_bytes)

    # two more uninstrumented passes of K steps: how much one pass varies on this box
    repeats = [total_s / steps * 1e3]
    for _ in range(2):
        _, again_s = tp.bench_transfer(cpipe, spipe, st, rt, warmup=0, iters=steps)
        repeats.append(again_s / steps * 1e3)
    torch.cuda.synchronize()

    # practical ceiling: the runtime's own D2D copy of the same size, same timing method
    e0, e1 = hip.TimedEvent(), hip.TimedEvent()
    for _ in range(5):
        hip.memcpy_async(dst, src, nbytes, stream=recv_stream)
    e0.record(recv_stream)
    for _ in range(50):
        hip.memcpy_async(dst, src, nbytes, stream=recv_stream)
    e1.record(recv_stream)
    e1.synchronize()
    memcpy_us = e0.elapsed_ms(e1) / 50 * 1e3
    destroy(objs)

    kernel_us = kernel_ms / launches * 1e3
    achieved = 2.0 * nbytes / (kernel_us * 1e-6) / 1e9
    per_us.sort()
    return {
        "value": nbytes * steps / total_s / 1e9,
        "ms_per_step": total_s / steps * 1e3,
        "step_p50_us": float(per_us[int(0.5 * len(per_us))]),
        "profiled_pass_ms_per_step": prof_total_s / steps * 1e3,
        "ms_per_step_repeats": repeats,
        "roofline": {
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            # HBM-side bytes per launch from the two rocprofv3 --pmc passes over this command
            # (FETCH_SIZE and WRITE_SIZE, scaled as the named summary says), read from that file
            "traffic": traffic_from_profile(TRAFFIC_PROFILE, "tphip::single_copy_kernel<4, 0>"),
            "traffic_source": TRAFFIC_PROFILE,
            "kernel": "tphip::single_copy_kernel<4, 0>", "kernel_avg_us": kernel_us,
            "algorithmic_bytes_per_launch": 2 * nbytes,
        },
        "hipMemcpyAsync_d2d_us": memcpy_us,
        "hipMemcpyAsync_d2d_hbm_GBps": 2.0 * nbytes / (memcpy_us * 1e-6) / 1e9,
    }


def bench_d2d_in_flight(depth=4, transfers=400):
    """configs[1]'s tensor with several transfers in flight on the same pipes: `depth` chains of
    write/read run side by side (one caller thread each), every chain with a receive buffer and
    stream of its own; all copies are queued on the sender's one stream."""
    import threading

    import torch

    from tensorpipe_amd import datagen
    from tensorpipe_amd import pipe as tp

    nbytes = 64 * MIB
    src = torch.from_numpy(datagen.uniform_u8(datagen.SEED_BASE + 2, nbytes)).cuda()
    dsts = [torch.zeros(nbytes, dtype=torch.uint8, device="cuda") for _ in range(depth)]
    objs = make_pair("basic:0,hip_xth:10")
    cpipe, spipe = objs[0], objs[1]
    send_stream = torch.cuda.Stream()
    recv_streams = [torch.cuda.Stream() for _ in range(depth)]
    st = [tp.make_tensor(src, stream=send_stream, target=(tp.HIP, 0))]
    rts = [[tp.make_tensor(d, stream=s)] for d, s in zip(dsts, recv_streams)]
    torch.cuda.synchronize()
    tp.bench_transfer(cpipe, spipe, st, rts[0], warmup=0, iters=20)
    per_chain = transfers // depth
    lined_up = threading.Barrier(depth + 1)

    def chain(k):
        lined_up.wait()
        tp.bench_transfer(cpipe, spipe, st, rts[k], warmup=0, iters=per_chain)

    threads = [threading.Thread(target=chain, args=(k,)) for k in range(depth)]
    for t in threads:
        t.start()
    lined_up.wait()  # every caller thread is up: the clock starts with the first write
    t0 = time.perf_counter()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ok = all(bool(torch.equal(src, d)) for d in dsts)
    destroy(objs)
    done = per_chain * depth
    return {"in_flight": depth, "transfers": done, "us_per_transfer": dt / done * 1e6,
            "payload_GBps": nbytes * done / dt / 1e9,
            "hbm_frac": 2.0 * nbytes * done / dt / 1e9 / HBM_PEAK_GBPS, "byte_exact": ok}


def bench_rpc_message(messages=500, warmup=20):
    """configs[4]: 256 fp16 tensors, log-uniform sizes, 4 KiB payload, one launch per message."""
    import numpy as np
    import torch

    from tensorpipe_amd import datagen
    from tensorpipe_amd import pipe as tp

    sizes = [int(s) for s in datagen.loguniform_sizes(datagen.SEED_BASE + 5, 256, 4 * MIB, 256)]
    total = sum(sizes)
    arena_src = torch.zeros(total + 16 * len(sizes), dtype=torch.uint8, device="cuda")
    arena_dst = torch.zeros_like(arena_src)  # the padding between tensors stays zero in both
    st, rt, off = [], [], 0
    for i, n in enumerate(sizes):
        h = datagen.normal(1000 + i, n // 2, "f16", sigma=0.02).view(np.uint8)
        arena_src[off:off + n] = torch.from_numpy(h).cuda()
        st.append(tp.make_tensor(arena_src.data_ptr() + off, nbytes=n, device=tp.HIP,
                                 target=(tp.HIP, 0)))
        rt.append(tp.make_tensor(arena_dst.data_ptr() + off, nbytes=n, device=tp.HIP))
        off += (n + 15) // 16 * 16
    payload = datagen.bench_pattern(4096)
    pout = np.zeros(4096, np.uint8)
    objs = make_pair("basic:0,hip_xth:10")
    torch.cuda.synchronize()
    tp.bench_transfer(objs[0], objs[1], st, rt, payloads=[payload], recv_payloads=[pout],
                      warmup=0, iters=warmup)
    per_us, total_s = tp.bench_transfer(objs[0], objs[1], st, rt, payloads=[payload],
                                        recv_payloads=[pout], warmup=0, iters=messages)
    _, launches, kernel_ms, _ = profiled(
        lambda: tp.bench_transfer(objs[0], objs[1], st, rt, payloads=[payload],
                                  recv_payloads=[pout], warmup=0, iters=messages), messages + 8)
    torch.cuda.synchronize()
    ok = bool(torch.equal(arena_src[:off], arena_dst[:off])) and bytes(pout) == bytes(payload)
    destroy(objs)

    # the same message between two processes (hip_ipc), as a round trip
    arena_dst.zero_()
    peer = PeerRun("basic:0,hip_ipc:11")
    try:
        torch.cuda.synchronize()
        ipc_us, _ = peer.pingpong(st, rt, sizes, "gpu", 10, 200)
        torch.cuda.synchronize()
        ipc_ok = bool(torch.equal(arena_src[:off], arena_dst[:off]))
    finally:
        peer.close()
    ipc_us.sort()
    ipc_p50 = float(ipc_us[int(0.5 * len(ipc_us))])
    per_us.sort()
    kernel_us = kernel_ms / max(launches, 1) * 1e3
    return {
        "tensors": len(sizes), "total_bytes": total, "messages": messages,
        "launches_per_message": launches / messages,
        "payload_GBps": total * messages / total_s / 1e9,
        "message_p50_us": float(per_us[int(0.5 * len(per_us))]),
        "kernel_avg_us": kernel_us,
        "kernel_hbm_GBps": 2.0 * total / (kernel_us * 1e-6) / 1e9,
        "kernel_hbm_frac": 2.0 * total / (kernel_us * 1e-6) / 1e9 / HBM_PEAK_GBPS,
        "byte_exact": ok,
        "ipc_round_trip_p50_us": ipc_p50,
        "ipc_payload_GBps": 2.0 * total / (ipc_p50 * 1e-6) / 1e9,
        "ipc_byte_exact": ipc_ok,
    }


def bench_rpc_message_in_flight(depth=3, messages=1200):
    """configs[4]'s message with several in flight on the same pipes: `depth` chains of write/read
    side by side (one caller thread each, receive buffers and stream of their own)."""
    import threading

    import torch

    from tensorpipe_amd import datagen
    from tensorpipe_amd import pipe as tp

    sizes = [int(s) for s in datagen.loguniform_sizes(datagen.SEED_BASE + 5, 256, 4 * MIB, 256)]
    total = sum(sizes)
    arena_src = torch.zeros(total + 16 * len(sizes), dtype=torch.uint8, device="cuda")
    arena_src.random_(0, 256)
    dsts = [torch.zeros_like(arena_src) for _ in range(depth)]
    send_stream = torch.cuda.Stream()
    recv_streams = [torch.cuda.Stream() for _ in range(depth)]
    st, rts, off = [], [[] for _ in range(depth)], 0
    for n in sizes:
        st.append(tp.make_tensor(arena_src.data_ptr() + off, nbytes=n, device=tp.HIP, stream=send_stream,
                                 target=(tp.HIP, 0)))
        for k in range(depth):
            rts[k].append(tp.make_tensor(dsts[k].data_ptr() + off, nbytes=n, device=tp.HIP,
                                         stream=recv_streams[k]))
        off += (n + 15) // 16 * 16
    objs = make_pair("basic:0,hip_xth:10")
    torch.cuda.synchronize()
    for k in range(depth):  # every chain's buffers and stream have been used once before the clock starts
        tp.bench_transfer(objs[0], objs[1], st, rts[k], warmup=0, iters=10)
    per_chain = messages // depth
    lined_up = threading.Barrier(depth + 1)

    def chain(k):
        lined_up.wait()
        tp.bench_transfer(objs[0], objs[1], st, rts[k], warmup=0, iters=per_chain)

    threads = [threading.Thread(target=chain, args=(k,)) for k in range(depth)]
    for t in threads:
        t.start()
    lined_up.wait()
    t0 = time.perf_counter()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    done = per_chain * depth
    ok, o = True, 0
    for n in sizes:  # the padding between tensors is not part of any message
        ok = ok and all(bool(torch.equal(arena_src[o:o + n], d[o:o + n])) for d in dsts)
        o += (n + 15) // 16 * 16
    destroy(objs)
    return {"in_flight": depth, "messages": done, "tensors": len(sizes), "total_bytes": total,
            "us_per_message": dt / done * 1e6, "payload_GBps": total * done / dt / 1e9,
            "hbm_frac": 2.0 * total * done / dt / 1e9 / HBM_PEAK_GBPS, "byte_exact": ok}


class PeerRun:
    """A bench_peer child process connected through one pipe."""

    def __init__(self, channels, env=None, transport="shm"):
        from tensorpipe_amd import pipe as tp

        self.tp = tp
        saved = {k: os.environ.get(k) for k in (env or {})}
        os.environ.update(env or {})
        try:
            self.ctx = tp.Context("bench_main", transports=transport + ":0", channels=channels)
        finally:
            for k, v in saved.items():
                if v is None:
                    os.environ.pop(k, None)
                else:
                    os.environ[k] = v
        self.listener = self.ctx.listen("uv://127.0.0.1" if transport == "uv" else "shm://")
        # "shm_stock" (the reference's shm protocol) registers under the name "shm"
        self.transport = "shm" if transport == "shm_stock" else transport
        child_env = dict(os.environ)
        child_env.update(env or {})
        child_env["TP_BENCH_PEER_TRANSPORT"] = transport
        child_env["PYTHONPATH"] = ROOT + os.pathsep + child_env.get("PYTHONPATH", "")
        self.proc = subprocess.Popen(
            [sys.executable, os.path.join(ROOT, "bench_peer.py"), self.listener.url(self.transport), channels],
            env=child_env, cwd=ROOT)
        self.pipe = self.listener.accept(180000)

    def pingpong(self, send, recv, sizes, device, warmup, iters, payloads=(), recv_payloads=()):
        cmd = {"op": "pingpong", "sizes": sizes, "device": device, "warmup": warmup,
               "iters": iters, "payload": payloads[0].nbytes if payloads else 0}
        self.pipe.write([], metadata=json.dumps(cmd)).wait()
        d = self.pipe.read_descriptor(120000)
        self.pipe.read([], []).wait()
        assert d.metadata.decode() == "ready"
        return self.tp.bench_pingpong(self.pipe, True, send, recv, payloads=payloads,
                                      recv_payloads=recv_payloads, warmup=warmup, iters=iters)

    def open_more(self, count):
        """`count` more pipes between the two processes (same contexts, same channels)."""
        self.pipe.write([], metadata=json.dumps({"op": "connect", "count": count})).wait()
        more = [self.listener.accept(60000) for _ in range(count)]
        d = self.pipe.read_descriptor(120000)
        self.pipe.read([], []).wait()
        assert d.metadata.decode() == "connected"
        self.more = getattr(self, "more", []) + more
        return more

    def pingpong_multi(self, sends, recvs, size, warmup, iters):
        """One ping-pong chain per pipe, all at once; returns (seconds from the first chain's start
        to the last chain's end, round trips in that time). The warm-up rounds are a run of their
        own before it: first use maps the peer's buffers."""
        import threading

        pipes = [self.pipe] + getattr(self, "more", [])

        def run(rounds):
            cmd = {"op": "pingpong_multi", "sizes": [size], "warmup": 0, "iters": rounds}
            self.pipe.write([], metadata=json.dumps(cmd)).wait()
            d = self.pipe.read_descriptor(120000)
            self.pipe.read([], []).wait()
            assert d.metadata.decode() == "ready"
            lined_up = threading.Barrier(len(pipes) + 1)
            began, ended = [0.0] * len(pipes), [0.0] * len(pipes)

            def chain(k, q, st, rt):
                lined_up.wait()
                began[k] = time.perf_counter()
                # 2: each chain waits for its receive stream on a thread of its own, not on the context's
                self.tp.bench_pingpong(q, 2, st, rt, warmup=0, iters=rounds)
                ended[k] = time.perf_counter()

            threads = [threading.Thread(target=chain, args=(k,) + a)
                       for k, a in enumerate(zip(pipes, sends, recvs))]
            for t in threads:
                t.start()
            lined_up.wait()
            for t in threads:
                t.join()
            return max(ended) - min(began)

        run(warmup)
        return run(iters), len(pipes) * iters

    def close(self):
        try:
            try:
                self.pipe.write([], metadata=json.dumps({"op": "quit"})).wait(10000)
            except self.tp.PipeError:
                pass  # the peer read it and left before the write's callback ran
            self.proc.wait(30)
        finally:
            if self.proc.poll() is None:
                self.proc.kill()
            destroy(getattr(self, "more", []) + [self.pipe, self.listener, self.ctx])


def bench_ipc(iters=100, warmup=5, max_bytes=1 << 30, min_bytes=4096):
    """configs[2]: hip_ipc, one fp32 tensor, 4 KiB * 4^k up to 1 GiB, ping-pong with a peer process."""
    import numpy as np
    import torch

    from tensorpipe_amd import datagen
    from tensorpipe_amd import pipe as tp

    peer = PeerRun("basic:0,hip_ipc:11")
    out = {"sizes": {}}
    try:
        size = min_bytes
        while size <= max_bytes:
            # seeded N(0,1) over the whole tensor, no two 16 MiB blocks alike
            host = datagen.normal_large(datagen.SEED_BASE + 3, size // 4, "f32").view(np.uint8)
            src = torch.from_numpy(host).cuda()
            del host
            dst = torch.zeros(size, dtype=torch.uint8, device="cuda")
            st = [tp.make_tensor(src, target=(tp.HIP, 0))]
            rt = [tp.make_tensor(dst)]
            torch.cuda.synchronize()
            # latency-sized transfers get more round trips (clocks and the
            # polling threads settle within the first few milliseconds)
            n_it = iters * 10 if size <= MIB else iters if size <= 256 * MIB else max(iters // 4, 10)
            per_us, total_s = peer.pingpong(st, rt, [size], "gpu", warmup * 10 if size <= MIB else warmup, n_it)
            torch.cuda.synchronize()
            ok = bool(torch.equal(src, dst))
            per_us.sort()
            p50 = float(per_us[int(0.5 * len(per_us))])
            # one round trip carries the tensor once in each direction
            gbps = 2.0 * size / (p50 * 1e-6) / 1e9
            out["sizes"][str(size)] = {
                "rtt_p50_us": p50, "payload_GBps": gbps, "hbm_GBps": 2 * gbps,
                "hbm_frac": 2 * gbps / HBM_PEAK_GBPS, "byte_exact": ok, "iters": n_it}
            if size >= 64 * MIB:
                # the copy kernel alone (this side launches the copies of the echo direction)
                _, launches, kernel_ms, _ = profiled(
                    lambda: peer.pingpong(st, rt, [size], "gpu", 1, 10), 16)
                k_us = kernel_ms / max(launches, 1) * 1e3
                out["sizes"][str(size)].update({
                    "kernel_avg_us": k_us,
                    "kernel_hbm_GBps": 2.0 * size / (k_us * 1e-6) / 1e9,
                    "kernel_hbm_frac": 2.0 * size / (k_us * 1e-6) / 1e9 / HBM_PEAK_GBPS})
            log(f"  ipc {size:>11d} B  rtt p50 {p50:10.1f} us  payload {gbps:8.1f} GB/s  exact={ok}")
            del src, dst
            size *= 4
        if "4096" in out["sizes"]:
            out["rtt_4KiB_p50_us"] = out["sizes"]["4096"]["rtt_p50_us"]
    finally:
        peer.close()
    return out


def bench_ipc_in_flight(depth=4, sizes=(64 * MIB, 256 * MIB, 1 << 30)):
    """configs[2]'s large tensors with `depth` transfers in flight between the two processes:
    `depth` pipes over the same pair of contexts, one ping-pong chain on each, every chain with
    buffers and a stream of its own on both sides. What the channel moves when it is kept busy,
    beside the one-at-a-time round trips of the sweep."""
    import numpy as np
    import torch

    from tensorpipe_amd import datagen
    from tensorpipe_amd import pipe as tp

    peer = PeerRun("basic:0,hip_ipc:11")
    out = {"in_flight": depth, "sizes": {}}
    try:
        peer.open_more(depth - 1)
        for size in sizes:
            host = datagen.normal_large(datagen.SEED_BASE + 3, size // 4, "f32").view(np.uint8)
            srcs = [torch.from_numpy(host).cuda() for _ in range(depth)]
            del host
            dsts = [torch.zeros(size, dtype=torch.uint8, device="cuda") for _ in range(depth)]
            streams = [torch.cuda.Stream() for _ in range(depth)]
            sends = [[tp.make_tensor(s, stream=st, target=(tp.HIP, 0))] for s, st in zip(srcs, streams)]
            recvs = [[tp.make_tensor(d, stream=st)] for d, st in zip(dsts, streams)]
            torch.cuda.synchronize()
            iters = 200 if size <= 64 * MIB else 60 if size <= 256 * MIB else 16
            warm = 10
            dt, trips = peer.pingpong_multi(sends, recvs, size, warm, iters)
            torch.cuda.synchronize()
            ok = all(bool(torch.equal(s, d)) for s, d in zip(srcs, dsts))
            # every round trip carries the tensor once in each direction
            gbps = 2.0 * size * trips / dt / 1e9
            out["sizes"][str(size)] = {
                "round_trips": trips, "us_per_transfer": dt / (2 * trips) * 1e6, "payload_GBps": gbps,
                "hbm_frac": 2.0 * gbps / HBM_PEAK_GBPS, "byte_exact": ok}
            log(f"  ipc {depth} in flight {size:>11d} B  {dt / (2 * trips) * 1e6:9.1f} us per transfer  "
                f"payload {gbps:8.1f} GB/s  hbm {2.0 * gbps / HBM_PEAK_GBPS:.3f}  exact={ok}")
            del srcs, dsts, sends, recvs
            torch.cuda.empty_cache()
    finally:
        peer.close()
    return out


def bench_staged(iters=50, warmup=3, nbytes=256 * MIB):
    """configs[3]: hip_basic, 256 MiB bf16, GPU -> pinned -> shm -> pinned -> GPU, 4-deep ring."""
    import numpy as np
    import torch

    from tensorpipe_amd import datagen
    from tensorpipe_amd import pipe as tp

    out = {}
    # seeded N(0,1) in bf16 over the whole tensor, no two 8 MiB blocks alike
    host = datagen.normal_large(datagen.SEED_BASE + 4, nbytes // 2, "bf16").view(np.uint8)
    src = torch.from_numpy(host).cuda()
    del host
    dst = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    for chunk in (1 * MIB, 4 * MIB):
        env = {"TP_HIP_BASIC_SLOT_BYTES": str(chunk), "TP_HIP_BASIC_NUM_SLOTS": "4"}
        peer = PeerRun("basic:0,hip_basic:10", env=env)
        try:
            dst.zero_()
            st = [tp.make_tensor(src, target=(tp.HIP, 0))]
            rt = [tp.make_tensor(dst)]
            torch.cuda.synchronize()
            per_us, total_s = peer.pingpong(st, rt, [nbytes], "gpu", warmup, iters)
            torch.cuda.synchronize()
            ok = bool(torch.equal(src, dst))
            per_us.sort()
            p50 = float(per_us[int(0.5 * len(per_us))])
            # a round trip is two staged transfers back to back
            gbps = 2.0 * nbytes / (p50 * 1e-6) / 1e9
            out[f"chunk_{chunk // MIB}MiB"] = {
                "rtt_p50_ms": p50 / 1e3, "payload_GBps": gbps, "pcie_frac": gbps / PCIE_PEAK_GBPS,
                "byte_exact": ok, "iters": iters}
            log(f"  staged chunk {chunk // MIB} MiB: {gbps:.2f} GB/s ({gbps / PCIE_PEAK_GBPS:.1%} of PCIe) exact={ok}")
        finally:
            peer.close()
    return out


def bench_cpu_path(stock_wire_tcp=False, stock_wire_shm=False):
    """configs[0] on this library's own CPU side (Pipe + shm transport + basic channel, two
    processes): the control plane the device channels ride on, next to the reference's. With
    `stock_wire_tcp` the same over the TCP transport with the reference's encodings on the wire,
    with `stock_wire_shm` over the transport that speaks the reference's shm protocol: what the
    two routes to unmodified peers cost (both ends here are this library's)."""
    import numpy as np

    from tensorpipe_amd import datagen
    from tensorpipe_amd import pipe as tp

    out = {}
    if stock_wire_tcp or stock_wire_shm:
        peer = PeerRun("basic:0", env={"TP_STOCK_WIRE": "1"}, transport="uv" if stock_wire_tcp else "shm_stock")
    else:
        peer = PeerRun("basic:0")
    try:
        for name, n, iters in (("4KiB", 4096, 2000), ("1MiB", MIB, 1000), ("64MiB", 64 * MIB, 40)):
            src = datagen.uniform_u8(datagen.SEED_BASE + 1, n)
            dst = np.zeros(n, np.uint8)
            payload = datagen.bench_pattern(64)
            pout = np.zeros(64, np.uint8)
            per_us, _ = peer.pingpong([tp.make_tensor(src)], [tp.make_tensor(dst)], [n], "cpu", 5, iters,
                                      payloads=[payload], recv_payloads=[pout])
            per_us.sort()
            p50 = float(per_us[int(0.5 * len(per_us))])
            out[name] = {"rtt_p50_us": p50, "payload_GBps": 2.0 * n / (p50 * 1e-6) / 1e9,
                         "byte_exact": bool((src == dst).all()) and bytes(pout) == bytes(payload)}
            log(f"  own CPU path {name}: rtt p50 {p50:.1f} us  exact={out[name]['byte_exact']}")
    finally:
        peer.close()
    return out


def bench_torch_rpc():
    """torch.distributed.rpc round trips (PyTorch's own TensorPipe agent) with GPU tensors on this
    library's channels, next to CPU tensors on the agent's stock channels."""
    import tempfile

    from tensorpipe_amd import torch_rpc as tp_rpc

    if not os.path.exists(tp_rpc.library_path()):
        return {"error": "libtensorpipe_amd_torch_rpc.so is not built"}
    def run(mode):
        meeting = os.path.join(tempfile.mkdtemp(prefix="tp_rpc_"), "rendezvous")
        ranks = [subprocess.Popen([sys.executable, os.path.join(ROOT, "bench_rpc_peer.py"), str(r), meeting, mode],
                                  stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, cwd=ROOT)
                 for r in (1, 0)]
        try:
            out, _ = ranks[1].communicate(timeout=180)
            ranks[0].communicate(timeout=30)
        finally:
            for p in ranks:
                if p.poll() is None:
                    p.kill()
                    p.wait()
        if ranks[1].returncode != 0:
            raise RuntimeError(f"rank 0 of the RPC group ({mode}) ended with {ranks[1].returncode}")
        return json.loads(out.decode().strip().splitlines()[-1])

    out = run("all")
    staged = run("staged")
    out["gpu_tensors_hip_basic"] = staged["gpu_tensors_hip_basic"]
    for k, v in staged["gpu_buffers_by_channel"].items():
        out["gpu_buffers_by_channel"][k] = out["gpu_buffers_by_channel"].get(k, 0) + v
    return out


def bench_cold_copy():
    """The headline loop sends the same source every step, and 64 MiB stays resident in the
    256 MiB Infinity Cache between steps. The same kernel over rotating source/destination pairs
    (working set 1.25 GiB and more) shows what it does when every byte comes from HBM: the
    headline's 64 MiB, and 256 MiB and 1 GiB as in the cross-process sweep."""
    import torch

    from tensorpipe_amd import hip

    out = {}
    for name, nbytes, npairs, rounds in (("64MiB", 64 * MIB, 10, 4), ("256MiB", 256 * MIB, 4, 4),
                                         ("1GiB", 1 << 30, 2, 4)):
        pairs = [(torch.empty(nbytes // 8, dtype=torch.int64, device="cuda").random_().view(torch.uint8),
                  torch.empty(nbytes, dtype=torch.uint8, device="cuda")) for _ in range(npairs)]
        torch.cuda.synchronize()

        def rotate():
            for _ in range(rounds):
                for a, b in pairs:
                    hip.copy(b, a, nbytes)
            torch.cuda.synchronize()

        rotate()
        _, cold_n, cold_ms, _ = profiled(rotate, 64)
        cold_us = cold_ms / max(cold_n, 1) * 1e3
        ok = all(bool(torch.equal(a, b)) for a, b in pairs[:2])
        gbps = 2.0 * nbytes / (cold_us * 1e-6) / 1e9
        out[name] = {"kernel_avg_us": cold_us, "hbm_GBps": gbps, "hbm_frac": gbps / HBM_PEAK_GBPS,
                     "working_set_bytes": 2 * npairs * nbytes, "byte_exact": ok}
        # The same with loads and stores both streaming past the caches, whatever the size:
        # what a caller gets who knows that neither side will be touched again soon. (The
        # channels keep cached stores up to 64 MiB: what arrives is what the receiver reads next.)
        tables = [hip.make_table([(a, b, nbytes)])[0] for a, b in pairs]
        stream = torch.cuda.current_stream().cuda_stream

        def rotate_streaming():
            for _ in range(rounds):
                for t in tables:
                    hip.batched_copy_table(t, 1, stream=stream, unroll=4, blocks=0, nontemporal=3)
            torch.cuda.synchronize()

        rotate_streaming()
        _, s_n, s_ms, _ = profiled(rotate_streaming, 64)
        s_us = s_ms / max(s_n, 1) * 1e3
        out[name]["streaming_kernel_avg_us"] = s_us
        out[name]["streaming_hbm_frac"] = 2.0 * nbytes / (s_us * 1e-6) / 1e9 / HBM_PEAK_GBPS
        del pairs
        torch.cuda.empty_cache()
    # the figures of the 64 MiB case at the top level, where they have always been
    out.update(out["64MiB"])
    return out


def bench_hbm_streams(nbytes=256 * MIB, nbuffers=8, rounds=4):
    """What bounds a copy whose bytes all come from and go to HBM: a kernel that only reads and
    one that only writes, with the copy kernels' access pattern, over rotating 256 MiB buffers
    (2 GiB working set: nothing comes from the 256 MiB Infinity Cache), and the copy kernel over
    the same buffers. A copy reads a byte for every byte it writes, so it cannot beat the mix of
    the two one-directional rates, 2RW/(R+W)."""
    import ctypes

    import torch

    from tensorpipe_amd import _native, hip

    lib = _native.tphip()
    bufs = [torch.empty(nbytes // 8, dtype=torch.int64, device="cuda").random_().view(torch.uint8)
            for _ in range(nbuffers)]
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()

    def measure(fn):
        fn()
        _, n, ms, _ = profiled(fn, nbuffers * rounds + 8)
        return ms / max(n, 1) * 1e3

    def reads():
        for _ in range(rounds):
            for b in bufs:
                _native.check(lib.tphip_bench_stream(0, 0, b.data_ptr(), nbytes, stream))
        torch.cuda.synchronize()

    def writes():
        for _ in range(rounds):
            for b in bufs:
                _native.check(lib.tphip_bench_stream(0, 1, b.data_ptr(), nbytes, stream))
        torch.cuda.synchronize()

    def copies():
        for _ in range(rounds):
            for k in range(0, nbuffers, 2):
                hip.copy(bufs[k + 1], bufs[k], nbytes)
                hip.copy(bufs[k], bufs[k + 1], nbytes)
        torch.cuda.synchronize()

    read_us = measure(reads)
    copy_us = measure(copies)
    write_us = measure(writes)  # last: it overwrites the buffers
    r = nbytes / (read_us * 1e-6) / 1e9
    w = nbytes / (write_us * 1e-6) / 1e9
    c = 2.0 * nbytes / (copy_us * 1e-6) / 1e9
    mix = 2.0 * r * w / (r + w)
    return {"bytes": nbytes, "working_set_bytes": nbuffers * nbytes,
            "read_only_us": read_us, "read_only_GBps": r, "read_only_frac": r / HBM_PEAK_GBPS,
            "write_only_us": write_us, "write_only_GBps": w, "write_only_frac": w / HBM_PEAK_GBPS,
            "mix_bound_GBps": mix, "mix_bound_frac": mix / HBM_PEAK_GBPS,
            "copy_us": copy_us, "copy_hbm_GBps": c, "copy_frac": c / HBM_PEAK_GBPS,
            "copy_frac_of_mix_bound": c / mix}


def bench_link_duplex(nbytes=256 * MIB):
    """What the one host link of the one GPU gives when both directions run at once, which is
    what a staged transfer between two processes on one GPU does all the time (the sender's
    device-to-host chunks and the receiver's host-to-device chunks cross the same link): the copy
    kernel towards pinned host memory on one stream and from it on another, as one launch each
    and as back-to-back launches of 1 MiB and 4 MiB like the channel's chunks."""
    import ctypes
    import time

    import torch

    from tensorpipe_amd import _native, hip

    lib = _native.tphip()
    dsrc = torch.empty(nbytes // 8, dtype=torch.int64, device="cuda").random_().view(torch.uint8)
    ddst = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    up = torch.empty(nbytes, dtype=torch.uint8).pin_memory()
    down = torch.empty(nbytes // 8, dtype=torch.int64).random_().view(torch.uint8).pin_memory()
    s_up, s_down = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    out = {}
    for name, chunk in (("one_launch", nbytes), ("chunks_4MiB", 4 * MIB), ("chunks_1MiB", 1 * MIB)):
        n = nbytes // chunk
        tables = []
        for k in range(n):
            tables.append((hip.make_table([(dsrc.data_ptr() + k * chunk, up.data_ptr() + k * chunk, chunk)])[0],
                           hip.make_table([(down.data_ptr() + k * chunk, ddst.data_ptr() + k * chunk, chunk)])[0]))
        for mode in ("d2h_alone", "h2d_alone", "both"):
            best = 0.0
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for t_up, t_down in tables:
                    if mode != "h2d_alone":
                        _native.check(lib.tphip_batched_copy_tuned(0, t_up, 1, s_up.cuda_stream, 4, 32, 3))
                    if mode != "d2h_alone":
                        _native.check(lib.tphip_batched_copy_tuned(0, t_down, 1, s_down.cuda_stream, 4, 32, 3))
                torch.cuda.synchronize()
                best = max(best, nbytes / (time.perf_counter() - t0) / 1e9)
            out[f"{name}_{mode}_GBps"] = best
    ok = bool(torch.equal(up.cuda(), dsrc)) and bool(torch.equal(down.cuda(), ddst))
    out["byte_exact"] = ok
    out["duplex_ceiling_GBps"] = max(out["one_launch_both_GBps"], out["chunks_4MiB_both_GBps"],
                                     out["chunks_1MiB_both_GBps"])
    return out


def bench_link_ceiling(nbytes=256 * MIB):
    """Pinned D2H / H2D: the copy kernel against the runtime's copy engine path."""
    import torch

    from tensorpipe_amd import hip

    dev = torch.empty(nbytes, dtype=torch.uint8, device="cuda").random_()
    pinned = torch.empty(nbytes, dtype=torch.uint8).pin_memory()
    out = {}
    for name, fn in (
        ("d2h_kernel", lambda: hip.copy(pinned, dev, nbytes)),
        ("d2h_hipMemcpyAsync", lambda: hip.memcpy_async(pinned, dev, nbytes)),
        ("h2d_kernel", lambda: hip.copy(dev, pinned, nbytes)),
        ("h2d_hipMemcpyAsync", lambda: hip.memcpy_async(dev, pinned, nbytes)),
    ):
        fn()
        torch.cuda.synchronize()
        e0, e1 = hip.TimedEvent(), hip.TimedEvent()
        e0.record()
        for _ in range(5):
            fn()
        e1.record()
        e1.synchronize()
        out[name + "_GBps"] = nbytes / (e0.elapsed_ms(e1) / 5 * 1e-3) / 1e9
    return out


def cpu_baseline():
    """CPU figures beside the GPU ones, on this box's host cores: the genuine reference
    (TensorPipe prebuilt inside PyTorch's libtorch_cpu.so: shm transport + basic channel,
    driven by oracle/_ref/ref_pipe_bench) when it is there, and always the port
    (oracle/cpu_shm_basic)."""

    def run(exe, tensor, payload, warmup, iters):
        r = subprocess.run([exe, str(tensor), str(payload), str(warmup), str(iters)],
                           stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
        return json.loads(r.stdout.strip().splitlines()[-1])

    def suite(exe):
        same = run(exe, 64 * MIB, 0, 2, 400)   # the headline workload's tensor, bounded sample (~5 s)
        cfg1 = run(exe, 1 * MIB, 64, 5, 1000)  # configs[0]
        rtt = run(exe, 4096, 64, 5, 2000)      # 4 KiB round trip
        return {"payload_GBps_64MiB": same["payload_GBps"],
                "config1_1MiB_rtt_p50_us": cfg1["rtt_p50_us"],
                "config1_payload_GBps": cfg1["payload_GBps"],
                "rtt_4KiB_p50_us": rtt["rtt_p50_us"]}

    port_exe = os.path.join(ROOT, "oracle", "cpu_shm_basic")
    ref_exe = os.path.join(ROOT, "oracle", "_ref", "ref_pipe_bench")
    port = ref = None
    if os.path.exists(port_exe):
        try:
            port = suite(port_exe)
        except Exception as e:  # reported, and the reference's figures stand alone
            log(f"[bench] CPU port FAILED: {e!r}")
    if os.path.exists(ref_exe):
        try:
            ref = suite(ref_exe)
        except Exception as e:  # e.g. a box whose torch lacks the tensorpipe symbols
            ref = {"error": repr(e)}
    if ref and "error" not in ref:
        main_, kind, cores = ref, "reference", 4
        threads = "2 processes x (1 busy-polling shm reactor + 1 epoll loop thread)"
    elif port:
        main_, kind, cores = port, "port", 2
        threads = "2 processes x 1 busy-polling thread"
    else:
        return {"error": "neither oracle/cpu_shm_basic nor oracle/_ref/ref_pipe_bench is built"}
    return {
        "value": main_["payload_GBps_64MiB"], "unit": "GB/s", "cores": cores, "kind": kind,
        "sample": "400 ping-pong round trips (800 transfers, 53.7 GB) of one 64 MiB CPU tensor through "
                  "Pipe + shm transport + basic channel; " + threads,
        "config1_1MiB_rtt_p50_us": main_["config1_1MiB_rtt_p50_us"],
        "config1_payload_GBps": main_["config1_payload_GBps"],
        "rtt_4KiB_p50_us": main_["rtt_4KiB_p50_us"],
        "host_cpus": os.cpu_count(),
        "affinity_cpus": sorted(os.sched_getaffinity(0)),
        "reference": ref, "port": port,
    }


# The configurations besides the headline. Each runs in a process of its own so that
# none inherits runtime state from another (streams a process has used change what the
# runtime does on later launches, which shifts small-transfer latencies by microseconds).
LEGS = {
    "rpc_message": bench_rpc_message,
    "rpc_message_in_flight": bench_rpc_message_in_flight,
    "d2d_in_flight": bench_d2d_in_flight,
    "ipc": bench_ipc,
    "ipc_in_flight": bench_ipc_in_flight,
    "staged": bench_staged,
    "staged_short": lambda: bench_staged(iters=20),
    "host_link": bench_link_ceiling,
    "host_link_duplex": bench_link_duplex,
    "hbm_streams": bench_hbm_streams,
    "ipc_rtt": lambda: bench_ipc(iters=300, warmup=30, max_bytes=4096),
    "ipc_large": lambda: bench_ipc(iters=40, warmup=3, min_bytes=256 * MIB),
    "cpu_path": bench_cpu_path,
    "cpu_path_stock_wire_tcp": lambda: bench_cpu_path(stock_wire_tcp=True),
    "cpu_path_stock_wire_shm": lambda: bench_cpu_path(stock_wire_shm=True),
    "cold_copy": bench_cold_copy,
    "torch_rpc": bench_torch_rpc,
}


def run_leg(name, timeout_s=600, env=None):
    """One configuration in a process (group) of its own; whatever happens, nothing of it is
    left running afterwards."""
    import signal

    proc = subprocess.Popen([sys.executable, os.path.abspath(__file__), "--leg", name],
                            stdout=subprocess.PIPE, env=dict(os.environ, **(env or {})),
                            start_new_session=True)
    try:
        out, _ = proc.communicate(timeout=timeout_s)
    finally:
        try:
            os.killpg(proc.pid, signal.SIGKILL)  # the leg's peer process too, should it still be there
        except ProcessLookupError:
            pass
        proc.wait()
    if proc.returncode != 0:
        raise RuntimeError(f"bench leg {name} failed with exit code {proc.returncode}")
    return json.loads(out.decode().strip().splitlines()[-1])


def extra_leg(name, env=None):
    """One of the other configurations; a failure there is reported in its place and on
    stderr, and does not take the headline line with it."""
    try:
        return run_leg(name, env=env)
    except Exception as e:  # noqa: BLE001 - any failure of a side measurement
        log(f"[bench] leg {name} FAILED: {e}")
        return {"error": f"{type(e).__name__}: {e}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-extras", action="store_true",
                    help="only the headline configuration and the CPU baseline")
    ap.add_argument("--leg", choices=sorted(LEGS), default=None,
                    help="run one of the other configurations alone and print its JSON (internal)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; every configuration of the device "
                 "channels is single-GPU (run with --gpus 1)")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    from tensorpipe_amd import _native

    _native.tphip()  # fails loudly if the HIP library is not built

    if args.leg is not None:
        print(json.dumps(LEGS[args.leg]()), flush=True)
        return

    t_start = time.time()
    log("[bench] same-process D2D, 64 MiB (headline)")
    d2d = bench_d2d(args.steps, args.warmup)
    extra = {
        "d2d_step_p50_us": d2d["step_p50_us"],
        "d2d_profiled_pass_ms_per_step": d2d["profiled_pass_ms_per_step"],
        # the timed pass (= ms_per_step) and two more passes of the same K steps
        "d2d_ms_per_step_repeats": d2d["ms_per_step_repeats"],
        "hipMemcpyAsync_d2d_us": d2d["hipMemcpyAsync_d2d_us"],
        "hipMemcpyAsync_d2d_hbm_GBps": d2d["hipMemcpyAsync_d2d_hbm_GBps"],
    }
    if not args.skip_extras:
        log("[bench] many-tensor message (256 tensors, one launch per message)")
        extra["rpc_message"] = extra_leg("rpc_message")
        extra["rpc_message_in_flight"] = extra_leg("rpc_message_in_flight")
        log("[bench] cross-process IPC sweep")
        extra["ipc"] = extra_leg("ipc")
        # the large tensors of the sweep with four transfers in flight between the processes
        extra["ipc_in_flight"] = extra_leg("ipc_in_flight")
        log("[bench] host-staged 256 MiB")
        extra["staged"] = extra_leg("staged")
        # the same transfers with the runtime's hipMemcpyAsync instead of the copy kernel
        extra["staged_hipMemcpyAsync"] = extra_leg("staged_short", env={"TP_HIP_BASIC_ENGINE": "sdma"})
        # ... and with the copy kernel launched per chunk by the host (one launch, one polled
        # event and two control messages per chunk) instead of the two kernels that walk the ring
        extra["staged_host_driven"] = extra_leg("staged_short", env={"TP_HIP_BASIC_GPU_RING": "0"})
        extra["host_link"] = extra_leg("host_link")
        # both directions of the one host link at once: what bounds a staged transfer on one GPU
        duplex = extra_leg("host_link_duplex")
        extra["host_link_duplex"] = duplex
        if "duplex_ceiling_GBps" in duplex and "error" not in extra["staged"]:
            for name, leg in extra["staged"].items():
                if isinstance(leg, dict) and "payload_GBps" in leg:
                    # against the link with both directions busy: as one launch per direction, and
                    # as back-to-back launches of this leg's chunk size
                    leg["frac_of_duplex_one_launch"] = leg["payload_GBps"] / duplex["one_launch_both_GBps"]
                    same = duplex.get("chunks_" + name.split("_", 1)[1] + "_both_GBps")
                    if same:
                        leg["frac_of_duplex_same_chunks"] = leg["payload_GBps"] / same
        # the 4 KiB round trip in three more pairs of processes: it moves by a third from one
        # pair of processes to the next on the same box (where the hypervisor puts the threads)
        rtts = [extra["ipc"].get("rtt_4KiB_p50_us")] if "error" not in extra["ipc"] else []
        for _ in range(3):
            again = extra_leg("ipc_rtt")
            if "rtt_4KiB_p50_us" in again:
                rtts.append(again["rtt_4KiB_p50_us"])
        rtts = sorted(r for r in rtts if r is not None)
        if rtts:
            extra["ipc_rtt_4KiB"] = {"p50_us_per_process_pair": rtts,
                                     "median_us": rtts[len(rtts) // 2], "best_us": rtts[0]}
        # the headline's tensor with four transfers in flight instead of one
        extra["d2d_in_flight"] = extra_leg("d2d_in_flight")
        extra["d2d_cold_source"] = extra_leg("cold_copy")
        # what HBM gives a kernel that only reads or only writes: the bound of any copy
        extra["hbm_streams"] = extra_leg("hbm_streams")
        log("[bench] this library's CPU path (shm + basic)")
        extra["cpu_path"] = extra_leg("cpu_path")
        log("[bench] the same over TCP in the reference's wire format")
        extra["cpu_path_stock_wire_tcp"] = extra_leg("cpu_path_stock_wire_tcp")
        extra["cpu_path_stock_wire_shm"] = extra_leg("cpu_path_stock_wire_shm")
        log("[bench] torch.distributed.rpc with GPU tensors on these channels")
        extra["torch_rpc"] = extra_leg("torch_rpc")
    log("[bench] CPU baseline (port of shm + basic)")
    cpu = cpu_baseline()
    extra["bench_wall_s"] = time.time() - t_start

    roofline = d2d["roofline"]
    # Next to the kernel's own figure (achieved / frac, from the launches' begin and end): the
    # same bytes over the whole timed step, host time included, and what the kernel does when
    # nothing can come from the Infinity Cache.
    roofline["step_frac"] = 2.0 * 64 * MIB / (d2d["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBPS
    cold = extra.get("d2d_cold_source", {})
    if "hbm_frac" in cold:
        roofline["hbm_only_frac"] = cold["hbm_frac"]
    roofline["note"] = ("achieved/frac: one launch of the copy kernel, source resident in the 256 MiB Infinity "
                        "Cache as in any loop that re-sends a 64 MiB tensor; step_frac: the whole write/read "
                        "step; hbm_only_frac: the same kernel over rotating buffers, every byte from HBM")

    line = {
        "metric": "payload GB/s, same-process D2D channel (fraction of HBM roofline under roofline.frac; "
                  "p50 RTT at 4 KiB under extra.ipc)",
        "value": d2d["value"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": d2d["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic (seeded uniform bytes)",
        "config": {"workload": "configs[1]: hip_xth same-process D2D, 1 x 64 MiB uint8 tensor, "
                               "two connected pipes in one process, write/read per step, byte-exact"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
