"""The resident copy agent and the signal words of the tphip C ABI: copies posted to the agent
are byte-identical to the CPU oracle's for the same table, the notify word is raised after the
bytes are visible, an agent that left is started again, and a word raised in stream order is
seen by the host."""
import ctypes
import os
import time

import numpy as np
import pytest

from tensorpipe_amd import _native, datagen, hip

pytestmark = pytest.mark.gpu

FILL = 0xEE
BUSY = -6


class Agent:
    def __init__(self):
        self.lib = _native.tphip()
        self.h = ctypes.c_void_p()
        _native.check(self.lib.tphip_agent_create(0, ctypes.byref(self.h)), "tphip_agent_create")

    def submit(self, entries, notify=None, value=0):
        table, n = hip.make_table(entries)
        ticket = ctypes.c_uint64()
        rc = self.lib.tphip_agent_submit(self.h, table, n, notify, value, ctypes.byref(ticket))
        return rc, ticket.value

    def wait(self, ticket, timeout=5.0):
        done = ctypes.c_int(0)
        t0 = time.time()
        while True:
            _native.check(self.lib.tphip_agent_done(self.h, ticket, ctypes.byref(done)), "tphip_agent_done")
            if done.value:
                return
            assert time.time() - t0 < timeout, "the agent never served the command"

    def close(self):
        if self.h:
            _native.check(self.lib.tphip_agent_destroy(self.h), "tphip_agent_destroy")
            self.h = None


@pytest.fixture()
def agent():
    a = Agent()
    yield a
    a.close()


def _pinned_words(n):
    import torch

    t = torch.zeros(n, dtype=torch.int64).pin_memory()
    return t


def test_agent_copies_match_the_oracle(agent, oracle):
    import torch

    sizes = [1, 2, 15, 16, 17, 63, 64, 255, 256, 4096, 4099, 65536, 70001, 0, 33]
    rng = np.random.default_rng(5)
    layout, so, do = [], 0, 0
    for n in sizes:
        so = (so + 15) // 16 * 16 + int(rng.integers(0, 16))
        do = (do + 15) // 16 * 16 + int(rng.integers(0, 16))
        layout.append((so, do, n))
        so += n + 24
        do += n + 24
    host_src = datagen.uniform_u8(901, so + 64)
    src = torch.from_numpy(host_src).cuda()
    dst = torch.full((do + 64,), FILL, dtype=torch.uint8, device="cuda")
    ref = np.full(do + 64, FILL, dtype=np.uint8)
    torch.cuda.synchronize()
    words = _pinned_words(8)
    last = 0
    for k in range(0, len(layout), 4):
        part = layout[k:k + 4]
        rc, last = agent.submit([(src.data_ptr() + s, dst.data_ptr() + d, n) for s, d, n in part],
                                notify=words.data_ptr() + 8, value=1000 + k)
        assert rc == 0
        agent.wait(last)
        # the word is raised before the ticket is reported done
        assert int(words[1]) == 1000 + k
    oracle.xth_message([(host_src[s:], ref[d:], n) for s, d, n in layout])
    got = dst.cpu().numpy()
    bad = np.nonzero(got != ref)[0]
    assert bad.size == 0, f"{bad.size} bytes differ, first at {bad[0]}"
    assert (src.cpu().numpy() == host_src).all()


def test_agent_restarts_after_leaving_and_serves_bursts(agent):
    import torch

    src = torch.arange(4096, dtype=torch.int32, device="cuda")
    dst = torch.zeros(64, 4096, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    posted = 0
    tickets = []
    for burst in range(6):
        for _ in range(9):
            row = posted % 64
            while True:
                rc, t = agent.submit([(src.data_ptr(), dst[row].data_ptr(), 4096 * 4)])
                if rc != BUSY:
                    break
                agent.wait(tickets[-1])
            assert rc == 0
            tickets.append(t)
            posted += 1
        agent.wait(tickets[-1])
        time.sleep(0.005)  # far beyond the idle limit: the agent has left and must come back
    assert tickets == list(range(1, posted + 1))
    torch.cuda.synchronize()
    assert bool((dst[:min(posted, 64)] == src).all())


def test_agent_rejects_what_it_cannot_take(agent):
    import torch

    a = torch.zeros(64, dtype=torch.uint8, device="cuda")
    rc, _ = agent.submit([(a.data_ptr(), a.data_ptr() + 32, 0)])
    assert rc == -1  # nothing to copy
    rc, _ = agent.submit([(0, a.data_ptr(), 16)])
    assert rc == -1
    rc, _ = agent.submit([(a.data_ptr(), a.data_ptr() + 32, 16)] * 33)
    assert rc == -1  # more than one submission may carry


def test_two_agents_and_destroy_while_running():
    import torch

    src = torch.full((1 << 16,), 7, dtype=torch.uint8, device="cuda")
    dst = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    a, b = Agent(), Agent()
    rc, ta = a.submit([(src.data_ptr(), dst.data_ptr(), 1 << 15)])
    assert rc == 0
    rc, tb = b.submit([(src.data_ptr() + (1 << 15), dst.data_ptr() + (1 << 15), 1 << 15)])
    assert rc == 0
    a.wait(ta)
    b.wait(tb)
    a.close()  # right away: the agent is still inside its idle window
    b.close()
    torch.cuda.synchronize()
    assert bool((dst == 7).all())


def test_stream_signal_is_seen_by_the_host_in_stream_order():
    import torch

    lib = _native.tphip()
    words = _pinned_words(4)
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.Stream()
    for v in (5, 6, 7):
        with torch.cuda.stream(stream):
            buf.add_(1)
        _native.check(lib.tphip_stream_signal(0, stream.cuda_stream, words.data_ptr() + 16, v), "tphip_stream_signal")
        t0 = time.time()
        while int(words[2]) != v:
            assert time.time() - t0 < 5.0
        # the add enqueued before the signal has finished: the stream has nothing pending
    stream.synchronize()
    assert int(buf[0]) == 3


def _gated(lib, table, n, stream, event, gate_ptr, value, max_wait_us, expired_ptr):
    _native.check(
        lib.tphip_batched_copy_gated(0, table, n, stream, event, gate_ptr, value, max_wait_us, expired_ptr),
        "tphip_batched_copy_gated")


@pytest.mark.parametrize("shape", ["single", "inline", "table"])
def test_gated_copy_waits_for_the_word_and_gives_up_in_time(oracle, shape):
    """A gated copy starts when the word is raised in stream order on another stream, and one
    whose word never comes ends by itself, reports it, and has copied nothing."""
    import torch

    lib = _native.tphip()
    sizes = {"single": [3 << 20], "inline": [70001, 4096, 33, 1 << 20], "table": [4096 + 3 * k for k in range(200)]}[shape]
    total = sum((s + 31) // 16 * 16 for s in sizes) + 64
    host_src = datagen.uniform_u8(950, total)
    src = torch.zeros(total, dtype=torch.uint8, device="cuda")
    dst = torch.full((total,), FILL, dtype=torch.uint8, device="cuda")
    staging = torch.from_numpy(host_src).cuda()
    entries, off = [], 0
    layout = []
    for s in sizes:
        entries.append((src.data_ptr() + off + 1, dst.data_ptr() + off + 2, s))
        layout.append((off + 1, off + 2, s))
        off += (s + 31) // 16 * 16
    table, n = hip.make_table(entries)
    words = _pinned_words(8)
    gate, expired = words.data_ptr(), words.data_ptr() + 8
    producer, consumer = torch.cuda.Stream(), torch.cuda.Stream()
    ev = hip.TimedEvent()
    torch.cuda.synchronize()

    # 1) never raised: gives up after ~2 ms, nothing copied
    t0 = time.time()
    _gated(lib, table, n, consumer.cuda_stream, ev.handle, gate, 1, 2000, expired)
    ev.synchronize()
    assert time.time() - t0 < 2.0
    assert int(words[1]) == 1, "the copy must report that it gave up"
    assert bool((dst == FILL).all()), "a copy that gave up must not have written"

    if (os.environ.get("GPU_MAX_HW_QUEUES") == "1" or os.environ.get("AMD_SERIALIZE_KERNEL", "0") != "0"
            or os.environ.get("HIP_LAUNCH_BLOCKING", "0") != "0"):
        # One hardware queue for every stream, or launches that return only when the kernel has
        # ended: the producer's work could not start before the waiting gate has given up, which
        # is what the first half has just shown.
        return
    # 2) raised behind the producer's work: the copy sees what the producer wrote
    words[1] = 0
    _gated(lib, table, n, consumer.cuda_stream, ev.handle, gate, 1, 2_000_000, expired)
    time.sleep(0.01)  # the gated kernel is up and waiting
    with torch.cuda.stream(producer):
        src.copy_(staging, non_blocking=True)
    _native.check(lib.tphip_stream_signal(0, producer.cuda_stream, gate, 1), "tphip_stream_signal")
    ev.synchronize()
    torch.cuda.synchronize()
    assert int(words[1]) == 0
    ref = np.full(total, FILL, dtype=np.uint8)
    oracle.xth_message([(host_src[s:], ref[d:], b) for s, d, b in layout])
    got = dst.cpu().numpy()
    bad = np.nonzero(got != ref)[0]
    assert bad.size == 0, f"{bad.size} bytes differ, first at {bad[0]}"
