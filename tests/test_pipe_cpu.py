"""CPU-only tests of the pipe layer (shm transport, basic and xth channels):
the reference's generic channel cases (tensorpipe/test/channel/channel_test.cc)
driven through Pipe::write/read, plus close/error behaviour."""
import numpy as np
import pytest

from tensorpipe_amd import pipe as tp


@pytest.fixture
def pair():
    made = []

    def make(channels="basic:0"):
        server = tp.Context("server", channels=channels)
        client = tp.Context("client", channels=channels)
        listener = server.listen()
        cpipe = client.connect(listener.url())
        spipe = listener.accept()
        made.append((cpipe, spipe, listener, client, server))
        return cpipe, spipe

    yield make
    for cpipe, spipe, listener, client, server in made:
        cpipe.destroy()
        spipe.destroy()
        listener.destroy()
        client.destroy()
        server.destroy()


def _roundtrip(sender, receiver, arrays, payloads=(), targets=False):
    tensors = [tp.make_tensor(a, target=(tp.CPU, 0) if targets else None) for a in arrays]
    w = sender.write(tensors, payloads=payloads, metadata="meta")
    d = receiver.read_descriptor()
    assert d.metadata.decode() == "meta"
    assert d.num_tensors == len(arrays) and d.num_payloads == len(payloads)
    outs = [np.full(d.tensor_lengths[i], 0xEE, np.uint8) for i in range(d.num_tensors)]
    pouts = [np.zeros(d.payload_lengths[i], np.uint8) for i in range(d.num_payloads)]
    r = receiver.read([tp.make_tensor(o) for o in outs], pouts)
    r.wait()
    w.wait()
    return outs, pouts


@pytest.mark.parametrize("channels", ["basic:0", "xth:5,basic:0"])
def test_client_to_server_and_back(pair, channels):
    cpipe, spipe = pair(channels)
    assert spipe.remote_name() == "client"
    data = np.arange(256, dtype=np.uint8)
    outs, _ = _roundtrip(cpipe, spipe, [data])
    assert (outs[0] == data).all()
    outs, _ = _roundtrip(spipe, cpipe, [data[::-1].copy()])
    assert (outs[0] == data[::-1]).all()


@pytest.mark.parametrize("channels", ["basic:0", "xth:5,basic:0"])
@pytest.mark.parametrize("targets", [False, True])
def test_send_multiple_tensors(pair, channels, targets):
    cpipe, spipe = pair(channels)
    n = 256 * 1024
    src = (np.arange(n) % 256).astype(np.uint8)
    outs, _ = _roundtrip(cpipe, spipe, [src] * 20, targets=targets)
    for o in outs:
        assert (o == src).all()


def test_some_tensors_name_a_target_device(pair):
    # tensorpipe/test/core/pipe_test.cc:281-359 (SimpleWriteReadWithSomeTargetDevices): the first
    # tensor names the device it is to land on, the second leaves it to the receiver; the descriptor
    # tells the receiver which is which
    cpipe, spipe = pair()
    a = np.frombuffer(b"tensor #1", np.uint8).copy()
    b = np.frombuffer(b"tensor #2", np.uint8).copy()
    w = cpipe.write([tp.make_tensor(a, target=(tp.CPU, 0)), tp.make_tensor(b)],
                    payloads=[b"payload #1"], metadata="pipe metadata")
    d = spipe.read_descriptor()
    assert d.metadata.decode() == "pipe metadata" and d.num_tensors == 2 and d.num_payloads == 1
    assert (d.tensor_target_type[0], d.tensor_target_index[0]) == (tp.CPU, 0)
    assert d.tensor_target_type[1] == -1  # no target named
    assert d.tensor_source_type[0] == tp.CPU and d.tensor_source_type[1] == tp.CPU
    outs = [np.zeros(d.tensor_lengths[i], np.uint8) for i in range(2)]
    pout = np.zeros(d.payload_lengths[0], np.uint8)
    spipe.read([tp.make_tensor(o) for o in outs], [pout]).wait()
    w.wait()
    assert bytes(outs[0]) == b"tensor #1" and bytes(outs[1]) == b"tensor #2" and bytes(pout) == b"payload #1"


def test_payloads_and_empty_tensors(pair):
    cpipe, spipe = pair()
    a, z, b = np.array([7], np.uint8), np.zeros(0, np.uint8), np.array([9], np.uint8)
    outs, pouts = _roundtrip(cpipe, spipe, [a, z, b], payloads=[b"payload #0", b"", b"payload #2"])
    assert outs[0][0] == 7 and outs[1].size == 0 and outs[2][0] == 9
    assert bytes(pouts[0]) == b"payload #0" and bytes(pouts[2]) == b"payload #2"
    outs, _ = _roundtrip(cpipe, spipe, [z])
    assert outs[0].size == 0
    outs, pouts = _roundtrip(cpipe, spipe, [], payloads=[b"only payload"])
    assert bytes(pouts[0]) == b"only payload"


def test_large_message_exceeds_ring(pair):
    cpipe, spipe = pair()
    rng = np.random.default_rng(0)
    big = rng.integers(0, 256, 9 * 1024 * 1024 + 13, dtype=np.uint8)
    outs, _ = _roundtrip(cpipe, spipe, [big])
    assert (outs[0] == big).all()


def test_both_ways_interleaved(pair):
    cpipe, spipe = pair()
    a = np.full(100000, 1, np.uint8)
    b = np.full(50000, 2, np.uint8)
    w1 = cpipe.write([tp.make_tensor(a)])
    w2 = spipe.write([tp.make_tensor(b)])
    d1 = spipe.read_descriptor()
    d2 = cpipe.read_descriptor()
    o1 = np.zeros(d1.tensor_lengths[0], np.uint8)
    o2 = np.zeros(d2.tensor_lengths[0], np.uint8)
    r1 = spipe.read([tp.make_tensor(o1)])
    r2 = cpipe.read([tp.make_tensor(o2)])
    for op in (r1, r2, w1, w2):
        op.wait()
    assert (o1 == 1).all() and (o2 == 2).all()


def test_many_messages_in_order(pair):
    cpipe, spipe = pair()
    sources = [np.full(1000, i, np.uint8) for i in range(50)]  # must outlive the writes
    writes = [cpipe.write([tp.make_tensor(sources[i])], metadata=str(i)) for i in range(50)]
    for i in range(50):
        d = spipe.read_descriptor()
        assert d.metadata.decode() == str(i)
        o = np.zeros(1000, np.uint8)
        spipe.read([tp.make_tensor(o)]).wait()
        assert (o == i).all()
    for w in writes:
        w.wait()


@pytest.mark.parametrize("initiator", [1, 2])
def test_ping_pong_chains_side_by_side(initiator):
    """The benchmark harness's echo loop (tensorpipe/benchmark/benchmark_pipe.cc:463-468,571-577),
    three chains at once over one pair of contexts, the initiator finishing its rounds on the
    pipe's thread (1) or on a thread of the chain's own (2): every chain's last echo is its
    own source, byte for byte."""
    import threading

    server = tp.Context("server", channels="basic:0")
    client = tp.Context("client", channels="basic:0")
    listener = server.listen()
    pipes = []
    for _ in range(3):
        c = client.connect(listener.url())
        pipes.append((c, listener.accept()))
    rng = np.random.default_rng(7)
    srcs = [rng.integers(0, 256, 70000 + 13 * k, dtype=np.uint8) for k in range(3)]
    backs = [np.zeros_like(s) for s in srcs]
    echo_bufs = [np.zeros_like(s) for s in srcs]
    errors = []

    def side(fn, *args, **kwargs):
        try:
            fn(*args, **kwargs)
        except Exception as e:  # noqa: BLE001 - reported by the assertion below
            errors.append(e)

    threads = []
    for (c, s), src, back, buf in zip(pipes, srcs, backs, echo_bufs):
        t = [tp.make_tensor(buf)]
        threads.append(threading.Thread(target=side, args=(tp.bench_pingpong, s, 0, t, t),
                                        kwargs={"warmup": 2, "iters": 20}))
        threads.append(threading.Thread(target=side, args=(tp.bench_pingpong, c, initiator,
                                                           [tp.make_tensor(src)], [tp.make_tensor(back)]),
                                        kwargs={"warmup": 2, "iters": 20}))
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
    assert not errors and not any(t.is_alive() for t in threads), errors
    for src, back in zip(srcs, backs):
        assert (src == back).all()
    for c, s in pipes:
        c.destroy()
        s.destroy()
    listener.destroy()
    client.destroy()
    server.destroy()


@pytest.mark.parametrize("stock_wire", [False, True])
@pytest.mark.parametrize("client_transports,server_transports,opened_on,ends_on", [
    ("uv:1,shm:2", "uv:1,shm:2", "uv", "shm"),   # both prefer shm: the pipe moves there
    ("uv:2,shm:1", "uv:1,shm:2", "uv", "shm"),   # the server's order decides
    ("uv:1,shm:2", "uv:2,shm:1", "uv", "uv"),    # the server prefers what the pipe is on
    ("uv:1", "uv:1,shm:2", "uv", "uv"),          # the client lacks the better one
    ("uv:1,shm:2", "uv:1,shm:2", "shm", "shm"),  # already on the best
])
def test_pipe_moves_to_the_best_common_transport(stock_wire, client_transports, server_transports,
                                                 opened_on, ends_on):
    """tensorpipe/core/pipe_impl.cc:987-1042 (the server picks the transport, by its own
    priorities, among those both ends have and it listens on) and :1108-1125 (the client opens
    the pipe's connection again there): messages flow both ways afterwards, on the transport
    the rule names."""
    server = tp.Context("server", transports=server_transports, channels="basic:0", stock_wire=stock_wire)
    client = tp.Context("client", transports=client_transports, channels="basic:0", stock_wire=stock_wire)
    listener = server.listen("uv://127.0.0.1:0,shm://")
    cpipe = client.connect(listener.url(opened_on))
    spipe = listener.accept()
    try:
        rng = np.random.default_rng(11)
        for sender, receiver in ((cpipe, spipe), (spipe, cpipe), (cpipe, spipe)):
            data = rng.integers(0, 256, 3 * 1024 * 1024 + 5, dtype=np.uint8)
            outs, pouts = _roundtrip(sender, receiver, [data, data[:77].copy()], payloads=[b"payload"])
            assert (outs[0] == data).all() and (outs[1] == data[:77]).all()
            assert bytes(pouts[0]) == b"payload"
        assert cpipe.transport() == ends_on and spipe.transport() == ends_on
        assert spipe.remote_name() == "client"
    finally:
        for o in (cpipe, spipe, listener, client, server):
            o.destroy()


def test_close_fails_pending_and_future_ops(pair):
    cpipe, spipe = pair()
    # make sure the pipe is established first
    _roundtrip(cpipe, spipe, [np.arange(10, dtype=np.uint8)])
    cpipe.close()
    with pytest.raises(tp.PipeError):
        cpipe.write([tp.make_tensor(np.zeros(10, np.uint8))]).wait()
    # the peer notices the closed connection
    with pytest.raises(tp.PipeError):
        spipe.read_descriptor(timeout_ms=5000)


def test_context_close_fails_pipes(pair):
    cpipe, spipe = pair()
    _roundtrip(cpipe, spipe, [np.arange(10, dtype=np.uint8)])
    # last tuple created by the fixture holds the contexts
    with pytest.raises(tp.PipeError):
        # closing the remote context makes our reads fail
        import threading

        t = threading.Timer(0.2, lambda: spipe.close())
        t.start()
        cpipe.read_descriptor(timeout_ms=5000)


def test_peer_process_dies_mid_message():
    # the other process disappears (no close, no goodbye) after it has seen a descriptor and before
    # it has read the tensor: what is pending here fails, later operations fail too, nothing hangs
    import multiprocessing as mp

    from tests import peer_process

    ctx = tp.Context("main", channels="basic:0")
    listener = ctx.listen()
    spawn = mp.get_context("spawn")
    ready, errors = spawn.Event(), spawn.Queue()
    proc = spawn.Process(target=peer_process.echo_peer,
                         args=(listener.url(), "basic:0", {}, ready, errors))
    proc.start()
    try:
        assert ready.wait(120), "peer did not start"
        pipe = listener.accept(60000)
        a = np.arange(100000, dtype=np.uint8)
        w = pipe.write([tp.make_tensor(a)], metadata="cpu")
        d = pipe.read_descriptor(60000)
        out = np.zeros(d.tensor_lengths[0], np.uint8)
        pipe.read([tp.make_tensor(out)], []).wait(60000)
        w.wait(60000)
        assert (out == a).all()
        big = np.zeros(8 << 20, np.uint8)  # larger than the transport's ring: cannot complete alone
        w = pipe.write([tp.make_tensor(big)], metadata="die")
        with pytest.raises(tp.PipeError) as failed:
            pipe.read_descriptor(timeout_ms=20000)
        assert "timed out" not in str(failed.value)  # an error was delivered, not a time-out
        with pytest.raises(tp.PipeError) as failed:
            w.wait(20000)
        assert "timed out" not in str(failed.value)
        with pytest.raises(tp.PipeError) as failed:
            pipe.write([tp.make_tensor(a)], metadata="cpu").wait(20000)
        assert "timed out" not in str(failed.value)
        proc.join(30)
        assert proc.exitcode == 3
    finally:
        if proc.is_alive():
            proc.kill()
        pipe.destroy()
        listener.destroy()
        ctx.destroy()


def test_contexts_come_and_go_without_leaking_descriptors_or_threads():
    # every context brings a reactor thread, sockets, an epoll set and ring segments:
    # all of it must be gone after destroy()
    import os
    import threading

    def one_round(k):
        server = tp.Context("server", channels="xth:5,basic:0")
        client = tp.Context("client", channels="xth:5,basic:0")
        listener = server.listen()
        cpipe = client.connect(listener.url())
        spipe = listener.accept()
        outs, _ = _roundtrip(cpipe, spipe, [np.full(70000 + k, k % 251, np.uint8)])
        assert (outs[0] == k % 251).all()
        for o in (cpipe, spipe, listener, client, server):
            o.destroy()

    one_round(0)
    fds_before = len(os.listdir("/proc/self/fd"))
    threads_before = len(os.listdir("/proc/self/task"))
    for k in range(1, 40):
        one_round(k)
    assert len(os.listdir("/proc/self/fd")) <= fds_before
    assert len(os.listdir("/proc/self/task")) <= threads_before
    assert threading.active_count() >= 1


def test_idle_contexts_do_not_spin(pair):
    # the reactor threads busy-poll only while traffic flows (a 200 us window); an open, idle pipe
    # costs no CPU
    import resource
    import time

    cpipe, spipe = pair()
    _roundtrip(cpipe, spipe, [np.arange(1000, dtype=np.uint8)])
    time.sleep(0.2)
    before = resource.getrusage(resource.RUSAGE_SELF)
    time.sleep(1.0)
    after = resource.getrusage(resource.RUSAGE_SELF)
    used = (after.ru_utime - before.ru_utime) + (after.ru_stime - before.ru_stime)
    assert used < 0.2, f"{used:.3f} CPU seconds in one idle second"
    # and it still works afterwards (the threads wake up)
    outs, _ = _roundtrip(cpipe, spipe, [np.arange(77, dtype=np.uint8)])
    assert (outs[0] == np.arange(77, dtype=np.uint8)).all()


def test_unknown_channel_and_missing_gpu():
    with pytest.raises(tp.PipeError):
        tp.Context("x", channels="nope:0")
    # Without a GPU the HIP channels are not viable and are skipped, like a
    # reference context skips a non-viable channel (core/context_impl.cc:89-110).
    import torch

    ctx = tp.Context("y", channels="basic:0,hip_xth:10,hip_ipc:11,hip_basic:12")
    assert ctx.has_channel("basic")
    if not torch.cuda.is_available():
        assert not ctx.has_channel("hip_xth")
        assert not ctx.has_channel("hip_ipc")
        assert not ctx.has_channel("hip_basic")
    ctx.destroy()
