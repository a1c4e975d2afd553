"""The three HIP channels driven through Pipe::write/read, checked against the
CPU oracle's restatement of the corresponding reference channel. Cases follow
tensorpipe/test/channel/channel_test.cc, channel_test_cuda.cc and
channel_test_cuda_xdtt.cc."""
import multiprocessing as mp
import os

import numpy as np
import pytest

from tensorpipe_amd import _native, datagen
from tensorpipe_amd import pipe as tp

pytestmark = pytest.mark.gpu

FILL = 0xEE


def _gpu(arr):
    import torch

    return torch.from_numpy(np.ascontiguousarray(arr)).cuda()


# ---------------------------------------------------------------------------
# hip_xth: two pipes in this process
# ---------------------------------------------------------------------------

@pytest.fixture(scope="module")
def xth_pair():
    server = tp.Context("server", channels="basic:0,hip_xth:10")
    client = tp.Context("client", channels="basic:0,hip_xth:10")
    assert server.has_channel("hip_xth"), "hip_xth must be viable on a GPU box"
    listener = server.listen()
    cpipe = client.connect(listener.url())
    spipe = listener.accept()
    yield cpipe, spipe
    cpipe.destroy()
    spipe.destroy()
    listener.destroy()
    client.destroy()
    server.destroy()


def _xth_send(oracle, sender, receiver, host_arrays, with_target, offsets=None):
    """Send GPU copies of host_arrays; compare what arrives with the oracle's copy."""
    import torch

    srcs = [_gpu(a) if a.size else torch.empty(1, dtype=torch.uint8, device="cuda")
            for a in host_arrays]
    target = (tp.HIP, 0) if with_target else None
    tensors = [tp.make_tensor(s, nbytes=a.size, target=target) for s, a in zip(srcs, host_arrays)]
    w = sender.write(tensors, payloads=[b"payload #0"], metadata="m")
    d = receiver.read_descriptor()
    assert d.num_tensors == len(host_arrays)
    pad = 32
    dsts = [torch.full((int(d.tensor_lengths[i]) + 2 * pad,), FILL, dtype=torch.uint8, device="cuda")
            for i in range(d.num_tensors)]
    pout = np.zeros(int(d.payload_lengths[0]), np.uint8)
    rt = [tp.make_tensor(dsts[i].data_ptr() + pad, nbytes=int(d.tensor_lengths[i]), device=tp.HIP)
          for i in range(d.num_tensors)]
    r = receiver.read(rt, [pout])
    r.wait()
    w.wait()
    torch.cuda.synchronize()
    assert bytes(pout) == b"payload #0"
    # oracle: the same message through the CPU restatement of cuda_xth
    refs = [np.full(a.size + 2 * pad, FILL, np.uint8) for a in host_arrays]
    oracle.xth_message([(a, ref[pad:], a.size) for a, ref in zip(host_arrays, refs)])
    for dst, ref in zip(dsts, refs):
        assert (dst.cpu().numpy() == ref).all()


@pytest.mark.parametrize("with_target", [True, False])
def test_xth_client_to_server_and_back(oracle, xth_pair, with_target):
    cpipe, spipe = xth_pair
    iota = np.arange(256, dtype=np.uint8)
    _xth_send(oracle, cpipe, spipe, [iota], with_target)
    _xth_send(oracle, spipe, cpipe, [iota], with_target)


def test_xth_send_multiple_tensors(oracle, xth_pair):
    cpipe, spipe = xth_pair
    n = 256 * 1024
    src = (np.arange(n) % 256).astype(np.uint8)
    _xth_send(oracle, cpipe, spipe, [src] * 100, True)


def test_xth_empty_and_nonempty(oracle, xth_pair):
    cpipe, spipe = xth_pair
    a, z, b = np.array([7], np.uint8), np.zeros(0, np.uint8), np.array([9], np.uint8)
    _xth_send(oracle, cpipe, spipe, [a, z, b], True)
    _xth_send(oracle, cpipe, spipe, [z], True)


def test_xth_rpc_message(oracle, xth_pair):
    # 256 fp16 tensors, log-uniform sizes, N(0, 0.02): the many-tensor message
    cpipe, spipe = xth_pair
    sizes = datagen.loguniform_sizes(datagen.SEED_BASE + 5, 256, 4 << 20, 256)
    arrays = [datagen.normal(1000 + i, int(s) // 2, "f16", sigma=0.02).view(np.uint8)
              for i, s in enumerate(sizes)]
    _xth_send(oracle, cpipe, spipe, arrays, True)


def test_xth_64mib(oracle, xth_pair):
    cpipe, spipe = xth_pair
    _xth_send(oracle, cpipe, spipe, [datagen.uniform_u8(datagen.SEED_BASE + 2, 64 << 20)], True)


def test_xth_both_ways_concurrently(oracle, xth_pair):
    import torch

    cpipe, spipe = xth_pair
    a = _gpu(np.full(300000, 1, np.uint8))
    b = _gpu(np.full(200000, 2, np.uint8))
    w1 = cpipe.write([tp.make_tensor(a, target=(tp.HIP, 0))])
    w2 = spipe.write([tp.make_tensor(b, target=(tp.HIP, 0))])
    d1, d2 = spipe.read_descriptor(), cpipe.read_descriptor()
    o1 = torch.zeros(int(d1.tensor_lengths[0]), dtype=torch.uint8, device="cuda")
    o2 = torch.zeros(int(d2.tensor_lengths[0]), dtype=torch.uint8, device="cuda")
    ops = [spipe.read([tp.make_tensor(o1)]), cpipe.read([tp.make_tensor(o2)]), w1, w2]
    for op in ops:
        op.wait()
    torch.cuda.synchronize()
    assert (o1 == 1).all().item() and (o2 == 2).all().item()


def test_xth_receiver_waits_for_start_event(xth_pair):
    # channel_test_cuda.cc:19-94: slow kernel, then fill 0x42 on the sender's
    # stream; the receiver must see only 0x42.
    import torch

    cpipe, spipe = xth_pair
    lib = _native.tphip()
    n = 1024
    src = torch.zeros(n, dtype=torch.uint8, device="cuda")
    send_stream, recv_stream = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    _native.check(lib.tphip_test_slow_kernel(0, src.data_ptr(), n, send_stream.cuda_stream))
    _native.check(lib.tphip_fill(0, src.data_ptr(), 0x42, n, send_stream.cuda_stream))
    w = cpipe.write([tp.make_tensor(src, stream=send_stream, target=(tp.HIP, 0))])
    spipe.read_descriptor()
    dst = torch.zeros(n, dtype=torch.uint8, device="cuda")
    torch.cuda.current_stream().synchronize()
    r = spipe.read([tp.make_tensor(dst, stream=recv_stream)])
    r.wait()
    w.wait()
    recv_stream.synchronize()
    assert (dst.cpu().numpy() == 0x42).all()


def test_xth_send_offset_allocation(oracle, xth_pair):
    # channel_test_cuda.cc:96-139: 256 B of 0x42 from base+128 of a 384 B allocation
    import torch

    cpipe, spipe = xth_pair
    alloc = torch.full((384,), 0xFF, dtype=torch.uint8, device="cuda")
    alloc[128:] = 0x42
    w = cpipe.write([tp.make_tensor(alloc.data_ptr() + 128, nbytes=256, device=tp.HIP,
                                    target=(tp.HIP, 0))])
    spipe.read_descriptor()
    dst = torch.full((256 + 64,), FILL, dtype=torch.uint8, device="cuda")
    spipe.read([tp.make_tensor(dst.data_ptr() + 32, nbytes=256, device=tp.HIP)]).wait()
    w.wait()
    torch.cuda.synchronize()
    got = dst.cpu().numpy()
    assert (got[32:288] == 0x42).all() and (got[:32] == FILL).all() and (got[288:] == FILL).all()


# ---------------------------------------------------------------------------
# hip_ipc and hip_basic: echo peer in a second process
# ---------------------------------------------------------------------------

class Peer:
    def __init__(self, channels, env=None):
        from tests import peer_process

        self.mp = mp.get_context("spawn")
        self.ctx = tp.Context("main", channels=channels)
        self.listener = self.ctx.listen()
        self.ready = self.mp.Event()
        self.errors = self.mp.Queue()
        self.proc = self.mp.Process(
            target=peer_process.echo_peer,
            args=(self.listener.url(), channels, env or {}, self.ready, self.errors))
        self.proc.start()
        assert self.ready.wait(120), "peer did not start"
        self._check()
        self.pipe = self.listener.accept(60000)

    def _check(self):
        if not self.errors.empty():
            raise AssertionError("peer failed:\n" + self.errors.get())

    def echo(self, tensors, metadata, payloads=()):
        """Send tensors, receive the echo into fresh buffers; returns (gpu/cpu buffers, payloads)."""
        import torch

        w = self.pipe.write(tensors, payloads=list(payloads), metadata=metadata)
        d = self.pipe.read_descriptor(60000)
        self._check()
        outs, rts = [], []
        for i, t in enumerate(tensors):
            n = int(d.tensor_lengths[i])
            assert n == t.length
            if t.device_type == tp.HIP:
                o = torch.full((max(n, 1) + 64,), FILL, dtype=torch.uint8, device="cuda")
                rts.append(tp.make_tensor(o.data_ptr() + 32, nbytes=n, device=tp.HIP))
            else:
                o = np.full(n + 64, FILL, np.uint8)
                rts.append(tp.make_tensor(o.ctypes.data + 32, nbytes=n, device=tp.CPU))
            outs.append(o)
        pouts = [np.zeros(int(d.payload_lengths[i]), np.uint8) for i in range(d.num_payloads)]
        r = self.pipe.read(rts, pouts)
        r.wait(60000)
        w.wait(60000)
        torch.cuda.synchronize()
        return outs, pouts

    def close(self):
        try:
            try:
                self.pipe.write([], metadata="quit").wait(10000)
            except tp.PipeError:
                # the peer may read the message and exit before this side's write callback has
                # run; a pipe whose peer is gone fails what is still pending, as the reference's does
                pass
            self.proc.join(30)
        finally:
            if self.proc.is_alive():
                self.proc.kill()
            self.pipe.destroy()
            self.listener.destroy()
            self.ctx.destroy()
        self._check()
        assert self.proc.exitcode == 0, f"peer exited with {self.proc.exitcode}"


def _check_echo(out, host, length):
    got = out.cpu().numpy() if hasattr(out, "cpu") else out
    assert (got[32:32 + length] == host[:length]).all(), "payload bytes differ"
    assert (got[:32] == FILL).all() and (got[32 + length:32 + length + 32] == FILL).all()


@pytest.fixture(scope="module")
def ipc_peer():
    peer = Peer("basic:0,hip_ipc:11")
    assert peer.ctx.has_channel("hip_ipc")
    yield peer
    peer.close()


@pytest.fixture(scope="module")
def ipc_outbox_peer():
    # the reference's staging geometry (4 slots of 8 MiB), so that the sizes below cross slot
    # boundaries and reuse slots
    env = {"TP_HIP_IPC_MODE": "outbox", "TP_HIP_IPC_SLOT_BYTES": str(8 << 20), "TP_HIP_IPC_NUM_SLOTS": "4"}
    os.environ.update(env)
    try:
        peer = Peer("basic:0,hip_ipc:11", env=env)
    finally:
        for k in env:
            del os.environ[k]
    yield peer
    peer.close()


@pytest.fixture(scope="module")
def ipc_outbox_default_peer():
    # default geometry on this side, a small odd one on the peer's: each receiver follows the
    # geometry the sender announced
    os.environ["TP_HIP_IPC_MODE"] = "outbox"
    try:
        peer = Peer("basic:0,hip_ipc:11", env={"TP_HIP_IPC_MODE": "outbox",
                                               "TP_HIP_IPC_SLOT_BYTES": str((1 << 20) + 48),
                                               "TP_HIP_IPC_NUM_SLOTS": "3"})
    finally:
        del os.environ["TP_HIP_IPC_MODE"]
    yield peer
    peer.close()


@pytest.fixture(scope="module")
def basic_peer():
    peer = Peer("basic:0,hip_basic:10")
    assert peer.ctx.has_channel("hip_basic")
    yield peer
    peer.close()


@pytest.fixture(scope="module")
def basic_inner_peer():
    # the reference's route for every chunk: through the wrapped CPU channel
    os.environ["TP_HIP_BASIC_NO_SHARED_RING"] = "1"
    try:
        peer = Peer("basic:0,hip_basic:10", env={"TP_HIP_BASIC_NO_SHARED_RING": "1"})
    finally:
        del os.environ["TP_HIP_BASIC_NO_SHARED_RING"]
    yield peer
    peer.close()


@pytest.fixture(scope="module")
def basic_small_ring_peer():
    # 4-deep ring of 64 KiB slots: many chunks per tensor, constant slot reuse
    env = {"TP_HIP_BASIC_SLOT_BYTES": str(64 << 10), "TP_HIP_BASIC_NUM_SLOTS": "4"}
    os.environ.update(env)
    try:
        peer = Peer("basic:0,hip_basic:10", env=env)
    finally:
        for k in env:
            del os.environ[k]
    yield peer
    peer.close()


@pytest.fixture(scope="module")
def basic_mixed_ring_peer():
    # the default ring on this side (16 x 1 MiB), 3 slots of 256 KiB + 48 B on the peer's: the two
    # ends agree on the smaller slot as chunk size, and each ring keeps its own depth
    peer = Peer("basic:0,hip_basic:10", env={"TP_HIP_BASIC_SLOT_BYTES": str((256 << 10) + 48),
                                             "TP_HIP_BASIC_NUM_SLOTS": "3"})
    yield peer
    peer.close()


def _ipc_cases(oracle, peer, slot, sizes):
    for k, n in enumerate(sizes):
        host = datagen.normal(datagen.SEED_BASE + 3 + k, max(n // 4, 1), "f32").view(np.uint8)
        if n % 4 or n < 4:
            host = datagen.uniform_u8(k, max(n, 1))
        src = _gpu(host)
        outs, _ = peer.echo([tp.make_tensor(src, nbytes=n, target=(tp.HIP, 0))], "gpu")
        # oracle: cuda_ipc moves the tensor chunk by chunk through the outbox
        ref = np.full(n, FILL, np.uint8)
        oracle.ipc_tensor(host, ref, n, slot=slot, num_slots=4, in_flight=4)
        _check_echo(outs[0], ref, n)


def test_ipc_direct_sizes(oracle, ipc_peer):
    _ipc_cases(oracle, ipc_peer, 8 << 20,
               [256, 4096, 16384, 65536, 1 << 20, (8 << 20) + 4, 64 << 20, 1, 17, 0])


def test_ipc_sweep_points_between_the_others(oracle, ipc_peer):
    # the sizes of the benchmark's sweep (4 KiB * 4^k) that the case above leaves out
    _ipc_cases(oracle, ipc_peer, 8 << 20, [256 << 10, 4 << 20, 16 << 20])


def test_ipc_at_the_boundary_between_copy_agent_and_launched_copy(oracle, ipc_peer):
    """A unit of at most 128 KiB and 16 tensors is copied by the receiver's resident agent and
    acknowledged by a signal word, anything larger by a launched kernel and a message: both sides
    of both limits, every tensor against the oracle's per-tensor transfer."""
    limit = 128 << 10
    _ipc_cases(oracle, ipc_peer, 8 << 20, [limit - 1, limit, limit + 1, limit + 16])
    for count in (16, 17):
        for each in (limit // count, limit // count + 1):  # in all just inside / just outside the byte limit
            hosts = [datagen.uniform_u8(900 + 31 * count + i, each) for i in range(count)]
            srcs = [_gpu(h) for h in hosts]
            outs, _ = ipc_peer.echo([tp.make_tensor(s, nbytes=each, target=(tp.HIP, 0)) for s in srcs], "gpu")
            for o, h in zip(outs, hosts):
                ref = np.full(each, FILL, np.uint8)
                oracle.ipc_tensor(h, ref, each, slot=8 << 20, num_slots=4, in_flight=4)
                _check_echo(o, ref, each)


def test_ipc_direct_many_tensors_and_offsets(oracle, ipc_peer):
    import torch

    sizes = [int(s) for s in datagen.loguniform_sizes(9, 64, 1 << 20, 48)]
    host = [datagen.uniform_u8(50 + i, s) for i, s in enumerate(sizes)]
    arena = torch.empty(sum(sizes) + 16 * len(sizes) + 128, dtype=torch.uint8, device="cuda")
    tensors, off = [], 128  # nothing starts at the allocation base
    for h in host:
        arena[off:off + h.size] = torch.from_numpy(h).cuda()
        tensors.append(tp.make_tensor(arena.data_ptr() + off, nbytes=h.size, device=tp.HIP,
                                      target=(tp.HIP, 0)))
        off += h.size + 3
    outs, pouts = ipc_peer.echo(tensors, "gpu", payloads=[b"x" * 4096])
    assert bytes(pouts[0]) == b"x" * 4096
    for o, h in zip(outs, host):
        _check_echo(o, h, h.size)


def test_ipc_outbox_sizes(oracle, ipc_outbox_peer):
    # multi-chunk (> 8 MiB) and slot reuse (> 4 chunks in flight) included
    _ipc_cases(oracle, ipc_outbox_peer, 8 << 20,
               [256, 1 << 20, (8 << 20) - 1, 8 << 20, (8 << 20) + 1, (40 << 20) + 7, 0])


def test_ipc_outbox_mixed_geometries(oracle, ipc_outbox_default_peer):
    # 32 MiB slots this way, 1 MiB + 48 B slots (three of them) on the way back
    _ipc_cases(oracle, ipc_outbox_default_peer, 32 << 20,
               [4096, (1 << 20) + 48, (1 << 20) + 49, (32 << 20) + 5, (70 << 20) + 1, 0])


def test_ipc_refuses_same_process():
    # cuda_ipc_test.cc:37-57: two contexts of one process cannot use the channel;
    # the pipe falls back to the next channel (none for GPU here), so a GPU send fails.
    import torch

    server = tp.Context("s", channels="basic:0,hip_ipc:11")
    client = tp.Context("c", channels="basic:0,hip_ipc:11")
    listener = server.listen()
    cpipe = client.connect(listener.url())
    spipe = listener.accept()
    src = torch.zeros(16, dtype=torch.uint8, device="cuda")
    with pytest.raises(tp.PipeError, match="no channel"):
        cpipe.write([tp.make_tensor(src, target=(tp.HIP, 0))]).wait()
    for o in (cpipe, spipe, listener, client, server):
        o.destroy()


def _staged_cases(oracle, peer, sizes, slot=1 << 20, num_slots=16):
    for k, n in enumerate(sizes):
        host = datagen.normal(datagen.SEED_BASE + 4 + k, max((n + 1) // 2, 1), "bf16").view(np.uint8)
        src = _gpu(host)
        outs, _ = peer.echo([tp.make_tensor(src, nbytes=n, target=(tp.HIP, 0))], "gpu")
        ref = np.full(n, FILL, np.uint8)
        oracle.staged_tensor(host, ref, n, slot=slot, num_slots=num_slots)
        _check_echo(outs[0], ref, n)


def test_basic_staged_sizes(oracle, basic_peer):
    _staged_cases(oracle, basic_peer, [1024, 1 << 20, (1 << 20) + 1, (5 << 20) + 3, 40 << 20, 1, 0])


def test_basic_staged_inner_route(oracle, basic_inner_peer):
    _staged_cases(oracle, basic_inner_peer, [1024, (1 << 20) + 1, (20 << 20) + 3, 1, 0])


def test_basic_staged_small_ring(oracle, basic_small_ring_peer):
    _staged_cases(oracle, basic_small_ring_peer, [1024, (64 << 10) + 1, (3 << 20) + 5, 17],
                  slot=64 << 10, num_slots=4)
    # several tensors in one message share the 4 slots
    hosts = [datagen.uniform_u8(200 + i, (300 << 10) + i) for i in range(5)]
    srcs = [_gpu(h) for h in hosts]  # must stay alive until the echo is back
    outs, _ = basic_small_ring_peer.echo(
        [tp.make_tensor(s, target=(tp.HIP, 0)) for s in srcs], "gpu")
    for o, h in zip(outs, hosts):
        _check_echo(o, h, h.size)


def test_basic_staged_mixed_geometries(oracle, basic_mixed_ring_peer):
    chunk = (256 << 10) + 48
    _staged_cases(oracle, basic_mixed_ring_peer, [1024, chunk, chunk + 1, (3 << 20) + 7, 0],
                  slot=chunk, num_slots=3)


def test_basic_cross_device_types(oracle, basic_peer):
    # channel_test_cuda_xdtt.cc: CPU -> GPU and GPU -> CPU, 1024 bytes of 0x42
    host = np.full(1024, 0x42, np.uint8)
    outs, _ = basic_peer.echo([tp.make_tensor(host, target=(tp.HIP, 0))], "gpu")
    _check_echo(outs[0], host, 1024)  # CPU -> GPU there, GPU -> CPU back
    src = _gpu(host)
    outs, _ = basic_peer.echo([tp.make_tensor(src, target=(tp.CPU, 0))], "cpu")
    _check_echo(outs[0], host, 1024)  # GPU -> CPU there, CPU -> GPU back
    big = datagen.uniform_u8(77, (3 << 20) + 5)
    big_gpu = _gpu(big)
    outs, _ = basic_peer.echo([tp.make_tensor(big_gpu, target=(tp.CPU, 0)),
                               tp.make_tensor(big, target=(tp.HIP, 0))], "cpu,gpu")
    _check_echo(outs[0], big, big.size)
    _check_echo(outs[1], big, big.size)


def test_basic_refuses_cpu_to_cpu():
    # cuda_basic_test.cc:40-62
    ctx = tp.Context("only_staged", channels="hip_basic:10")
    other = tp.Context("other", channels="hip_basic:10")
    listener = ctx.listen()
    cpipe = other.connect(listener.url())
    spipe = listener.accept()
    a = np.zeros(16, np.uint8)
    with pytest.raises(tp.PipeError, match="no channel"):
        cpipe.write([tp.make_tensor(a, target=(tp.CPU, 0))]).wait()
    for o in (cpipe, spipe, listener, other, ctx):
        o.destroy()


def test_contexts_come_and_go_without_leaking_device_memory():
    # contexts with every HIP channel, pipes and transfers, created and destroyed over and over:
    # device memory in use must not grow (staging slabs, events and mappings are given back)
    import torch

    def one_round(k, peer_rounds):
        server = tp.Context("server", channels="basic:0,hip_xth:10,hip_ipc:11,hip_basic:12")
        client = tp.Context("client", channels="basic:0,hip_xth:10,hip_ipc:11,hip_basic:12")
        listener = server.listen()
        cpipe = client.connect(listener.url())
        spipe = listener.accept()
        src = torch.full((1 << 20,), k % 251, dtype=torch.uint8, device="cuda")
        dst = torch.zeros_like(src)
        w = cpipe.write([tp.make_tensor(src, target=(tp.HIP, 0))])
        spipe.read_descriptor()
        spipe.read([tp.make_tensor(dst)]).wait()
        w.wait()
        torch.cuda.synchronize()
        assert torch.equal(src, dst)
        for o in (cpipe, spipe, listener, client, server):
            o.destroy()
        if peer_rounds:
            # a second process, every tensor through the staging slab of hip_ipc
            env = {"TP_HIP_IPC_MODE": "outbox"}
            os.environ.update(env)
            try:
                peer = Peer("basic:0,hip_ipc:11,hip_basic:10", env=env)
            finally:
                del os.environ["TP_HIP_IPC_MODE"]
            host = datagen.uniform_u8(k, (3 << 20) + 1)
            keep = _gpu(host)
            outs, _ = peer.echo([tp.make_tensor(keep, target=(tp.HIP, 0))], "gpu")
            _check_echo(outs[0], host, host.size)
            outs, _ = peer.echo([tp.make_tensor(host, target=(tp.HIP, 0))], "gpu")  # hip_basic
            _check_echo(outs[0], host, host.size)
            peer.close()

    one_round(0, True)  # first use creates what lives as long as the process (copy plan ring)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    free_before, _ = torch.cuda.mem_get_info()
    for k in range(1, 25):
        one_round(k, k % 8 == 0)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_before - free_after < (32 << 20), (free_before, free_after)


def test_ipc_peer_mappings_do_not_pin_freed_memory():
    # sixty tensors, each out of its own 64 MiB allocation; all sixty stay alive until the last echo
    # is back (so that every one has an address of its own) and are freed together. The peer has
    # mapped every one of them; with a limit on what it keeps mapped (256 MiB here) the freed
    # memory goes back to the device instead of staying alive through the peer's mappings.
    import ctypes

    import torch

    lib = _native.tphip()
    peer = Peer("basic:0,hip_ipc:11", env={"TP_HIP_IPC_MAX_MAPPED_BYTES": str(256 << 20)})
    held = []
    try:
        n = 64 << 20
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        free_before, _ = torch.cuda.mem_get_info()
        for k in range(60):
            p = ctypes.c_void_p()
            _native.check(lib.tphip_malloc(0, n, ctypes.byref(p)))
            held.append(p)
            _native.check(lib.tphip_fill(0, p, k + 1, n, None))
            _native.check(lib.tphip_stream_sync(0, None))
            outs, _ = peer.echo([tp.make_tensor(p.value, nbytes=n, device=tp.HIP, target=(tp.HIP, 0))], "gpu")
            assert int(outs[0][32]) == k + 1 and int(outs[0][32 + n - 1]) == k + 1
            del outs
        while held:
            _native.check(lib.tphip_free(0, held.pop()))
        torch.cuda.empty_cache()
        free_after, _ = torch.cuda.mem_get_info()
        # without the limit the peer would still hold 60 x 64 MiB = 3.75 GiB of what was just freed
        assert free_before - free_after < (1 << 30), (free_before, free_after)
    finally:
        while held:
            lib.tphip_free(0, held.pop())
        peer.close()


def test_ipc_one_message_out_of_many_allocations(ipc_peer):
    # 1100 tensors in one message, each out of an allocation of its own: more allocations than the
    # sender's export table holds before it looks for freed ones (1024) and more than a receiving
    # channel keeps mapped (1024); the message names every one of them
    import ctypes

    import torch

    lib = _native.tphip()
    count, n = 1100, 4096
    held = []
    try:
        for k in range(count):
            p = ctypes.c_void_p()
            _native.check(lib.tphip_malloc(0, n, ctypes.byref(p)))
            held.append(p)
            _native.check(lib.tphip_fill(0, p, k % 251 + 1, n, None))
        _native.check(lib.tphip_stream_sync(0, None))
        tensors = [tp.make_tensor(p.value + 16 * (k % 3), nbytes=n - 64, device=tp.HIP, target=(tp.HIP, 0))
                   for k, p in enumerate(held)]
        outs, _ = ipc_peer.echo(tensors, "gpu")
        torch.cuda.synchronize()
        for k, o in enumerate(outs):
            got = o.cpu().numpy()
            assert (got[32:32 + n - 64] == k % 251 + 1).all(), k
            assert (got[:32] == FILL).all() and (got[32 + n - 64:] == FILL).all(), k
        # and again, now that the peer has dropped some of the mappings
        outs, _ = ipc_peer.echo(tensors[:40], "gpu")
        for k, o in enumerate(outs):
            assert (o.cpu().numpy()[32:32 + n - 64] == k % 251 + 1).all(), k
    finally:
        while held:
            lib.tphip_free(0, held.pop())


# ---------------------------------------------------------------------------
# The benchmark's own shapes at full size: same channels, geometries and tensor sizes as
# bench.py's cross-process legs. The source is seeded over its whole length with no two blocks
# alike (a chunk delivered from the wrong offset cannot compare equal); at these sizes the echo
# is compared with the source on the device, and a 1 MiB sample at each end and in the middle
# with the CPU oracle's result for the same chunking.
# ---------------------------------------------------------------------------

def _full_size_echo(oracle, peer, nbytes, dtype, kind, slot, num_slots):
    import torch

    elem = 4 if dtype == "f32" else 2
    host = datagen.normal_large(datagen.SEED_BASE + (3 if kind == "ipc" else 4), nbytes // elem, dtype).view(np.uint8)
    src = _gpu(host)
    outs, _ = peer.echo([tp.make_tensor(src, nbytes=nbytes, target=(tp.HIP, 0))], "gpu")
    out = outs[0]
    assert bool(torch.equal(out[32:32 + nbytes], src)), "echoed bytes differ from the source"
    assert bool((out[:32] == FILL).all()) and bool((out[32 + nbytes:] == FILL).all())
    # oracle on three windows of whole chunks
    win = max(slot, 1 << 20)
    for lo in (0, (nbytes // 2) // slot * slot, nbytes - win):
        ref = np.full(win, FILL, np.uint8)
        piece = host[lo:lo + win]
        if kind == "ipc":
            oracle.ipc_tensor(piece, ref, win, slot=slot, num_slots=num_slots, in_flight=num_slots)
        else:
            oracle.staged_tensor(piece, ref, win, slot=slot, num_slots=num_slots)
        got = out[32 + lo:32 + lo + win].cpu().numpy()
        assert (got == ref).all(), f"window at {lo} differs from the oracle"
    del src, out, outs


@pytest.mark.parametrize("nbytes", [256 << 20, 1 << 30])
def test_ipc_bench_shapes_full_size(oracle, ipc_peer, nbytes):
    # configs[2]'s two largest points: fp32 N(0,1), 256 MiB and 1 GiB through hip_ipc
    _full_size_echo(oracle, ipc_peer, nbytes, "f32", "ipc", 8 << 20, 4)


@pytest.mark.parametrize("slot_mib", [1, 4])
def test_staged_bench_shapes_full_size(oracle, slot_mib):
    # configs[3]: 256 MiB bf16 N(0,1) through hip_basic with a 4-deep ring of 1 MiB and of 4 MiB slots
    env = {"TP_HIP_BASIC_SLOT_BYTES": str(slot_mib << 20), "TP_HIP_BASIC_NUM_SLOTS": "4"}
    os.environ.update(env)
    try:
        peer = Peer("basic:0,hip_basic:10", env=env)
    finally:
        for k in env:
            del os.environ[k]
    try:
        _full_size_echo(oracle, peer, 256 << 20, "bf16", "staged", slot_mib << 20, 4)
    finally:
        peer.close()
