"""Parity of the batched multi-tensor copy kernel (through the tphip C ABI)
with the CPU oracle on the same seeded inputs: byte-identical destinations,
untouched bytes everywhere else, unchanged sources."""
import ctypes

import numpy as np
import pytest

from tensorpipe_amd import _native, datagen, hip

pytestmark = pytest.mark.gpu

FILL = 0xEE


def _run_case(oracle, layout, seed, tuned=None, arena_pad=64):
    """layout: list of (src_off, dst_off, nbytes) inside one src and one dst arena."""
    import torch

    src_size = max([s + n for s, _, n in layout] + [0]) + arena_pad
    dst_size = max([d + n for _, d, n in layout] + [0]) + arena_pad
    host_src = datagen.uniform_u8(seed, src_size)
    dev_src = torch.from_numpy(host_src).cuda()
    dev_dst = torch.full((dst_size,), FILL, dtype=torch.uint8, device="cuda")
    ref_dst = np.full(dst_size, FILL, dtype=np.uint8)

    entries = [(dev_src.data_ptr() + s, dev_dst.data_ptr() + d, n) for s, d, n in layout]
    for lo in range(0, len(entries), 4096):
        table, n = hip.make_table(entries[lo:lo + 4096])
        if tuned is None:
            hip.batched_copy_table(table, n)
        else:
            hip.batched_copy_table(table, n, unroll=tuned[0], blocks=tuned[1], nontemporal=tuned[2])
    torch.cuda.synchronize()

    oracle.xth_message([(host_src[s:], ref_dst[d:], n) for s, d, n in layout])
    got = dev_dst.cpu().numpy()
    bad = np.nonzero(got != ref_dst)[0]
    assert bad.size == 0, f"{bad.size} bytes differ, first at dst offset {bad[0]}"
    assert (dev_src.cpu().numpy() == host_src).all(), "source was modified"


def _pack(sizes, src_mis=lambda i: 0, dst_mis=lambda i: 0, gap=32):
    layout, so, do = [], 0, 0
    for i, n in enumerate(sizes):
        so = (so + 15) // 16 * 16 + src_mis(i)
        do = (do + 15) // 16 * 16 + dst_mis(i)
        layout.append((so, do, int(n)))
        so += int(n) + gap
        do += int(n) + gap
    return layout


def test_alignment_matrix(oracle):
    # every (src mod 16) x (dst mod 16) with lengths around vector and wave edges
    lengths = [0, 1, 2, 15, 16, 17, 31, 33, 63, 64, 65, 255, 256, 257, 1023, 1025, 4097]
    sizes, smis, dmis = [], [], []
    for a in range(16):
        for b in range(16):
            for n in lengths:
                sizes.append(n)
                smis.append(a)
                dmis.append(b)
    layout = _pack(sizes, lambda i: smis[i], lambda i: dmis[i])
    _run_case(oracle, layout, seed=11)


@pytest.mark.parametrize("mod64", range(0, 64, 7))
def test_length_mod_64(oracle, mod64):
    sizes = [4096 * k + mod64 for k in range(1, 40)]
    layout = _pack(sizes, lambda i: i % 16, lambda i: (i * 5) % 16)
    _run_case(oracle, layout, seed=100 + mod64)


def test_rpc_message_sizes(oracle):
    # 256 tensors, log-uniform in [256 B, 4 MiB], even byte counts (fp16 payloads)
    sizes = datagen.loguniform_sizes(datagen.SEED_BASE + 5, 256, 4 << 20, 256)
    assert all(int(s) % 2 == 0 and 256 <= int(s) <= (4 << 20) for s in sizes)
    layout = _pack(sizes, gap=0)
    _run_case(oracle, layout, seed=5)
    # same sizes, 2-byte aligned but otherwise arbitrary placement
    layout = _pack(sizes, lambda i: (i * 2) % 16, lambda i: (i * 6) % 16, gap=2)
    _run_case(oracle, layout, seed=6)


def test_many_tiny_tensors(oracle):
    rng = np.random.default_rng(7)
    sizes = rng.integers(0, 96, 4096)
    layout = _pack(sizes, lambda i: int(rng.integers(0, 16)), lambda i: int(rng.integers(0, 16)), gap=1)
    _run_case(oracle, layout, seed=7)


def test_reference_vectors(oracle):
    # 100 x 256 KiB from one source (channel_test.cc:127-189); 1, 0, 1 (:297-336);
    # 256 B from base+128 of a 384 B allocation (channel_test_cuda.cc:96-139)
    n = 256 * 1024
    layout = [(0, i * (n + 16), n) for i in range(100)]
    _run_case(oracle, layout, seed=21)
    _run_case(oracle, [(0, 0, 1), (5, 40, 0), (9, 80, 1)], seed=22)
    _run_case(oracle, [(128, 0, 256)], seed=23)
    _run_case(oracle, [(0, 0, 0)], seed=24)
    _run_case(oracle, [], seed=25)


@pytest.mark.parametrize("nbytes,soff,doff", [
    (64 << 20, 0, 0), ((64 << 20) + 3, 1, 0), ((64 << 20) - 5, 0, 7), (4096, 0, 0), (1, 3, 5),
    (15, 1, 2), (16, 0, 8), (1 << 20, 4, 4),
])
def test_single_tensor(oracle, nbytes, soff, doff):
    _run_case(oracle, [(soff, doff, nbytes)], seed=nbytes % 1000)


@pytest.mark.parametrize("unroll", [1, 2, 4, 8])
@pytest.mark.parametrize("nt", [0, 1, 2, 3])
def test_launch_shapes(oracle, unroll, nt):
    sizes = list(datagen.loguniform_sizes(77, 16, 1 << 20, 96)) + [0, 1, 5, 100000, 3 << 20]
    layout = _pack(sizes, lambda i: i % 16, lambda i: (i * 3) % 16)
    for blocks in (0, 1, 7, 300):
        _run_case(oracle, layout, seed=unroll * 10 + nt, tuned=(unroll, blocks, nt))
    _run_case(oracle, [(3, 5, (8 << 20) + 11)], seed=9, tuned=(unroll, 0, nt))
    _run_case(oracle, [(3, 5, (8 << 20) + 11)], seed=9, tuned=(unroll, 3, nt))


def test_plan_ring_reuse(oracle):
    # more launches than plan slots on one stream, all checked; 270 entries each, so that the
    # plans go through the ring (tables of up to 256 entries travel in the kernel arguments)
    for k in range(70):
        sizes = [1000 + k, 17, 4096 + k] + [64 + (i * 37 + k) % 900 for i in range(267)]
        _run_case(oracle, _pack(sizes, lambda i: (i + k) % 16, lambda i: (i * 3 + k) % 16), seed=k)


@pytest.mark.parametrize("n", [2, 3, 31, 63, 64, 65, 66, 130, 255, 256, 257, 300])
def test_inline_plan_boundary(oracle, n):
    # either side of the two sizes of table that travel in the kernel arguments (64 and 256
    # entries), default and tuned launches
    rng = np.random.default_rng(1000 + n)
    sizes = [int(x) for x in rng.integers(0, 70000, n)]
    sizes[0] = (2 << 20) + 3
    layout = _pack(sizes, lambda i: int(rng.integers(0, 16)), lambda i: int(rng.integers(0, 16)), gap=3)
    _run_case(oracle, layout, seed=n)
    for tuned in ((1, 0, 3), (2, 1, 0), (4, 5, 2), (8, 300, 1)):
        _run_case(oracle, layout, seed=n + 1, tuned=tuned)


def test_many_inline_launches_back_to_back(oracle):
    # the arguments of a launch belong to that launch alone: 200 different small tables in a row
    for k in range(200):
        sizes = [100 + k, 4096 + 3 * k, 0, 15 + k % 17]
        _run_case(oracle, _pack(sizes, lambda i: (i + k) % 16, lambda i: (i * 5 + k) % 16), seed=300 + k)


@pytest.mark.parametrize("limit", [1, 64, 1000, 70000])
def test_table_cut_into_several_launches(oracle, limit):
    # a table whose 16-byte vector total exceeds what one launch carries is cut into several
    # launches, and an entry above the limit goes to the single-entry kernel; driven here with a
    # lowered limit (the real one is just under 64 GiB) on tables with both kinds of entry
    lib = _native.tphip()
    rng = np.random.default_rng(4000 + limit)
    sizes = [int(x) for x in rng.integers(0, 40000, 90)] + [0, 15, 16 * limit, 16 * limit + 16,
                                                            16 * limit - 1, 3 << 20]
    order = rng.permutation(len(sizes))
    sizes = [sizes[i] for i in order]
    layout = _pack(sizes, lambda i: (i * 7) % 16, lambda i: (i * 3) % 16)
    _native.check(lib.tphip_test_set_table_limit(limit))
    try:
        _run_case(oracle, layout, seed=limit)
        _run_case(oracle, layout, seed=limit + 1, tuned=(2, 9, 3))
    finally:
        _native.check(lib.tphip_test_set_table_limit(0))
    assert lib.tphip_test_set_table_limit(1 << 33) == -1


def test_entry_larger_than_4GiB():
    # 64-bit byte counts in the single-entry kernel and in a table next to small entries: 5 GiB + 3
    # with unaligned ends, checked on the device
    import torch

    n = (5 << 30) + 3
    a = torch.empty((n + 16 + 7) // 8, dtype=torch.int64, device="cuda").random_().view(torch.uint8)
    b = torch.full((n + 32,), FILL, dtype=torch.uint8, device="cuda")
    hip.batched_copy([(a.data_ptr() + 1, b.data_ptr() + 7, n)])
    torch.cuda.synchronize()
    assert torch.equal(a[1:1 + n], b[7:7 + n])
    assert bool((b[:7] == FILL).all()) and bool((b[7 + n:] == FILL).all())
    b.fill_(FILL)
    small = torch.arange(1000, dtype=torch.int32, device="cuda").view(torch.uint8)
    out = torch.zeros(4000 + 8, dtype=torch.uint8, device="cuda")
    hip.batched_copy([(small, out.data_ptr() + 3, 4000), (a.data_ptr() + 1, b.data_ptr() + 7, n),
                      (small.data_ptr() + 5, out.data_ptr() + 4003, 2)])
    torch.cuda.synchronize()
    assert torch.equal(a[1:1 + n], b[7:7 + n])
    assert torch.equal(out[3:4003], small) and torch.equal(out[4003:4005], small[5:7])
    assert bool((b[:7] == FILL).all()) and bool((b[7 + n:] == FILL).all())


def test_stream_completion_callback():
    # tphip_stream_on_complete (the role of CudaLoop::addCallback, tensorpipe/common/cuda_loop.cc:86-124):
    # the function runs once, with status 0, after the work enqueued before it -- here a 64 MiB copy
    # behind a fill -- and the copied bytes are complete by then
    import threading

    import torch

    lib = _native.tphip()
    host_fn = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_int)
    lib.tphip_stream_on_complete.argtypes = [ctypes.c_int, ctypes.c_void_p, host_fn, ctypes.c_void_p]
    stream = ctypes.c_void_p()
    _native.check(lib.tphip_stream_create(0, ctypes.byref(stream)))
    n = 64 << 20
    src = torch.zeros(n, dtype=torch.uint8, device="cuda")
    dst = torch.zeros(n, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    calls, fired = [], threading.Event()

    def on_done(arg, status):
        calls.append((arg, status))
        fired.set()

    keep = host_fn(on_done)  # must outlive the call
    _native.check(lib.tphip_fill(0, src.data_ptr(), 0x5A, n, stream))
    _native.check(lib.tphip_copy(0, dst.data_ptr(), src.data_ptr(), n, stream))
    _native.check(lib.tphip_stream_on_complete(0, stream, keep, ctypes.c_void_p(1234)))
    assert fired.wait(30), "completion callback did not run"
    # read back on torch's stream: only the callback orders this after the copy
    got = dst.cpu()
    assert bool((got == 0x5A).all())
    assert calls == [(1234, 0)]
    assert lib.tphip_stream_on_complete(0, stream, host_fn(), None) == -1  # null function
    _native.check(lib.tphip_stream_sync(0, stream))
    _native.check(lib.tphip_stream_destroy(0, stream))


def test_random_tables_against_oracle(oracle):
    # randomised tables (hypothesis, fixed seed): sizes over six orders of magnitude, every alignment,
    # empty entries anywhere, random launch shapes; each compared byte for byte with the oracle
    from hypothesis import given, settings, strategies as st, seed, HealthCheck

    size = st.one_of(
        st.integers(0, 48), st.integers(49, 5000), st.integers(5001, 300000),
        st.integers(300001, 3 << 20))
    entry = st.tuples(size, st.integers(0, 15), st.integers(0, 15))
    shape = st.one_of(
        st.none(),
        st.tuples(st.sampled_from([1, 2, 4, 8]), st.sampled_from([0, 1, 3, 64, 500, 2048]),
                  st.integers(0, 3)))

    @seed(20240611)
    @settings(max_examples=150, deadline=None, derandomize=True, database=None,
              suppress_health_check=list(HealthCheck))
    @given(st.lists(entry, min_size=0, max_size=150), shape, st.integers(0, 1 << 30))
    def check(entries, tuned, data_seed):
        sizes = [e[0] for e in entries]
        layout = _pack(sizes, lambda i: entries[i][1], lambda i: entries[i][2], gap=1)
        _run_case(oracle, layout, seed=data_seed, tuned=tuned)

    check()


def test_copy_with_completion_event(oracle):
    # tphip_batched_copy_signal: the event covers everything the call enqueued, whichever kernel
    # (or none) the call ends with. The copies run on a non-blocking stream that nothing else waits
    # for, so only the event orders the read-back after them.
    import torch

    lib = _native.tphip()
    stream = ctypes.c_void_p()
    _native.check(lib.tphip_stream_create(0, ctypes.byref(stream)))
    event = ctypes.c_void_p()
    _native.check(lib.tphip_event_create(0, 0, ctypes.byref(event)))
    rng = np.random.default_rng(321)

    def run(sizes, seed, tuned=(0, 0, -1), limit=0):
        layout = _pack(sizes, lambda i: (i * 5) % 16, lambda i: (i * 9) % 16)
        src_size = max([s + n for s, _, n in layout] + [0]) + 64
        dst_size = max([d + n for _, d, n in layout] + [0]) + 64
        host_src = datagen.uniform_u8(seed, src_size)
        dev_src = torch.from_numpy(host_src).cuda()
        dev_dst = torch.full((dst_size,), FILL, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        table, n = hip.make_table([(dev_src.data_ptr() + s, dev_dst.data_ptr() + d, k)
                                   for s, d, k in layout])
        _native.check(lib.tphip_test_set_table_limit(limit))
        try:
            _native.check(lib.tphip_batched_copy_signal(0, table, n, stream, event, *tuned))
        finally:
            _native.check(lib.tphip_test_set_table_limit(0))
        _native.check(lib.tphip_event_sync(0, event))
        done = ctypes.c_int(0)
        _native.check(lib.tphip_event_query(0, event, ctypes.byref(done)))
        assert done.value == 1
        got = dev_dst.cpu().numpy()  # on torch's stream: ordered after the copies by the event alone
        ref = np.full(dst_size, FILL, dtype=np.uint8)
        oracle.xth_message([(host_src[s:], ref[d:], k) for s, d, k in layout])
        assert (got == ref).all()

    run([(96 << 20) + 5], 1)                                        # single-entry kernel
    run([int(x) for x in rng.integers(1, 3 << 20, 30)], 2)          # plan in the kernel arguments
    run([int(x) for x in rng.integers(1, 1 << 20, 200)], 3)         # plan ring: stage kernel + copy kernel
    run([int(x) for x in rng.integers(1, 1 << 20, 200)], 4, tuned=(4, 32, 3))
    run([], 5)                                                      # nothing to enqueue
    run([0, 0, 0], 6)
    run([int(x) for x in rng.integers(1, 200000, 50)] + [16 * 5000 + 16], 7, limit=5000)  # ends with a lone large entry
    run([16 * 5000 + 16] + [int(x) for x in rng.integers(1, 60000, 50)], 8, limit=5000)   # several launches
    # with launch profiling on, the event is recorded as a marker of its own
    _native.check(lib.tphip_profile_start(0, 8))
    run([(32 << 20) + 1], 9)
    launches, ms, nbytes = ctypes.c_uint32(), ctypes.c_double(), ctypes.c_uint64()
    _native.check(lib.tphip_profile_stop(0, ctypes.byref(launches), ctypes.byref(ms), ctypes.byref(nbytes)))
    assert launches.value == 1 and nbytes.value == (32 << 20) + 1
    assert lib.tphip_batched_copy_signal(0, None, 0, stream, None, 0, 0, -1) == -1
    _native.check(lib.tphip_event_destroy(0, event))
    _native.check(lib.tphip_stream_destroy(0, stream))


def test_graph_capture_and_replay(oracle):
    # launches whose plan travels in the kernel arguments can be captured; every replay must copy
    # what the sources hold at that moment. Eager work and synchronisation between the replays.
    import os

    import torch

    if os.environ.get("TPHIP_INLINE_PLANS") == "0":
        pytest.skip("plans in the kernel arguments are switched off: no table can be captured")
    lib = _native.tphip()
    rng = np.random.default_rng(77)
    sizes = [int(x) for x in rng.integers(1, 50000, 40)] + [0, 1, 15, 17, 1 << 20]
    layout = _pack(sizes, lambda i: (i * 3) % 16, lambda i: (i * 11) % 16)
    src_size = max(s + n for s, _, n in layout) + 64
    dst_size = max(d + n for _, d, n in layout) + 64
    one = (5 << 20) + 13
    src = torch.zeros(src_size, dtype=torch.uint8, device="cuda")
    dst = torch.zeros(dst_size, dtype=torch.uint8, device="cuda")
    big_src = torch.zeros(one + 16, dtype=torch.uint8, device="cuda")
    big_dst = torch.zeros(one + 16, dtype=torch.uint8, device="cuda")
    entries = [(src.data_ptr() + s, dst.data_ptr() + d, n) for s, d, n in layout]
    many = [(src.data_ptr() + i, dst.data_ptr() + i, 1) for i in range(270)]
    many_table, many_n = hip.make_table(many)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hip.batched_copy(entries)
        hip.copy(big_dst.data_ptr() + 3, big_src.data_ptr() + 1, one)
        # more entries than fit the kernel arguments: refused while capturing, nothing enqueued
        stream = torch.cuda.current_stream().cuda_stream
        assert lib.tphip_batched_copy(0, many_table, many_n, ctypes.c_void_p(stream)) == -5
    assert b"graph" in lib.tphip_strerror(-5)

    for replay in range(4):
        host_src = datagen.uniform_u8(900 + replay, src_size)
        host_big = datagen.uniform_u8(950 + replay, one + 16)
        src.copy_(torch.from_numpy(host_src))
        big_src.copy_(torch.from_numpy(host_big))
        dst.fill_(FILL)
        big_dst.fill_(FILL)
        graph.replay()
        torch.cuda.synchronize()
        ref = np.full(dst_size, FILL, dtype=np.uint8)
        oracle.xth_message([(host_src[s:], ref[d:], n) for s, d, n in layout])
        assert (dst.cpu().numpy() == ref).all(), f"replay {replay}: table copy differs"
        got = big_dst.cpu().numpy()
        assert (got[3:3 + one] == host_big[1:1 + one]).all(), f"replay {replay}: single copy differs"
        assert (got[:3] == FILL).all() and (got[3 + one:] == FILL).all()
        # eager launches between replays, through the plan ring as well
        _run_case(oracle, _pack([100 + replay] * 270), seed=replay)
    # outside capture the large table goes through as before
    _native.check(lib.tphip_batched_copy(0, many_table, many_n, None))
    torch.cuda.synchronize()
    assert torch.equal(dst[:270], src[:270])


def test_full_size_roundtrip_property():
    # 1 GiB single tensor and the ~105 MiB many-tensor message at full size:
    # checked on the device (copy twice, compare), not against the CPU oracle.
    import torch

    n = 1 << 30
    a = torch.empty(n // 8, dtype=torch.int64, device="cuda").random_()
    b = torch.zeros_like(a)
    c = torch.zeros_like(a)
    hip.copy(b, a)
    hip.copy(c, b)
    torch.cuda.synchronize()
    assert torch.equal(a, c) and torch.equal(a, b)


def test_copies_that_leave_as_several_launches():
    # From twice 256 MiB on a single copy goes out as launches of 256 MiB, the last one with the
    # remainder: odd lengths, both ends misaligned, guard bytes on either side untouched, the
    # completion event behind the last piece, and a captured copy of that size replayed.
    import torch

    lib = _native.tphip()
    for nbytes, so, do in (((512 << 20) + 4099, 3, 5), ((768 << 20) - 1, 0, 13), (512 << 20, 16, 0)):
        src = torch.empty((nbytes + 64 + 7) // 8, dtype=torch.int64, device="cuda").random_().view(torch.uint8)
        dst = torch.full((nbytes + 64,), FILL, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        stream, event = ctypes.c_void_p(), ctypes.c_void_p()
        _native.check(lib.tphip_stream_create(0, ctypes.byref(stream)))
        _native.check(lib.tphip_event_create(0, 0, ctypes.byref(event)))
        table, n = hip.make_table([(src.data_ptr() + so, dst.data_ptr() + do, nbytes)])
        _native.check(lib.tphip_batched_copy_signal(0, table, n, stream, event, 0, 0, -1))
        done = ctypes.c_int(0)
        for _ in range(2000000):
            _native.check(lib.tphip_event_query(0, event, ctypes.byref(done)))
            if done.value:
                break
        assert done.value, "the completion event behind the last piece never completed"
        # the event says the bytes are there: no further synchronisation with that stream
        assert torch.equal(dst[do:do + nbytes], src[so:so + nbytes])
        assert bool((dst[:do] == FILL).all()) and bool((dst[do + nbytes:] == FILL).all())
        _native.check(lib.tphip_event_destroy(0, event))
        _native.check(lib.tphip_stream_destroy(0, stream))
        del src, dst
        torch.cuda.empty_cache()
    nbytes = (512 << 20) + 16
    src = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hip.copy(dst, src, nbytes)
    for replay in range(2):
        src.random_(0, 256)
        dst.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(src, dst), f"replay {replay} of a captured multi-launch copy differs"


def test_pinned_host_endpoints(oracle):
    # device -> mapped pinned host -> device, the staged channel's two hops
    import torch

    n = (3 << 20) + 77
    host_src = datagen.uniform_u8(31, n)
    dev_src = torch.from_numpy(host_src).cuda()
    pinned = torch.full((n + 64,), FILL, dtype=torch.uint8).pin_memory()
    dev_dst = torch.full((n + 64,), FILL, dtype=torch.uint8, device="cuda")
    hip.batched_copy([(dev_src, pinned.data_ptr() + 5, n)])
    torch.cuda.synchronize()
    assert (pinned.numpy()[5:5 + n] == host_src).all()
    assert (pinned.numpy()[:5] == FILL).all() and (pinned.numpy()[5 + n:] == FILL).all()
    hip.batched_copy([(pinned.data_ptr() + 5, dev_dst.data_ptr() + 9, n)])
    torch.cuda.synchronize()
    got = dev_dst.cpu().numpy()
    assert (got[9:9 + n] == host_src).all()
    assert (got[:9] == FILL).all() and (got[9 + n:] == FILL).all()


def test_argument_errors():
    lib = _native.tphip()
    table = (_native.CopyDesc * 1)()
    table[0].src, table[0].dst, table[0].bytes = None, None, 16
    assert lib.tphip_batched_copy(0, table, 1, None) == -1
    big = (_native.CopyDesc * 4097)()
    assert lib.tphip_batched_copy(0, big, 4097, None) == -2
    assert lib.tphip_batched_copy(0, None, 0, None) == 0
    assert b"invalid" in lib.tphip_strerror(-1)


def test_stream_ordering_with_slow_kernel(oracle):
    # ReceiverWaitsForStartEvent (channel_test_cuda.cc:19-94) at kernel level: the
    # copy is enqueued behind a slow kernel and a fill on the same stream and must
    # observe the fill.
    import torch

    lib = _native.tphip()
    n = 1024
    src = torch.zeros(n, dtype=torch.uint8, device="cuda")
    dst = torch.zeros(n, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.Stream()
    h = stream.cuda_stream
    _native.check(lib.tphip_test_slow_kernel(0, src.data_ptr(), n, h))
    _native.check(lib.tphip_fill(0, src.data_ptr(), 0x42, n, h))
    hip.copy(dst, src, n, stream=stream)
    stream.synchronize()
    assert (dst.cpu().numpy() == 0x42).all()
