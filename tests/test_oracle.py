"""Pins the CPU oracle against the reference's own test vectors and against
facts that do not depend on the oracle's code (memcmp with the input, guard
bands, brute-force chunk sums, a hand-worked allocator trace)."""
import numpy as np
import pytest

GUARD = 64


def _guarded(n, fill=0xEE):
    buf = np.full(n + 2 * GUARD, fill, dtype=np.uint8)
    return buf, buf[GUARD:GUARD + n]


def _check_guards(buf, n, fill=0xEE):
    assert (buf[:GUARD] == fill).all() and (buf[GUARD + n:] == fill).all()


def test_iota_256(oracle):
    # test/channel/channel_test.cc:45-125: 256 bytes of std::iota
    src = np.arange(256, dtype=np.uint8)
    buf, dst = _guarded(256)
    oracle.xth_message([(src, dst, 256)])
    assert dst.tolist() == list(range(256))
    _check_guards(buf, 256)


def test_send_multiple_tensors(oracle):
    # test/channel/channel_test.cc:127-189: 100 x 256 KiB, data[i] = i % 256
    n = 256 * 1024
    src = (np.arange(n) % 256).astype(np.uint8)
    dsts = [np.zeros(n, dtype=np.uint8) for _ in range(100)]
    oracle.xth_message([(src, d, n) for d in dsts])
    for d in dsts:
        assert (d == src).all()


def test_empty_and_nonempty(oracle):
    # test/channel/channel_test.cc:262-336: lengths 1, 0, 1 and a lone 0
    a, b = np.array([7], np.uint8), np.array([9], np.uint8)
    da, dz, db = (np.full(1, 0xEE, np.uint8) for _ in range(3))
    oracle.xth_message([(a, da, 1), (a, dz, 0), (b, db, 1)])
    assert (da[0], dz[0], db[0]) == (7, 0xEE, 9)


def test_offset_allocation(oracle):
    # test/channel/channel_test_cuda.cc:96-139: send 256 B of 0x42 from base+128
    alloc = np.full(384, 0xFF, np.uint8)
    alloc[128:] = 0x42
    buf, dst = _guarded(256)
    oracle.xth_message([(alloc[128:], dst, 256)])
    assert (dst == 0x42).all()
    _check_guards(buf, 256)


@pytest.mark.parametrize("slot", [1, 7, 8, 4096])
def test_chunk_arithmetic_bruteforce(oracle, slot):
    lib = oracle.lib
    for length in list(range(0, 6 * slot + 3)) + [slot * 1000 + 1]:
        n = lib.tp_oracle_num_chunks(length, slot)
        assert n == -(-length // slot)
        lens = [lib.tp_oracle_chunk_length(length, slot, k) for k in range(n)]
        assert sum(lens) == length
        assert all(l == slot for l in lens[:-1])
        if n:
            assert 1 <= lens[-1] <= slot


def test_chunk_counts_at_baseline_sizes(oracle):
    lib = oracle.lib
    assert lib.tp_oracle_num_chunks(1 << 30, 8 << 20) == 128  # ipc, 1 GiB
    assert lib.tp_oracle_num_chunks(256 << 20, 1 << 20) == 256  # staged, 1 MiB chunks
    assert lib.tp_oracle_num_chunks(256 << 20, 4 << 20) == 64


@pytest.mark.parametrize("in_flight", [1, 2, 4])
@pytest.mark.parametrize("length", [0, 1, 4095, 4096, 4097, 4 * 4096 + 7, 9 * 4096 + 1])
def test_ipc_tensor_identity(oracle, length, in_flight):
    rng = np.random.default_rng(length + in_flight)
    src = rng.integers(0, 256, max(length, 1), dtype=np.uint8)
    keep = src.copy()
    buf, dst = _guarded(length)
    chunks = oracle.ipc_tensor(src, dst, length, slot=4096, num_slots=4, in_flight=in_flight)
    assert chunks == -(-length // 4096)
    assert (dst == src[:length]).all()
    assert (src == keep).all()
    _check_guards(buf, length)


@pytest.mark.parametrize("length", [0, 1, 1023, 1024, 1025, 16 * 1024 + 5, 40 * 1024])
def test_staged_tensor_identity(oracle, length):
    rng = np.random.default_rng(length)
    src = rng.integers(0, 256, max(length, 1), dtype=np.uint8)
    buf, dst = _guarded(length)
    chunks = oracle.staged_tensor(src, dst, length, slot=1024, num_slots=16)
    assert chunks == -(-length // 1024)
    assert (dst == src[:length]).all()
    _check_guards(buf, length)


def test_staged_xdtt_vector(oracle):
    # test/channel/channel_test_cuda_xdtt.cc: 1024 bytes of 0x42
    src = np.full(1024, 0x42, np.uint8)
    buf, dst = _guarded(1024)
    oracle.staged_tensor(src, dst, 1024)
    assert (dst == 0x42).all()
    _check_guards(buf, 1024)


@pytest.mark.parametrize("ring", [64, 4096])
@pytest.mark.parametrize("length", [1, 63, 64, 65, 1000, 5 * 4096 + 3])
def test_basic_stream_wraps(oracle, ring, length):
    rng = np.random.default_rng(ring + length)
    src = rng.integers(0, 256, length, dtype=np.uint8)
    buf, dst = _guarded(length)
    oracle.basic_stream(src, dst, length, ring_bytes=ring)
    assert (dst == src).all()
    _check_guards(buf, length)


def test_bench_pattern(oracle):
    out = np.zeros(70000, np.uint8)
    oracle.lib.tp_oracle_bench_pattern(out.ctypes.data, out.size)
    i = np.arange(out.size)
    assert (out == (((i >> 8) ^ (i & 0xFF)) & 0xFF)).all()
    assert out[0] == 0 and out[255] == 255 and out[256] == 1 and out[257] == 0


def test_percentile(oracle):
    # measurements.h:51-53: samples[size_t(f * n)] after sorting
    s = np.array([5.0, 1.0, 4.0, 2.0, 3.0])
    assert oracle.lib.tp_oracle_percentile(s.ctypes.data, 5, 0.5) == 3.0
    s = np.array([4.0, 1.0, 3.0, 2.0])
    assert oracle.lib.tp_oracle_percentile(s.ctypes.data, 4, 0.5) == 3.0
    assert oracle.lib.tp_oracle_percentile(s.ctypes.data, 4, 0.95) == 4.0


def test_allocator_trace(oracle):
    # Hand-worked: 2 slots. Requests 0,1 get slots 0,1; 2 and 3 wait; releasing
    # slot 1 serves request 2 with slot 1; releasing 0 serves 3 with slot 0;
    # request 4 waits and is failed by close.
    ev = [("a", 0), ("a", 1), ("a", 2), ("a", 3), ("r", 1), ("r", 0), ("a", 4), ("c", 0)]
    assert oracle.allocator_trace(2, ev) == [(0, 0), (1, 1), (2, 1), (3, 0), (4, -1)]
    # lowest free slot first: free 2 then 0, next request takes 0
    ev = [("a", 0), ("a", 1), ("a", 2), ("r", 2), ("r", 0), ("a", 3), ("a", 4)]
    assert oracle.allocator_trace(3, ev) == [(0, 0), (1, 1), (2, 2), (3, 0), (4, 2)]
