"""The GPU-driven staging ring of the tphip C ABI (tphip_ring_push / tphip_ring_pull): a tensor
pushed through a ring of pinned host slots by one kernel and pulled out by another arrives
byte-identical to what the CPU oracle's staged transfer (tp_oracle_staged_tensor: the reference's
chunk-by-chunk walk through its pinned rings) delivers for the same bytes and geometry; a kernel
whose other side is not running gives up in time, says how far it got, and the transfer completes
when both are launched again from there."""
import ctypes

import numpy as np
import pytest

from tensorpipe_amd import _native, datagen
from tensorpipe_amd._native import RingEnd, check

pytestmark = pytest.mark.gpu

FILL = 0xEE
YIELDED = 1 << 63
HEADER = 4096
vp = ctypes.c_void_p


class Ring:
    """Both ends of one ring in this process, each with a stream of its own."""

    def __init__(self, slot, num_slots):
        import torch

        self.torch = torch
        self.lib = _native.tphip()
        self.slot, self.num_slots = slot, num_slots
        host, dev = vp(), vp()
        check(self.lib.tphip_host_alloc(0, HEADER + slot * num_slots, ctypes.byref(host), ctypes.byref(dev)))
        ctypes.memset(host.value, 0, HEADER)
        self.host, self.dev = host.value, dev.value
        self.words = (ctypes.c_uint64 * (HEADER // 8)).from_address(self.host)
        nbytes = self.lib.tphip_ring_scratch_bytes(num_slots)
        self.scratch = [torch.zeros(nbytes, dtype=torch.uint8, device="cuda") for _ in range(2)]
        self.streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        self.events = []
        for _ in range(2):
            ev = vp()
            check(self.lib.tphip_event_create(0, 0, ctypes.byref(ev)))
            self.events.append(ev)
        torch.cuda.synchronize()
        # words: 0 produced, 8 consumed, 16/24 status of push/pull, 32 abort
        self.ends = [
            RingEnd(self.dev + HEADER, slot, num_slots, self.dev, self.dev + 64, self.scratch[k].data_ptr(),
                    self.dev + 128 + 64 * k, self.dev + 256)
            for k in range(2)
        ]
        self.seq = 0

    def status(self, k):
        return int(self.words[16 + 8 * k])

    def push(self, src_ptr, nbytes, first_seq, yield_us=200000):
        check(self.lib.tphip_ring_push(0, ctypes.byref(self.ends[0]), src_ptr, nbytes, first_seq, yield_us, 0,
                                       self.streams[0].cuda_stream, self.events[0]), "tphip_ring_push")

    def pull(self, dst_ptr, nbytes, first_seq, yield_us=200000):
        check(self.lib.tphip_ring_pull(0, ctypes.byref(self.ends[1]), dst_ptr, nbytes, first_seq, yield_us, 0,
                                       self.streams[1].cuda_stream, self.events[1]), "tphip_ring_pull")

    def sync(self, k):
        check(self.lib.tphip_stream_sync(0, self.streams[k].cuda_stream))

    def transfer(self, src_ptr, dst_ptr, nbytes, yield_us=200000):
        """Both kernels, launched again from where they stopped for as long as one gave up (two
        streams of one process may share a hardware queue: then they take turns)."""
        chunks = (nbytes + self.slot - 1) // self.slot
        done = [0, 0]
        for _ in range(10000):
            if done[1] < chunks:
                off = done[1] * self.slot
                self.pull(dst_ptr + off, nbytes - off, self.seq + done[1], yield_us)
            if done[0] < chunks:
                off = done[0] * self.slot
                self.push(src_ptr + off, nbytes - off, self.seq + done[0], yield_us)
            for k in range(2):
                if done[k] < chunks:
                    self.sync(k)
                    done[k] = (self.status(k) & ~YIELDED) - self.seq
            if done == [chunks, chunks]:
                break
        assert done == [chunks, chunks], f"the transfer never completed: {done} of {chunks} chunks"
        self.seq += chunks

    def close(self):
        self.torch.cuda.synchronize()
        for ev in self.events:
            self.lib.tphip_event_destroy(0, ev)
        self.lib.tphip_host_free(self.host)


def expected(oracle, host_src, so, do, nbytes, total, slot, num_slots):
    want = np.full(total, FILL, dtype=np.uint8)
    chunks = oracle.staged_tensor(host_src[so:], want[do:], nbytes, slot=slot, num_slots=num_slots)
    assert chunks == (nbytes + slot - 1) // slot
    return want


@pytest.mark.parametrize("slot,num_slots", [(1 << 20, 16), (64 << 10, 3), (4 << 20, 4), (4096, 5)])
def test_pushed_and_pulled_tensors_match_the_oracle(oracle, slot, num_slots):
    import torch

    ring = Ring(slot, num_slots)
    try:
        # one chunk, a ragged tail, odd alignments on either side, several turns of the ring
        cases = [(slot, 0, 0), (1, 3, 5), (slot + 17, 0, 0), (slot * num_slots * 2 + 4099, 7, 1),
                 (3 * slot - 1, 16, 9), (slot * (num_slots + 1), 0, 13)]
        for k, (nbytes, so, do) in enumerate(cases):
            total = nbytes + 64
            host_src = datagen.uniform_u8(70 + k, total)
            src = torch.from_numpy(host_src).cuda()
            dst = torch.full((total,), FILL, dtype=torch.uint8, device="cuda")
            torch.cuda.synchronize()
            ring.transfer(src.data_ptr() + so, dst.data_ptr() + do, nbytes)
            want = expected(oracle, host_src, so, do, nbytes, total, slot, num_slots)
            got = dst.cpu().numpy()
            assert (got == want).all(), f"case {k}: {nbytes} bytes at +{so} -> +{do} differ from the oracle"
            assert (src.cpu().numpy() == host_src).all(), "the source changed"
    finally:
        ring.close()


def test_a_kernel_without_its_other_side_gives_up_and_the_transfer_resumes(oracle):
    import torch

    slot, num_slots = 256 << 10, 4
    ring = Ring(slot, num_slots)
    try:
        nbytes = 9 * slot + 100
        total = nbytes + 32
        host_src = datagen.uniform_u8(91, total)
        src = torch.from_numpy(host_src).cuda()
        dst = torch.full((total,), FILL, dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        # a pull with nothing in the ring: gives up, nothing written, nothing consumed
        ring.pull(dst.data_ptr(), nbytes, 0, yield_us=300)
        ring.sync(1)
        assert ring.status(1) == YIELDED | 0
        assert int(ring.words[8]) == 0 and (dst.cpu().numpy() == FILL).all()
        # a push with nobody pulling: fills the ring, then gives up
        ring.push(src.data_ptr(), nbytes, 0, yield_us=300)
        ring.sync(0)
        assert ring.status(0) == YIELDED | num_slots
        assert int(ring.words[0]) == num_slots
        # the pull alone drains what is there and gives up again
        ring.pull(dst.data_ptr(), nbytes, 0, yield_us=300)
        ring.sync(1)
        assert ring.status(1) == YIELDED | num_slots
        # ... and from there on both finish the tensor
        chunks = (nbytes + slot - 1) // slot
        off = num_slots * slot
        ring.pull(dst.data_ptr() + off, nbytes - off, num_slots)
        ring.push(src.data_ptr() + off, nbytes - off, num_slots)
        ring.seq = 0
        done = [num_slots, num_slots]
        for _ in range(1000):
            for k in range(2):
                ring.sync(k)
                done[k] = ring.status(k) & ~YIELDED
            if done == [chunks, chunks]:
                break
            o0, o1 = done[0] * slot, done[1] * slot
            if done[1] < chunks:
                ring.pull(dst.data_ptr() + o1, nbytes - o1, done[1])
            if done[0] < chunks:
                ring.push(src.data_ptr() + o0, nbytes - o0, done[0])
        assert done == [chunks, chunks]
        want = expected(oracle, host_src, 0, 0, nbytes, total, slot, num_slots)
        assert (dst.cpu().numpy() == want).all()
    finally:
        ring.close()


def test_a_raised_abort_word_ends_a_waiting_kernel():
    ring = Ring(1 << 20, 4)
    try:
        import torch

        dst = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
        ring.words[32] = 1
        ring.pull(dst.data_ptr(), 1 << 20, 0, yield_us=30_000_000)
        ring.sync(1)  # comes back long before the thirty seconds are over
        assert ring.status(1) == YIELDED | 0
        ring.words[32] = 0
    finally:
        ring.close()


def test_bad_arguments_are_refused():
    lib = _native.tphip()
    ring = Ring(1 << 20, 4)
    try:
        end = ring.ends[0]
        assert lib.tphip_ring_push(0, ctypes.byref(end), None, 16, 0, 100, 0, None, None) == -1
        assert lib.tphip_ring_push(0, ctypes.byref(end), ring.dev, 0, 0, 100, 0, None, None) == -1
        odd = RingEnd(end.slots, 1000, 4, end.produced, end.consumed, end.scratch, end.status, end.abort)
        assert lib.tphip_ring_pull(0, ctypes.byref(odd), ring.dev, 16, 0, 100, 0, None, None) == -1
    finally:
        ring.close()
