"""Loader of the CPU oracle (oracle/libtp_oracle.so). Test infrastructure only."""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class CopyDesc(ctypes.Structure):
    _fields_ = [("src", ctypes.c_void_p), ("dst", ctypes.c_void_p), ("bytes", ctypes.c_uint64)]


class AllocEvent(ctypes.Structure):
    _fields_ = [("op", ctypes.c_char), ("arg", ctypes.c_int32)]


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        vp, u32, u64 = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64
        lib.tp_oracle_xth_message.argtypes = [ctypes.POINTER(CopyDesc), u32]
        lib.tp_oracle_num_chunks.restype = u64
        lib.tp_oracle_num_chunks.argtypes = [u64, u64]
        lib.tp_oracle_chunk_length.restype = u64
        lib.tp_oracle_chunk_length.argtypes = [u64, u64, u64]
        lib.tp_oracle_ipc_tensor.restype = u64
        lib.tp_oracle_ipc_tensor.argtypes = [vp, vp, u64, vp, u64, u32, u32]
        lib.tp_oracle_staged_tensor.restype = u64
        lib.tp_oracle_staged_tensor.argtypes = [vp, vp, u64, vp, vp, u64, u32]
        lib.tp_oracle_basic_stream.argtypes = [vp, vp, u64, vp, u64]
        lib.tp_oracle_bench_pattern.argtypes = [vp, u64]
        lib.tp_oracle_percentile.restype = ctypes.c_double
        lib.tp_oracle_percentile.argtypes = [vp, u64, ctypes.c_double]
        lib.tp_oracle_allocator_trace.restype = u32
        lib.tp_oracle_allocator_trace.argtypes = [
            u32, ctypes.POINTER(AllocEvent), u32, ctypes.POINTER(ctypes.c_int32), u32]

    def xth_message(self, entries):
        """entries: list of (src ndarray u8, dst ndarray u8, nbytes); copies on the CPU."""
        table = (CopyDesc * max(len(entries), 1))()
        for i, (s, d, n) in enumerate(entries):
            table[i].src = s.ctypes.data
            table[i].dst = d.ctypes.data
            table[i].bytes = n
        self.lib.tp_oracle_xth_message(table, len(entries))

    def ipc_tensor(self, src, dst, length, slot=8 << 20, num_slots=4, in_flight=4):
        outbox = np.zeros(slot * num_slots, dtype=np.uint8)
        return self.lib.tp_oracle_ipc_tensor(
            src.ctypes.data, dst.ctypes.data, length, outbox.ctypes.data, slot, num_slots, in_flight)

    def staged_tensor(self, src, dst, length, slot=1 << 20, num_slots=16):
        sr = np.zeros(slot * num_slots, dtype=np.uint8)
        rr = np.zeros(slot * num_slots, dtype=np.uint8)
        return self.lib.tp_oracle_staged_tensor(
            src.ctypes.data, dst.ctypes.data, length, sr.ctypes.data, rr.ctypes.data, slot, num_slots)

    def basic_stream(self, src, dst, length, ring_bytes=2 << 20):
        ring = np.zeros(ring_bytes, dtype=np.uint8)
        self.lib.tp_oracle_basic_stream(
            src.ctypes.data, dst.ctypes.data, length, ring.ctypes.data, ring_bytes)

    def allocator_trace(self, num_slots, events):
        ev = (AllocEvent * len(events))()
        for i, (op, arg) in enumerate(events):
            ev[i].op = op.encode()
            ev[i].arg = arg
        out = (ctypes.c_int32 * (2 * len(events) + 2))()
        n = self.lib.tp_oracle_allocator_trace(num_slots, ev, len(events), out, len(out))
        return [(out[2 * i], out[2 * i + 1]) for i in range(n)]


def load():
    path = os.path.join(ROOT, "oracle", "libtp_oracle.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} missing: run __graft_entry__.build()")
    return Oracle(ctypes.CDLL(path))
