#!/usr/bin/env python3
"""Writes tests/golden/reference_vectors.json: the known-answer vectors that the
reference's own tests and benchmark hold for the device-channel path, re-expressed
as data (what each test sends, and therefore what must arrive), plus hand-worked
tables for the integer bookkeeping (chunking, slot allocation, percentiles).

Nothing here runs or imports the reference; every vector is spelled out from the
literal values in the cited test (relative to the root of pytorch/tensorpipe):

  channel_test.cc:45-125        256 bytes 0,1,...,255, each direction
  channel_test.cc:127-189       100 tensors of 256 KiB, byte i = i % 256
  channel_test.cc:295-336       lengths 1, 0, 1
  channel_test_cuda.cc:19-94    1024 bytes of 0x42 written behind a slow kernel
  channel_test_cuda.cc:96-139   256 bytes of 0x42 at base+128; the 128 bytes before are 0xff
  channel_test_cuda_xdtt.cc     1024 bytes of 0x42 between a CPU and a GPU endpoint
  benchmark_pipe.cc:86-91       payload byte i = (i >> 8) ^ (i & 0xff)
  measurements.h:51-53          percentile p of sorted samples = samples[floor(p * n)]
  cuda_ipc/channel_impl.cc:119-133, cuda_ipc/constants.h:22-24
                                chunks = ceil(len / slot); the last one holds the remainder
  allocator.cc:26-79            lowest free slot first; requests beyond capacity wait in FIFO order

Payloads are stored as a generator expression plus SHA-256 (and the first/last bytes),
so the file stays small; tests rebuild the bytes from the expression and check the hash.
"""
import hashlib
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def payload(kind, n, **kw):
    if kind == "iota":
        b = bytes(i % 256 for i in range(n))
    elif kind == "fill":
        b = bytes([kw["value"]]) * n
    elif kind == "bench":
        b = bytes(((i >> 8) ^ (i & 0xFF)) & 0xFF for i in range(n))
    else:
        raise ValueError(kind)
    d = {"kind": kind, "bytes": n, "sha256": hashlib.sha256(b).hexdigest(),
         "head": b[:8].hex(), "tail": b[-8:].hex()}
    d.update(kw)
    return d


def chunk_table(slot):
    rows = []
    for length in (0, 1, slot - 1, slot, slot + 1, 2 * slot, 4 * slot + 7, 10 * slot - 1):
        n = 0 if length == 0 else (length + slot - 1) // slot
        lengths = [slot] * (n - 1) + ([length - (n - 1) * slot] if n else [])
        rows.append({"length": length, "slot": slot, "chunks": n, "first": lengths[:1], "last": lengths[-1:]})
    return rows


def main():
    vectors = {
        "channel": [
            {"name": "ClientToServer / ServerToClient", "cite": "tensorpipe/test/channel/channel_test.cc:45-125",
             "tensors": [payload("iota", 256)]},
            {"name": "SendMultipleTensors", "cite": "tensorpipe/test/channel/channel_test.cc:127-189",
             "repeat": 100, "tensors": [payload("iota", 256 * 1024)]},
            {"name": "EmptyAndNonEmptyTensors", "cite": "tensorpipe/test/channel/channel_test.cc:295-336",
             "tensors": [payload("fill", 1, value=0xA1), payload("fill", 0, value=0), payload("fill", 1, value=0xC3)]},
            {"name": "ReceiverWaitsForStartEvent", "cite": "tensorpipe/test/channel/channel_test_cuda.cc:19-94",
             "tensors": [payload("fill", 1024, value=0x42)]},
            {"name": "SendOffsetAllocation", "cite": "tensorpipe/test/channel/channel_test_cuda.cc:96-139",
             "offset": 128, "guard_value": 0xFF, "tensors": [payload("fill", 256, value=0x42)]},
            {"name": "SendFromCpuToGpu / SendFromGpuToCpu",
             "cite": "tensorpipe/test/channel/channel_test_cuda_xdtt.cc:19-143",
             "tensors": [payload("fill", 1024, value=0x42)]},
        ],
        "bench_pattern": {"cite": "tensorpipe/benchmark/benchmark_pipe.cc:86-91",
                          "cases": [payload("bench", 64), payload("bench", 4096), payload("bench", 70000)]},
        "percentile": {"cite": "tensorpipe/benchmark/measurements.h:51-53",
                       "samples": [7.0, 1.0, 5.0, 3.0, 9.0, 11.0, 2.0, 8.0, 4.0, 6.0],
                       "expected": {"0.0": 1.0, "0.5": 6.0, "0.9": 11.0, "0.99": 11.0, "0.25": 3.0}},
        "chunking": {"cite": "tensorpipe/channel/cuda_ipc/channel_impl.cc:119-133",
                     "rows": chunk_table(8 << 20) + chunk_table(1 << 20) + chunk_table(4096)},
        # Hand-worked with 4 slots. ["a", k] = request k asks for a slot, ["r", s] = slot s is
        # returned, ["c", 0] = the allocator is closed. Requests 0-3 take slots 0-3; 4 and 5 wait;
        # returning 2 serves request 4 with slot 2, returning 0 serves 5 with slot 0; 6 waits and gets
        # slot 1 when it comes back; 3 comes back unclaimed and request 7 takes it; 0 and 2 come back,
        # request 8 takes the lowest (0), 9 takes 2; 10 waits and is failed (-1) by the close.
        "allocator": {"cite": "tensorpipe/common/allocator.cc:26-79", "slots": 4,
                      "events": [["a", 0], ["a", 1], ["a", 2], ["a", 3], ["a", 4], ["a", 5], ["r", 2], ["r", 0],
                                 ["a", 6], ["r", 1], ["r", 3], ["a", 7], ["r", 0], ["r", 2], ["a", 8], ["a", 9],
                                 ["a", 10], ["c", 0]],
                      "grants": [[0, 0], [1, 1], [2, 2], [3, 3], [4, 2], [5, 0], [6, 1], [7, 3], [8, 0], [9, 2],
                                 [10, -1]]},
    }
    path = os.path.join(HERE, "reference_vectors.json")
    with open(path, "w") as f:
        json.dump(vectors, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()
