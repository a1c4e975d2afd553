"""The committed golden vectors (tests/golden/reference_vectors.json) against the oracle
(CPU) and against the HIP copy path (GPU, through the C ABI)."""
import hashlib
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLDEN = json.load(f)


def build(p):
    n = p["bytes"]
    i = np.arange(n, dtype=np.int64)
    if p["kind"] == "iota":
        b = (i % 256).astype(np.uint8)
    elif p["kind"] == "fill":
        b = np.full(n, p["value"], np.uint8)
    elif p["kind"] == "bench":
        b = (((i >> 8) ^ (i & 0xFF)) & 0xFF).astype(np.uint8)
    else:
        raise ValueError(p["kind"])
    return b


def all_payloads():
    out = [t for c in GOLDEN["channel"] for t in c["tensors"]] + GOLDEN["bench_pattern"]["cases"]
    return out


@pytest.mark.parametrize("p", all_payloads(), ids=lambda p: f"{p['kind']}{p['bytes']}")
def test_fixture_is_self_consistent(p):
    b = build(p)
    assert hashlib.sha256(b.tobytes()).hexdigest() == p["sha256"]
    assert b[:8].tobytes().hex() == p["head"] and b[-8:].tobytes().hex() == p["tail"]


@pytest.mark.parametrize("case", GOLDEN["channel"], ids=lambda c: c["name"].split(" ")[0])
def test_oracle_channels_deliver_the_vectors(oracle, case):
    """Every channel restatement of the oracle is the identity on the reference's vectors."""
    for p in case["tensors"]:
        want = build(p)
        n = p["bytes"]
        for fn in ("xth", "ipc", "staged"):
            src = want.copy()
            dst = np.full(n + 64, 0xEE, np.uint8)
            view = dst[32:32 + n]
            if fn == "xth":
                oracle.xth_message([(src, view, n)])
            elif fn == "ipc":
                assert oracle.ipc_tensor(src, view, n, slot=4096, num_slots=4) == (n + 4095) // 4096
            else:
                assert oracle.staged_tensor(src, view, n, slot=4096, num_slots=4) == (n + 4095) // 4096
            assert np.array_equal(view, want), (case["name"], fn)
            assert (dst[:32] == 0xEE).all() and (dst[32 + n:] == 0xEE).all(), "guard bytes touched"
            assert np.array_equal(src, want), "source modified"


def test_oracle_chunking(oracle):
    for row in GOLDEN["chunking"]["rows"]:
        n = oracle.lib.tp_oracle_num_chunks(row["length"], row["slot"])
        assert n == row["chunks"], row
        if n:
            assert oracle.lib.tp_oracle_chunk_length(row["length"], row["slot"], 0) == row["first"][0]
            assert oracle.lib.tp_oracle_chunk_length(row["length"], row["slot"], n - 1) == row["last"][0]


def test_oracle_bench_pattern(oracle):
    for p in GOLDEN["bench_pattern"]["cases"]:
        out = np.zeros(p["bytes"], np.uint8)
        oracle.lib.tp_oracle_bench_pattern(out.ctypes.data, p["bytes"])
        assert hashlib.sha256(out.tobytes()).hexdigest() == p["sha256"]


def test_oracle_percentile(oracle):
    g = GOLDEN["percentile"]
    s = np.array(g["samples"], np.float64)
    for frac, want in g["expected"].items():
        assert oracle.lib.tp_oracle_percentile(s.copy().ctypes.data, len(s), float(frac)) == want


def test_oracle_allocator(oracle):
    g = GOLDEN["allocator"]
    got = oracle.allocator_trace(g["slots"], [(op, arg) for op, arg in g["events"]])
    assert got == [tuple(x) for x in g["grants"]]


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLDEN["channel"], ids=lambda c: c["name"].split(" ")[0])
def test_hip_copy_delivers_the_vectors(case):
    """The HIP copy path (C ABI: tphip_batched_copy) on the same vectors, guard bytes included."""
    import torch

    from tensorpipe_amd import hip

    repeat = case.get("repeat", 1)
    offset = case.get("offset", 0)
    entries, keep, checks = [], [], []
    for _ in range(repeat):
        for p in case["tensors"]:
            n = p["bytes"]
            want = build(p)
            alloc = torch.full((offset + max(n, 1),), case.get("guard_value", 0), dtype=torch.uint8, device="cuda")
            alloc[offset:offset + n] = torch.from_numpy(want).cuda()
            dst = torch.full((n + 64,), 0xEE, dtype=torch.uint8, device="cuda")
            keep += [alloc, dst]
            entries.append((alloc.data_ptr() + offset, dst.data_ptr() + 32, n))
            checks.append((dst, want, n))
    torch.cuda.synchronize()
    hip.batched_copy(entries)
    torch.cuda.synchronize()
    for dst, want, n in checks:
        host = dst.cpu().numpy()
        assert np.array_equal(host[32:32 + n], want), case["name"]
        assert (host[:32] == 0xEE).all() and (host[32 + n:] == 0xEE).all(), "guard bytes touched"
