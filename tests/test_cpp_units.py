"""Host-only unit checks of the C++ building blocks (tests/cpp/unit_tests.cc)."""
import json
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin", "unit_tests")
with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
    GOLDEN = json.load(f)


def run(*args):
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built (run __graft_entry__.build())")
    out = subprocess.run([BIN, *args], stdout=subprocess.PIPE, text=True, timeout=60)
    return out.returncode, out.stdout


def replay(slots, events):
    rc, out = run("allocator", str(slots), *[op + (str(arg) if op != "c" else "") for op, arg in events])
    assert rc == 0, out
    return [tuple(int(x) for x in tok.split(":")) for tok in out.split()]


def test_slot_allocator_matches_the_golden_trace():
    g = GOLDEN["allocator"]
    assert replay(g["slots"], g["events"]) == [tuple(x) for x in g["grants"]]


def test_slot_allocator_matches_the_oracle(oracle):
    import random

    rng = random.Random(1234)
    for trial in range(50):
        slots = rng.randint(1, 6)
        events, held, waiting, req = [], [], 0, 0
        for _ in range(rng.randint(1, 40)):
            if held and rng.random() < 0.45:
                s = held.pop(rng.randrange(len(held)))
                events.append(("r", s))
                if waiting:
                    waiting -= 1
                    held.append(s)  # the oldest waiter takes exactly the slot that came back
            else:
                events.append(("a", req))
                req += 1
                free = [i for i in range(slots) if i not in held]
                if free and not waiting:
                    held.append(min(free))
                else:
                    waiting += 1
        events.append(("c", 0))
        assert replay(slots, events) == oracle.allocator_trace(slots, events), (trial, slots, events)


def test_basics():
    rc, out = run("basics")
    assert rc == 0 and out.strip() == "OK", out


def test_on_demand_loops_never_wait_inside_a_task():
    """Two application threads, each in a task of one loop, defer to the other's loop at once (the
    previous executor waited there for good); a caller holding a lock the drainer's task wants; a
    task queued beside a draining application thread runs, and not on that thread; order and
    exactly-once under load; destruction with a helper on its way."""
    rc, out = run("loops")
    assert rc == 0 and out.strip() == "OK", out


def test_messages_of_a_departed_peer_are_delivered():
    # the writer exits before the reader posts its reads: the stream hands over what arrived,
    # then reports the end
    rc, out = run("departed_peer")
    assert rc == 0 and out.strip() == "OK", out


@pytest.mark.gpu
def test_host_pointer_in_a_hip_buffer_is_refused():
    rc, out = run("pointers")
    assert rc == 0 and out.strip().splitlines()[-1] == "OK", out


def test_remembered_pointer_answers_are_checked_again_per_message():
    """The same on the host-only stand-in runtime, where a freed device range can be mapped again
    as plain memory: after the next checkpoint the address is no longer taken for device memory."""
    fake = os.path.join(os.path.dirname(BIN), "fake")
    proc = subprocess.run([BIN, "pointers", "map_over"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120,
                          env=dict(os.environ, LD_LIBRARY_PATH=fake))
    lines = proc.stdout.strip().splitlines()
    assert proc.returncode == 0 and lines and lines[-1] == "OK", proc.stdout
    assert not any(l.startswith("note:") for l in lines), proc.stdout


@pytest.mark.parametrize("seed", [4, 5])
def test_garbage_on_new_connections_in_stock_wire_format(seed):
    # the same where the first packets are the reference's libnop objects
    out = subprocess.run([BIN, "garbage", str(seed), "100"], stdout=subprocess.PIPE, text=True, timeout=120,
                         env=dict(os.environ, TP_STOCK_WIRE="1"))
    assert out.returncode == 0 and out.stdout.strip() == "OK", out.stdout


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_garbage_on_new_connections(seed):
    # random bytes where the first packets of a pipe belong: the listening context survives them
    # and still serves a proper pipe
    out = subprocess.run([BIN, "garbage", str(seed), "100"], stdout=subprocess.PIPE, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.strip() == "OK", out.stdout


def test_nop_wire_decodes_and_reproduces_the_frames_of_a_stock_endpoint():
    """tests/golden/stock_wire_vectors.txt holds control frames written by the TensorPipe inside
    PyTorch (tests/cpp/stock_wire_interop.cc capture made it): every one decodes to what the
    capturing program sent and encodes back to the same bytes; cut or bent frames are refused."""
    rc, out = run("nop_wire", os.path.join(ROOT, "tests", "golden", "stock_wire_vectors.txt"))
    assert rc == 0, out
    facts = {}
    for line in out.splitlines():
        if line.startswith("VECTOR "):
            _, name, rest = line.split(" ", 2)
            facts[name] = rest
    assert out.strip().splitlines()[-1] == f"OK {len(facts)} vectors" and len(facts) >= 12
    assert facts["stock_client.spontaneous_connection"] == "name=stock_client"
    assert facts["stock_client.requested_connection_r"].startswith("token=")
    assert facts["stock_client.brochure"] == "transports=1 channels=1 first=uv:uv:*"
    assert facts["stock_server.brochure_answer"] == (
        "transport=uv domain=uv:* ids=1 channels=1 pairs=1 first_pair=cpu,cpu->basic")
    # the message of the capturing program: 300 B and empty payloads; 70001 B with the target named,
    # 129 B without, an empty tensor
    for who, salt in (("stock_client", 110), ("stock_server", 100)):
        assert facts[f"{who}.descriptor_0"] == (
            f"metadata=message metadata {salt} payloads=300[first payload]0[] "
            "tensors=70001@cpu>cpu[named target]129@cpu>?[]0@cpu>cpu[empty]")
        assert facts[f"{who}.descriptor_reply_0"] == "devices=1 cpu:0"


def test_compat_pipe_talks_to_itself():
    rc, out = run("compat_pipe")
    assert rc == 0 and out.strip() == "OK", out


def test_shm_transport_in_the_reference_protocol():
    """transport/shm_stock, both ends this library's: messages of every size class both ways
    (below, at and far above the 2 MiB ring), exact-length reads, a peer that wrote and left,
    closes, listeners by chosen and by kernel-picked name. (Against the unmodified build:
    tests/test_stock_wire_interop.py.)"""
    rc, out = run("shm_stock")
    assert rc == 0 and out.strip() == "OK", out


def test_shm_transport_with_a_peer_that_breaks_the_protocol():
    """A peer written in the test against the reference's protocol alone (socket, descriptors by
    SCM_RIGHTS, ring headers) first behaves, then misbehaves: a data segment smaller than its
    header says, markers that claim more bytes than a ring holds (inbox and outbox), the ring's
    size rewritten after set-up, a long message announced and abandoned. Every case ends in an
    error or in the bytes that were really sent; none reads outside a ring or waits for ever."""
    rc, out = run("shm_stock_hostile_peer")
    assert rc == 0 and out.strip() == "OK", out


@pytest.mark.parametrize("transport", ["shm", "shm_stock", "tcp"])
def test_transport_suite_after_the_reference(transport):
    """The reference's transport tests (tensorpipe/test/transport/listener_test.cc,
    connection_test.cc, context_test.cc, shm/connection_test.cc), case by case, on each of this
    library's transports: accepts and incoming connections are queued and served in order, a
    closed listener and the listener of a closed context, a peer that drops the connection at
    once, objects and raw bytes, writes that complete before any read, messages five times the
    ring, two messages that do not fit the ring together (raw and as objects)."""
    rc, out = run("transport_suite", transport)
    assert rc == 0 and out.strip() == "OK", out


def test_tcp_transport():
    """Messages of every size class both ways, exact-length reads, the reference's stream framing
    written and read by hand, a peer that wrote and left, and a pipe over it."""
    rc, out = run("tcp")
    assert rc == 0 and out.strip() == "OK", out
