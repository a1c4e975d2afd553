"""Runs the C++ test programs under tests/cpp and reports every case as a test.

The programs drive the product's C++ API directly: channel::Context::createChannel +
Channel::send/recv (channel_tests) and Context/Listener/Pipe with mixed CPU/GPU messages
(pipe_tests), following the reference's own suites (tensorpipe/test/channel/*.cc,
tensorpipe/test/core/pipe_cuda_test.cc). Each suite is started once; every endpoint of
every case prints a "RESULT <role> <case> OK|FAIL ..." line that is checked here.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin")

CPU_SUITES = [("channel_tests", "basic"), ("channel_tests", "xth"),
              ("pipe_tests", "cpu_same_process"), ("pipe_tests", "cpu_two_process")]
GPU_SUITES = [("channel_tests", "hip_xth"), ("channel_tests", "hip_ipc"), ("channel_tests", "hip_ipc_outbox"),
              ("channel_tests", "hip_ipc_gated"), ("channel_tests", "hip_ipc_messages"),
              ("channel_tests", "hip_basic"), ("channel_tests", "hip_basic_host_ring"),
              ("channel_tests", "hip_basic_small_ring"),
              ("pipe_tests", "same_process"), ("pipe_tests", "two_process")]

# tests/cpp/fake_tphip.cc: the C ABI of include/tphip.h with threads and memcpy behind it
STAND_IN = os.path.join(BIN, "fake")

_results = {}


def _binary(program):
    path = os.path.join(BIN, program)
    if not os.path.exists(path):
        pytest.fail(f"{path} is not built (run __graft_entry__.build())")
    return path


def list_cases(program, suite):
    path = os.path.join(BIN, program)
    if not os.path.exists(path):
        return ["<not built>"]
    out = subprocess.run([path, "--suite", suite, "--list"], stdout=subprocess.PIPE, text=True, timeout=30)
    return out.stdout.split()


def run_suite(program, suite, stock_wire=False, stand_in=False):
    """One run per suite and session; returns {case: [(role, ok, detail), ...]}."""
    key = (program, suite, stock_wire, stand_in)
    if key not in _results:
        print(f"running {program} --suite {suite}" + (" in stock wire format" if stock_wire else ""), flush=True)
        env = dict(os.environ, TP_STOCK_WIRE="1") if stock_wire else None
        if stand_in:
            if not os.path.exists(os.path.join(STAND_IN, "libtphip.so")):
                pytest.fail(f"{STAND_IN}/libtphip.so is not built (run __graft_entry__.build())")
            env = dict(env or os.environ, LD_LIBRARY_PATH=STAND_IN)
        proc = subprocess.run([_binary(program), "--suite", suite], stdout=subprocess.PIPE,
                              stderr=subprocess.PIPE, text=True, timeout=600, env=env)
        per_case = {}
        for line in proc.stdout.splitlines():
            parts = line.split(" ", 4)
            if len(parts) >= 4 and parts[0] == "RESULT":
                role, case, verdict = parts[1], parts[2], parts[3]
                per_case.setdefault(case, []).append((role, verdict == "OK", line))
        _results[key] = (proc.returncode, per_case, proc.stdout[-4000:], proc.stderr[-4000:])
    return _results[key]


def check_case(program, suite, case, stock_wire=False, stand_in=False):
    rc, per_case, out, err = run_suite(program, suite, stock_wire, stand_in)
    assert case in per_case, f"no result for {case}; exit code {rc}\n{out}\n{err}"
    bad = [line for _, ok, line in per_case[case] if not ok]
    assert not bad, "\n".join(bad) + "\n" + err
    two_process = suite in ("basic", "hip_ipc", "hip_ipc_outbox", "hip_ipc_gated", "hip_ipc_messages", "hip_basic",
                            "hip_basic_host_ring", "hip_basic_small_ring", "two_process", "cpu_two_process")
    assert len(per_case[case]) == (2 if two_process else 1), per_case[case]


def _params(suites):
    return [pytest.param(p, s, c, id=f"{s}-{c}") for p, s in suites for c in list_cases(p, s)]


@pytest.mark.parametrize("program,suite,case", _params(CPU_SUITES))
def test_cpu_suite(program, suite, case):
    check_case(program, suite, case)


@pytest.mark.gpu
@pytest.mark.parametrize("program,suite,case", _params(GPU_SUITES))
def test_gpu_suite(program, suite, case):
    check_case(program, suite, case)


# The suites of the device channels once more without a GPU: libtphip.so replaced by the host-only
# stand-in (streams are threads, copies memcpy), which leaves the channels' own host logic -- state
# machines, control messages, slot rings, signal words, error paths -- to be checked on the CPU.
# Parity of the kernels is NOT what these show; the -m gpu runs of the same suites are.
@pytest.mark.parametrize("program,suite,case", _params(GPU_SUITES))
def test_device_channel_host_logic_on_the_stand_in_runtime(program, suite, case):
    check_case(program, suite, case, stand_in=True)


# The pipe suites once more with the reference's encodings on the wire (TP_STOCK_WIRE=1: its
# handshake, libnop descriptors, descriptor replies on their own connection, no batching across
# the channel interface): the same cases must pass, both ends being this library's.
@pytest.mark.parametrize("program,suite,case", _params([s for s in CPU_SUITES if s[0] == "pipe_tests"]))
def test_cpu_suite_in_stock_wire_format(program, suite, case):
    check_case(program, suite, case, stock_wire=True)


@pytest.mark.gpu
@pytest.mark.parametrize("program,suite,case", _params([s for s in GPU_SUITES if s[0] == "pipe_tests"]))
def test_gpu_suite_in_stock_wire_format(program, suite, case):
    check_case(program, suite, case, stock_wire=True)
