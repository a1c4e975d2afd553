"""This library's device channels registered in an UNMODIFIED TensorPipe: the build that PyTorch
ships inside libtorch_cpu.so (its own Context, Pipe, shm transport and basic channel), with
hip_xth / hip_ipc / hip_basic added through Context::registerChannel exactly as the reference
registers its CUDA channels (tensorpipe/core/context.h:67-70,
tensorpipe/test/core/pipe_test.h:300-316). tests/cpp/stock_conformance.cc sends a message with a
payload, three GPU tensors and one CPU tensor each way and checks every byte.

The program only exists where PyTorch's TensorPipe headers were present at build time.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "tests", "cpp", "bin", "stock_conformance")


# tests/cpp/fake_tphip.cc, the host-only stand-in for libtphip.so: with it the same program runs on
# the CPU and checks the channels' host logic inside the stock pipe (not the kernels).
STAND_IN = os.path.join(ROOT, "tests", "cpp", "bin", "fake")

# every case twice: on the GPU, and on the CPU against the stand-in runtime
runtimes = pytest.mark.parametrize("runtime", [pytest.param("gpu", marks=pytest.mark.gpu), "stand_in"])


def _run(args, env=None, runtime="gpu", timeout=120):
    if not os.path.exists(PROGRAM):
        pytest.skip("tests/cpp/bin/stock_conformance is not built (no stock TensorPipe headers at build time)")
    print("running stock_conformance", *args, env or "", runtime, flush=True)
    env = dict(env or {})
    if runtime == "stand_in":
        env["LD_LIBRARY_PATH"] = STAND_IN
    proc = subprocess.run([PROGRAM, *args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout,
                          env=dict(os.environ, **env))
    results = [line for line in proc.stdout.splitlines() if line.startswith("RESULT ")]
    assert results, f"no result line; exit code {proc.returncode}\n{proc.stdout[-2000:]}\n{proc.stderr[-2000:]}"
    bad = [line for line in results if line.split()[2] != "OK"]
    assert not bad and proc.returncode == 0, "\n".join(bad) + f"\nexit code {proc.returncode}\n" + proc.stderr[-2000:]


@runtimes
def test_hip_xth_in_a_stock_context_same_process(runtime):
    _run(["same_process"], runtime=runtime)


@runtimes
@pytest.mark.parametrize("channel", ["hip_ipc", "hip_basic"])
def test_channel_in_stock_contexts_of_two_processes(channel, runtime):
    _run(["two_process", channel], runtime=runtime)


@runtimes
@pytest.mark.parametrize("channel,rounds", [("hip_basic", 40), ("hip_xth", 40)])
def test_one_stock_context_talking_to_itself_both_ways_at_once(channel, rounds, runtime):
    """What an RPC agent's call to its own rank does: one context, a pipe to itself, messages both
    ways at the same moment from application threads. With hip_basic every GPU tensor then goes
    through the wrapped CPU channel, so two of this library's loops are driven by threads that are
    all strangers to it (the host's transport threads included); a thread inside a task of one loop
    that defers to the other must never wait there."""
    _run(["to_self", channel, str(rounds)], runtime=runtime, timeout=300)


@runtimes
def test_hip_basic_inner_route_over_the_hosts_connections(runtime):
    """hip_basic without the shared ring: every chunk travels through the CPU channel it wraps, which
    here runs over the stock pipe's own connections (the route between machines, and to oneself)."""
    _run(["two_process", "hip_basic"], env={"TP_HIP_BASIC_NO_SHARED_RING": "1"}, runtime=runtime)


@runtimes
def test_endpoint_with_hip_channels_talks_to_an_unmodified_peer(runtime):
    """Registering the channels does not get in the way of a peer that has none of them: payloads
    and CPU tensors still travel on the stock channels."""
    _run(["unmodified_peer"], runtime=runtime)


@runtimes
@pytest.mark.parametrize("channel", ["hip_xth", "hip_ipc", "hip_basic"])
def test_native_pipe_in_stock_wire_format_with_a_stock_peer(channel, runtime):
    """One end is a context of this library with ContextOptions::stockWireFormat (its own pipe, its
    TCP transport registered as "uv", the channel natively), the other the stock TensorPipe with the
    same channel through the bridge: payload, GPU tensors and a CPU tensor both ways, byte for byte."""
    _run(["native_peer", channel], runtime=runtime)


@runtimes
@pytest.mark.parametrize("channel", ["hip_ipc", "hip_basic"])
def test_native_pipe_with_a_stock_peer_moves_to_the_reference_shm_transport(channel, runtime):
    """The same two processes when both ends also hold the reference's shm transport (this
    library's end through transport/shm_stock), preferred: the stock end connects over uv, the
    pipe moves to shm during the handshake, and payload, GPU tensors and a CPU tensor flow there."""
    _run(["native_peer", channel, "shm"], runtime=runtime)
