"""The stock-protocol endpoint (tensorpipe_amd/csrc/nopwire) against an unmodified TensorPipe: the
build inside PyTorch's libtorch_cpu.so, over its uv transport and basic channel on 127.0.0.1, and
over its shm transport (this library's transport/shm_stock speaks that protocol). Both
roles, messages both ways: payloads, CPU tensors with and without a target device named by the
sender, an empty tensor (tests/cpp/stock_wire_interop.cc). No GPU involved.

The program only exists where PyTorch's TensorPipe headers were present at build time.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAM = os.path.join(ROOT, "tests", "cpp", "bin", "stock_wire_interop")


def test_compat_endpoint_and_stock_endpoint_understand_each_other():
    if not os.path.exists(PROGRAM):
        pytest.skip("tests/cpp/bin/stock_wire_interop is not built (no stock TensorPipe headers at build time)")
    proc = subprocess.run([PROGRAM, "run"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    results = [line for line in proc.stdout.splitlines() if line.startswith("RESULT ")]
    assert [r.split()[1] for r in results] == [
        "compat_client_with_stock_server", "stock_client_with_compat_server",
        "native_client_with_stock_server", "stock_client_with_native_server",
        # both ends also hold a transport called "shm" that the other's does not understand:
        # the pipe stays on uv (tensorpipe/core/pipe_impl.cc:996-1012 goes by the domain descriptors)
        "native_client_with_stock_server_both_hold_shm", "stock_client_with_native_server_both_hold_shm",
        # the native end holds the transport that speaks the stock shm protocol
        # (transport/shm_stock): opened over uv, the pipe moves to shm in both roles
        "native_client_with_stock_server_moves_to_shm", "stock_client_with_native_server_moves_to_shm"], (
        proc.stdout[-2000:] + proc.stderr[-2000:])
    bad = [r for r in results if r.split()[2] != "OK"]
    assert not bad and proc.returncode == 0, "\n".join(bad) + proc.stderr[-2000:]
