"""torch.distributed.rpc moving GPU tensors between two processes (and to oneself) on this
library's channels, registered with PyTorch's own TensorPipe agent by
tensorpipe_amd/csrc/bridge/torch_rpc_plugin.cc: the counterpart of the registration the reference's
CUDA channels get in PyTorch's CUDA builds. Every tensor is compared bit for bit with what was sent,
and the module's counter proves that GPU buffers went through the hip_* channels."""
import pytest

from tests.test_torch_rpc import run_group

pytestmark = pytest.mark.gpu


# "staged": the agent's channel list cut down to hip_basic, so that calls to the other rank take the
# shared pinned ring and calls to this rank itself take the wrapped CPU channel, whose loop and the
# staged channel's own loop are then both driven by agent and transport threads that are strangers
# to this library (tests/cpp/unit_tests.cc `loops` holds the executor's side of that).
@pytest.mark.parametrize("mode", ["gpu", "staged"])
def test_gpu_tensors_over_rpc(mode):
    results, outs = run_group(mode)
    names = {line.split()[1] for line in results}
    assert {"echo_0", "echo_4097", "echo_67108864", "add_one", "checksum_at_callee", "mixed_devices_arrive_in_place",
            "mixed_echo", "in_flight_24", "view", "rref_to_here", "to_self", "to_self_used_the_channels",
            "channel_chosen", "callee_calls_back", "route"} <= names
    for rank, out in enumerate(outs):
        counts = [int(line.split()[3]) for line in out.splitlines() if line.startswith(f"RANK {rank} ")]
        assert counts and counts[0] > 50, f"rank {rank}: {counts}"


def test_calls_with_gpu_tensors_fail_when_the_peer_dies():
    """The other process ends abruptly with GPU tensors of several calls in flight on hip_ipc: every
    pending call reports an error, nothing waits for ever."""
    results, _ = run_group("peer_dies", timeout=120, rank1_exit=3)
    assert {"before", "calls_fail_instead_of_hanging"} <= {line.split()[1] for line in results}


def test_three_processes_share_the_gpu():
    """Three RPC workers on the one GPU, every pair connected: calls to both peers at once, and a
    call that the first peer relays to the second with the tensor on the GPU all the way."""
    results, _ = run_group("gpu3", timeout=180, world=3)
    assert {"both_peers", "relayed", "channel_chosen", "route"} <= {line.split()[1] for line in results}
