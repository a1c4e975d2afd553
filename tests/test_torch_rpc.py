"""torch.distributed.rpc with this library's module loaded, on a machine without a GPU: the hip_*
channels report themselves not viable, the agent leaves them out, and CPU tensors travel as
before. (The GPU cases are in test_zy_torch_rpc_gpu.py.)"""
import os
import subprocess
import sys
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CASES = os.path.join(ROOT, "tests", "torch_rpc_cases.py")
PLUGIN = os.path.join(ROOT, "tensorpipe_amd", "lib", "libtensorpipe_amd_torch_rpc.so")



def run_group(mode, timeout=120, rank1_exit=0, world=2):
    if not os.path.exists(PLUGIN):
        pytest.skip("libtensorpipe_amd_torch_rpc.so is not built (no RPC agent headers at build time)")
    meeting = tempfile.NamedTemporaryFile(prefix="tp_rpc_", suffix=".rendezvous", delete=False)
    meeting.close()
    os.unlink(meeting.name)  # the first rank creates it
    print(f"running torch_rpc_cases.py, mode {mode}, rendezvous {meeting.name}", flush=True)
    # The ranks keep a short timeline of what the channels did last and print it when they end;
    # a rank that stalls ends itself (torch_rpc_cases.py) well inside this function's time limit.
    env = dict(os.environ, TP_TIMELINE=os.environ.get("TP_TIMELINE", "400"))
    ranks = [
        subprocess.Popen([sys.executable, "-u", CASES, str(rank), meeting.name, mode],
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env)
        for rank in range(world)
    ]
    outs = []
    for p in ranks:
        try:
            outs.append(p.communicate(timeout=timeout))
        except subprocess.TimeoutExpired:
            p.kill()
            outs.append(p.communicate())
    if os.path.exists(meeting.name):
        os.unlink(meeting.name)
    text = outs[0][0]
    results = [line for line in text.splitlines() if line.startswith("RESULT ")]
    tail = "\n".join(f"--- rank {i}\n{o[-2500:]}\n{e[-12000:]}" for i, (o, e) in enumerate(outs))
    assert results, f"no result line\n{tail}"
    results += [line for o, _ in outs[1:] for line in o.splitlines() if line.startswith("RESULT stalled")]
    bad = [line for line in results if line.split()[2] != "OK"]
    codes = [p.returncode for p in ranks]
    want = [0, rank1_exit] + [0] * (world - 2)
    assert not bad and codes == want, "\n".join(bad) + f"\nexit codes {codes}\n" + tail
    return results, [o for o, _ in outs]


def test_cpu_rpc_is_undisturbed_by_the_module():
    results, _ = run_group("cpu")
    names = {line.split()[1] for line in results}
    assert {"echo_0", "echo_67108864", "mixed_echo", "in_flight_24", "callee_calls_back", "route"} <= names


def test_cpu_calls_fail_when_the_peer_dies():
    results, _ = run_group("cpu_peer_dies", timeout=120, rank1_exit=3)
    assert {"before", "calls_fail_instead_of_hanging"} <= {line.split()[1] for line in results}
