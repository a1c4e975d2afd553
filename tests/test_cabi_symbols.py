"""The C-ABI libraries load and export every function their headers declare."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

HEADERS = {
    "tphip.h": "libtphip.so",
    "tp_datagen.h": "libtpdatagen.so",
    "tensorpipe_c.h": "libtensorpipe_amd.so",
}


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    names = re.findall(r"\b((?:tphip|tpdg|tpc)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(n for n in names if not n.endswith("_fn")))


@pytest.mark.parametrize("header", sorted(HEADERS))
def test_exports(header):
    path = os.path.join(ROOT, "include", header)
    if not os.path.exists(path):
        pytest.skip(f"{header} not present")
    lib = ctypes.CDLL(os.path.join(ROOT, "tensorpipe_amd", "lib", HEADERS[header]))
    names = _declared(header)
    assert len(names) >= 5
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_copy_desc_layout():
    from tensorpipe_amd import _native

    assert ctypes.sizeof(_native.CopyDesc) == 24
    assert _native.CopyDesc.dst.offset == 8 and _native.CopyDesc.bytes.offset == 16


def test_one_hip_runtime_per_process():
    """Loading the native library before torch must not leave two HIP runtimes in the process
    (each would be blind to the other's allocations)."""
    import subprocess
    import sys

    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "from tensorpipe_amd import _native\n"
        "_native.tphip()\n"
        "import torch\n"
        "libs = sorted({l.split()[-1] for l in open('/proc/self/maps') if 'libamdhip64' in l})\n"
        "print(len(libs), libs)\n" % ROOT
    )
    out = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, text=True, timeout=300)
    assert out.returncode == 0
    assert out.stdout.split()[0] == "1", out.stdout
