"""In-tree build of the native libraries (no cmake; hipcc and gcc directly).

  libtphip.so       HIP kernels + C ABI (include/tphip.h)           hipcc, gfx950
  libtpdatagen.so   seeded payload generator (include/tp_datagen.h)  gcc
  libtensorpipe_amd.so            channels, transports, pipe, C harness API        g++
  libtensorpipe_amd_torch_rpc.so  the channels registered with PyTorch's RPC agent g++
"""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "lib")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def run(cmd, **kw):
    print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    out = "\n".join(
        l for l in proc.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l
    )
    if out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}")


def build_tphip():
    os.makedirs(LIB, exist_ok=True)
    run([HIPCC, *HIP_FLAGS, "-shared", f"-I{INCLUDE}", f"-I{CSRC}/hip",
         "-o", os.path.join(LIB, "libtphip.so"), os.path.join(CSRC, "hip", "tphip.hip")])


def build_datagen():
    os.makedirs(LIB, exist_ok=True)
    run(["gcc", "-O2", "-fPIC", "-shared", f"-I{INCLUDE}",
         "-o", os.path.join(LIB, "libtpdatagen.so"),
         os.path.join(CSRC, "datagen", "tp_datagen.c"), "-lm"])


HOST_SOURCES = [
    "tensorpipe/common/common.cc",
    "tensorpipe/transport/shm/shm.cc",
    "tensorpipe/channel/basic/basic.cc",
    "tensorpipe/channel/xth/xth.cc",
    "tensorpipe/channel/hip_common.cc",
    "tensorpipe/channel/hip_xth/hip_xth.cc",
    "tensorpipe/channel/hip_ipc/hip_ipc.cc",
    "tensorpipe/channel/hip_basic/hip_basic.cc",
    "tensorpipe/core/core.cc",
    "capi/tensorpipe_c.cc",
    "bridge/bridge_amd.cc",
    "tensorpipe/transport/tcp/tcp.cc",
    "tensorpipe/transport/shm_stock/shm_stock.cc",
    "nopwire/nop_wire.cc",
    "nopwire/compat_pipe.cc",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter", "-pthread"]


def build_host(jobs=8):
    """libtensorpipe_amd.so: channels, shm transport, core and the C harness API (g++)."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(PKG, "build")
    os.makedirs(objdir, exist_ok=True)
    os.makedirs(LIB, exist_ok=True)
    sources = [s for s in HOST_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = [os.path.join(objdir, s.replace("/", "_") + ".o") for s in sources]

    def compile_one(pair):
        src, obj = pair
        run(["g++", *HOST_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    run(["g++", "-shared", "-pthread", "-o", os.path.join(LIB, "libtensorpipe_amd.so"), *objs,
         f"-L{LIB}", "-ltphip", "-Wl,-rpath,$ORIGIN", "-Wl,--no-undefined"])


CPP_TESTS = ["channel_tests", "pipe_tests", "unit_tests"]


def build_cpp_tests():
    """The C++ test programs under tests/cpp (plain executables driving the C++ API)."""
    src_dir = os.path.join(ROOT, "tests", "cpp")
    bin_dir = os.path.join(src_dir, "bin")
    os.makedirs(bin_dir, exist_ok=True)
    for name in CPP_TESTS:
        run(["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-Wno-unused-parameter", "-pthread",
             f"-I{INCLUDE}", f"-I{CSRC}", os.path.join(src_dir, name + ".cc"),
             "-o", os.path.join(bin_dir, name), f"-L{LIB}", "-ltensorpipe_amd", "-ltphip",
             "-Wl,-rpath,$ORIGIN/../../../tensorpipe_amd/lib"])


def build_fake_tphip(extra_flags=()):
    """tests/cpp/bin/fake/libtphip.so: the C ABI of include/tphip.h without a GPU behind it
    (tests/cpp/fake_tphip.cc). The C++ test programs load it instead of the real library when
    LD_LIBRARY_PATH names its directory, so the channels' host logic runs on the CPU."""
    out_dir = os.path.join(ROOT, "tests", "cpp", "bin", "fake")
    os.makedirs(out_dir, exist_ok=True)
    run(["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-Wno-unused-parameter",
         "-pthread", *extra_flags, f"-I{INCLUDE}", os.path.join(ROOT, "tests", "cpp", "fake_tphip.cc"),
         "-o", os.path.join(out_dir, "libtphip.so")])
    return out_dir


def stock_tensorpipe():
    """(include dir, lib dir) of the TensorPipe that PyTorch ships prebuilt, or None."""
    try:
        import importlib.util

        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        return None
    if spec is None or not spec.origin:
        return None
    root = os.path.dirname(spec.origin)
    inc, lib = os.path.join(root, "include"), os.path.join(root, "lib")
    if os.path.exists(os.path.join(inc, "tensorpipe", "tensorpipe.h")) and \
            os.path.exists(os.path.join(lib, "libtorch_cpu.so")):
        return inc, lib
    return None


def build_stock_conformance():
    """tests/cpp/bin/stock_conformance: this library's channels registered in the unmodified
    TensorPipe inside libtorch_cpu.so. The adapter is compiled against the STOCK headers (listed
    first, so that <tensorpipe/...> means theirs) and reaches this library through
    csrc/bridge/bridge.h only. Skipped where PyTorch's headers are not installed."""
    found = stock_tensorpipe()
    if found is None:
        print("stock TensorPipe headers not found: skipping tests/cpp/bin/stock_conformance", flush=True)
        return False
    inc, lib = found
    src_dir = os.path.join(ROOT, "tests", "cpp")
    bin_dir = os.path.join(src_dir, "bin")
    os.makedirs(bin_dir, exist_ok=True)
    run(["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-Wno-unused-parameter", "-pthread",
         f"-I{inc}", f"-I{INCLUDE}", f"-I{CSRC}",
         os.path.join(CSRC, "bridge", "stock_adapter.cc"), os.path.join(src_dir, "stock_conformance.cc"),
         "-o", os.path.join(bin_dir, "stock_conformance"),
         f"-L{LIB}", "-ltensorpipe_amd", "-ltphip", f"-L{lib}", "-ltorch_cpu", "-lc10",
         "-Wl,-rpath,$ORIGIN/../../../tensorpipe_amd/lib", f"-Wl,-rpath,{lib}"])
    # tests/cpp/bin/stock_wire_interop: the stock-protocol endpoint of csrc/nopwire against the same
    # unmodified TensorPipe, over TCP (no GPU); `capture` mode wrote tests/golden/stock_wire_vectors.txt.
    run(["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-Wno-unused-parameter", "-pthread",
         f"-I{inc}", f"-I{INCLUDE}", f"-I{CSRC}",
         os.path.join(src_dir, "stock_wire_interop.cc"),
         "-o", os.path.join(bin_dir, "stock_wire_interop"),
         f"-L{LIB}", "-ltensorpipe_amd", "-ltphip", f"-L{lib}", "-ltorch_cpu", "-lc10",
         "-Wl,-rpath,$ORIGIN/../../../tensorpipe_amd/lib", f"-Wl,-rpath,{lib}"])
    return True


def build_torch_rpc_plugin():
    """lib/libtensorpipe_amd_torch_rpc.so: registers hip_xth / hip_ipc / hip_basic and a GPU tensor
    converter with the TensorPipe agent of the installed PyTorch (torch.distributed.rpc), whose ROCm
    builds come without GPU channels. g++ against PyTorch's own headers (its TensorPipe's listed
    first); skipped where they are not installed."""
    found = stock_tensorpipe()
    if found is None or not os.path.exists(
            os.path.join(found[0], "torch", "csrc", "distributed", "rpc", "tensorpipe_agent.h")):
        print("PyTorch's RPC agent headers not found: skipping libtensorpipe_amd_torch_rpc.so", flush=True)
        return False
    inc, lib = found
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    run(["g++", "-O1", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-Wno-unused-parameter", "-pthread",
         "-DUSE_TENSORPIPE", "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__", "-DUSE_DISTRIBUTED", "-DUSE_RPC",
         f"-I{inc}", f"-I{inc}/torch/csrc/api/include", f"-I{rocm}/include", f"-I{INCLUDE}", f"-I{CSRC}",
         os.path.join(CSRC, "bridge", "torch_rpc_plugin.cc"), os.path.join(CSRC, "bridge", "stock_adapter.cc"),
         "-o", os.path.join(LIB, "libtensorpipe_amd_torch_rpc.so"),
         f"-L{LIB}", "-ltensorpipe_amd", "-ltphip",
         f"-L{lib}", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
         "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{lib}"])
    return True


def build_all():
    build_tphip()
    build_datagen()
    build_host()
    build_cpp_tests()
    build_fake_tphip()
    build_stock_conformance()
    build_torch_rpc_plugin()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
