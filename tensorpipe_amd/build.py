"""In-tree build of the native libraries (no cmake; hipcc and gcc directly).

  libtphip.so       HIP kernels + C ABI (include/tphip.h)           hipcc, gfx950
  libtpdatagen.so   seeded payload generator (include/tp_datagen.h)  gcc
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


def build_all():
    build_tphip()
    build_datagen()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
