#!/bin/sh
# Writes tests/golden/stock_wire_vectors.txt: the control frames an unmodified TensorPipe endpoint (the build
# inside PyTorch's libtorch_cpu.so) puts on its TCP connections, read off the wire by
# tests/cpp/stock_wire_interop.cc while it exchanges its test messages with that endpoint in both roles.
# Needs tests/cpp/bin/stock_wire_interop (built by __graft_entry__.build() where PyTorch's TensorPipe headers
# are installed). Ports and registration tokens in the frames are those of the capturing run.
set -e
here=$(cd "$(dirname "$0")" && pwd)
"$here/../cpp/bin/stock_wire_interop" capture "$here/stock_wire_vectors.txt"
