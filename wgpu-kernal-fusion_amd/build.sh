#!/bin/bash
# Builds libwkf_hip.so (C ABI levels 0 and 1) in-tree with hipcc.  The GPU kernels
# themselves are generated at run time and JIT-compiled by hiprtc for gfx950.
set -euo pipefail
here="$(cd "$(dirname "$0")" && pwd)"
cd "$here/csrc"
hipcc -O2 -std=c++17 -fPIC -shared -Wall -Wno-unused-function -Wno-unused-value -Wno-unused-result \
  --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
  -I"$here/../include" -I. \
  hip_ffi.cpp core.cpp codegen.cpp graph.cpp gemm.cpp tensor_api.cpp \
  -o "$here/libwkf_hip.so" -lhiprtc -Wl,-rpath,/opt/rocm/lib \
  2> >(grep -v "packed-fp32-ops' is not a recognized feature" >&2)
echo "built $here/libwkf_hip.so"
