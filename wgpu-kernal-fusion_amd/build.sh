#!/bin/bash
# Builds libwkf_hip.so (C ABI levels 0 and 1) in-tree with hipcc.  The GPU kernels
# themselves are generated at run time and JIT-compiled by hiprtc for gfx950.
set -euo pipefail
here="$(cd "$(dirname "$0")" && pwd)"
cd "$here/csrc"
# hip_ffi.cpp is HIP source (it holds a file-scope device array, compiled for gfx950); the layers above it are
# plain C++.  The two kinds are compiled in separate commands: given both in one, hipcc drops the offload target.
obj="$here/build"
mkdir -p "$obj"
flags=(-O2 -std=c++17 -fPIC -Wall -Wno-unused-function -Wno-unused-value -Wno-unused-result -I"$here/../include" -I.)
hipcc "${flags[@]}" --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops -x hip -c hip_ffi.cpp -o "$obj/hip_ffi.o" \
  2> >(grep -v "packed-fp32-ops' is not a recognized feature" >&2)
pids=()
for f in core codegen graph gemm tensor_api; do
  hipcc "${flags[@]}" -x c++ -c "$f.cpp" -o "$obj/$f.o" &
  pids+=($!)
done
for p in "${pids[@]}"; do wait "$p"; done
hipcc --hip-link --offload-arch=gfx950 -shared -fPIC "$obj"/hip_ffi.o "$obj"/core.o "$obj"/codegen.o "$obj"/graph.o "$obj"/gemm.o "$obj"/tensor_api.o \
  -o "$here/libwkf_hip.so" -lhiprtc -Wl,-rpath,/opt/rocm/lib
echo "built $here/libwkf_hip.so"
