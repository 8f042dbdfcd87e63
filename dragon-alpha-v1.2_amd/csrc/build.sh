#!/bin/bash
# Builds libdragon_hip.so (kernels + C ABI + runtime bridge) for gfx950, in-tree.
set -euo pipefail
cd "$(dirname "$0")"
HIPCC=${HIPCC:-/opt/rocm/bin/hipcc}
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Wall -Wno-unused-function \
  -Xclang -target-feature -Xclang -packed-fp32-ops"
SRCS="gemm_mfma.hip skbuf_summary.hip c_abi_gemm.hip runtime.hip"
OBJS=""
mkdir -p build
for s in $SRCS; do
  o=build/${s%.hip}.o
  $HIPCC $FLAGS -c "$s" -o "$o" 2> >(grep -v "packed-fp32-ops" >&2) &
  OBJS="$OBJS $o"
done
wait
$HIPCC --offload-arch=gfx950 -shared -fPIC -o ../libdragon_hip.so $OBJS
echo "built $(cd .. && pwd)/libdragon_hip.so"
