#!/bin/bash
# Builds libag_hip.so for gfx950 next to this script.  Usage: build.sh [extra hipcc flags]
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
out="$here/../libag_hip.so"
srcs=(common.hip im2col.hip gemm.hip conv.hip pool.hip reduce.hip adam.hip elementwise.hip)
flags=(--offload-arch=gfx950 -O3 -std=c++17 -fPIC -fvisibility=hidden
       -Xclang -target-feature -Xclang -packed-fp32-ops
       -I"$here/../../include" -I"$here" -Wall -Wno-unused-function "$@")
mkdir -p "$here/obj"
pids=()
for s in "${srcs[@]}"; do
  extra=()
  # adam.hip must keep the reference's separately rounded multiplies and adds
  [ "$s" = adam.hip ] && extra=(-ffp-contract=off)
  /opt/rocm/bin/hipcc "${flags[@]}" "${extra[@]}" -c "$here/$s" -o "$here/obj/${s%.hip}.o" &
  pids+=($!)
done
for p in "${pids[@]}"; do wait "$p"; done
/opt/rocm/bin/hipcc --offload-arch=gfx950 -shared -fPIC -o "$out" "$here"/obj/*.o
echo "built $out"
