#!/bin/bash
# Builds libag_hip.so for gfx950 next to this script, its test flavour libag_hip_test.so (the same sources with
# the tuning hooks of ag_test_hooks.h compiled in: -DAG_TEST_HOOKS) and the host operator layer libag_host.so.
# Usage: build.sh [extra hipcc flags]
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
out="$here/../libag_hip.so"
srcs=(common.hip im2col.hip gemm.hip gemm_dl.hip conv.hip conv_s2.hip pool.hip reduce.hip adam.hip elementwise.hip)
hooked=(gemm.hip pool.hip)   # the sources that hold test hooks: compiled a second time for the test flavour
flags=(--offload-arch=gfx950 -O3 -std=c++17 -fPIC -fvisibility=hidden
       -Xclang -target-feature -Xclang -packed-fp32-ops
       -I"$here/../../include" -I"$here" -Wall -Wno-unused-function "$@")
mkdir -p "$here/obj" "$here/obj/hooks"
pids=()
compile() {  # source, object, extra flags...
  local s="$1" o="$2"; shift 2
  local extra=("$@")
  # adam.hip must keep the reference's separately rounded multiplies and adds
  [ "$s" = adam.hip ] && extra+=(-ffp-contract=off)
  # keep the MFMA accumulators in ordinary VGPRs (no copies to and from AGPRs around the epilogue)
  [ "$s" = gemm_dl.hip ] && extra+=(-Wno-inline-asm -Wno-pass-failed)
  /opt/rocm/bin/hipcc "${flags[@]}" "${extra[@]}" -c "$here/$s" -o "$o" &
  pids+=($!)
}
for s in "${srcs[@]}"; do compile "$s" "$here/obj/${s%.hip}.o"; done
for s in "${hooked[@]}"; do compile "$s" "$here/obj/hooks/${s%.hip}.o" -DAG_TEST_HOOKS; done
for p in "${pids[@]}"; do wait "$p"; done
/opt/rocm/bin/hipcc --offload-arch=gfx950 -shared -fPIC -o "$out" "$here"/obj/*.o
echo "built $out"
test_objs=()
for s in "${srcs[@]}"; do
  o="$here/obj/${s%.hip}.o"
  for h in "${hooked[@]}"; do [ "$s" = "$h" ] && o="$here/obj/hooks/${s%.hip}.o"; done
  test_objs+=("$o")
done
/opt/rocm/bin/hipcc --offload-arch=gfx950 -shared -fPIC -o "$here/../libag_hip_test.so" "${test_objs[@]}"
echo "built $here/../libag_hip_test.so"

# Host-side operator layer (C++ mirror of the reference's Op / graph / optimizer code); links the
# kernel library next to it.
host_out="$here/../libag_host.so"
/opt/rocm/bin/hipcc -O2 -std=c++17 -fPIC -fvisibility=hidden -Wall -I"$here/../../include" -I"$here/host" -I/opt/rocm/include \
    -x c++ "$here/host/runtime.cpp" "$here/host/ops.cpp" "$here/host/gradient.cpp" "$here/host/persist.cpp" "$here/host/capi_host.cpp" \
    -D__HIP_PLATFORM_AMD__ -shared -o "$host_out" -L"$here/.." -lag_hip -L/opt/rocm/lib -lamdhip64 \
    -Wl,-rpath,'$ORIGIN' -Wl,-rpath,/opt/rocm/lib
echo "built $host_out"
