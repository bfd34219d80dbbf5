#!/bin/bash
# Builds libFastKron.so (the C-ABI library) for gfx950 with hipcc, in-tree.
#   fastkron_amd/csrc/build.sh           (takes no arguments: the kernels have no build-time switches)
set -euo pipefail
if (( $# )); then echo "build.sh takes no arguments" >&2; exit 2; fi
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
OUT="$HERE/../lib"
OBJ="$HERE/../lib/obj"
mkdir -p "$OUT" "$OBJ"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
# -packed-fp32-ops is switched off: hipcc must not form v_pk_*_f32 from scalar float code.
FLAGS=(-O3 -std=c++17 -fPIC --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops
       -Wall -Wno-unused-function -Wno-unused-value -Wno-unused-result -Wno-unused-command-line-argument -I"$HERE/../../include")
SRCS=("$HERE"/api.cpp "$HERE"/handle.cpp "$HERE"/kernel_db.cpp "$HERE"/autotuner.cpp "$HERE"/static_scratch.hip "$HERE"/kernels/*.hip)
pids=()
objs=()
for s in "${SRCS[@]}"; do
  o="$OBJ/$(basename "$s").o"
  objs+=("$o")
  "$HIPCC" "${FLAGS[@]}" -x hip -c "$s" -o "$o" &
  pids+=($!)
  if (( ${#pids[@]} >= 8 )); then wait "${pids[0]}"; pids=("${pids[@]:1}"); fi
done
for p in "${pids[@]}"; do wait "$p"; done
"$HIPCC" -shared -fPIC --offload-arch=gfx950 -o "$OUT/libFastKron.so" "${objs[@]}"
echo "built $OUT/libFastKron.so"
