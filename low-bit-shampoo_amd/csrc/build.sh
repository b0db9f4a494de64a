#!/usr/bin/env bash
# Builds qtensor/libqtensor_hip.so for gfx950 (cross-compiles without a GPU).
# Sources compile in parallel to objects under csrc/build/, then link.
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
out="${QT_OUT:-${here}/../qtensor/libqtensor_hip.so}"
obj="${QT_OBJ:-${here}/build}"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
# -ffp-contract=off: the nearest-entry rule needs two separately rounded fp32 subtractions.
# packed-fp32-ops is switched off for the device pass on this pool.
FLAGS=(-O3 -std=c++17 --offload-arch=gfx950 -fPIC -ffp-contract=off -fno-fast-math
       -Xclang -target-feature -Xclang -packed-fp32-ops
       -Wall -Wno-unused-command-line-argument -I"${here}" -I"${here}/../../include")
mkdir -p "${obj}"
pids=()
objs=()
for src in "${here}"/qt_*.hip; do
  o="${obj}/$(basename "${src%.hip}").o"
  objs+=("${o}")
  "${HIPCC}" "${FLAGS[@]}" "$@" -c "${src}" -o "${o}" &
  pids+=($!)
done
for p in "${pids[@]}"; do wait "${p}"; done
"${HIPCC}" --offload-arch=gfx950 -shared -fPIC "${objs[@]}" -o "${out}"
echo "built ${out}"
