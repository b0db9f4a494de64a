#!/usr/bin/env bash
# Builds qtensor/libqtensor_hip.so for gfx950 (cross-compiles without a GPU).
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
out="${QT_OUT:-${here}/../qtensor/libqtensor_hip.so}"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
# -ffp-contract=off: the nearest-entry rule needs two separately rounded fp32 subtractions.
# packed-fp32-ops is switched off for the device pass on this pool.
FLAGS=(-O3 -std=c++17 --offload-arch=gfx950 -fPIC -shared -ffp-contract=off -fno-fast-math
       -Xclang -target-feature -Xclang -packed-fp32-ops
       -Wall -Wno-unused-command-line-argument -I"${here}" -I"${here}/../../include")
srcs=("${here}"/qt_*.hip)
"${HIPCC}" "${FLAGS[@]}" "${srcs[@]}" -o "${out}" "$@"
echo "built ${out}"
