#!/bin/bash
# Builds libfwp_hip.so for gfx950 next to the package (in-tree, so it travels with the tree).
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
root="$(cd "$here/../.." && pwd)"
out="$here/../libfwp_hip.so"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
"$HIPCC" --offload-arch=gfx950 -O3 -std=c++17 -fPIC -shared \
    -Xclang -target-feature -Xclang -packed-fp32-ops -mllvm -amdgpu-mfma-vgpr-form \
    -I"$root/include" -I"$here" \
    "$here"/fwp_api.hip "$here"/fwp_generic.hip "$here"/fwp_delta_reg.hip "$here"/fwp_delta_mfma.hip "$here"/fwp_delta_split.hip "$here"/fwp_rnn_reg.hip "$here"/fwp_lstm_reg.hip "$here"/fwp_rec_reg.hip "$here"/fwp_layer.hip \
    -o "$out" "$@"
echo "built $out"
