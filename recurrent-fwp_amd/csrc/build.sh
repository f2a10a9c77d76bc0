#!/bin/bash
# Builds libfwp_hip.so for gfx950 next to the package (in-tree, so it travels with the tree).
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
root="$(cd "$here/../.." && pwd)"
out="$here/../libfwp_hip.so"
HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
common=(--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops
        -I"$root/include" -I"$here")
# the widest sum-rule kernels crash the compiler pass that -amdgpu-mfma-vgpr-form adds: compiled apart
wide="$(mktemp -d)/fwp_sum_wide.o"
"$HIPCC" "${common[@]}" -c "$here"/fwp_sum_wide.hip -o "$wide" "$@"
"$HIPCC" "${common[@]}" -shared -mllvm -amdgpu-mfma-vgpr-form "$wide" \
    "$here"/fwp_api.hip "$here"/fwp_generic.hip "$here"/fwp_delta_reg.hip "$here"/fwp_delta_mfma.hip "$here"/fwp_delta_split.hip "$here"/fwp_delta_phase.hip "$here"/fwp_rnn_reg.hip "$here"/fwp_lstm_reg.hip "$here"/fwp_rec_reg.hip "$here"/fwp_layer.hip "$here"/fwp_static.hip "$here"/fwp_step.hip \
    -o "$out" "$@"
echo "built $out"
