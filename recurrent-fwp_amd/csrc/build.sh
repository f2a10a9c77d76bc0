#!/bin/bash
# Builds libfwp_hip.so for gfx950 next to the package (in-tree, so it travels with the tree).
# Every source file is compiled to an object of its own, FWP_JOBS at a time (default 8), then linked.
# Arguments go to every compile line; FWP_OUT names another output file (a build for a measurement, e.g.
# FWP_OUT=/tmp/libfwp_nb.so build.sh -DFWP_TIMING_WITHOUT_BARRIERS, timed with bench.py --lib).
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
root="$(cd "$here/../.." && pwd)"
out="${FWP_OUT:-$here/../libfwp_hip.so}"
export HIPCC="${HIPCC:-/opt/rocm/bin/hipcc}"
export FWP_OBJ="$(mktemp -d)"
trap 'rm -rf "$FWP_OBJ"' EXIT
export FWP_COMMON="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops -I$root/include -I$here $*"
# the widest sum-rule kernels crash the compiler pass that -amdgpu-mfma-vgpr-form adds: compiled without it
compile_one() {
    src="$1"
    extra="-mllvm -amdgpu-mfma-vgpr-form"
    [ "$(basename "$src")" = fwp_sum_wide.hip ] && extra=""
    # shellcheck disable=SC2086
    "$HIPCC" $FWP_COMMON $extra -c "$src" -o "$FWP_OBJ/$(basename "$src" .hip).o"
}
export -f compile_one
ls "$here"/*.hip | xargs -P "${FWP_JOBS:-8}" -I{} bash -c 'compile_one "$@"' _ {}
# shellcheck disable=SC2086
"$HIPCC" --offload-arch=gfx950 -shared -fPIC "$FWP_OBJ"/*.o -o "$out"
echo "built $out"
