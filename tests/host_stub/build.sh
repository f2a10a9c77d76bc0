#!/bin/bash
# Builds, into the directory given as $1, the stand-in libfwp_hip.so (fwp_stub.c) and _fwp_torch_host.so:
# csrc/fwp_torch.cpp compiled with -DFWP_HOST_STUB against it (host tensors, no GPU).  $2 = "asan" adds
# -fsanitize=address to both (the Python process that imports the module then needs libasan preloaded).
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
root="$(cd "$here/../.." && pwd)"
out="$1"
san=""
[ "${2:-}" = asan ] && san="-fsanitize=address -fno-omit-frame-pointer -g"
mkdir -p "$out"
PY="${PYTHON:-python3}"
read -r TORCH_INC TORCH_LIB PY_INC CXX11 <<<"$("$PY" - <<'PYEOF'
import sysconfig, torch
from torch.utils import cpp_extension as ce
print(" ".join("-I" + p for p in ce.include_paths()).replace(" ", ","), ce.library_paths()[0],
      sysconfig.get_paths()["include"], int(torch._C._GLIBCXX_USE_CXX11_ABI))
PYEOF
)"
# shellcheck disable=SC2086
gcc -O1 -std=c11 -fPIC -shared $san -I"$root/include" "$here/fwp_stub.c" -o "$out/libfwp_hip.so"
# shellcheck disable=SC2086
g++ -O1 -std=c++17 -fPIC -shared -fvisibility=hidden $san \
    -DFWP_HOST_STUB=1 -DTORCH_EXTENSION_NAME=_fwp_torch_host -DTORCH_API_INCLUDE_EXTENSION_H \
    -D_GLIBCXX_USE_CXX11_ABI="$CXX11" \
    ${TORCH_INC//,/ } -I"$PY_INC" -I"$root/include" \
    "$root/recurrent-fwp_amd/csrc/fwp_torch.cpp" \
    -L"$TORCH_LIB" -ltorch -ltorch_cpu -ltorch_python -lc10 \
    -L"$out" -lfwp_hip -Wl,-rpath,'$ORIGIN' \
    -o "$out/_fwp_torch_host.so"
echo "built $out/_fwp_torch_host.so"
