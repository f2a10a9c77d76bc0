#!/bin/bash
# Builds _fwp_torch.so (the C++ autograd binding over libfwp_hip.so) next to the package.
# Host code only: g++ against PyTorch's headers; libfwp_hip.so must have been built first.
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
root="$(cd "$here/../.." && pwd)"
pkg="$here/.."
PY="${PYTHON:-python3}"
read -r TORCH_INC TORCH_LIB PY_INC CXX11 <<<"$("$PY" - <<'PYEOF'
import sysconfig, torch
from torch.utils import cpp_extension as ce
print(" ".join("-I" + p for p in ce.include_paths()).replace(" ", ","), ce.library_paths()[0],
      sysconfig.get_paths()["include"], int(torch._C._GLIBCXX_USE_CXX11_ABI))
PYEOF
)"
g++ -O2 -std=c++17 -fPIC -shared -fvisibility=hidden \
    -D__HIP_PLATFORM_AMD__=1 -DUSE_ROCM=1 -DTORCH_EXTENSION_NAME=_fwp_torch -DTORCH_API_INCLUDE_EXTENSION_H \
    -D_GLIBCXX_USE_CXX11_ABI="$CXX11" \
    ${TORCH_INC//,/ } -I"$PY_INC" -I/opt/rocm/include -I"$root/include" \
    "$here"/fwp_torch.cpp \
    -L"$TORCH_LIB" -ltorch -ltorch_cpu -ltorch_python -lc10 -lc10_hip \
    -L"$pkg" -lfwp_hip -Wl,-rpath,'$ORIGIN' \
    -o "$pkg/_fwp_torch.so" "$@"
echo "built $pkg/_fwp_torch.so"
