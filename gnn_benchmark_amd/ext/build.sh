#!/usr/bin/env bash
# Builds the pybind11 module `computation_ops` (computation_ops.cpp) against the installed PyTorch-ROCm headers and
# links it with ../csrc/libgnnagg.so (found at run time through an rpath relative to this directory).  Host code
# only: g++ is enough, no GPU and no hipcc needed.  The counterpart of the reference's model/ops/setup.py.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
ROOT="$(cd "$HERE/../.." && pwd)"
PY=${PYTHON:-python3}
TORCH_DIR="$($PY -c 'import torch,os;print(os.path.dirname(torch.__file__))')"
PY_INC="$($PY -c 'import sysconfig;print(sysconfig.get_paths()["include"])')"
EXT="$($PY -c 'import sysconfig;print(sysconfig.get_config_var("EXT_SUFFIX"))')"
ROCM=${ROCM_PATH:-/opt/rocm}
CXX=${CXX:-g++}
test -f "$HERE/../csrc/libgnnagg.so" || { echo "build libgnnagg.so first (make -C gnn_benchmark_amd/csrc)"; exit 1; }
"$CXX" -O2 -std=c++17 -fPIC -shared -w \
    -D__HIP_PLATFORM_AMD__=1 -DUSE_ROCM=1 -DTORCH_EXTENSION_NAME=computation_ops -DTORCH_API_INCLUDE_EXTENSION_H \
    -D_GLIBCXX_USE_CXX11_ABI=1 \
    -I"$ROOT/include" -I"$TORCH_DIR/include" -I"$TORCH_DIR/include/torch/csrc/api/include" -I"$ROCM/include" -I"$PY_INC" \
    "$HERE/computation_ops.cpp" -o "$HERE/computation_ops$EXT" \
    -L"$HERE/../csrc" -lgnnagg -Wl,-rpath,'$ORIGIN/../csrc' \
    -L"$TORCH_DIR/lib" -Wl,-rpath,"$TORCH_DIR/lib" -lc10 -lc10_hip -ltorch_cpu -ltorch_hip -ltorch -ltorch_python
echo "wrote $HERE/computation_ops$EXT"
