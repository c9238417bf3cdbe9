#!/usr/bin/env bash
# TEST INFRASTRUCTURE -- not part of the product.
#
# Builds the reference's own native operator module (pybind11; `computation_ops` in the
# reference's setup.py) straight from its sources where they lie under /root/reference, with g++ only
# (no reference build system is run).  The output goes to oracle/_ref/ which is
# git-ignored; no reference source is copied into this repository.
#
# Sources compiled (unchanged, in place):
#   self_benchmark/a64fx/model/ops/src/{spmm.cpp,utils.cpp,ops.cpp,quantization_x86.cpp}
# The x86 path of the reference requires AVX-512 (spmm.cpp:62, kernel_1xN exists
# only under __AVX512F__ or SVE), so the flags below name the AVX-512 subsets it uses.
#
# The module is built under the name `reference_computation_ops` (the name is a macro in the
# reference's ops.cpp:11): pybind11 keeps one module object per module NAME in a process, so a
# second pybind11 module called `computation_ops` -- the product's drop-in is one -- would get
# this module's object back from its own init, or the other way round.
#
# Usage: oracle/build_ref.sh            (silently skips when /root/reference is absent)
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
REF="${GNN_REFERENCE_ROOT:-/root/reference}/self_benchmark/a64fx/model/ops/src"
OUT="$HERE/_ref"
if [ ! -f "$REF/spmm.cpp" ]; then
    echo "build_ref: $REF not present, skipping reference build"
    exit 0
fi
mkdir -p "$OUT"
PY=${PYTHON:-python3}
TORCH_DIR="$($PY -c 'import torch,os;print(os.path.dirname(torch.__file__))')"
PY_INC="$($PY -c 'import sysconfig;print(sysconfig.get_paths()["include"])')"
EXT="$($PY -c 'import sysconfig;print(sysconfig.get_config_var("EXT_SUFFIX"))')"
CXX=${CXX:-g++}
FLAGS=(-O3 -std=c++17 -fPIC -shared -fopenmp
       -mavx512f -mavx512cd -mavx512bw -mavx512dq -mavx512vl -mfma
       -DTORCH_EXTENSION_NAME=reference_computation_ops -DTORCH_API_INCLUDE_EXTENSION_H
       -D_GLIBCXX_USE_CXX11_ABI=1 -w
       -I"$TORCH_DIR/include" -I"$TORCH_DIR/include/torch/csrc/api/include" -I"$PY_INC")
LIBS=(-L"$TORCH_DIR/lib" -Wl,-rpath,"$TORCH_DIR/lib" -lc10 -ltorch_cpu -ltorch -ltorch_python)
"$CXX" "${FLAGS[@]}" "$REF/spmm.cpp" "$REF/utils.cpp" "$REF/ops.cpp" "$REF/quantization_x86.cpp" \
    -o "$OUT/reference_computation_ops$EXT" "${LIBS[@]}"
rm -f "$OUT"/computation_ops*.so
echo "build_ref: wrote $OUT/reference_computation_ops$EXT"
