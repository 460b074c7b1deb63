#!/usr/bin/env bash
# TEST INFRASTRUCTURE ONLY.  Compiles the two dependency-free x86 kernels of the
# reference (code+score, weighted gather-add) straight from the sources where
# they lie under $REF, into oracle/_ref/ as Python extension modules.  They are
# used by the tests to pin the C restatement in this directory and, optionally,
# as the "reference" CPU baseline.  Nothing is copied out of the reference tree.
#
#   compute_code_score/torch_extension.cc  -> oracle/_ref/ccs_cpu.so
#   gather/cpu/torch_extension.cpp         -> oracle/_ref/gather_add_cpu.so
#
# The third x86 source (bh4/cpu/torch_extension.cpp) needs libxsmm, which this
# image does not have: it is unbuildable here and is not attempted.
set -euo pipefail
REF="${LFFN_REFERENCE_ROOT:-/root/reference}"
PL="$REF/src/roberta/models/prenorm_lookup"
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
OUT="$HERE/_ref"
if [ ! -d "$PL" ]; then
  echo "build_ref: $PL not present, nothing to do"; exit 0
fi
mkdir -p "$OUT"
PYINC="$(python3 -c 'import sysconfig; print(sysconfig.get_paths()["include"])')"
TORCH="$(python3 -c 'import torch, os; print(os.path.dirname(torch.__file__))')"
PYB="$(python3 -c 'import pybind11; print(pybind11.get_include())')"
ABI="$(python3 -c 'import torch; print(int(torch._C._GLIBCXX_USE_CXX11_ABI))')"
COMMON=(-O3 -mavx2 -mfma -fopenmp -fPIC -shared -std=c++17 -w
        -D_GLIBCXX_USE_CXX11_ABI="$ABI" -DTORCH_API_INCLUDE_EXTENSION_H
        -I"$PYINC" -I"$PYB" -I"$TORCH/include" -I"$TORCH/include/torch/csrc/api/include"
        -L"$TORCH/lib" -Wl,-rpath,"$TORCH/lib"
        -ltorch -ltorch_cpu -ltorch_python -lc10 -lgomp)
build_one() {  # name source
  g++ "$2" -o "$OUT/$1.so" -DTORCH_EXTENSION_NAME="$1" "${COMMON[@]}"
  echo "build_ref: built $OUT/$1.so"
}
build_one ccs_cpu        "$PL/compute_code_score/torch_extension.cc" &
build_one gather_add_cpu "$PL/gather/cpu/torch_extension.cpp" &
wait
