#!/usr/bin/env bash
# TEST INFRASTRUCTURE ONLY. Compiles the reference's own x86 C++ extension, from the sources
# where they lie under /root/reference, into oracle/_ref/ (git-ignored). Nothing is copied.
# The result is used by tests/ and bench.py's cpu_baseline leg as a checker / CPU baseline;
# the product never loads it.
#
# Built files (reference tree, read-only): super_gnn/ops/csrc/{utils,spmm,ops,vertex_cover,
# quantization_x86}.cpp -- the file set and flags super_gnn/ops/setup.py:11-36,52-55 selects
# on an AVX-512 host. The ARM/SVE half (quantization_arm.cpp) needs <arm_sve.h> and cannot be
# built on x86, so *_for_all_procs has no executable reference here.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
REF="${SGNN_REFERENCE_ROOT:-/root/reference}"
SRC="$REF/super_gnn/ops/csrc"
OUT="$HERE/_ref"
if [ ! -d "$SRC" ]; then echo "build_ref: $SRC not present, skipping"; exit 0; fi
if ! grep -q avx512f /proc/cpuinfo; then echo "build_ref: host has no avx512f, skipping"; exit 0; fi
mkdir -p "$OUT/obj"
PY=python3
INC=$($PY - <<'PY'
import sysconfig
from torch.utils.cpp_extension import include_paths
print(" ".join("-I" + p for p in include_paths() + [sysconfig.get_paths()["include"]]))
PY
)
TLIB=$($PY -c "from torch.utils.cpp_extension import library_paths; print(library_paths()[0])")
ABI=$($PY -c "import torch; print(int(torch._C._GLIBCXX_USE_CXX11_ABI))")
EXT=$($PY -c "import sysconfig; print(sysconfig.get_config_var('EXT_SUFFIX'))")
FLAGS="-O3 -std=c++17 -fPIC -fopenmp -mavx512f -mavx512cd -mavx512bw -mavx512dq -mavx512vl -mavx512ifma -mavx512vbmi \
 -DTORCH_EXTENSION_NAME=supergnn_ops -DTORCH_API_INCLUDE_EXTENSION_H -D_GLIBCXX_USE_CXX11_ABI=$ABI -w"
pids=()
for f in utils spmm ops vertex_cover quantization_x86; do
  g++ $FLAGS $INC -I"$SRC" -c "$SRC/$f.cpp" -o "$OUT/obj/$f.o" &
  pids+=($!)
done
for p in "${pids[@]}"; do wait "$p"; done
g++ -shared -fopenmp "$OUT"/obj/*.o -L"$TLIB" -Wl,-rpath,"$TLIB" -ltorch -ltorch_cpu -ltorch_python -lc10 \
  -o "$OUT/supergnn_ops$EXT"
rm -rf "$OUT/obj"
echo "build_ref: wrote $OUT/supergnn_ops$EXT"
