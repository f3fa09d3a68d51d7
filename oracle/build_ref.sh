#!/bin/bash
# Builds the reference's own CPU path (its pybind dispatcher + scalar CPU loops)
# straight from the sources where they lie under /root/reference into
# oracle/_ref/window_matmul_kernel_ref.so.  Nothing is copied; only the two .cpp
# files that make up the reference's CPU-only build are compiled
# (reference setup.py:22-32 selects exactly these when no CUDA toolkit exists).
#
# The result is test infrastructure: it pins the C restatement in
# oracle/window_matmul_oracle.c and may serve as the timed CPU baseline.
# It is never imported by the product path.
set -euo pipefail
REF=${WM_REFERENCE_ROOT:-/root/reference}
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
OUT="$HERE/_ref"
if [ ! -d "$REF/csrc/window_matmul" ]; then
  echo "build_ref: $REF not present, skipping" >&2
  exit 0
fi
mkdir -p "$OUT"
TORCH_DIR=$(python3 -c "import torch, os; print(os.path.dirname(torch.__file__))")
PY_INC=$(python3 -c "import sysconfig; print(sysconfig.get_paths()['include'])")
g++ -O3 -std=c++17 -fPIC -shared -Wno-sign-compare -Wno-deprecated-declarations \
  -DTORCH_EXTENSION_NAME=window_matmul_kernel_ref -DTORCH_API_INCLUDE_EXTENSION_H \
  -D_GLIBCXX_USE_CXX11_ABI=1 \
  -I"$REF/csrc/window_matmul" \
  -I"$TORCH_DIR/include" -I"$TORCH_DIR/include/torch/csrc/api/include" -I"$PY_INC" \
  "$REF/csrc/window_matmul/window_matmul.cpp" \
  "$REF/csrc/window_matmul/cpu/window_matmul_cpu.cpp" \
  -L"$TORCH_DIR/lib" -Wl,-rpath,"$TORCH_DIR/lib" \
  -ltorch_python -ltorch -ltorch_cpu -lc10 \
  -o "$OUT/window_matmul_kernel_ref.so"
echo "build_ref: wrote $OUT/window_matmul_kernel_ref.so"
