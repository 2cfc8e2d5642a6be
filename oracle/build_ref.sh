#!/bin/sh
# Compiles the reference's own native/ranges/ranges.cpp, from where it lies, into
# oracle/_ref/km_ranges_ref.so (a Python extension exporting make_ranges,
# make_ranges_symmetric, transpose_ranges).  Used only to validate ranges_oracle.c and to
# write the golden vectors under tests/golden/.  Needs g++, the installed torch headers and
# the reference tree; does nothing (exit 0) when the reference tree is absent.
#
# The CUDA operators of the reference (native/*/*.cu) are not buildable here: they need nvcc
# and the CUDA toolkit headers, which this image does not have.
set -e
REF="${KM_REFERENCE_ROOT:-/root/reference}"
HERE="$(cd "$(dirname "$0")" && pwd)"
SRC="$REF/native/ranges/ranges.cpp"
if [ ! -f "$SRC" ]; then
    echo "build_ref.sh: $SRC not found, skipping"
    exit 0
fi
TORCH_DIR="$(python3 -c 'import os, torch; print(os.path.dirname(torch.__file__))')"
PY_INC="$(python3 -c 'import sysconfig; print(sysconfig.get_paths()["include"])')"
mkdir -p "$HERE/_ref"
g++ -O2 -std=c++17 -shared -fPIC -DTORCH_EXTENSION_NAME=km_ranges_ref \
    -DTORCH_API_INCLUDE_EXTENSION_H -D_GLIBCXX_USE_CXX11_ABI=1 \
    -I"$TORCH_DIR/include" -I"$TORCH_DIR/include/torch/csrc/api/include" -I"$PY_INC" \
    "$SRC" -o "$HERE/_ref/km_ranges_ref.so" \
    -L"$TORCH_DIR/lib" -ltorch -ltorch_cpu -ltorch_python -lc10 -Wl,-rpath,"$TORCH_DIR/lib"
echo "build_ref.sh: built $HERE/_ref/km_ranges_ref.so"
