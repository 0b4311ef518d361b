#!/bin/bash
# TEST INFRASTRUCTURE ONLY.
# Compiles the SMaLL reference (header-only C++17) from where it lies into two
# shared objects under oracle/_ref/ through oracle/ref_shim.cpp:
#   libsmall_ref_REF.so   REF platform  (scalar; float + quint8)
#   libsmall_ref_ZEN2.so  ZEN2 platform (AVX2/FMA; float only)
# Flags follow the reference's CMakeLists.txt (-fopenmp -O3 -fpermissive,
# -DUARCH_REF for REF, -mavx2 -mfma for ZEN2) except that -march=native is
# dropped so the binary built in one container runs on another x86-64 host
# with AVX2.  Nothing is copied out of the reference tree.
set -euo pipefail
REF_ROOT="${1:-/root/reference}"
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
OUT="$HERE/_ref"
if [ ! -f "$REF_ROOT/include/small.h" ]; then
    echo "build_ref.sh: $REF_ROOT/include/small.h not found; skipping" >&2
    exit 3
fi
mkdir -p "$OUT"
COMMON="-std=c++17 -O3 -fopenmp -fpermissive -w -shared -fPIC -I $REF_ROOT/include"
g++ $COMMON -DUARCH_REF -I "$REF_ROOT/include/small/platforms/reference" \
    "$HERE/ref_shim.cpp" -o "$OUT/libsmall_ref_REF.so" &
g++ $COMMON -mavx2 -mfma -I "$REF_ROOT/include/small/platforms/zen2" \
    "$HERE/ref_shim.cpp" -o "$OUT/libsmall_ref_ZEN2.so" &
wait
ls -la "$OUT"
