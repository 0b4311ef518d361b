#!/bin/bash
# TEST INFRASTRUCTURE ONLY.
# Drop-in proof: compiles the reference's own unit-test programs (test/test_*.cpp), unmodified and from
# where they lie, against THIS repository's include/ (the small:: API over the C ABI) and links them to
# smallframework_amd/lib/libsmall_hip.so.  Outputs go to oracle/_ref/tests/ (binaries only; nothing is
# copied out of the reference tree).  tests/test_reference_programs.py runs them on the GPU.
#
# Left out: test_ukernel_CONV.cpp, which tests the CPU platforms' micro-kernel macros
# (FLOAT_DEF_TILE_C ...), i.e. the part of the reference this library replaces.
set -uo pipefail
REF_ROOT="${1:-/root/reference}"
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
ROOT="$(dirname "$HERE")"
OUT="$HERE/_ref/tests"
LIBDIR="$ROOT/smallframework_amd/lib"
if [ ! -d "$REF_ROOT/test" ]; then
    echo "build_ref_tests.sh: $REF_ROOT/test not found; skipping" >&2
    exit 3
fi
mkdir -p "$OUT"
JOBS="${JOBS:-8}"
fail=0
pids=()
names=()
for src in "$REF_ROOT"/test/test_*.cpp; do
    name="$(basename "$src" .cpp)"
    [ "$name" = "test_ukernel_CONV" ] && continue
    g++ -std=c++17 -O1 -w -fpermissive -I "$ROOT/include" -I "$REF_ROOT/test/include" -I "$REF_ROOT/test" \
        "$src" -o "$OUT/$name" -L"$LIBDIR" -lsmall_hip -Wl,-rpath,'$ORIGIN/../../../smallframework_amd/lib' \
        > "$OUT/$name.log" 2>&1 &
    pids+=($!)
    names+=("$name")
    if [ "${#pids[@]}" -ge "$JOBS" ]; then
        wait "${pids[0]}" || { echo "FAILED ${names[0]}" >&2; fail=1; }
        pids=("${pids[@]:1}")
        names=("${names[@]:1}")
    fi
done
for i in "${!pids[@]}"; do
    wait "${pids[$i]}" || { echo "FAILED ${names[$i]}" >&2; fail=1; }
done
find "$OUT" -name '*.log' -size 0 -delete
ls "$OUT"
exit $fail
