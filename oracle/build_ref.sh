#!/bin/bash
# Builds the reference's DSL front end + CUDA code generator (plain C++14, no CUDA needed to *run the generator*)
# from the sources where they lie under /root/reference into oracle/_ref/.  Used only as a text oracle for the
# code-generation tests (which stages fuse, operand order of emitted expressions); never for numerics, never shipped.
# The reference's device code (CUDA inside modified NCCL, MPI host code) cannot be built in this image.
set -euo pipefail
REF=${REF:-/root/reference}
HERE="$(cd "$(dirname "$0")" && pwd)"
OUT="$HERE/_ref"
mkdir -p "$OUT"
CXX=${CXX:-g++}
FLAGS="-std=c++14 -O1 -w -fPIC -I $REF/src"
for o in codegen dsl pipeline utils; do
  if [ ! -f "$OUT/$o.o" ] || [ "$REF/src/$o.cpp" -nt "$OUT/$o.o" ]; then
    $CXX $FLAGS -c "$REF/src/$o.cpp" -o "$OUT/$o.o" &
  fi
done
wait
# one shared object for the generator, so that the four example programs stay a few KB each (the directory travels with
# every GPU run although only CPU tests use it)
$CXX -shared -s -o "$OUT/libccnref.so" "$OUT"/codegen.o "$OUT"/dsl.o "$OUT"/pipeline.o "$OUT"/utils.o
for ex in sgd adam lamb model-parallel; do
  $CXX $FLAGS "$REF/examples/$ex/$ex.cpp" -L"$OUT" -lccnref -Wl,-rpath,'$ORIGIN' -s -o "$OUT/ref-$ex" &
done
wait
echo "built: $(ls "$OUT" | tr '\n' ' ')"
