#!/bin/sh
# Builds oracle/_ref/libtokspur_ref.so from the reference's own CPU sources where they lie
# (read-only tree, default /root/reference) plus ref_shim.cpp. Nothing is copied; outputs go to
# oracle/_ref/ only. Without the reference tree this is a no-op that reports so.
set -e
HERE="$(cd "$(dirname "$0")" && pwd)"
REF="${TOKSPUR_REFERENCE:-/root/reference}/native"
if [ ! -d "$REF/src" ]; then echo "reference tree absent: oracle/_ref not rebuilt"; exit 0; fi
mkdir -p "$HERE/_ref"
SRCS="gguf numeric routing operators q8_many expert_lanes grouped_mm moe_mm_many_plan sampling"
OBJS=""
for s in $SRCS; do
  g++ -std=c++20 -O2 -fPIC -ffp-contract=off -DTOKSPUR_PRIVATE_GROUPED_MM=1 -I"$REF/include" \
      -c "$REF/src/$s.cpp" -o "$HERE/_ref/$s.o"
  OBJS="$OBJS $HERE/_ref/$s.o"
done
g++ -std=c++20 -O2 -fPIC -ffp-contract=off -DTOKSPUR_PRIVATE_GROUPED_MM=1 -I"$REF/include" \
    -c "$HERE/ref_shim.cpp" -o "$HERE/_ref/ref_shim.o"
g++ -shared -o "$HERE/_ref/libtokspur_ref.so" "$HERE/_ref/ref_shim.o" $OBJS -Wl,-z,defs -lpthread
rm -f "$HERE"/_ref/*.o
echo "built $HERE/_ref/libtokspur_ref.so"
