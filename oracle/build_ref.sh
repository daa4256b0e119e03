#!/bin/sh
# Compile plow's own CPU kernel library (runtime/cpu/dev) straight from the mounted plow tree into
# oracle/_ref/libplow_ref.so, plus the thin driver ref_shim.c. Outputs go only to oracle/_ref/
# (git-ignored). Flags follow runtime/CMakeLists.txt:92-118; AMD clang is used because gcc 11
# cannot build the AVX-512 BF16 tier.
set -e
REF="${1:-/root/reference}"
HERE="$(cd "$(dirname "$0")" && pwd)"
R="$REF/runtime"
[ -d "$R/cpu/dev" ] || { echo "build_ref: no plow tree at $REF (skipped)"; exit 0; }
CC="${REFCC:-/opt/rocm/lib/llvm/bin/clang}"
OUT="$HERE/_ref"
OBJ="$OUT/obj"
mkdir -p "$OBJ"
CF="-std=c11 -O2 -w -fPIC -I$R/common -I$R/cpu/dev -I$R/cpu"
for f in "$R"/cpu/dev/*.c "$R"/cpu/dev/golden/*.c; do
  $CC $CF -c "$f" -o "$OBJ/$(basename "$(dirname "$f")")_$(basename "$f" .c).o"
done
for f in "$R"/cpu/dev/avx512/*.c; do
  $CC $CF -mavx512f -mavx512bw -mavx512vl -mavx512bf16 -mavx512vnni -c "$f" -o "$OBJ/avx512_$(basename "$f" .c).o"
done
for f in "$R"/cpu/dev/amx/*.c; do
  $CC $CF -mavx512f -mavx512bw -mavx512vl -mavx512bf16 -mavx512vnni -mamx-tile -mamx-bf16 -mamx-int8 \
      -c "$f" -o "$OBJ/amx_$(basename "$f" .c).o"
done
$CC $CF -c "$HERE/ref_shim.c" -o "$OBJ/ref_shim.o"
$CC -shared -o "$OUT/libplow_ref.so" "$OBJ"/*.o -lm -lpthread
echo "build_ref: wrote $OUT/libplow_ref.so"
