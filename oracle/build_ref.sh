#!/bin/bash
# Compiles the reference library from the sources where they lie and uses it
# to lower the hot path's pipelines on the CPU.  Everything it writes goes to
# oracle/_ref/ (git-ignored).  Needs the reference tree; a no-op without it.
set -euo pipefail
REF=${GERN_REFERENCE:-/root/reference}
HERE=$(cd "$(dirname "$0")" && pwd)
OUT=$HERE/_ref
if [ ! -d "$REF/src" ]; then
    echo "reference tree not present at $REF: skipping oracle/_ref"
    exit 0
fi
mkdir -p "$OUT/obj"
cat > "$OUT/config.h" <<EOC
#pragma once
#define GERN_ROOT_DIR "$REF"
#define GERN_CUDA_ARCH ""
#define ORACLE_DIR "$HERE"
EOC
objs=()
for dir in annotations compose codegen utils; do
    for f in "$REF"/src/$dir/*.cpp; do
        o="$OUT/obj/${dir}_$(basename "${f%.cpp}").o"
        objs+=("$o")
        if [ ! -f "$o" ] || [ "$f" -nt "$o" ]; then
            echo "g++ -c $f"
            g++ -std=c++20 -O1 -w -I"$REF/include/gern" -c "$f" -o "$o" &
            # at most 8 compilers at once
            while [ "$(jobs -r | wc -l)" -ge 8 ]; do sleep 0.2; done
        fi
    done
done
wait
ar rcs "$OUT/libGernRef.a" "${objs[@]}"
g++ -std=c++20 -O1 -w -I"$REF/include/gern" -I"$REF/test" -I"$OUT" -I"$HERE" \
    "$HERE/ref_driver.cpp" "$OUT/libGernRef.a" -ldl -o "$OUT/ref_driver"
"$OUT/ref_driver" "$OUT"
echo "oracle/_ref built:"; cat "$OUT/manifest.txt"
