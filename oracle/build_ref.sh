#!/bin/sh
# Builds oracle/_ref/libref_sampler.so from the reference's own sampler.cpp, read in
# place under /root/reference (never copied).  Only works where /root/reference is
# mounted; the result is git-ignored but travels to the GPU box as a built file.
set -e
HERE="$(cd "$(dirname "$0")" && pwd)"
REF="${ET_REFERENCE_ROOT:-/root/reference}"
OUT="$HERE/_ref"
if [ ! -f "$REF/extension/llm/sampler/sampler.cpp" ]; then
  echo "build_ref: $REF not present, skipping" >&2
  exit 0
fi
mkdir -p "$OUT/inc"
ln -sfn "$REF" "$OUT/inc/executorch"   # provides the <executorch/...> include prefix
g++ -std=c++17 -O2 -w -fPIC -shared \
    -I "$OUT/inc" -I "$REF/runtime/core/portable_type/c10" \
    -DC10_USING_CUSTOM_GENERATED_MACROS \
    "$REF/extension/llm/sampler/sampler.cpp" "$HERE/ref_shim.cpp" \
    -o "$OUT/libref_sampler.so"
rm -rf "$OUT/inc"
echo "build_ref: wrote $OUT/libref_sampler.so"
