#!/bin/bash
# Compiles, from the reference tree where it lies, the part of the reference's own
# CPU code that builds from a few source files with g++ alone, into oracle/_ref/
# (git-ignored). Test infrastructure only: the outputs validate the oracle.
#   libref_hash.so : FarmHash Fingerprint64 + MurMurHash64 (column-io dataset helpers)
# Usage: oracle/ref_build.sh [reference_root]   (default /root/reference)
set -euo pipefail
HERE="$(cd "$(dirname "$0")" && pwd)"
REF="${1:-/root/reference}"
SRC="$REF/third_party/column-io/cc/column-io/dataset"
if [ ! -f "$SRC/farmhash.cc" ]; then
  echo "reference tree not found at $REF: skipping oracle/_ref" >&2
  exit 0
fi
mkdir -p "$HERE/_ref"
g++ -O2 -fPIC -shared -std=c++17 -fvisibility=hidden -w -I"$SRC" \
  "$HERE/ref_hash_driver.cc" "$SRC/farmhash.cc" "$SRC/hash_utils.cc" \
  -o "$HERE/_ref/libref_hash.so"
echo "built $HERE/_ref/libref_hash.so"
