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

#   ref_ops        : the reference's CPU operators (csrc/ops/*.cc) and its CPU table and sparse
#                    optimizers (csrc/embedding/*.cc), and the parts of its checkpoint code that
#                    need no CUDA header (csrc/serialize: writer of one data file, reader of the
#                    directory's index and headers; csrc/platform: the file system layer) compiled against the installed torch headers and driven by
#                    ref_ops_driver.cc. Their CUDA counterparts (*_cuda / *_gpu, defined in .cu
#                    files that need nvcc) stay unresolved: the binary binds lazily and every
#                    tensor it sees is on the CPU, so they are never reached.
TORCH="$(python3 -c 'import torch, os; print(os.path.dirname(torch.__file__))')"
PYINC="$(python3 -c 'import sysconfig; print(sysconfig.get_paths()["include"])')"
ABI="$(python3 -c 'import torch; print(int(torch._C._GLIBCXX_USE_CXX11_ABI))')"
CSRC="$REF/csrc"
OBJ="$HERE/_ref/obj"
mkdir -p "$OBJ"
CXXFLAGS="-std=c++17 -O2 -fPIC -fopenmp -w -D_GLIBCXX_USE_CXX11_ABI=$ABI -I$CSRC -I$CSRC/ops -I$REF/third_party -I$TORCH/include -I$TORCH/include/torch/csrc/api/include -I$PYINC"
SOURCES="ops/block_apply_adamw_op.cc ops/hashtable_ops.cc ops/block_ops.cc ops/ids_partition.cc ops/ids_encode.cc
         ops/fused_uint64_mod.cc ops/fused_bucketized.cc ops/multi_hash.cc ops/dense_to_ragged.cc
         embedding/id_allocator.cc embedding/cpu_id_map.cc embedding/parallel_util.cc
         embedding/hashtable.cc embedding/slot_group.cc embedding/initializer.cc embedding/children_info.cc
         embedding/slice_info.cc embedding/optim.cc embedding/adam.cc embedding/adamw.cc embedding/adamw_tf.cc
         serialize/string_sep.cc serialize/register_preserved_key.cc utils/str_util.cc utils/scanner.cc
         serialize/block_info.cc serialize/index_info.cc serialize/load_bundle.cc serialize/name.cc
         serialize/table_reader.cc serialize/table_writer.cc serialize/write_block.cc serialize/dtype_serialize.cc
         platform/env.cc platform/filesystem.cc platform/path.cc platform/status.cc platform/fileoutput_buffer.cc
         platform/file_system_helper.cc platform/posix/env.cc platform/posix/posix_filesystem.cc"
# Objects are kept between runs and recompiled only when their source is newer (each file takes
# about 25 s against the torch headers).
pids=()
compile() {  # source, object
  if [ ! -f "$2" ] || [ "$1" -nt "$2" ] || [ "$HERE/ref_build.sh" -nt "$2" ]; then
    ( g++ $CXXFLAGS -c "$1" -o "$2" ) &
    pids+=($!)
    if [ "${#pids[@]}" -ge 7 ]; then wait "${pids[0]}"; pids=("${pids[@]:1}"); fi
  fi
}
for s in $SOURCES; do
  compile "$CSRC/$s" "$OBJ/$(echo "$s" | tr '/' '_' | sed 's/\.cc$/.o/')"
done
compile "$HERE/ref_ops_driver.cc" "$OBJ/driver.o"
for p in "${pids[@]}"; do wait "$p"; done
PYLIB="$(python3 -c 'import sysconfig; print(sysconfig.get_config_var("LIBDIR"))')"
# The reference objects go into a shared library, where undefined symbols are allowed; the driver
# links against it with lazy binding, so a function that is never called is never looked up.
g++ -shared -fopenmp -o "$HERE/_ref/libref_ops.so" $(ls "$OBJ"/*.o | grep -v driver.o) \
  -Wl,-z,lazy -Wl,-rpath,"$TORCH/lib" \
  -L"$TORCH/lib" -ltorch -ltorch_cpu -lc10 -ltorch_python -L"$PYLIB" -lpython3.10
g++ -fopenmp -o "$HERE/_ref/ref_ops" "$OBJ/driver.o" \
  -Wl,--allow-shlib-undefined -Wl,-z,lazy -Wl,-rpath,'$ORIGIN' -Wl,-rpath,"$TORCH/lib" \
  -L"$HERE/_ref" -lref_ops -L"$TORCH/lib" -ltorch -ltorch_cpu -lc10 -L"$PYLIB" -lpython3.10
echo "built $HERE/_ref/ref_ops"
