#!/usr/bin/env bash
# Build oracle/_ref/libcake_ref_parts.so: the parts of the reference that
# compile from their own sources where they lie under /root/reference, with
# g++ directly (the reference's build system is not run).
#
# What builds:  src/pack_*.cpp, src/unpack_*.cpp (packing layouts and sizes),
#               src/kernels/haswell/dense.cpp (6x16 micro-kernel; needs only
#               <immintrin.h>, supplied with -include),
#               examples/cake_gemv.cpp (schedule_mvm + 8-row kernel),
#               examples/cake_conv.cpp (im_2_col).
# What does not: src/block_sizing.cpp (needs the grid_dims table that
#               python/grid_gen.py prepends to tiling.h), src/cake_sgemm*.cpp
#               (need the generated include/kernels.h).  Those stay unbuilt.
#
# Test infrastructure only; outputs go to oracle/_ref/ (git-ignored).
set -euo pipefail
REF="${CAKE_REFERENCE_DIR:-/root/reference}"
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
OUT="$HERE/_ref"
if [ ! -d "$REF/src" ]; then
    echo "build_ref.sh: $REF not present, nothing built" >&2
    exit 0
fi
mkdir -p "$OUT/obj"
CXX="${CXX:-g++}"
# Makefile:129 flags of the reference (-O2 -mavx -mfma -fopenmp) + -mavx2 for the gemv example
FLAGS="-O2 -mavx -mavx2 -mfma -mtune=haswell -fopenmp -fPIC -w -I$REF/include -fvisibility=hidden -ffunction-sections"
for f in pack_ob pack_k_first pack_m_first pack_n_first pack_helper unpack_k_first unpack_m_first unpack_n_first; do
    $CXX $FLAGS -c "$REF/src/$f.cpp" -o "$OUT/obj/$f.o"
done
$CXX $FLAGS -include immintrin.h -c "$REF/src/kernels/haswell/dense.cpp" -o "$OUT/obj/dense.o"
$CXX $FLAGS -Dmain=cake_gemv_example_main -c "$REF/examples/cake_gemv.cpp" -o "$OUT/obj/gemv.o"
$CXX $FLAGS -Dmain=cake_conv_example_main -c "$REF/examples/cake_conv.cpp" -o "$OUT/obj/conv.o"
$CXX $FLAGS -c "$HERE/ref_shim.cpp" -o "$OUT/obj/ref_shim.o"
# hidden visibility + section GC drops the example mains (and their calls into
# the parts of the library that were not built) from the link
$CXX -shared -fopenmp -Wl,--gc-sections -Wl,-z,defs -o "$OUT/libcake_ref_parts.so" "$OUT"/obj/*.o -lm
echo "built $OUT/libcake_ref_parts.so"
