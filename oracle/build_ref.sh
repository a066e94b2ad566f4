#!/usr/bin/env bash
# Builds the reference's own CPU contraction and CPU permutation (host-only, no GPU
# needed) from the sources where they lie under /root/reference, plus a small C-ABI shim of ours,
# into oracle/_ref/libref_cpu.so.  TEST INFRASTRUCTURE ONLY: the product never
# loads this library.  Nothing from the reference is copied into this repository;
# only the compiled object leaves this script.
#
# The reference's CPU path needs the Composable Kernel host headers, which it
# does not vendor; the ROCm image carries CK under /opt/rocm/include/ck.
set -euo pipefail
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
REF="${HIPTENSOR_REFERENCE_ROOT:-/root/reference}"
OUT="$HERE/_ref"
R="$REF/library"
if [ ! -d "$R/src/contraction" ]; then
  echo "build_ref.sh: reference tree not found at $REF; skipping" >&2
  exit 0
fi
mkdir -p "$OUT/obj"
CKCM=/opt/rocm/lib/cmake/composable_kernel
INC=$(grep -h INTERFACE_INCLUDE_DIRECTORIES \
        "$CKCM/composable_kerneldevice_other_operationsTargets.cmake" \
        "$CKCM/composable_kerneldevice_contraction_operationsTargets.cmake" \
      | sed 's/.*DIRECTORIES "//; s/"$//' | tr ';' '\n' \
      | sed 's#${_IMPORT_PREFIX}#/opt/rocm#' | sort -u | sed 's/^/-I/' | tr '\n' ' ')
CXX=/opt/rocm/bin/hipcc
# HIPTENSOR_DATA_LAYOUT_COL_MAJOR=1 is the definition the reference's own build passes by
# default (CMakeLists.txt:69,119-120); its permutation sources do not compile without it.
# NDEBUG as in a release build: without it the permutation sources print a line per call.
FLAGS="-std=c++17 -x hip --cuda-host-only -O2 -fPIC -w -DNDEBUG -DHIPTENSOR_DATA_LAYOUT_COL_MAJOR=1 -I$R/include -I$R/src/include -I$R/src/contraction -I$R/src/permutation $INC"
# The reference's CPU permutation class derives from a Composable Kernel device operation
# (library/src/permutation/permutation_cpu_reference_impl.hpp:47-63), so its instance files
# carry device code and are compiled in full for gfx950; everything else is host-only.
DEVFLAGS="${FLAGS/--cuda-host-only/--offload-arch=gfx950}"
pids=()
for f in contraction/contraction_cpu_reference.cpp \
         contraction/contraction_cpu_reference_instances.cpp \
         contraction/contraction_solution.cpp \
         contraction/contraction_solution_registry.cpp \
         contraction/contraction_types.cpp \
         permutation/permutation_cpu_reference.cpp \
         permutation/permutation_cpu_reference_instances.cpp \
         permutation/permutation_solution.cpp \
         permutation/permutation_solution_registry.cpp \
         permutation/permutation_types.cpp \
         data_types.cpp; do
  o="$OUT/obj/ref_$(basename "$f" .cpp).o"
  $CXX $FLAGS -c "$R/src/$f" -o "$o" &
  pids+=($!)
done
for r in 2 3 4 5 6; do
  f="permutation/permutation_cpu_reference_rank${r}_instances.cpp"
  $CXX $DEVFLAGS -c "$R/src/$f" -o "$OUT/obj/ref_$(basename "$f" .cpp).o" &
  pids+=($!)
done
$CXX $FLAGS -c "$HERE/ref_shim.cpp" -o "$OUT/obj/ref_shim.o" &
pids+=($!)
for p in "${pids[@]}"; do wait "$p"; done
$CXX -shared -o "$OUT/libref_cpu.so" "$OUT"/obj/*.o
echo "built $OUT/libref_cpu.so"
