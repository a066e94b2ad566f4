#!/usr/bin/env bash
# Builds the reference's own CPU contraction (host-only, no GPU needed) from the
# sources where they lie under /root/reference, plus a small C-ABI shim of ours,
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
FLAGS="-std=c++17 -x hip --cuda-host-only -O2 -fPIC -w -I$R/include -I$R/src/include -I$R/src/contraction $INC"
pids=()
for f in contraction/contraction_cpu_reference.cpp \
         contraction/contraction_cpu_reference_instances.cpp \
         contraction/contraction_solution.cpp \
         contraction/contraction_solution_registry.cpp \
         contraction/contraction_types.cpp \
         data_types.cpp; do
  o="$OUT/obj/ref_$(basename "$f" .cpp).o"
  $CXX $FLAGS -c "$R/src/$f" -o "$o" &
  pids+=($!)
done
$CXX $FLAGS -c "$HERE/ref_shim.cpp" -o "$OUT/obj/ref_shim.o" &
pids+=($!)
for p in "${pids[@]}"; do wait "$p"; done
$CXX -shared -o "$OUT/libref_cpu.so" "$OUT"/obj/*.o
echo "built $OUT/libref_cpu.so"
