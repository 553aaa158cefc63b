#!/bin/bash
# Compiles the reference's CPU fp32 GEMM path straight from its own sources under
# $DECX_REFERENCE (default /root/reference) into oracle/_ref/libdecx_ref_cpu.so.
# Nothing is copied into the repository and no stand-in is written for anything the
# reference needs: the one assembly file (a CPUID helper that needs NASM, absent
# here) is simply left out, and its symbol stays unresolved in the shared object --
# it is reached only from de::InitCPUInfo(), which ref_driver.cpp never calls.
# Skips quietly (exit 0) when the reference tree is not mounted.
set -e
REF="${DECX_REFERENCE:-/root/reference}"
HERE="$(cd "$(dirname "$0")" && pwd)"
if [ ! -d "$REF/srcs" ]; then echo "build_ref: no reference tree at $REF, skipping"; exit 0; fi
OUT="$HERE/_ref"; OBJ="$OUT/obj"; mkdir -p "$OBJ"
S="$REF/srcs"; CORE="$S/modules/core"; GEMM="$S/modules/BLAS/GEMM/CPU"
COMMON="-O2 -mavx2 -mfma -fPIC -w -D_CPP_EXPORT_ENABLED_=1 -D_C_EXPORT_ENABLED_=0 -I$S/modules/core -I$S/common"
CORE_DEFS="-D_DECX_CPU_PARTS_ -D_DECX_CORE_CPU_"
BLAS_DEFS="-D_DECX_CPU_PARTS_ -D_DECX_BLAS_CPU_"
n=0
cc() { # std defs src
  n=$((n+1)); g++ -std=$1 $COMMON $2 -c "$3" -o "$OBJ/o$n.o" & 
  if (( n % 8 == 0 )); then wait; fi
}
for f in "$CORE/global_vars.cxx" "$CORE/pre_post_proc_CPUcoreModule.cxx" "$CORE/classes/Matrix.cxx" \
         "$CORE"/resources_manager/*.cxx "$CORE/configs/config.cxx" "$CORE"/thread_management/*.cxx \
         "$CORE"/allocators/*.cxx "$CORE"/memory_management/*.cxx; do
  cc c++11 "$CORE_DEFS" "$f"
done
n=$((n+1)); gcc -O2 -fPIC -w $CORE_DEFS -c "$CORE/configs/x86_64/decx_CPUID_x86.c" -o "$OBJ/o$n.o" &
for f in "$S/common/FMGR/fragment_arangement.cxx" "$GEMM/GEMM.cxx" "$GEMM/cpu_GEMM_config.cxx" \
         "$GEMM"/fp32/*.cxx "$GEMM"/fp64/*.cxx; do
  cc c++17 "$BLAS_DEFS" "$f"
done
wait
g++ -std=c++17 -O2 -fPIC -w -I"$S/includes" -c "$HERE/ref_driver.cpp" -o "$OBJ/driver.o"
g++ -shared -Wl,-z,lazy -o "$OUT/libdecx_ref_cpu.so" "$OBJ"/*.o -lpthread
gcc -O2 -fPIC -shared -o "$OUT/libref_loader.so" "$HERE/ref_loader.c" -ldl
rm -rf "$OBJ"
echo "build_ref: built $OUT/libdecx_ref_cpu.so"
