#!/bin/sh
# Builds the C-ABI layer over the CPU thread harness (tests only): libflashpop_emu.so, or, with
# EMU_MAIN=<source with a main()>, an executable EMU_OUT.  The translation units are compiled in
# parallel.  EMU_FLAGS: extra compiler flags (sanitizers); EMU_OPT: optimisation level (default -O2).
set -e
here=$(cd "$(dirname "$0")" && pwd)
csrc="$here/../../flash-pop_amd/csrc"
cxx=${EMU_CXX:-/opt/rocm/llvm/bin/clang++}
out=${EMU_OUT:-$here/libflashpop_emu.so}
obj=$(mktemp -d)
trap 'rm -rf "$obj"' EXIT
flags="-std=c++17 ${EMU_OPT:--O2} -g -fPIC -pthread $EMU_FLAGS -I$here -I$csrc"
pids=""
for w in 64 128 192 256; do
  "$cxx" $flags -DEMU_FAMILY=$w -c "$here/pass_family.cpp" -o "$obj/pass_$w.o" & pids="$pids $!"
done
for dk in 64 128; do
  for dv in 64 128; do
    "$cxx" $flags -DEMU_DK=$dk -DEMU_DV=$dv -c "$here/fused_family.cpp" -o "$obj/fused_${dk}_$dv.o" & pids="$pids $!"
  done
done
"$cxx" $flags -c "$here/launch_emu.cpp" -o "$obj/launch_emu.o" & pids="$pids $!"
"$cxx" $flags -c "$csrc/flashpop_api.cpp" -o "$obj/flashpop_api.o" & pids="$pids $!"
if [ -n "$EMU_MAIN" ]; then
  "$cxx" $flags -c "$EMU_MAIN" -o "$obj/main.o" & pids="$pids $!"
fi
for p in $pids; do wait "$p"; done
if [ -n "$EMU_MAIN" ]; then
  "$cxx" -pthread $EMU_FLAGS "$obj"/*.o -o "$out"
else
  "$cxx" -shared -pthread $EMU_FLAGS "$obj"/*.o -o "$out"
fi
