#!/bin/sh
# Builds libflashpop_emu.so: the C-ABI layer over the CPU thread harness (tests only).
set -e
here=$(cd "$(dirname "$0")" && pwd)
csrc="$here/../../flash-pop_amd/csrc"
cxx=${EMU_CXX:-/opt/rocm/llvm/bin/clang++}
"$cxx" -std=c++17 -O2 -g -fPIC -shared -pthread $EMU_FLAGS -I"$here" -I"$csrc" \
  "$here/launch_emu.cpp" "$csrc/flashpop_api.cpp" -o "$here/libflashpop_emu.so"
