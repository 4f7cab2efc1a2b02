#!/bin/sh
# Host build of the kernels for CPU testing: same sources as libamoe.so, with the stand-in
# headers of this directory ahead of the HIP ones.  $1 = "asan" adds the host sanitizers.
set -e
here="$(cd "$(dirname "$0")" && pwd)"
root="$(cd "$here/../.." && pwd)"
CXX=/opt/rocm/llvm/bin/clang++
flags="-x c++ -std=c++20 -O1 -g -fPIC -shared -pthread -Wno-psabi -I $here -I $root/include -I $root/analog_moe_amd/csrc"
out="$here/libamoe_emu.so"
if [ "$1" = "asan" ]; then
  flags="$flags -fsanitize=address,undefined -fno-omit-frame-pointer -shared-libasan"
  out="$here/libamoe_emu_asan.so"
fi
$CXX $flags "$root/analog_moe_amd/csrc/amoe.hip" -o "$out"
echo "$out"
