#!/bin/bash
# Builds the host side in-tree:
#   libmoodist.so   host core (g++, links neither HIP nor torch; loads both
#                   libamdhip64.so and libmoodist_hip.so at first GPU use)
#   _C*.so          pybind11 module on PyTorch-ROCm (skipped with MOODIST_SKIP_WRAPPER=1: the _C
#                   of an earlier build then refuses the new core, whose build magic differs,
#                   unless MOODIST_BUILD_MAGIC repeats that build's)
set -euo pipefail
here="$(cd "$(dirname "$0")" && pwd)"
root="$(cd "$here/../.." && pwd)"
pkg="$here/.."
cxx="${CXX:-g++}"
# A build magic of its own for every build, as the reference draws one at configure time
# (CMakeLists.txt:97-106): the core carries it in its API table, the Python module compares it
# with its own, and a libmoodist.so left over from another build beside a new _C is refused.
# MOODIST_BUILD_MAGIC=0x... overrides it (the reference's -DMOODIST_BUILD_MAGIC).
magic="${MOODIST_BUILD_MAGIC:-0x$(od -An -N8 -tx1 /dev/urandom | tr -d ' \n')ULL}"
export MOODIST_BUILD_MAGIC="$magic"
common=(-O2 -std=c++20 -fPIC -Wall -Wextra -fvisibility=hidden -DMOODIST_BUILD_MAGIC="$magic" -I"$root/include" -I"$here/core")
mkdir -p "$here/build"
objs=()
for f in hip_loader planner processgroup c_api plugin; do
  o="$here/build/core_$f.o"
  "$cxx" "${common[@]}" -c "$here/core/$f.cc" -o "$o" &
  objs+=("$o")
done
wait
# exports: the plugin entry and the plain C functions, nothing else (no C++ symbols leak out)
printf '{ global: moodist*; local: *; };\n' > "$here/build/exports.map"
"$cxx" -shared -o "$pkg/libmoodist.so" "${objs[@]}" -ldl -lpthread -Wl,--no-undefined \
  -Wl,--version-script="$here/build/exports.map"
echo "built $pkg/libmoodist.so (build magic $magic)"
if [ "${MOODIST_SKIP_WRAPPER:-0}" != "1" ] && [ -f "$here/wrapper/module.cc" ]; then
  python3 "$here/wrapper/build_wrapper.py"
fi
