#!/bin/bash
# Builds libmoodist_hip.so (gfx950 kernels + thin C ABI) in-tree.
#   build.sh [output.so]      MDH_EXTRA_FLAGS adds compiler flags (e.g. -DMDH_NT_LOAD=0)
set -euo pipefail
here="$(cd "$(dirname "$0")" && pwd)"
root="$(cd "$here/../.." && pwd)"
out="${1:-$here/../libmoodist_hip.so}"
extra="${MDH_EXTRA_FLAGS:-}"
tag="$(echo "$extra" | tr -c 'A-Za-z0-9\n' '_')"
jobs="${MDH_BUILD_JOBS:-8}"
# -amdgpu-kernarg-preload-count: a kernel's leading scalar arguments (14 dwords at most) are in
# registers when a wave starts; reduce_vec_kernel's are laid out for it.
flags=(-O3 -std=c++17 -fPIC --offload-arch=gfx950 -ffp-contract=off
       -Xclang -target-feature -Xclang -packed-fp32-ops
       -mllvm -amdgpu-kernarg-preload-count=14
       -I"$root/include" -I"$here/kernels" -Wall -Wno-unused-function -Wno-unused-const-variable $extra)
bdir="$here/build"
mkdir -p "$bdir"
cmds=()
objs=()
for f in abi copy reduce workspace; do
  o="$bdir/$f$tag.o"
  objs+=("$o")
  cmds+=("/opt/rocm/bin/hipcc ${flags[*]} -c $here/kernels/$f.hip -o $o")
done
for t in f32 bf16 f16 f64 i32 i64; do
  for f in sum min max; do
    o="$bdir/reduce_${t}_${f}$tag.o"
    objs+=("$o")
    cmds+=("/opt/rocm/bin/hipcc ${flags[*]} -DMDH_TNAME=$t -DMDH_FNAME=$f -c $here/kernels/reduce_inst.hip -o $o")
  done
done
printf '%s\n' "${cmds[@]}" | xargs -P "$jobs" -I{} bash -c '{} 2> >(grep -v "packed-fp32-ops" >&2)'
/opt/rocm/bin/hipcc -shared -fPIC --offload-arch=gfx950 -o "$out" "${objs[@]}"
echo "built $out"
