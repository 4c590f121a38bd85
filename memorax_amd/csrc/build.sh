#!/usr/bin/env bash
# Builds libmemorax_amd.so (HIP kernels + C ABI) for gfx950, in-tree.
#   memorax_amd/csrc/build.sh
set -euo pipefail
cd "$(dirname "$0")"
HIPCC=${HIPCC:-/opt/rocm/bin/hipcc}
FLAGS=(--offload-arch=gfx950 -O3 -std=c++17 -fPIC -I../../include
       -Xclang -target-feature -Xclang -packed-fp32-ops -Wall -Wno-unused-function)
objs=()
pids=()
for src in api.hip scan.hip chunk_fwd.hip chunk_bwd.hip step.hip delta_tm.hip; do
    [ -f "$src" ] || continue
    obj="${src%.hip}.o"
    extra=()
    # delta_tm.hip: MFMA results feed the vector ALU at once, keep them out of accumulation registers
    [ "$src" = delta_tm.hip ] && extra=(-mllvm -amdgpu-mfma-vgpr-form)
    "$HIPCC" "${FLAGS[@]}" "${extra[@]}" -c "$src" -o "$obj" 2> >(grep -v "packed-fp32-ops' is not a recognized feature" >&2) &
    pids+=($!)
    objs+=("$obj")
done
for p in "${pids[@]}"; do wait "$p"; done
"$HIPCC" --offload-arch=gfx950 -shared -fPIC -o libmemorax_amd.so "${objs[@]}"
rm -f "${objs[@]}"
echo "built $(pwd)/libmemorax_amd.so"
