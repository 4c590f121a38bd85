#!/usr/bin/env bash
# Builds, in-tree and for gfx950:
#   libmemorax_amd.so      the library (HIP kernels + C ABI)
#   libmemorax_amd_c64.so  the same sources with the delta rule's bf16 kernels on 64-step chunks; only
#                          bench.py loads it, to time that chunk length beside the default 32
#   libmemorax_amd_clk.so  the library with chunk_bwd.hip compiled for measurement (MRX_PHASE_CLOCKS: shader-clock
#                          brackets around every matrix product) and with pattern_probe.hip (the memory side of the
#                          chunked kernels without their arithmetic); only bench.py loads it, for the share of a
#                          wave's time that delta_bwd_kernel spends inside products and for what the kernels'
#                          access pattern alone costs
#   memorax_amd/csrc/build.sh
set -euo pipefail
cd "$(dirname "$0")"
HIPCC=${HIPCC:-/opt/rocm/bin/hipcc}
FLAGS=(--offload-arch=gfx950 -O3 -std=c++17 -fPIC -I../../include
       -Xclang -target-feature -Xclang -packed-fp32-ops -Wall -Wno-unused-function)
SRCS=(api.hip scan.hip chunk_fwd.hip chunk_bwd.hip step.hip delta_tm.hip la_states.hip mlstm_gates.hip rms_norm.hip gate.hip)
pids=()
compile() {  # compile <object suffix> <extra flags...>
    local suf=$1; shift
    for src in "${SRCS[@]}"; do
        local extra=()
        # delta_tm.hip: MFMA results feed the vector ALU at once, keep them out of accumulation registers
        [ "$src" = delta_tm.hip ] && extra=(-mllvm -amdgpu-mfma-vgpr-form)
        "$HIPCC" "${FLAGS[@]}" "${extra[@]}" "$@" -c "$src" -o "${src%.hip}$suf.o" \
            2> >(grep -v "packed-fp32-ops' is not a recognized feature" >&2) &
        pids+=($!)
    done
}
# the chunked and single-step kernels once more for head dim 32 (hd.h); both libraries link these objects
HD32_SRCS=(chunk_fwd.hip chunk_bwd.hip step.hip delta_tm.hip la_states.hip)
compile ""
compile _c64 -DMRX_DELTA_BF16_CHUNK=64
ALL_SRCS=("${SRCS[@]}"); SRCS=("${HD32_SRCS[@]}")
compile _hd32 -DMRX_HD=32
SRCS=(chunk_bwd.hip)
compile _clk -DMRX_PHASE_CLOCKS=1
SRCS=(pattern_probe.hip)
compile ""
SRCS=("${ALL_SRCS[@]}")
for p in "${pids[@]}"; do wait "$p"; done
HD32_OBJS=$(printf '%s_hd32.o ' "${HD32_SRCS[@]%.hip}")
"$HIPCC" --offload-arch=gfx950 -shared -fPIC -o libmemorax_amd.so $(printf '%s.o ' "${SRCS[@]%.hip}") $HD32_OBJS
"$HIPCC" --offload-arch=gfx950 -shared -fPIC -o libmemorax_amd_c64.so $(printf '%s_c64.o ' "${SRCS[@]%.hip}") $HD32_OBJS
CLK_OBJS=$(printf '%s.o ' "${SRCS[@]%.hip}" | sed 's/chunk_bwd\.o/chunk_bwd_clk.o/')
"$HIPCC" --offload-arch=gfx950 -shared -fPIC -o libmemorax_amd_clk.so $CLK_OBJS pattern_probe.o $HD32_OBJS
rm -f ./*.o
echo "built $(pwd)/libmemorax_amd.so, libmemorax_amd_c64.so and libmemorax_amd_clk.so"
