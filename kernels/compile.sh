#!/usr/bin/env bash
# Builds kernels/libternaspmm.so for MI355X (gfx950) and the tests/test_kernel harness.
# Run from anywhere:  bash kernels/compile.sh
# One hipcc compile per translation unit, all at once (each kernel family is instantiated in a
# file of its own), then one link.  -amdgpu-kernarg-preload-count: the first 16 dwords of a kernel's
# arguments arrive in scalar registers with the wave instead of being fetched by its first instructions
# (every launch of a decode step starts 0.05 - 0.3 us earlier).
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
src="$here/../ternainfer_amd/csrc"
obj="$here/build"
mkdir -p "$obj"

flags=(-std=c++17 -O3 -fPIC --offload-arch=gfx950
       -Xclang -target-feature -Xclang -packed-fp32-ops
       -mllvm -amdgpu-kernarg-preload-count=16
       -Wall -Wno-unused-function)

pids=()
compile() {  # compile <source> <object> [extra flags]
    local s="$1" o="$2"; shift 2
    hipcc "${flags[@]}" "$@" -c "$src/$s" -o "$obj/$o" 2> >(grep -v "packed-fp32-ops' is not a recognized feature" >&2) &
    pids+=($!)
}
compile ternaspmm.hip ternaspmm.o
compile launch_reference.hip launch_reference.o
compile launch_decode_packed.hip launch_decode_packed.o
compile launch_prefill_packed.hip launch_prefill_packed_i8.o -DTERNA_PREFILL_ACT=int8_t
compile launch_prefill_packed.hip launch_prefill_packed_bf16.o -DTERNA_PREFILL_ACT=uint16_t
compile abi_fused.hip abi_fused.o
compile abi_chain.hip abi_chain.o
compile abi_attention.hip abi_attention.o
# accumulators of the prompt-pass attention in ordinary vector registers (they are rescaled between matrix instructions)
compile abi_prefill_attention.hip abi_prefill_attention.o -mllvm -amdgpu-mfma-vgpr-form
compile abi_head.hip abi_head.o
compile abi_probe.hip abi_probe.o
compile format_host.cpp format_host.o
for p in "${pids[@]}"; do wait "$p"; done

hipcc -shared -fPIC --offload-arch=gfx950 "$obj"/*.o -o "$here/libternaspmm.so"

if [ -f "$here/../tests/test_kernel.hip" ]; then
    hipcc -std=c++17 -O2 --offload-arch=gfx950 \
        "$here/../tests/test_kernel.hip" \
        -L"$here" -lternaspmm -lhipblas \
        -Wl,-rpath,'$ORIGIN/../kernels' \
        -o "$here/../tests/test_kernel"
fi
