#!/usr/bin/env bash
# Builds kernels/libternaspmm.so for MI355X (gfx950) and the tests/test_kernel harness.
# Run from anywhere:  bash kernels/compile.sh
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
src="$here/../ternainfer_amd/csrc"

hipcc -std=c++17 -O3 -fPIC -shared --offload-arch=gfx950 \
    -Xclang -target-feature -Xclang -packed-fp32-ops \
    -Wall -Wno-unused-function \
    "$src/ternaspmm.hip" "$src/format_host.cpp" \
    -o "$here/libternaspmm.so"

if [ -f "$here/../tests/test_kernel.hip" ]; then
    hipcc -std=c++17 -O2 --offload-arch=gfx950 \
        "$here/../tests/test_kernel.hip" \
        -L"$here" -lternaspmm -lhipblas \
        -Wl,-rpath,'$ORIGIN/../kernels' \
        -o "$here/../tests/test_kernel"
fi
