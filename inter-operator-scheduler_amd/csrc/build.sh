#!/bin/bash
# Builds libios_runtime.so for gfx950 into csrc/build/.  hipcc cross-compiles without a GPU.
set -euo pipefail
cd "$(dirname "$0")"
mkdir -p build
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops -mllvm -amdgpu-mfma-vgpr-form=1 -Wno-unused-result"
pids=()
for src in conv_mfma.hip pointwise.hip fused.hip runtime.hip c_api.hip; do
    hipcc $FLAGS -c "$src" -o "build/${src%.hip}.o" &
    pids+=($!)
done
hipcc $FLAGS -x hip -c plan.cpp -o build/plan.o &
pids+=($!)
for pid in "${pids[@]}"; do wait "$pid"; done
hipcc --offload-arch=gfx950 -shared -fPIC -o build/libios_runtime.so build/conv_mfma.o build/pointwise.o build/fused.o build/runtime.o build/c_api.o build/plan.o
echo "built $(pwd)/build/libios_runtime.so"
