#!/bin/bash
# Builds libios_runtime.so for gfx950 into csrc/build/.  hipcc cross-compiles without a GPU.
set -euo pipefail
cd "$(dirname "$0")"
mkdir -p build
# -amdgpu-kernarg-preload-count: the leading scalar kernel arguments arrive in registers (the fused stage kernel's item
# starts), which takes one scalar-load round trip out of every fused launch
FLAGS="--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Xclang -target-feature -Xclang -packed-fp32-ops -mllvm -amdgpu-mfma-vgpr-form=1 -mllvm -amdgpu-kernarg-preload-count=16 -Wno-unused-result"
# The stand-alone convolution kernels are scheduled for instruction-level parallelism (more of a K step's loads ahead of its
# MFMAs): 0.3 % of an Inception-v3 pass in same-device A/B runs with identical kernel configurations.  The same for the
# 512-thread form of the fused stage kernel, which holds most convolution levels (another 0.4 % there and on NASNet); the other
# two forms spill or slow the memory-bound bodies down with it (NASNet +0.8 %), so they keep the default.
declare -A FILE_FLAGS=([conv_mfma.hip]="-mllvm -amdgpu-sched-strategy=max-ilp" [fused_512.hip]="-mllvm -amdgpu-sched-strategy=max-ilp")
pids=()
for src in conv_mfma.hip pointwise.hip fused.hip fused_512.hip fused_wide.hip runtime.hip c_api.hip; do
    # the resource remarks go to a log: a kernel that spills registers to scratch memory is reported below
    hipcc $FLAGS ${FILE_FLAGS[$src]:-} -Rpass-analysis=kernel-resource-usage -c "$src" -o "build/${src%.hip}.o" 2> "build/${src%.hip}.log" &
    pids+=($!)
done
hipcc $FLAGS -x hip -c plan.cpp -o build/plan.o &
pids+=($!)
status=0
for pid in "${pids[@]}"; do wait "$pid" || status=1; done
if [ "$status" -ne 0 ]; then
    grep -h -B2 -A8 "error" build/*.log >&2 || cat build/*.log >&2
    exit 1
fi
if grep -h "ScratchSize \[bytes/lane\]: [1-9]" build/*.log > /dev/null; then
    echo "warning: kernels spilling to scratch memory (bytes per lane):" >&2
    awk '/Function Name:/ { name = $0; sub(/.*Function Name: /, "", name); sub(/ \[-R.*/, "", name) }
         /ScratchSize \[bytes\/lane\]: [1-9]/ { size = $0; sub(/.*lane\]: /, "", size); sub(/ .*/, "", size); print "  " size "  " name }' build/*.log >&2
fi
hipcc --offload-arch=gfx950 -shared -fPIC -o build/libios_runtime.so build/conv_mfma.o build/pointwise.o build/fused.o build/fused_512.o build/fused_wide.o build/runtime.o build/c_api.o build/plan.o
echo "built $(pwd)/build/libios_runtime.so"
