#!/bin/bash
# Compiles libagpu_hip.so for gfx950 in-tree (no GPU needed: hipcc cross-compiles).
set -euo pipefail
cd "$(dirname "$0")"
HIPCC=${HIPCC:-/opt/rocm/bin/hipcc}
FLAGS=(--offload-arch=gfx950 -O3 -std=c++17 -fPIC -fvisibility=hidden -ffp-contract=off
       -Xclang -target-feature -Xclang -packed-fp32-ops -Wall -Wno-unused-function)
mkdir -p build
rm -f build/*.o build/trace/*.o  # objects of sources that no longer exist must not be linked
pids=()
for src in *.hip; do
  obj="build/${src%.hip}.o"
  "$HIPCC" "${FLAGS[@]}" -c "$src" -o "$obj" &
  pids+=($!)
done
g++ -O2 -std=c++17 -fPIC -fopenmp -fvisibility=hidden -ffp-contract=off -c quantize_host.cpp -o build/quantize_host.o &
pids+=($!)
for p in "${pids[@]}"; do wait "$p"; done
"$HIPCC" --offload-arch=gfx950 -shared -fPIC -o ../libagpu_hip.so build/*.o -fopenmp
echo "built $(cd .. && pwd)/libagpu_hip.so"
# The same library with time stamps inside the one-launch decode step (bench_configs.py --stamps): the two sources that
# know about them compiled again with -DAGPU_PK_TRACE, every other object shared.
mkdir -p build/trace
cp build/*.o build/trace/
"$HIPCC" "${FLAGS[@]}" -DAGPU_PK_TRACE -c decode_xcd.hip -o build/trace/decode_xcd.o &
"$HIPCC" "${FLAGS[@]}" -DAGPU_PK_TRACE -c gpt2_model.hip -o build/trace/gpt2_model.o &
wait
"$HIPCC" --offload-arch=gfx950 -shared -fPIC -o ../libagpu_hip_trace.so build/trace/*.o -fopenmp
echo "built $(cd .. && pwd)/libagpu_hip_trace.so"
# C++ host-layer test (include/agpu_nn.hpp); runs on the GPU box from tests/test_gpu_cpp.py
g++ -O1 -std=c++17 -I../../include ../../tests/cpp/test_nn.cpp -o ../../tests/cpp/test_nn \
    -L.. -lagpu_hip -Wl,-rpath,'$ORIGIN/../../async-gpu_amd' -Wl,-rpath,/opt/rocm/lib -L/opt/rocm/lib -lamdhip64
echo "built tests/cpp/test_nn"
g++ -O1 -std=c++17 -I../../include ../../tests/cpp/test_gpu_array_host.cpp -o ../../tests/cpp/test_gpu_array_host \
    -L.. -lagpu_hip -Wl,-rpath,'$ORIGIN/../../async-gpu_amd' -Wl,-rpath,/opt/rocm/lib -L/opt/rocm/lib -lamdhip64
echo "built tests/cpp/test_gpu_array_host"
# The GPT-2 example program over include/agpu_nn.hpp (tests/test_cpp_example.py, tests/test_gpu_model.py)
g++ -O1 -std=c++17 -I../../include ../examples/gpt2_inference.cpp -o ../examples/gpt2_inference \
    -L.. -lagpu_hip -Wl,-rpath,'$ORIGIN/..' -Wl,-rpath,/opt/rocm/lib -L/opt/rocm/lib -lamdhip64
echo "built async-gpu_amd/examples/gpt2_inference"
