#!/bin/bash
# Builds the C++ test of the ZukuExecuteContext mirror against libmmreshard.so
# and the C restatement of the reshard, and the host emulation of the kernels.
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
root="${here}/../.."
g++ -O2 -std=c++20 -Wall -Wextra -Wno-unknown-pragmas -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -I"${root}/include" \
  -I"${root}/multimesh-jax_amd/csrc" "${here}/hip_execute_context_test.cc" \
  -L"${root}/multimesh-jax_amd" -lmmreshard -L"${root}/oracle" -lreshard_oracle -L/opt/rocm/lib -lamdhip64 \
  -Wl,-rpath,'$ORIGIN/../../multimesh-jax_amd' -Wl,-rpath,'$ORIGIN/../../oracle' -Wl,-rpath,/opt/rocm/lib \
  -o "${here}/hip_execute_context_test"
echo "built ${here}/hip_execute_context_test"
g++ -O2 -std=c++20 -Wall -Wextra -Wno-unknown-pragmas -D__HIP_PLATFORM_AMD__ -I/opt/rocm/include -I"${root}/include" \
  -I"${root}/multimesh-jax_amd/csrc" "${here}/context_bench.cc" \
  -L"${root}/multimesh-jax_amd" -lmmreshard -L/opt/rocm/lib -lamdhip64 \
  -Wl,-rpath,'$ORIGIN/../../multimesh-jax_amd' -Wl,-rpath,/opt/rocm/lib \
  -o "${here}/context_bench"
echo "built ${here}/context_bench"
g++ -O2 -std=c++17 -Wall -Wextra -Wno-unknown-pragmas -fPIC -shared -I"${root}/include" -I"${root}/multimesh-jax_amd/csrc" \
  "${here}/kernel_emulation.cc" -L"${root}/multimesh-jax_amd" -lmmreshard \
  -Wl,-rpath,'$ORIGIN/../../multimesh-jax_amd' -Wl,-rpath,/opt/rocm/lib \
  -o "${here}/libmmr_emulation.so"
echo "built ${here}/libmmr_emulation.so"
# the same with the span kernel's two optional variations (source-aligned loads, cacheable edge lines) switched on
g++ -O2 -std=c++17 -Wall -Wextra -Wno-unknown-pragmas -fPIC -shared -DMMR_SPAN_ALIGNED_LOADS=1 -DMMR_SPAN_KEEP_EDGES=1 \
  -I"${root}/include" -I"${root}/multimesh-jax_amd/csrc" \
  "${here}/kernel_emulation.cc" -L"${root}/multimesh-jax_amd" -lmmreshard \
  -Wl,-rpath,'$ORIGIN/../../multimesh-jax_amd' -Wl,-rpath,/opt/rocm/lib \
  -o "${here}/libmmr_emulation_span_options.so"
echo "built ${here}/libmmr_emulation_span_options.so"
# Host-only sanitizer build: planner + descriptor geometry + the emulation of the kernels + a random sweep.
g++ -O1 -g -std=c++17 -fsanitize=address,undefined -fno-sanitize-recover=undefined -fno-omit-frame-pointer \
  -Wall -Wextra -Wno-unknown-pragmas -I"${root}/include" -I"${root}/multimesh-jax_amd/csrc" \
  "${root}/multimesh-jax_amd/csrc/geometry.cc" "${root}/multimesh-jax_amd/csrc/sharding_frontend.cc" \
  "${root}/multimesh-jax_amd/csrc/planner.cc" "${here}/kernel_emulation.cc" "${here}/sanitize_sweep.cc" \
  -o "${here}/sanitize_sweep"
echo "built ${here}/sanitize_sweep"
