#!/bin/bash
# Builds the C++ test of the ZukuExecuteContext mirror against libmmreshard.so
# and the C restatement of the reshard.
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
root="${here}/../.."
g++ -O2 -std=c++20 -Wall -Wextra -I"${root}/include" -I"${root}/multimesh-jax_amd/csrc" \
  "${here}/hip_execute_context_test.cc" \
  -L"${root}/multimesh-jax_amd" -lmmreshard -L"${root}/oracle" -lreshard_oracle \
  -Wl,-rpath,'$ORIGIN/../../multimesh-jax_amd' -Wl,-rpath,'$ORIGIN/../../oracle' -Wl,-rpath,/opt/rocm/lib \
  -o "${here}/hip_execute_context_test"
echo "built ${here}/hip_execute_context_test"
