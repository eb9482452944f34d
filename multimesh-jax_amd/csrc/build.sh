#!/bin/bash
# Builds libmmreshard.so (C ABI + gfx950 kernels) next to the Python package.
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
out="${here}/../libmmreshard.so"
hipcc --offload-arch=gfx950 -O3 -std=c++17 -fPIC -shared \
  -Xclang -target-feature -Xclang -packed-fp32-ops \
  -Wall -Wextra -Wno-unused-command-line-argument \
  -I"${here}/../../include" -I"${here}" \
  "${here}/geometry.cc" "${here}/sharding_frontend.cc" "${here}/planner.cc" \
  "${here}/context.cc" "${here}/hip_execute_context.cc" "${here}/kernels.hip" \
  -o "${out}"
echo "built ${out}"
