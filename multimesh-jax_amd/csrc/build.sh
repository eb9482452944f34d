#!/bin/bash
# Builds libmmreshard.so (C ABI + gfx950 kernels) next to the Python package.
set -euo pipefail
here="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
# digest of everything the library is built from (file names and contents, sorted): mmr_version() reports it
digest="$(cd "${here}/../.." && for f in $(ls include/*.h multimesh-jax_amd/csrc/* | LC_ALL=C sort); do echo "$f"; cat "$f"; done | sha256sum | cut -c1-16)"
out="${MMR_BUILD_OUT:-${here}/../libmmreshard.so}"  # MMR_BUILD_OUT: build to another place
hipcc --offload-arch=gfx950 -O3 -std=c++17 -fPIC -shared \
  -Xclang -target-feature -Xclang -packed-fp32-ops \
  -Wall -Wextra -Wno-unused-command-line-argument -DMMR_SOURCE_DIGEST="\"${digest}\"" ${MMR_EXTRA_FLAGS:-} \
  -I"${here}/../../include" -I"${here}" \
  "${here}/geometry.cc" "${here}/sharding_frontend.cc" "${here}/planner.cc" \
  "${here}/context.cc" "${here}/hip_execute_context.cc" "${here}/shard_buffer.cc" "${here}/kernels.hip" \
  -o "${out}"
# no kernel may touch scratch memory (a lane-indexed local array would put it there and cost most of the bandwidth)
usage="$(hipcc --offload-arch=gfx950 -O3 -std=c++17 --cuda-device-only -c -o /dev/null \
  -Xclang -target-feature -Xclang -packed-fp32-ops -Rpass-analysis=kernel-resource-usage ${MMR_EXTRA_FLAGS:-} \
  -I"${here}/../../include" -I"${here}" "${here}/kernels.hip" 2>&1 | grep -E "Function Name|ScratchSize|VGPRs:|Occupancy" || true)"
echo "${usage}" | sed 's/^.*remark: /  /'
if echo "${usage}" | grep -E "ScratchSize \[bytes/lane\]: [1-9]" >/dev/null; then
  echo "error: a kernel uses scratch memory" >&2
  exit 1
fi
echo "built ${out}"
