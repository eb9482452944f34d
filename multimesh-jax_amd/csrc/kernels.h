// Launchers of the gfx950 data-movement kernels. One launch consumes one chunk
// table of a plan: workgroup i executes chunk i.
#ifndef MMR_CSRC_KERNELS_H_
#define MMR_CSRC_KERNELS_H_

#include <hip/hip_runtime_api.h>

#include "mmreshard.h"

namespace mmr {

// Chunks whose offsets, strides and widths are all multiples of 16 bytes.
// xcd_split: false = chunk i runs as workgroup i (the hardware deals consecutive
// workgroups round-robin over the 8 XCDs); true = each XCD takes a contiguous
// eighth of the table, so chunks that are neighbours in the table share an L2.
hipError_t launch_copy16(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, bool xcd_split,
                         hipStream_t stream);
// Chunks of any alignment (chunk.align picks the access width).
hipError_t launch_copy_generic(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, bool xcd_split,
                               hipStream_t stream);
// LDS-staged tile transposes.
hipError_t launch_transpose(const mmr_transpose_chunk* d_chunks, int64_t n, void* const* d_ptrs, bool xcd_split,
                            hipStream_t stream);

}  // namespace mmr

#endif  // MMR_CSRC_KERNELS_H_
