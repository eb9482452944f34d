// Launchers of the gfx950 data-movement kernels. One launch consumes one chunk
// table of a plan: workgroup i executes chunk i.
#ifndef MMR_CSRC_KERNELS_H_
#define MMR_CSRC_KERNELS_H_

#include <hip/hip_runtime_api.h>

#include "mmreshard.h"
#include "group_ops.h"

namespace mmr {

// Flat device-to-device copy; both pointers and the size must be multiples of 16 (hipErrorInvalidValue otherwise).
hipError_t launch_flat_copy(const void* src, void* dst, size_t bytes, hipStream_t stream);
// Copy groups (every offset, stride and width a multiple of 16 bytes) of a bound table: n workgroups, one per
// chunk, each decoding its chunk from the table.  d_hints: the group of the first chunk of every block of 64 chunks.
// xcd_mode: 0/1 = chunk i runs as workgroup i (the hardware deals consecutive
// workgroups round-robin over the 8 XCDs); 2 = each XCD takes a contiguous
// eighth of the table; G >= 16 = runs of G consecutive chunks share an XCD (and
// so an L2), runs dealt round-robin.
// starts: host array of every group's first chunk (or null); tables of up to kMaxDirectGroups groups get it by value.
hipError_t launch_copy_groups(const CopyGroup* d_groups, uint32_t n_groups, const CopyPiece* d_pieces,
                              const uint32_t* d_hints, const uint32_t* starts, int64_t n, uint32_t xcd_mode,
                              hipStream_t stream);
// Tables of very many chunks leave as several launches over consecutive pieces of the table (copy_piece_chunks,
// chunk_ops.h).
// The same for a table small enough to travel in the kernel's argument block.
hipError_t launch_copy_groups_inline(const InlineCopyTable& table, uint32_t xcd_mode, hipStream_t stream);
// Span groups (ragged rows into dense destination tiles), staged through LDS.
hipError_t launch_spans(const SpanGroup* d_groups, uint32_t n_groups, const SpanMember* d_members,
                        const SpanPiece* d_pieces, const uint32_t* d_hints, int64_t n, uint32_t xcd_mode,
                        hipStream_t stream);
hipError_t launch_spans_inline(const InlineSpanTable& table, uint32_t xcd_mode, hipStream_t stream);
// Chunks of any alignment (chunk.align picks the access width).
hipError_t launch_copy_generic(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, uint32_t xcd_mode,
                               hipStream_t stream);
// LDS-staged tile transposes of elements of `itemsize` bytes (1, 2, 4, 8 or
// 16); every chunk of the table must carry that itemsize, and with
// `vector_only` every chunk must satisfy transpose_is_vector (chunk_ops.h).
hipError_t launch_transpose(const mmr_transpose_chunk* d_chunks, int64_t n, void* const* d_ptrs, uint32_t xcd_mode,
                            uint32_t itemsize, bool vector_only, hipStream_t stream);

// Device address of this GPU's static scratch array (MMR_STATIC_SCRATCH_BYTES long, 256-byte aligned), looked up once
// per device; `device` must be the current device of the calling thread.
hipError_t static_scratch_address(int device, void** out);

}  // namespace mmr

#endif  // MMR_CSRC_KERNELS_H_
