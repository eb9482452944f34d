// Launcher of the gfx950 data-movement kernel.  One launch consumes all chunk
// tables of a plan: the grid is the tables back to back, one workgroup per chunk.
#ifndef MMR_CSRC_KERNELS_H_
#define MMR_CSRC_KERNELS_H_

#include <hip/hip_runtime_api.h>

#include "mmreshard.h"

namespace mmr {

// Device-resident chunk tables of one plan, as the kernel receives them (by value).
struct PlanTables {
  struct Table {
    const void* chunks;  // device pointer to the records
    uint32_t n;          // records
    uint32_t group;      // XCD grouping: runs of `group` table neighbours share an XCD
    uint32_t grid;       // workgroups reserved for the table (n padded to the grouping)
  };
  Table copy16;     // mmr_copy_chunk, every offset/stride/width a multiple of 16
  Table span;       // mmr_span_chunk
  Table generic;    // mmr_copy_chunk, any alignment
  Table transpose;  // mmr_transpose_chunk
};

// xcd_mode: 0/1 = chunk i runs as workgroup i (the hardware deals consecutive
// workgroups round-robin over the 8 XCDs); 2 = each XCD takes a contiguous
// eighth of the table; G >= 16 = runs of G consecutive chunks share an XCD (and
// so an L2), runs dealt round-robin.
void set_table(PlanTables::Table* t, const void* d_chunks, int64_t n, uint32_t xcd_mode);

hipError_t launch_plan(const PlanTables& tables, void* const* d_ptrs, hipStream_t stream);

}  // namespace mmr

#endif  // MMR_CSRC_KERNELS_H_
