// Shard-intersection planner: (source descriptor, destination descriptor) pairs
// -> flat chunk tables one kernel launch per class consumes.  Host only.
//
// Stands in for the planning half of zuku::Reshard (call site
// zuku_execute_context_impl.cc:450-451); the result of a reshard does not
// depend on the plan, only its speed does.
#ifndef MMR_CSRC_PLANNER_H_
#define MMR_CSRC_PLANNER_H_

#include <string>
#include <vector>

#include "common.h"
#include "group_ops.h"

// Four launch classes.  Copy groups and span groups are decoded by arithmetic on the device (group_ops.h) and name
// their buffers by slot + offset until a launch binds them to addresses; generic and transpose chunks are one
// record per workgroup and go through the launch's pointer table.
struct mmr_plan {
  mmr_plan_options options{};
  std::vector<mmr_sharded_shape> srcs, dsts;
  std::vector<int64_t> slot_bases;  // first slot of every array
  int64_t n_slots = 0;
  std::vector<mmr::CopyGroup> copy_groups;  // every offset, stride and width a multiple of 16
  std::vector<mmr::CopyPiece> copy_pieces;
  uint32_t n_copy_chunks = 0;
  std::vector<mmr::SpanGroup> span_groups;  // ragged rows into dense destination tiles
  std::vector<mmr::SpanMember> span_members;
  std::vector<mmr::SpanPiece> span_pieces;
  uint32_t n_span_chunks = 0;
  std::vector<mmr_copy_chunk> generic;  // ragged boxes the span kernel does not take
  std::vector<mmr_transpose_chunk> transposes;
  mmr_plan_stats stats{};
};

namespace mmr {

constexpr uint32_t kDefaultChunkBytes = 8 * 1024;
constexpr uint32_t kDefaultSpanBytes = 4 * 1024;      // destination bytes per workgroup (one wavefront) of the span kernel
constexpr int64_t kDefaultSpanFractionKib = 4;        // interleave round of the span groups, per tile: one span of
                                                      // each tile in turn, so the spans that read the two sides of a source
                                                      // line run together (configuration 5: 13 % -> 8 % over-fetch, same time)
constexpr int64_t kTransposeChunkBytes = 32 * 1024;  // a transpose chunk batches small tiles up to this many bytes

// Cache key of a batch of descriptor pairs under given options.
std::string plan_key(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int n,
                     const mmr_plan_options& options);

int build_plan(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int n,
               const mmr_plan_options& options, mmr_plan* plan);

// Chunk ci of the plan's copy-group launch as a chunk record with slot-relative offsets (what the kernel works out
// on the device from the bound table).
mmr_copy_chunk decoded_copy_chunk(const mmr_plan& plan, uint32_t ci);
// Hints for find_group: the group of the first chunk of every block of 64 chunks.
template <class G>
std::vector<uint32_t> group_hints(const std::vector<G>& groups, uint32_t n_chunks) {
  std::vector<uint32_t> hints((n_chunks + (1u << kHintShift) - 1) >> kHintShift);
  uint32_t g = 0;
  for (size_t b = 0; b < hints.size(); ++b) {
    const uint32_t ci = static_cast<uint32_t>(b) << kHintShift;
    while (g + 1 < groups.size() && groups[g + 1].first_chunk <= ci) ++g;
    hints[b] = g;
  }
  return hints;
}

}  // namespace mmr

#endif  // MMR_CSRC_PLANNER_H_
