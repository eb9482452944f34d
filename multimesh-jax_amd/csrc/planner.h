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

struct mmr_plan {
  mmr_plan_options options{};
  std::vector<mmr_sharded_shape> srcs, dsts;
  std::vector<int64_t> slot_bases;  // first slot of every array
  int64_t n_slots = 0;
  std::vector<mmr_copy_chunk> copy16;   // every offset, stride and width a multiple of 16
  std::vector<mmr_copy_chunk> generic;  // anything else
  std::vector<mmr_transpose_chunk> transposes;
  mmr_plan_stats stats{};
};

namespace mmr {

constexpr uint32_t kDefaultChunkBytes = 8 * 1024;
constexpr int64_t kTransposeChunkBytes = 32 * 1024;  // a transpose chunk batches small tiles up to this many bytes

// Cache key of a batch of descriptor pairs under given options.
std::string plan_key(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int n,
                     const mmr_plan_options& options);

int build_plan(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int n,
               const mmr_plan_options& options, mmr_plan* plan);

}  // namespace mmr

#endif  // MMR_CSRC_PLANNER_H_
