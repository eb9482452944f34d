// Shared host-side helpers of the reshard library: status + error text, and the
// geometry of one side of a reshard derived from a sharded-shape descriptor.
#ifndef MMR_CSRC_COMMON_H_
#define MMR_CSRC_COMMON_H_

#include <cstdarg>
#include <cstdint>
#include <string>

#include "mmreshard.h"

namespace mmr {

constexpr int kMaxRank = MMR_MAX_DIMS - 1;

// Records the message mmr_last_error() returns on this thread; returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
const char* last_error();

int itemsize_of(int32_t dtype);  // 0 if unknown

// One side (source or destination) of a reshard.  Follows how the reference
// fills zuku::ShardedShape (mm_sharding.cc:345-372, 638-654): dims[i].size is
// the global extent, .sharding the tile count, .permutation the rank of the dim
// in device-id significance; a trailing {1, R>1} entry replicates.  Tile extent
// is ceil(size / sharding), the XLA convention the plugin's local shapes come
// from (spmd::MakePartitionedShape, mm_pjrt_executable.cc:537).
struct Side {
  int32_t dtype = 0;
  int itemsize = 0;
  int rank = 0;   // tensor dims
  int ndims = 0;  // descriptor entries (rank or rank + 1)
  int64_t size[kMaxRank] = {};
  int64_t tiles[kMaxRank] = {};
  int64_t ext[kMaxRank] = {};          // tile extent per dim, padding included
  int64_t dev_stride[MMR_MAX_DIMS] = {};  // stride of every descriptor entry in the device id
  int64_t replication = 1;
  int64_t dev_start = 0;
  int64_t dev_count = 0;
  int64_t stride[kMaxRank] = {};  // element stride of every logical dim inside a shard buffer
  int64_t shard_elems = 0;
  int64_t shard_bytes = 0;
};

// Validates the descriptor and derives the geometry. MMR_OK or an error code.
int make_side(const mmr_sharded_shape& s, Side* out);

// Byte-exact key of a descriptor (only the used entries), for plan/cache maps.
std::string descriptor_key(const mmr_sharded_shape& s);

}  // namespace mmr

#endif  // MMR_CSRC_COMMON_H_
