// Descriptor validation and shard geometry (host only).
#include <cstdio>
#include <cstring>

#include "common.h"

namespace mmr {

namespace {
thread_local std::string g_error;
}

int fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_error = buf;
  return code;
}

const char* last_error() { return g_error.c_str(); }

int itemsize_of(int32_t dtype) {
  switch (dtype) {
    case MMR_PRED: case MMR_S8: case MMR_U8: case MMR_F8E4M3FN: case MMR_F8E5M2:
      return 1;
    case MMR_F16: case MMR_BF16: case MMR_S16: case MMR_U16:
      return 2;
    case MMR_F32: case MMR_S32: case MMR_U32:
      return 4;
    case MMR_F64: case MMR_S64: case MMR_U64: case MMR_C64:
      return 8;
    case MMR_C128:
      return 16;
    default:
      return 0;
  }
}

int make_side(const mmr_sharded_shape& s, Side* out) {
  Side side;
  side.dtype = s.dtype;
  side.itemsize = itemsize_of(s.dtype);
  if (side.itemsize == 0) return fail(MMR_UNSUPPORTED, "Unsupported type: %d", s.dtype);
  if (s.ndims < 0 || s.ndims > MMR_MAX_DIMS)
    return fail(MMR_INVALID_ARGUMENT, "descriptor has %d entries, at most %d are supported", s.ndims, MMR_MAX_DIMS);
  side.ndims = s.ndims;
  const bool replicated = s.ndims > 0 && s.dims[s.ndims - 1].size == 1 && s.dims[s.ndims - 1].sharding > 1;
  side.rank = replicated ? s.ndims - 1 : s.ndims;
  if (side.rank > kMaxRank) return fail(MMR_INVALID_ARGUMENT, "tensor rank %d exceeds %d", side.rank, kMaxRank);
  if (s.dev_count < 1 || s.dev_start < 0)
    return fail(MMR_INVALID_ARGUMENT, "device list [%lld, +%lld) is not valid", (long long)s.dev_start, (long long)s.dev_count);
  side.dev_start = s.dev_start;
  side.dev_count = s.dev_count;

  // `permutation` must order the entries: 0 = most significant digit of the device id.
  int64_t acc = 1;
  for (int rank_in_id = s.ndims - 1; rank_in_id >= 0; --rank_in_id) {
    int found = -1;
    for (int i = 0; i < s.ndims; ++i) {
      if (s.dims[i].permutation == rank_in_id) {
        if (found >= 0) return fail(MMR_INVALID_ARGUMENT, "permutation value %d appears twice", rank_in_id);
        found = i;
      }
    }
    if (found < 0) return fail(MMR_INVALID_ARGUMENT, "permutation fields are not a permutation of 0..%d", s.ndims - 1);
    if (s.dims[found].sharding < 1)
      return fail(MMR_INVALID_ARGUMENT, "dim %d has sharding %lld", found, (long long)s.dims[found].sharding);
    side.dev_stride[found] = acc;
    acc *= s.dims[found].sharding;
  }
  if (acc != s.dev_count)
    return fail(MMR_INVALID_ARGUMENT, "product of shardings %lld differs from device count %lld", (long long)acc,
                (long long)s.dev_count);
  side.replication = replicated ? s.dims[s.ndims - 1].sharding : 1;

  side.shard_elems = 1;
  for (int i = 0; i < side.rank; ++i) {
    if (s.dims[i].size < 0) return fail(MMR_INVALID_ARGUMENT, "dim %d has size %lld", i, (long long)s.dims[i].size);
    side.size[i] = s.dims[i].size;
    side.tiles[i] = s.dims[i].sharding;
    side.ext[i] = (s.dims[i].size + s.dims[i].sharding - 1) / s.dims[i].sharding;
    side.shard_elems *= side.ext[i];
  }
  side.shard_bytes = side.shard_elems * side.itemsize;

  // physical strides: minor_to_major[0] is the fastest-varying logical dim
  bool seen[kMaxRank] = {};
  int64_t st = 1;
  for (int k = 0; k < side.rank; ++k) {
    int dim = s.has_layout ? s.minor_to_major[k] : side.rank - 1 - k;
    if (dim < 0 || dim >= side.rank || seen[dim])
      return fail(MMR_INVALID_ARGUMENT, "minor_to_major is not a permutation of 0..%d", side.rank - 1);
    seen[dim] = true;
    side.stride[dim] = st;
    st *= side.ext[dim];
  }
  *out = side;
  return MMR_OK;
}

std::string descriptor_key(const mmr_sharded_shape& s) {
  std::string k;
  auto put = [&k](const void* p, size_t n) { k.append(static_cast<const char*>(p), n); };
  put(&s.dtype, sizeof(s.dtype));
  put(&s.ndims, sizeof(s.ndims));
  int n = s.ndims < 0 ? 0 : (s.ndims > MMR_MAX_DIMS ? MMR_MAX_DIMS : s.ndims);
  put(s.dims, sizeof(mmr_sharding_dim) * n);
  put(&s.dev_start, sizeof(s.dev_start));
  put(&s.dev_count, sizeof(s.dev_count));
  int32_t has_layout = s.has_layout ? 1 : 0;
  put(&has_layout, sizeof(has_layout));
  if (has_layout) put(s.minor_to_major, sizeof(int32_t) * n);
  return k;
}

}  // namespace mmr

using mmr::fail;

extern "C" {

const char* mmr_last_error(void) { return mmr::last_error(); }
#ifndef MMR_SOURCE_DIGEST
#define MMR_SOURCE_DIGEST "unknown"
#endif
// "mmreshard <version> (gfx950) sources <digest>": the digest of the sources this binary was built from, so that a
// loader can tell a stale binary from a current one.
const char* mmr_version(void) { return "mmreshard 0.2 (gfx950) sources " MMR_SOURCE_DIGEST; }
int mmr_itemsize(int32_t dtype) { return mmr::itemsize_of(dtype); }

int mmr_validate_sharded_shape(const mmr_sharded_shape* s) {
  if (!s) return fail(MMR_INVALID_ARGUMENT, "null descriptor");
  mmr::Side side;
  return mmr::make_side(*s, &side);
}

int mmr_shard_extents(const mmr_sharded_shape* s, int64_t* extents, int32_t* rank) {
  if (!s || !extents || !rank) return fail(MMR_INVALID_ARGUMENT, "null argument");
  mmr::Side side;
  if (int rc = mmr::make_side(*s, &side)) return rc;
  for (int i = 0; i < side.rank; ++i) extents[i] = side.ext[i];
  *rank = side.rank;
  return MMR_OK;
}

int mmr_shard_bytes(const mmr_sharded_shape* s, int64_t* bytes) {
  if (!s || !bytes) return fail(MMR_INVALID_ARGUMENT, "null argument");
  mmr::Side side;
  if (int rc = mmr::make_side(*s, &side)) return rc;
  *bytes = side.shard_bytes;
  return MMR_OK;
}

int mmr_device_of_tile(const mmr_sharded_shape* s, const int64_t* tile_coord, int64_t* device) {
  if (!s || !tile_coord || !device) return fail(MMR_INVALID_ARGUMENT, "null argument");
  mmr::Side side;
  if (int rc = mmr::make_side(*s, &side)) return rc;
  int64_t dev = side.dev_start;
  for (int i = 0; i < side.ndims; ++i) {
    if (tile_coord[i] < 0 || tile_coord[i] >= s->dims[i].sharding)
      return fail(MMR_INVALID_ARGUMENT, "tile coordinate %lld of dim %d is outside [0, %lld)", (long long)tile_coord[i], i,
                  (long long)s->dims[i].sharding);
    dev += tile_coord[i] * side.dev_stride[i];
  }
  *device = dev;
  return MMR_OK;
}

int mmr_tile_of_device(const mmr_sharded_shape* s, int64_t device, int64_t* tile_coord) {
  if (!s || !tile_coord) return fail(MMR_INVALID_ARGUMENT, "null argument");
  mmr::Side side;
  if (int rc = mmr::make_side(*s, &side)) return rc;
  int64_t rel = device - side.dev_start;
  if (rel < 0 || rel >= side.dev_count)
    return fail(MMR_NOT_FOUND, "device %lld is outside the device list [%lld, +%lld)", (long long)device,
                (long long)side.dev_start, (long long)side.dev_count);
  for (int i = 0; i < side.ndims; ++i) tile_coord[i] = (rel / side.dev_stride[i]) % s->dims[i].sharding;
  return MMR_OK;
}

}  // extern "C"
