// Descriptor front-end (host only): how an XLA sharding plus a shape becomes the
// sharded-shape descriptor the reshard consumes.  Follows the reference's
// src/pjrt_client/mm_sharding.{h,cc} and mpmd_insert_reshard.cc:33-43 with the
// XLA proto types flattened to the PODs of mmreshard.h.
#include <algorithm>
#include <cstring>
#include <numeric>
#include <vector>

#include "common.h"

using mmr::fail;

namespace {

bool is_replicated(const mmr_op_sharding& s) { return s.type == MMR_SHARDING_REPLICATED; }
bool is_maximal(const mmr_op_sharding& s) { return s.type == MMR_SHARDING_MAXIMAL; }

// mm_sharding.cc:19-33
bool replicated_on_assigned_submesh(const mmr_op_sharding& s) {
  if (is_replicated(s)) return true;
  if (s.replicate_on_last_tile_dim) {
    for (int d = 0; d + 1 < s.n_tile_dims; ++d)
      if (s.tile_dims[d] != 1) return false;
    return true;
  }
  return false;
}

// mm_sharding.cc:35-38
bool replicated_or_submesh_replicate(const mmr_op_sharding& s) {
  return is_replicated(s) || replicated_on_assigned_submesh(s) || is_maximal(s);
}

int check_sharding(const mmr_op_sharding* s) {
  if (!s) return fail(MMR_INVALID_ARGUMENT, "null sharding");
  if (s->n_tile_dims < 0 || s->n_tile_dims > MMR_MAX_DIMS || s->n_iota_dims < 0 || s->n_iota_dims > MMR_MAX_DIMS)
    return fail(MMR_INVALID_ARGUMENT, "sharding has too many dims");
  return MMR_OK;
}

// XLA's IotaTileAssignment::Create canonical form, which is what the reference
// walks (HloSharding::FromProto builds every assignment through it): size-1
// iota dims are dropped and iota dims that stay adjacent and in order after the
// transpose are merged.
void canonical_iota(const std::vector<int64_t>& d, const std::vector<int>& p, std::vector<int64_t>* dims,
                    std::vector<int>* perm) {
  std::vector<int> renum(d.size(), -1);
  std::vector<int64_t> kept;
  for (size_t i = 0; i < d.size(); ++i)
    if (d[i] != 1) {
      renum[i] = static_cast<int>(kept.size());
      kept.push_back(d[i]);
    }
  std::vector<int> kp;
  for (int v : p)
    if (v >= 0 && v < static_cast<int>(renum.size()) && renum[v] >= 0) kp.push_back(renum[v]);
  if (kept.empty()) {
    *dims = {1};
    *perm = {0};
    return;
  }
  std::vector<std::vector<int>> groups;  // runs of consecutive iota dims, in transposed order
  for (int v : kp) {
    if (!groups.empty() && groups.back().back() + 1 == v) groups.back().push_back(v);
    else groups.push_back({v});
  }
  std::vector<int> order(groups.size());
  std::iota(order.begin(), order.end(), 0);
  std::sort(order.begin(), order.end(), [&](int a, int b) { return groups[a][0] < groups[b][0]; });
  std::vector<int> new_index(groups.size());
  dims->clear();
  for (size_t i = 0; i < order.size(); ++i) {
    new_index[order[i]] = static_cast<int>(i);
    int64_t n = 1;
    for (int v : groups[order[i]]) n *= kept[v];
    dims->push_back(n);
  }
  perm->clear();
  for (size_t g = 0; g < groups.size(); ++g) perm->push_back(new_index[g]);
}

void canonical_iota(const mmr_op_sharding& s, std::vector<int64_t>* dims, std::vector<int>* perm) {
  canonical_iota(std::vector<int64_t>(s.iota_reshape_dims, s.iota_reshape_dims + s.n_iota_dims),
                 std::vector<int>(s.iota_transpose_perm, s.iota_transpose_perm + s.n_iota_dims), dims, perm);
}

int map_type(int32_t dtype) {
  // mm_sharding.cc:376-425: only these fifteen types have a runtime type
  if (dtype < MMR_PRED || dtype > MMR_C128) return fail(MMR_UNSUPPORTED, "Unsupported type: %d", dtype);
  return MMR_OK;
}

// mm_sharding.cc:275-432
int canonicalize_iota(const mmr_op_sharding& s, const std::vector<int64_t>& reshape_dims, const std::vector<int>& perm,
                      int64_t offset, const int64_t* shape, int rank, int32_t dtype, bool shape_is_global,
                      mmr_sharded_shape* out) {
  const int nta = s.n_tile_dims;
  std::vector<int64_t> permuted(reshape_dims.size());
  for (size_t i = 0; i < perm.size(); ++i) permuted[i] = reshape_dims[perm[i]];

  // :297-325  tile dims that one iota dim spans form a group
  std::vector<std::vector<int>> groups(1);
  size_t iota_dim = 0;
  int64_t spanned = 1;
  int ta = 0;
  for (; ta < nta && iota_dim < permuted.size(); ++ta) {
    spanned *= s.tile_dims[ta];
    const int64_t span = permuted[iota_dim];
    if (span < s.tile_dims[ta])
      return fail(MMR_INVALID_ARGUMENT,
                  "CanonicalizeSharding: sharding has multiple iota dims within a single tensor dimension, which is "
                  "not yet supported");
    groups.back().push_back(ta);
    if (spanned >= span) {
      ++iota_dim;
      if (iota_dim < permuted.size()) groups.emplace_back();
      spanned = 1;
    }
  }
  for (; ta < nta; ++ta) groups.back().push_back(ta);

  // :327-339  the reference picks group transpose_perm[k] as the k-th most significant
  std::vector<int> full;
  for (size_t k = 0; k < perm.size(); ++k) {
    if (perm[k] < 0 || perm[k] >= static_cast<int>(groups.size()))
      return fail(MMR_INVALID_ARGUMENT, "CanonicalizeSharding: iota transpose does not match the tile dims");
    for (int d : groups[perm[k]]) full.push_back(d);
  }
  if (static_cast<int>(full.size()) != nta)
    return fail(MMR_INVALID_ARGUMENT, "CanonicalizeSharding: iota dims do not cover the tile dims");

  // :341-369
  const int num_shape_dims = s.replicate_on_last_tile_dim ? nta - 1 : nta;
  if (num_shape_dims > rank) return fail(MMR_INVALID_ARGUMENT, "sharding has more tile dims than the shape has dims");
  mmr_sharded_shape r{};
  r.dtype = dtype;
  r.ndims = nta;
  for (int k = 0; k < nta; ++k) {
    const int tdim = full[k];
    const int64_t extent = s.tile_dims[tdim];
    if (tdim == num_shape_dims) {
      r.dims[tdim] = mmr_sharding_dim{1, extent, k};
    } else {
      int64_t size = shape[tdim];
      if (!shape_is_global) size *= extent;
      r.dims[tdim] = mmr_sharding_dim{size, extent, k};
    }
  }
  int64_t n = 1;
  for (int64_t d : reshape_dims) n *= d;
  r.dev_start = offset;
  r.dev_count = n;
  if (int rc = map_type(dtype)) return rc;
  *out = r;
  return MMR_OK;
}

}  // namespace

extern "C" {

int mmr_compute_index_set(int64_t global_index, const int64_t* dims, int32_t n, int64_t* out) {
  if (n < 0 || (n > 0 && (!dims || !out))) return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  int64_t remainder = global_index, stride = 1;
  for (int d = 0; d < n; ++d) stride *= dims[d];
  for (int d = 0; d < n; ++d) {
    if (dims[d] <= 0) return fail(MMR_INVALID_ARGUMENT, "dim %d has extent %lld", d, (long long)dims[d]);
    stride /= dims[d];
    out[d] = remainder / stride;
    remainder -= out[d] * stride;
  }
  return MMR_OK;
}

int mmr_compute_global_index(const int64_t* indices, const int64_t* dims, int32_t n, int64_t* out) {
  if (n < 0 || !out || (n > 0 && (!dims || !indices))) return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  int64_t stride = 1, index = 0;
  for (int d = n - 1; d >= 0; --d) {
    index += stride * indices[d];
    stride *= dims[d];
  }
  *out = index;
  return MMR_OK;
}

int mmr_logical_to_physical_sharding(const int32_t* axes_flat, const int32_t* axes_begin, int32_t n_logical,
                                     int64_t dev_start, int64_t dev_count, const int64_t* mesh_dims, int32_t n_mesh,
                                     int32_t list_all_devices, mmr_op_sharding* out) {
  (void)dev_count;
  if (!out || n_logical < 0 || n_mesh < 0 || n_mesh > MMR_MAX_DIMS || (n_logical > 0 && !axes_begin))
    return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  std::vector<int> used(n_mesh, 0);
  bool fully_replicated = true;
  for (int l = 0; l < n_logical; ++l) {
    for (int k = axes_begin[l]; k < axes_begin[l + 1]; ++k) {
      const int ax = axes_flat[k];
      if (ax < 0 || ax >= n_mesh) return fail(MMR_INVALID_ARGUMENT, "device axis %d is outside the %d-axis mesh", ax, n_mesh);
      used[ax] = 1;
      if (mesh_dims[ax] > 1) fully_replicated = false;
    }
  }
  mmr_op_sharding r{};
  if (n_logical == 0 || (fully_replicated && !list_all_devices)) {  // :204-209
    r.type = MMR_SHARDING_REPLICATED;
    *out = r;
    return MMR_OK;
  }
  int64_t replication = 1, total = 1;
  bool any_unused = false;
  for (int d = 0; d < n_mesh; ++d) {
    if (!used[d]) {
      any_unused = true;
      replication *= mesh_dims[d];
    }
    total *= mesh_dims[d];
  }
  if (n_logical + (any_unused ? 1 : 0) > MMR_MAX_DIMS) return fail(MMR_INVALID_ARGUMENT, "too many tile dims");
  std::vector<int> dim_perm;
  for (int l = 0; l < n_logical; ++l) {
    std::vector<int> assigned(axes_flat + axes_begin[l], axes_flat + axes_begin[l + 1]);
    std::sort(assigned.begin(), assigned.end());
    int64_t t = 1;
    for (int ax : assigned) {
      t *= mesh_dims[ax];
      dim_perm.push_back(ax);
    }
    r.tile_dims[l] = t;
  }
  r.n_tile_dims = n_logical;
  for (int d = 0; d < n_mesh; ++d)
    if (!used[d]) dim_perm.push_back(d);
  if (any_unused) r.tile_dims[r.n_tile_dims++] = replication;
  r.type = MMR_SHARDING_OTHER;
  bool need_perm = false;
  for (int i = 0; i < n_mesh; ++i) need_perm |= dim_perm[i] != i;
  if (need_perm) {
    r.n_iota_dims = n_mesh;
    for (int i = 0; i < n_mesh; ++i) {
      r.iota_reshape_dims[i] = mesh_dims[i];
      r.iota_transpose_perm[i] = dim_perm[i];
    }
  } else {
    r.n_iota_dims = 1;
    r.iota_reshape_dims[0] = total;
    r.iota_transpose_perm[0] = 0;
  }
  r.replicate_on_last_tile_dim = any_unused;
  r.iota_offset = dev_start;  // :270
  *out = r;
  return MMR_OK;
}

int mmr_logical_sharding_to_op_sharding(const int64_t* mesh_dims, const char* const* mesh_axis_names, int32_t n_mesh,
                                        const char* const* logical_names, const char* const* logical_device_axes,
                                        int32_t n_logical_axes, const char* const* spec_names, const int32_t* spec_begin,
                                        int32_t rank, const int64_t* shape, int64_t dev_start, int64_t dev_count,
                                        int64_t total_devices, mmr_op_sharding* out) {
  if (!out || n_mesh < 0 || n_mesh > MMR_MAX_DIMS || rank < 0 || rank > MMR_MAX_DIMS || n_logical_axes < 0 ||
      (rank > 0 && (!spec_begin || !shape)))
    return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  std::vector<std::vector<int32_t>> to_device(rank);
  std::vector<int> used(n_mesh, 0);
  std::vector<int64_t> sharding_on_axis(rank, 1);
  for (int p = 0; p < n_logical_axes; ++p) {  // mpmd_logical_to_gspmd_sharding.cc:40-85, in the pairs' order
    for (int idx = 0; idx < rank; ++idx) {
      for (int k = spec_begin[idx]; k < spec_begin[idx + 1]; ++k) {
        if (std::strcmp(spec_names[k], logical_names[p]) != 0) continue;
        int di = -1;
        for (int a = 0; a < n_mesh; ++a)
          if (std::strcmp(mesh_axis_names[a], logical_device_axes[p]) == 0) {
            di = a;
            break;
          }
        if (di < 0) return fail(MMR_INVALID_ARGUMENT, "unknown device axis '%s' in autosharding", logical_device_axes[p]);
        const int64_t total = sharding_on_axis[idx] * mesh_dims[di];
        if (total <= shape[idx] && !used[di]) {
          to_device[idx].push_back(di);
          used[di] = 1;
          sharding_on_axis[idx] = total;
        }
        break;
      }
    }
  }
  std::vector<int32_t> flat, begin{0};
  for (auto& axes : to_device) {
    flat.insert(flat.end(), axes.begin(), axes.end());
    begin.push_back(static_cast<int32_t>(flat.size()));
  }
  const int32_t list_all = dev_count < total_devices;  // :87-88
  if (int rc = mmr_logical_to_physical_sharding(flat.data(), begin.data(), rank, dev_start, dev_count, mesh_dims, n_mesh,
                                                list_all, out))
    return rc;
  if (out->type == MMR_SHARDING_OTHER) {  // :101-113: the sharding must divide every dim
    for (int d = 0; d < rank; ++d)
      if (shape[d] % out->tile_dims[d])
        return fail(MMR_INVALID_ARGUMENT, "sharding does not evenly divide shape: dim %d of extent %lld over %lld tiles", d,
                    (long long)shape[d], (long long)out->tile_dims[d]);
  }
  return MMR_OK;
}

int mmr_tile_assignment_devices(const mmr_op_sharding* s, int64_t* out, int64_t capacity, int64_t* n_out) {
  if (int rc = check_sharding(s)) return rc;
  if (!out || !n_out) return fail(MMR_INVALID_ARGUMENT, "null output");
  int64_t n = 1;
  for (int d = 0; d < s->n_tile_dims; ++d) n *= s->tile_dims[d];
  if (n > capacity) return fail(MMR_INVALID_ARGUMENT, "%lld tiles do not fit a buffer of %lld", (long long)n, (long long)capacity);
  if (s->n_iota_dims == 0) {
    if (s->n_devices != n || !s->tile_assignment_devices)
      return fail(MMR_INVALID_ARGUMENT, "explicit device list has %lld entries for %lld tiles", (long long)s->n_devices, (long long)n);
    std::copy(s->tile_assignment_devices, s->tile_assignment_devices + n, out);
    *n_out = n;
    return MMR_OK;
  }
  const int k = s->n_iota_dims;
  int64_t total = 1, stride[MMR_MAX_DIMS];
  for (int d = k - 1; d >= 0; --d) {
    stride[d] = total;
    total *= s->iota_reshape_dims[d];
  }
  if (total != n) return fail(MMR_INVALID_ARGUMENT, "iota dims hold %lld devices for %lld tiles", (long long)total, (long long)n);
  // walk the transposed iota array in row-major order
  int64_t tdims[MMR_MAX_DIMS], idx[MMR_MAX_DIMS] = {};
  for (int d = 0; d < k; ++d) tdims[d] = s->iota_reshape_dims[s->iota_transpose_perm[d]];
  for (int64_t i = 0; i < n; ++i) {
    int64_t v = 0;
    for (int d = 0; d < k; ++d) v += idx[d] * stride[s->iota_transpose_perm[d]];
    out[i] = v + s->iota_offset;
    for (int d = k - 1; d >= 0; --d) {
      if (++idx[d] < tdims[d]) break;
      idx[d] = 0;
    }
  }
  *n_out = n;
  return MMR_OK;
}

int mmr_canonicalize_sharding(const mmr_op_sharding* s, const int64_t* shape, int32_t rank, int32_t dtype,
                              int32_t shape_is_global, mmr_sharded_shape* out) {
  if (int rc = check_sharding(s)) return rc;
  if (!out || rank < 0 || (rank > 0 && !shape)) return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  if (s->n_iota_dims > 0) {  // :438-441
    std::vector<int64_t> dims;
    std::vector<int> perm;
    canonical_iota(*s, &dims, &perm);
    return canonicalize_iota(*s, dims, perm, s->iota_offset, shape, rank, dtype, shape_is_global != 0, out);
  }
  // :443-455  an explicit list is accepted only if it counts up by one
  if (!s->tile_assignment_devices || s->n_devices < 1)
    return fail(MMR_INVALID_ARGUMENT, "CanonicalizeSharding: sharding has no tile assignment");
  int64_t prev = s->tile_assignment_devices[0] - 1;
  for (int64_t i = 0; i < s->n_devices; ++i) {
    if (s->tile_assignment_devices[i] != prev + 1)
      return fail(MMR_INVALID_ARGUMENT, "CanonicalizeSharding: only supported for iota tile assignment");
    prev = s->tile_assignment_devices[i];
  }
  return canonicalize_iota(*s, {s->n_devices}, {0}, s->tile_assignment_devices[0], shape, rank, dtype,
                           shape_is_global != 0, out);
}

int mmr_xla_shape_to_sharded_shape(const int64_t* shape, int32_t rank, int32_t dtype, int64_t dev_start,
                                   int64_t dev_count, const mmr_op_sharding* s, int32_t shape_is_global,
                                   mmr_sharded_shape* out) {
  if (int rc = check_sharding(s)) return rc;
  if (!out || rank < 0 || (rank > 0 && !shape)) return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  if (int rc = map_type(dtype)) return rc;  // :586-636
  if (is_replicated(*s) || is_maximal(*s)) {  // :638-654
    if (rank + (dev_count > 1 ? 1 : 0) > MMR_MAX_DIMS) return fail(MMR_INVALID_ARGUMENT, "rank %d is too large", rank);
    mmr_sharded_shape r{};
    r.dtype = dtype;
    for (int d = 0; d < rank; ++d) r.dims[d] = mmr_sharding_dim{shape[d], 1, d};
    r.ndims = rank;
    if (dev_count > 1) r.dims[r.ndims++] = mmr_sharding_dim{1, dev_count, rank};
    r.dev_start = dev_start;
    r.dev_count = dev_count;
    *out = r;
    return MMR_OK;
  }
  mmr_sharded_shape r{};
  if (int rc = mmr_canonicalize_sharding(s, shape, rank, dtype, shape_is_global, &r)) return rc;
  if (r.dev_start != dev_start || r.dev_count != dev_count) {  // :659-668
    if (r.dev_count != dev_count)
      return fail(MMR_INVALID_ARGUMENT, "devices=[%lld...%lld) given to XlaShapeToZukuShape differs from sharding",
                  (long long)dev_start, (long long)(dev_start + dev_count));
    r.dev_start = dev_start;  // same-shaped meshes can be resharded across
  }
  *out = r;
  return MMR_OK;
}

int mmr_mesh_equivalent_sharding(const mmr_op_sharding* lhs, const mmr_op_sharding* rhs, int32_t* out) {
  if (int rc = check_sharding(lhs)) return rc;
  if (int rc = check_sharding(rhs)) return rc;
  if (!out) return fail(MMR_INVALID_ARGUMENT, "null output");
  if (replicated_or_submesh_replicate(*lhs)) {
    *out = replicated_or_submesh_replicate(*rhs);
  } else if (replicated_or_submesh_replicate(*rhs)) {
    *out = 0;
  } else {
    *out = lhs->n_tile_dims == rhs->n_tile_dims &&
           std::equal(lhs->tile_dims, lhs->tile_dims + lhs->n_tile_dims, rhs->tile_dims);
  }
  return MMR_OK;
}

int mmr_needs_reshard(int64_t operand_dev_start, int64_t operand_dev_count, int64_t dev_start, int64_t dev_count,
                      const mmr_op_sharding* operand_sharding, const mmr_op_sharding* sharding, int32_t* out) {
  if (int rc = check_sharding(operand_sharding)) return rc;
  if (int rc = check_sharding(sharding)) return rc;
  if (!out) return fail(MMR_INVALID_ARGUMENT, "null output");
  const bool contains = operand_dev_start <= dev_start && dev_start + dev_count <= operand_dev_start + operand_dev_count;
  if (is_replicated(*operand_sharding) && is_replicated(*sharding) && contains) {
    *out = 0;
    return MMR_OK;
  }
  int32_t equivalent = 0;
  if (int rc = mmr_mesh_equivalent_sharding(operand_sharding, sharding, &equivalent)) return rc;
  *out = operand_dev_start != dev_start || operand_dev_count != dev_count || !equivalent;
  return MMR_OK;
}

int mmr_device_list_of_sharding(const mmr_op_sharding* s, int64_t* dev_start, int64_t* dev_count) {
  if (int rc = check_sharding(s)) return rc;
  if (!dev_start || !dev_count) return fail(MMR_INVALID_ARGUMENT, "null output");
  if (s->n_iota_dims > 0) {  // mpmd_utils.cc:158-165
    int64_t n = 1;
    for (int i = 0; i < s->n_iota_dims; ++i) n *= s->iota_reshape_dims[i];
    *dev_start = s->iota_offset;
    *dev_count = n;
    return MMR_OK;
  }
  if (s->n_devices < 1 || !s->tile_assignment_devices) return fail(MMR_INVALID_ARGUMENT, "sharding names no devices");
  for (int64_t i = 1; i < s->n_devices; ++i)  // :167-175
    if (s->tile_assignment_devices[i] != s->tile_assignment_devices[i - 1] + 1)
      return fail(MMR_UNSUPPORTED, "non-iota tile assignments not yet supported for DeviceList");
  *dev_start = s->tile_assignment_devices[0];
  *dev_count = s->n_devices;
  return MMR_OK;
}

int mmr_to_mpmd_sharding(int32_t rank, const mmr_op_sharding* sharding, int64_t task_dev_start, int64_t task_dev_count,
                         int64_t global_dev_start, int64_t global_dev_count, mmr_op_sharding* out, int64_t* devices_out,
                         int64_t devices_capacity) {
  if (int rc = check_sharding(sharding)) return rc;
  if (!out) return fail(MMR_INVALID_ARGUMENT, "null output");
  if (rank < 0 || rank >= MMR_MAX_DIMS) return fail(MMR_INVALID_ARGUMENT, "rank %d", rank);
  if (task_dev_count < 1) return fail(MMR_INVALID_ARGUMENT, "empty task device list");
  mmr_op_sharding r{};
  const bool same_devices = task_dev_start == global_dev_start && task_dev_count == global_dev_count;
  // :132-134  replicated over the whole machine stays replicated
  if (is_replicated(*sharding) && same_devices) {
    r.type = MMR_SHARDING_REPLICATED;
    *out = r;
    return MMR_OK;
  }
  // :136-139  one device: the array lives on that device
  if (task_dev_count == 1 && (is_maximal(*sharding) || is_replicated(*sharding))) {
    if (!devices_out || devices_capacity < 1) return fail(MMR_INVALID_ARGUMENT, "device list output too small");
    devices_out[0] = task_dev_start;
    r.type = MMR_SHARDING_MAXIMAL;
    r.tile_assignment_devices = devices_out;
    r.n_devices = 1;
    *out = r;
    return MMR_OK;
  }
  r = *sharding;
  r.tile_assignment_devices = nullptr;
  r.n_devices = 0;
  if (sharding->n_iota_dims > 0) {
    r.iota_offset = task_dev_start;  // :143-144
  } else if (sharding->n_devices > 0) {
    // :145-150  ids relative to the task's device list -> global ids
    if (!devices_out || devices_capacity < sharding->n_devices)
      return fail(MMR_INVALID_ARGUMENT, "device list output too small");
    for (int64_t i = 0; i < sharding->n_devices; ++i) {
      const int64_t rel = sharding->tile_assignment_devices[i];
      if (rel < 0 || rel >= task_dev_count)
        return fail(MMR_INVALID_ARGUMENT, "relative device id %lld outside the task's %lld devices", (long long)rel,
                    (long long)task_dev_count);
      devices_out[i] = task_dev_start + rel;
    }
    r.tile_assignment_devices = devices_out;
    r.n_devices = sharding->n_devices;
  }
  // :152-163  replicated on a subset of the devices: one tile per tensor dim, all of the task's devices as replicas
  if (is_replicated(*sharding) && rank > 0) {
    r = mmr_op_sharding{};
    r.type = MMR_SHARDING_OTHER;
    r.n_tile_dims = rank + 1;
    for (int i = 0; i < rank; ++i) r.tile_dims[i] = 1;
    r.tile_dims[rank] = task_dev_count;
    r.n_iota_dims = 1;
    r.iota_reshape_dims[0] = task_dev_count;
    r.iota_transpose_perm[0] = 0;
    r.iota_offset = task_dev_start;
    r.replicate_on_last_tile_dim = 1;
  }
  *out = r;
  return MMR_OK;
}

int mmr_replicate_dims(const mmr_op_sharding* sharding, const int64_t* replicated_dims, int32_t n_replicated,
                       mmr_op_sharding* out) {
  if (int rc = check_sharding(sharding)) return rc;
  if (!out || n_replicated < 0 || (n_replicated > 0 && !replicated_dims)) return fail(MMR_INVALID_ARGUMENT, "null argument");
  if (sharding->n_iota_dims <= 0)  // mm_sharding.cc:465-468
    return fail(MMR_INVALID_ARGUMENT, "ReplicateDims only supported for iota tile assignment");
  const int n_ta = sharding->n_tile_dims;
  const int64_t* ta = sharding->tile_dims;
  for (int i = 0; i < n_replicated; ++i)
    if (replicated_dims[i] < 0 || replicated_dims[i] >= n_ta)
      return fail(MMR_INVALID_ARGUMENT, "replicated dim %lld of %d tile dims", (long long)replicated_dims[i], n_ta);
  std::vector<int64_t> reshape;
  std::vector<int> perm;
  canonical_iota(*sharding, &reshape, &perm);
  // :476-514  un-group the iota dims into tile-assignment dims, then order the groups as the transpose does
  std::vector<std::vector<int>> groups(1);
  size_t iota_dim = 0;
  int64_t spanned = 1;
  int ta_dim = 0;
  for (; ta_dim < n_ta && iota_dim < perm.size(); ++ta_dim) {
    spanned *= ta[ta_dim];
    const int64_t span = reshape[static_cast<size_t>(perm[iota_dim])];
    groups.back().push_back(ta_dim);
    if (spanned >= span) {
      ++iota_dim;
      if (iota_dim < perm.size()) groups.emplace_back();
      spanned = 1;
    }
  }
  for (; ta_dim < n_ta; ++ta_dim) groups.back().push_back(ta_dim);
  if (groups.size() != perm.size()) return fail(MMR_INVALID_ARGUMENT, "iota dims do not group into tile assignment dims");
  std::vector<int> current;
  for (int src : perm)
    for (int d : groups[static_cast<size_t>(src)]) current.push_back(d);
  // :516-540
  std::vector<int64_t> new_reshape;
  for (int d : current) new_reshape.push_back(ta[d]);
  for (int i = 0; i < n_replicated; ++i) new_reshape.push_back(1);
  const bool repl_last = sharding->replicate_on_last_tile_dim != 0;
  const int num_shape_dims = repl_last ? n_ta - 1 : n_ta;
  std::vector<int> new_perm(current);
  int extra = static_cast<int>(new_perm.size());
  for (int i = 0; i < n_replicated; ++i) {
    const size_t dim = static_cast<size_t>(replicated_dims[i]);
    if (dim >= current.size()) return fail(MMR_INVALID_ARGUMENT, "replicated dim outside the permutation");
    new_perm.push_back(current[dim]);
    new_perm[dim] = extra++;
  }
  int64_t total = repl_last ? ta[num_shape_dims] : 1, elements = 1;  // :542-552
  for (int i = 0; i < n_replicated; ++i) total *= ta[replicated_dims[i]];
  for (int i = 0; i < n_ta; ++i) elements *= ta[i];
  mmr_op_sharding r{};
  if (total == elements) {  // :554-557
    r.type = MMR_SHARDING_REPLICATED;
    *out = r;
    return MMR_OK;
  }
  std::vector<int64_t> ta_dims(ta, ta + n_ta);  // :559-571
  if (repl_last) ta_dims[static_cast<size_t>(num_shape_dims)] = total;
  else ta_dims.push_back(total);
  for (int i = 0; i < n_replicated; ++i) ta_dims[static_cast<size_t>(replicated_dims[i])] = 1;
  // The reference hands the raw lists to HloSharding::FromProto, which keeps the canonical iota; so does this.
  std::vector<int64_t> cd;
  std::vector<int> cp;
  canonical_iota(new_reshape, new_perm, &cd, &cp);
  if (ta_dims.size() > MMR_MAX_DIMS || cd.size() > MMR_MAX_DIMS)
    return fail(MMR_UNSUPPORTED, "more than %d tile or iota dims", MMR_MAX_DIMS);
  r.type = MMR_SHARDING_OTHER;
  r.n_tile_dims = static_cast<int32_t>(ta_dims.size());
  for (size_t i = 0; i < ta_dims.size(); ++i) r.tile_dims[i] = ta_dims[i];
  r.n_iota_dims = static_cast<int32_t>(cd.size());
  for (size_t i = 0; i < cd.size(); ++i) {
    r.iota_reshape_dims[i] = cd[i];
    r.iota_transpose_perm[i] = cp[i];
  }
  r.replicate_on_last_tile_dim = 1;
  r.iota_offset = sharding->iota_offset;
  *out = r;
  return MMR_OK;
}

int mmr_resize_sharding(const int64_t* shape, int32_t rank, const mmr_op_sharding* sharding, int64_t num_elements,
                        int64_t dev_start, int64_t dev_count, mmr_op_sharding* out, int64_t* devices_out,
                        int64_t devices_capacity, int32_t* found) {
  if (int rc = check_sharding(sharding)) return rc;
  if (!out || !found || (rank > 0 && !shape)) return fail(MMR_INVALID_ARGUMENT, "null argument");
  *found = 0;
  const int n_ta = sharding->n_tile_dims;
  if (n_ta > rank) return fail(MMR_INVALID_ARGUMENT, "%d tile dims for a shape of rank %d", n_ta, rank);
  if (num_elements < 1) return fail(MMR_INVALID_ARGUMENT, "%lld tiles", (long long)num_elements);
  const bool has_devices = dev_count > 0;
  const bool iota = sharding->n_iota_dims > 0;
  if (iota) {  // mm_sharding.cc:101-109  no answer under a transposed device order
    std::vector<int64_t> d;
    std::vector<int> p;
    canonical_iota(*sharding, &d, &p);
    for (size_t i = 0; i < p.size(); ++i)
      if (p[i] != static_cast<int>(i)) return MMR_OK;
  }
  int64_t src_size = 1;
  for (int i = 0; i < n_ta; ++i) src_size *= sharding->tile_dims[i];
  const int64_t dst_size = num_elements;
  mmr_op_sharding r{};
  r.type = MMR_SHARDING_OTHER;
  bool matched = false;
  for (int dim = 0; dim < n_ta; ++dim) {  // :120-142
    const int64_t old_size = sharding->tile_dims[dim];
    const int64_t new_size = old_size * dst_size / src_size;
    if (!matched && old_size > 1 && new_size > 0 && new_size <= shape[dim]) {
      if ((src_size > dst_size && src_size % dst_size) || (src_size < dst_size && dst_size % src_size)) continue;
      r.tile_dims[r.n_tile_dims++] = new_size;
      matched = true;
    } else {
      r.tile_dims[r.n_tile_dims++] = old_size;
    }
    // the reference indexes the dims written so far by `dim`; after a skipped dim that entry does not exist
    if (dim == n_ta - 1 && sharding->replicate_on_last_tile_dim && r.n_tile_dims == dim + 1 && r.tile_dims[dim] > 1)
      r.replicate_on_last_tile_dim = 1;
  }
  if (!matched) return MMR_OK;
  int64_t tiles = 1;
  for (int i = 0; i < r.n_tile_dims; ++i) tiles *= r.tile_dims[i];
  if (iota || !has_devices) {  // :144-150
    r.n_iota_dims = 1;
    r.iota_reshape_dims[0] = num_elements;
    r.iota_transpose_perm[0] = 0;
    if (has_devices) r.iota_offset = dev_start;
    if (tiles != num_elements) return MMR_OK;  // HloSharding::FromProto refuses it
  } else {  // :151-154
    if (tiles != dev_count) return MMR_OK;
    if (!devices_out || devices_capacity < dev_count) return fail(MMR_INVALID_ARGUMENT, "device list output too small");
    for (int64_t i = 0; i < dev_count; ++i) devices_out[i] = dev_start + i;
    r.tile_assignment_devices = devices_out;
    r.n_devices = dev_count;
  }
  *out = r;
  *found = 1;
  return MMR_OK;
}

}  // extern "C"
