// Shard-intersection planner (host only).
//
// For every destination tile the overlapping source tiles are found by
// per-dimension interval intersection; each overlap is an N-d box with a byte
// stride per dim on either side.  Boxes are canonicalised (extent-1 dims
// dropped, dims that are contiguous on both sides merged) and lowered to
// workgroup-sized chunks:
//   * copy chunks     - n2 x n1 rows of w contiguous bytes (minor dim kept),
//   * transpose chunks - workgroup tiles (128 x 128 elements for 2-byte types) staged through LDS (source and
//                        destination disagree on the minor dim),
//   * fill chunks      - copy chunks without a source, zeroing the pad of short
//                        edge tiles.
#include "planner.h"

#include "chunk_ops.h"

#include <algorithm>
#include <cstring>

namespace mmr {
namespace {

struct BoxDim {
  int64_t n;  // extent in elements
  int64_t s;  // source byte stride
  int64_t d;  // destination byte stride
};

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

constexpr int64_t kGenericMaxPairs = 768;  // (row, slot) pairs of one generic chunk

class Builder {
 public:
  Builder(mmr_plan* plan, uint32_t chunk_bytes, uint32_t generic_chunk_bytes, bool force_generic)
      : plan_(plan), chunk_bytes_(chunk_bytes), generic_chunk_bytes_(generic_chunk_bytes), force_generic_(force_generic) {}

  void add_box(uint32_t src_slot, uint32_t dst_slot, int64_t src_off, int64_t dst_off, const BoxDim* in, int rank,
               int itemsize) {
    std::vector<BoxDim> dims;
    int64_t volume = 1;
    for (int i = 0; i < rank; ++i) {
      if (in[i].n <= 0) return;
      volume *= in[i].n;
      if (in[i].n > 1) dims.push_back(in[i]);
    }
    const bool fill = src_slot == MMR_SLOT_FILL;
    if (fill) {
      plan_->stats.bytes_filled += volume * itemsize;
    } else {
      plan_->stats.bytes_moved += volume * itemsize;
      plan_->stats.n_boxes += 1;
    }
    // destination-major order, then merge dims that are contiguous on both sides
    std::stable_sort(dims.begin(), dims.end(), [](const BoxDim& a, const BoxDim& b) {
      return a.d != b.d ? a.d > b.d : a.s > b.s;
    });
    for (int i = static_cast<int>(dims.size()) - 1; i > 0; --i) {
      if (dims[i - 1].s == dims[i].s * dims[i].n && dims[i - 1].d == dims[i].d * dims[i].n) {
        dims[i - 1] = BoxDim{dims[i - 1].n * dims[i].n, dims[i].s, dims[i].d};
        dims.erase(dims.begin() + i);
      }
    }
    int run = -1, x = -1, y = -1;
    for (int i = 0; i < static_cast<int>(dims.size()); ++i) {
      if (dims[i].s == itemsize && dims[i].d == itemsize) run = i;
      else if (dims[i].s == itemsize) x = i;
      else if (dims[i].d == itemsize) y = i;
    }
    if (run < 0 && x >= 0 && y >= 0 && !fill) {
      lower_transpose(src_slot, dst_slot, src_off, dst_off, dims, x, y, itemsize);
      return;
    }
    int64_t w = itemsize;
    if (run >= 0) {
      w = dims[run].n * itemsize;
      dims.erase(dims.begin() + run);
    }
    lower_copy(src_slot, dst_slot, src_off, dst_off, dims, w, fill);
  }

 private:
  // index of the dim whose rows are closest together on either side
  static int pick_row_dim(const std::vector<BoxDim>& dims, int skip) {
    int best = -1;
    for (int i = 0; i < static_cast<int>(dims.size()); ++i) {
      if (i == skip) continue;
      if (best < 0) { best = i; continue; }
      const int64_t a_lo = std::min(dims[i].s, dims[i].d), a_hi = std::max(dims[i].s, dims[i].d);
      const int64_t b_lo = std::min(dims[best].s, dims[best].d), b_hi = std::max(dims[best].s, dims[best].d);
      if (a_lo < b_lo || (a_lo == b_lo && a_hi < b_hi)) best = i;
    }
    return best;
  }

  // Calls fn(src_delta, dst_delta) for every index combination of `dims`.
  template <class Fn>
  static void for_each_index(const std::vector<BoxDim>& dims, Fn&& fn) {
    std::vector<int64_t> idx(dims.size(), 0);
    int64_t so = 0, dof = 0;
    while (true) {
      fn(so, dof);
      int k = static_cast<int>(dims.size()) - 1;
      for (; k >= 0; --k) {
        idx[k]++;
        so += dims[k].s;
        dof += dims[k].d;
        if (idx[k] < dims[k].n) break;
        so -= dims[k].s * dims[k].n;
        dof -= dims[k].d * dims[k].n;
        idx[k] = 0;
      }
      if (k < 0) break;
    }
  }

  void emit_copy(uint32_t src_slot, uint32_t dst_slot, int64_t so, int64_t dof, int64_t w, int64_t n1, int64_t n2,
                 int64_t s1, int64_t d1, int64_t s2, int64_t d2, bool fill) {
    mmr_copy_chunk c{};
    c.src_slot = src_slot;
    c.dst_slot = dst_slot;
    c.src_off = fill ? 0 : static_cast<uint64_t>(so);
    c.dst_off = static_cast<uint64_t>(dof);
    c.w = static_cast<uint32_t>(w);
    c.n1 = static_cast<uint32_t>(n1);
    c.n2 = static_cast<uint32_t>(n2);
    c.s1 = (n1 > 1 && !fill) ? s1 : 0;
    c.d1 = n1 > 1 ? d1 : 0;
    c.s2 = (n2 > 1 && !fill) ? s2 : 0;
    c.d2 = n2 > 1 ? d2 : 0;
    uint64_t bits = c.src_off | c.dst_off | c.w | static_cast<uint64_t>(c.s1) | static_cast<uint64_t>(c.d1) |
                    static_cast<uint64_t>(c.s2) | static_cast<uint64_t>(c.d2);
    c.align = (bits & 15u) ? static_cast<uint32_t>(bits & (~bits + 1)) : 16u;
    if (fill) plan_->stats.n_fill_chunks += 1;
    (c.align == 16 && !force_generic_ ? plan_->copy16 : plan_->generic).push_back(c);
  }

  void lower_copy(uint32_t src_slot, uint32_t dst_slot, int64_t so, int64_t dof, std::vector<BoxDim>& outer, int64_t w,
                  bool fill) {
    // Rows that are not 16-byte aligned on both sides go to the generic kernel,
    // which spends one lane per 16-byte slot plus ragged ends: give it half the
    // bytes per workgroup so its workgroups live about as long as aligned ones.
    uint64_t bits = static_cast<uint64_t>(so | dof | w);
    for (const BoxDim& d : outer) bits |= static_cast<uint64_t>(d.s | d.d);
    const bool aligned = (bits & 15u) == 0 && !force_generic_;
    const int64_t cb = aligned ? chunk_bytes_ : generic_chunk_bytes_;
    if (w > cb) {
      // long rows: split columns into near-equal segments on 256-byte boundaries of the row
      const int64_t nseg = ceil_div(w, cb);
      const int64_t seg = ceil_div(ceil_div(w, nseg), 256) * 256;
      for_each_index(outer, [&](int64_t ds, int64_t dd) {
        for (int64_t c0 = 0; c0 < w; c0 += seg)
          emit_copy(src_slot, dst_slot, so + ds + c0, dof + dd + c0, std::min(seg, w - c0), 1, 1, 0, 0, 0, 0, fill);
      });
      return;
    }
    int64_t rows = std::max<int64_t>(1, cb / w);
    if (!aligned) {
      // The generic kernel spends one lane per (row, 16-byte slot) pair whatever the row holds: a chunk of very
      // narrow rows sized by bytes alone (the one-byte pad column of a short edge tile: 5,632 rows) keeps its
      // workgroup busy long after its neighbours have finished and becomes the tail of the launch.  Bound the
      // pairs per chunk (3 per lane of a 256-lane workgroup) as well as the bytes.
      const int64_t slots = (w + 15) / 16 + 1;
      rows = std::max<int64_t>(1, std::min(rows, kGenericMaxPairs / slots));
    }
    int i1 = pick_row_dim(outer, -1);
    if (i1 < 0) {
      emit_copy(src_slot, dst_slot, so, dof, w, 1, 1, 0, 0, 0, 0, fill);
      return;
    }
    BoxDim dim1 = outer[i1];
    int64_t n1 = std::min(dim1.n, rows);
    if (aligned && n1 < dim1.n && (dim1.d == w || dim1.s == w)) {
      // Rows that abut on one side, cut into several chunks along this dim: keep the cuts on 128-byte lines of that
      // side where a few rows less achieve it, so no line is shared by two workgroups (832-byte rows: 8 per chunk
      // instead of 9 measured +3 %).
      int64_t g = w, h = 128;
      while (h != 0) {
        const int64_t t = g % h;
        g = h;
        h = t;
      }
      const int64_t m = 128 / g;
      if (n1 > m) n1 = n1 / m * m;
    }
    BoxDim dim2{1, 0, 0};
    int64_t n2 = 1;
    int i2 = -1;
    // Rows that continue the run on the destination side along one dim (A) and on
    // the source side along another (B), as a fused layout permutation produces:
    // take a 2-D block so both sides see runs of several rows instead of one side
    // seeing single rows at a large stride.
    int ia = -1, ib = -1;
    if (aligned && !fill && outer.size() >= 2) {
      for (int i = 0; i < static_cast<int>(outer.size()); ++i) {
        if (outer[i].d == w && outer[i].s != w) ia = i;
        if (outer[i].s == w && outer[i].d != w) ib = i;
      }
    }
    if (ia >= 0 && ib >= 0 && rows >= 4) {
      const BoxDim da = outer[ia], db = outer[ib];
      int64_t na = 1;
      while (na * 2 <= da.n && na * na * 4 <= rows) na *= 2;  // about sqrt(rows), a power of two
      if (da.n * da.n <= 4 * rows) na = da.n;                  // or the whole of a short dim
      const int64_t nb = std::max<int64_t>(1, std::min(db.n, rows / na));
      i1 = ia;
      dim1 = da;
      n1 = std::min(na, da.n);
      i2 = ib;
      dim2 = db;
      n2 = nb;
    } else if (aligned && n1 == dim1.n && rows / n1 >= 2) {  // the generic kernel walks a single row dimension
      i2 = pick_row_dim(outer, i1);
      if (i2 >= 0) {
        dim2 = outer[i2];
        n2 = std::min(dim2.n, rows / n1);
      }
    }
    std::vector<BoxDim> rest;
    for (int i = 0; i < static_cast<int>(outer.size()); ++i)
      if (i != i1 && i != i2) rest.push_back(outer[i]);
    for_each_index(rest, [&](int64_t ds, int64_t dd) {
      for (int64_t b2 = 0; b2 < dim2.n; b2 += n2) {
        const int64_t m2 = std::min(n2, dim2.n - b2);
        for (int64_t b1 = 0; b1 < dim1.n; b1 += n1) {
          const int64_t m1 = std::min(n1, dim1.n - b1);
          emit_copy(src_slot, dst_slot, so + ds + b2 * dim2.s + b1 * dim1.s, dof + dd + b2 * dim2.d + b1 * dim1.d, w, m1,
                    m2, dim1.s, dim1.d, dim2.s, dim2.d, fill);
        }
      }
    });
  }

  void lower_transpose(uint32_t src_slot, uint32_t dst_slot, int64_t so, int64_t dof, const std::vector<BoxDim>& dims,
                       int x, int y, int itemsize) {
    uint32_t tx = 0, ty = 0;
    transpose_tile_extent(static_cast<uint32_t>(itemsize), &tx, &ty);
    int64_t tile_x = tx, tile_y = ty;
    const BoxDim dx = dims[x], dy = dims[y];
    // A box thinner than one 16-byte vector one way (3 channels moving out of the minor position, say) goes through
    // the kernel's thin path, which takes any tile that fits the workgroup's LDS: make the tile long the other way
    // instead of leaving chunks of a few hundred bytes.  That path works element by element, so its chunks are
    // sized by elements (32 per thread at most), and a small box is cut into about a thousand chunks or more so
    // that it still spreads over the 256 CUs.
    const int64_t vec = 16 / itemsize;
    const bool thin = dx.n < vec || dy.n < vec;
    int64_t chunk_bytes = kTransposeChunkBytes;
    if (thin) {
      int64_t box_bytes = itemsize;
      for (const BoxDim& d : dims) box_bytes *= d.n;
      chunk_bytes = std::min<int64_t>(chunk_bytes, 8192 * itemsize);
      chunk_bytes = std::max<int64_t>(std::min<int64_t>(chunk_bytes, box_bytes / 1024), 1024);
      if (dx.n < vec) tile_y = std::max<int64_t>(tile_y, chunk_bytes / (dx.n * itemsize) / tile_y * tile_y);
      else tile_x = std::max<int64_t>(tile_x, chunk_bytes / (dy.n * itemsize) / tile_x * tile_x);
    }
    std::vector<BoxDim> outer;
    for (int i = 0; i < static_cast<int>(dims.size()); ++i)
      if (i != x && i != y) outer.push_back(dims[i]);
    int ib = pick_row_dim(outer, -1);
    BoxDim db{1, 0, 0};
    if (ib >= 0) {
      db = outer[ib];
      outer.erase(outer.begin() + ib);
    }
    // tiles narrower than the workgroup tile (a short x or y extent) are batched along the next dimension
    const int64_t tile_bytes = std::min(tile_x, dx.n) * std::min(tile_y, dy.n) * itemsize;
    const int64_t nb = std::max<int64_t>(1, std::min<int64_t>(db.n, chunk_bytes / tile_bytes));
    for_each_index(outer, [&](int64_t ds, int64_t dd) {
      for (int64_t b0 = 0; b0 < db.n; b0 += nb) {
        for (int64_t y0 = 0; y0 < dy.n; y0 += tile_y) {
          for (int64_t x0 = 0; x0 < dx.n; x0 += tile_x) {
            mmr_transpose_chunk c{};
            c.src_slot = src_slot;
            c.dst_slot = dst_slot;
            c.src_off = static_cast<uint64_t>(so + ds + b0 * db.s + y0 * dy.s + x0 * dx.s);
            c.dst_off = static_cast<uint64_t>(dof + dd + b0 * db.d + y0 * dy.d + x0 * dx.d);
            c.nx = static_cast<uint32_t>(std::min(tile_x, dx.n - x0));
            c.ny = static_cast<uint32_t>(std::min(tile_y, dy.n - y0));
            c.nb = static_cast<uint32_t>(std::min(nb, db.n - b0));
            c.itemsize = static_cast<uint32_t>(itemsize);
            c.src_ystride = dy.s;
            c.dst_xstride = dx.d;
            c.src_bstride = db.s;
            c.dst_bstride = db.d;
            plan_->transposes.push_back(c);
          }
        }
      }
    });
  }

  mmr_plan* plan_;
  uint32_t chunk_bytes_;
  uint32_t generic_chunk_bytes_;
  bool force_generic_;
};

int plan_one_array(Builder& b, const Side& S, const Side& D, uint32_t slot_base) {
  const int rank = S.rank;
  const int item = S.itemsize;
  for (int i = 0; i < rank; ++i)
    if (S.size[i] == 0) return MMR_OK;  // empty array: nothing to move, nothing to pad
  for (int64_t dd = 0; dd < D.dev_count; ++dd) {
    const uint32_t dslot = slot_base + static_cast<uint32_t>(S.dev_count + dd);
    int64_t lo[kMaxRank], hi[kMaxRank], valid[kMaxRank];
    bool padded = false, empty = false;
    for (int i = 0; i < rank; ++i) {
      const int64_t c = (dd / D.dev_stride[i]) % D.tiles[i];
      lo[i] = std::min(c * D.ext[i], D.size[i]);
      hi[i] = std::min(lo[i] + D.ext[i], D.size[i]);
      valid[i] = hi[i] - lo[i];
      padded |= valid[i] < D.ext[i];
      empty |= valid[i] == 0;
    }
    if (padded) {
      // the pad of a short tile is rank slabs: dim i beyond its valid extent,
      // dims before it inside theirs, dims after it whole
      for (int i = 0; i < rank; ++i) {
        if (valid[i] == D.ext[i]) continue;
        BoxDim dims[kMaxRank];
        for (int j = 0; j < rank; ++j) {
          const int64_t n = j < i ? valid[j] : (j == i ? D.ext[i] - valid[i] : D.ext[j]);
          dims[j] = BoxDim{n, D.stride[j] * item, D.stride[j] * item};
        }
        b.add_box(MMR_SLOT_FILL, dslot, 0, valid[i] * D.stride[i] * item, dims, rank, item);
      }
    }
    if (empty) continue;
    int64_t t_lo[kMaxRank], t_n[kMaxRank], combos = 1;
    for (int i = 0; i < rank; ++i) {
      t_lo[i] = lo[i] / S.ext[i];
      t_n[i] = (hi[i] - 1) / S.ext[i] - t_lo[i] + 1;
      combos *= t_n[i];
    }
    for (int64_t c = 0; c < combos; ++c) {
      int64_t rem = c, sdev = 0, soff = 0, doff = 0;
      BoxDim dims[kMaxRank];
      for (int i = rank - 1; i >= 0; --i) {
        const int64_t t = t_lo[i] + rem % t_n[i];
        rem /= t_n[i];
        const int64_t s_lo = t * S.ext[i];
        const int64_t b_lo = std::max(lo[i], s_lo);
        const int64_t b_hi = std::min(hi[i], std::min(s_lo + S.ext[i], S.size[i]));
        dims[i] = BoxDim{b_hi - b_lo, S.stride[i] * item, D.stride[i] * item};
        soff += (b_lo - s_lo) * S.stride[i] * item;
        doff += (b_lo - lo[i]) * D.stride[i] * item;
        sdev += t * S.dev_stride[i];  // of R source replicas the lowest device id is read
      }
      b.add_box(slot_base + static_cast<uint32_t>(sdev), dslot, soff, doff, dims, rank, item);
    }
  }
  return MMR_OK;
}

}  // namespace

std::string plan_key(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int n,
                     const mmr_plan_options& options) {
  std::string k;
  k.append(reinterpret_cast<const char*>(&options), sizeof(options));
  k.append(reinterpret_cast<const char*>(&n), sizeof(n));
  for (int a = 0; a < n; ++a) {
    k += descriptor_key(srcs[a]);
    k += descriptor_key(dsts[a]);
  }
  return k;
}

int build_plan(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int n, const mmr_plan_options& options,
               mmr_plan* plan) {
  if (n < 0 || (n > 0 && (!srcs || !dsts))) return fail(MMR_INVALID_ARGUMENT, "bad descriptor arrays");
  uint32_t chunk_bytes = options.chunk_bytes ? options.chunk_bytes : kDefaultChunkBytes;
  chunk_bytes = std::min<uint32_t>(std::max<uint32_t>(chunk_bytes, 256), 16u << 20) & ~255u;
  plan->options = options;
  // Ragged rows cost more instructions per byte, so their chunks are half the aligned size when a size is asked
  // for.  By default 7 KiB (8 rows of configuration 5's 820-byte rows), measured best on large arrays (360 MB of
  // them: 5.13 TB/s against 5.00 at 5.5 KiB); a plan under ~58 MB gets proportionally smaller chunks, so that it
  // still has some 8,000 of them to spread over 256 CUs (configuration 5, 45 MB, buffers not in the Infinity Cache:
  // 4.35 TB/s at 5 KiB against 4.23 at 7 KiB and 3.95 at 8 KiB).
  uint32_t generic_chunk_bytes = std::max<uint32_t>(chunk_bytes / 2, 256);
  if (options.chunk_bytes == 0) {
    int64_t payload = 0;
    for (int a = 0; a < n; ++a) {
      int64_t bytes = mmr_itemsize(srcs[a].dtype) > 0 ? mmr_itemsize(srcs[a].dtype) : 1;
      for (int i = 0; i < srcs[a].ndims && i < MMR_MAX_DIMS; ++i) bytes *= std::max<int64_t>(srcs[a].dims[i].size, 1);
      payload += bytes;
    }
    generic_chunk_bytes = static_cast<uint32_t>(std::min<int64_t>(std::max<int64_t>(payload / 8192, 2048), 7168)) & ~255u;
  }
  Builder builder(plan, chunk_bytes, generic_chunk_bytes, (options.flags & MMR_PLAN_ALL_GENERIC) != 0);
  struct SlotInfo {
    int array;
    int64_t shard_bytes;
  };
  std::vector<SlotInfo> slot_info;  // by slot
  for (int a = 0; a < n; ++a) {
    Side S, D;
    if (int rc = make_side(srcs[a], &S)) return rc;
    if (int rc = make_side(dsts[a], &D)) return rc;
    if (S.dtype != D.dtype)
      return fail(MMR_INVALID_ARGUMENT, "array %d: source type %d differs from destination type %d", a, S.dtype, D.dtype);
    if (S.rank != D.rank)
      return fail(MMR_INVALID_ARGUMENT, "array %d: source rank %d differs from destination rank %d", a, S.rank, D.rank);
    for (int i = 0; i < S.rank; ++i)
      if (S.size[i] != D.size[i])
        return fail(MMR_INVALID_ARGUMENT, "array %d: dim %d is %lld in the source and %lld in the destination", a, i,
                    (long long)S.size[i], (long long)D.size[i]);
    if (plan->n_slots + S.dev_count + D.dev_count >= static_cast<int64_t>(MMR_SLOT_FILL))
      return fail(MMR_INVALID_ARGUMENT, "too many shard buffers in one plan");
    plan->srcs.push_back(srcs[a]);
    plan->dsts.push_back(dsts[a]);
    plan->slot_bases.push_back(plan->n_slots);
    for (int64_t k = 0; k < S.dev_count; ++k) slot_info.push_back({a, S.shard_bytes});
    for (int64_t k = 0; k < D.dev_count; ++k) slot_info.push_back({a, D.shard_bytes});
    if (int rc = plan_one_array(builder, S, D, static_cast<uint32_t>(plan->n_slots))) return rc;
    plan->n_slots += S.dev_count + D.dev_count;
  }
  // A plan that is mostly ragged rows: its few aligned chunks ride along in the
  // generic table (the generic kernel handles aligned rows too), one launch less.
  if (!plan->generic.empty() && !plan->copy16.empty()) {
    int64_t aligned_bytes = 0, generic_bytes = 0;
    bool one_dim = true;
    for (const mmr_copy_chunk& c : plan->copy16) {
      aligned_bytes += static_cast<int64_t>(c.w) * c.n1 * c.n2;
      one_dim &= c.n2 == 1;
    }
    for (const mmr_copy_chunk& c : plan->generic) generic_bytes += static_cast<int64_t>(c.w) * c.n1 * c.n2;
    if (one_dim && aligned_bytes * 4 < generic_bytes) {
      plan->generic.insert(plan->generic.end(), plan->copy16.begin(), plan->copy16.end());
      plan->copy16.clear();
    }
  }
  // Default order: aligned chunks and transpose tiles by destination address; ragged (generic) chunks by
  // destination with the tiles of an array interleaved (4), measured +12 % on configuration 5.
  const uint32_t order = options.order ? options.order : 2;
  const uint32_t generic_order = options.order ? options.order : 4;
  if (order == 2 || order == 3) {
    // Sorting 72-byte records directly dominated the planning time of large batches: sort (key, index) triples
    // and permute once.  The index as last key keeps equal keys (fill chunks share FILL as source) in emission order.
    auto sort_copy = [order](std::vector<mmr_copy_chunk>& table) {
      struct Key {
        uint64_t slot, off;
        uint32_t index;
      };
      std::vector<Key> keys(table.size());
      bool sorted = true;
      for (size_t i = 0; i < table.size(); ++i) {
        const mmr_copy_chunk& c = table[i];
        keys[i] = order == 2 ? Key{c.dst_slot, c.dst_off, static_cast<uint32_t>(i)}
                             : Key{c.src_slot, c.src_off, static_cast<uint32_t>(i)};
        if (i > 0 && std::tie(keys[i].slot, keys[i].off) < std::tie(keys[i - 1].slot, keys[i - 1].off)) sorted = false;
      }
      if (sorted) return;
      std::sort(keys.begin(), keys.end(), [](const Key& a, const Key& b) {
        return std::tie(a.slot, a.off, a.index) < std::tie(b.slot, b.off, b.index);
      });
      std::vector<mmr_copy_chunk> out(table.size());
      for (size_t i = 0; i < keys.size(); ++i) out[i] = table[keys[i].index];
      table.swap(out);
    };
    sort_copy(plan->copy16);
    if (generic_order == order) sort_copy(plan->generic);
  }
  if (order == 4 || generic_order == 4) {
    // Ragged rows: chunks of different destination tiles that cover the same rows read the same source lines at
    // the edges of their column ranges.  Cut every destination buffer into equal fractions and keep the chunks of
    // one fraction of all tiles of an array together (inside a fraction: by destination address), so that they
    // run at the same time on the same XCD and the shared lines are fetched once.
    const int64_t fraction_kib = (options.flags >> 8) & 0xffffu;  // tuning knob; 0 = default
    const int64_t fraction_bytes = (fraction_kib ? fraction_kib : 64) * 1024;
    auto sort_interleaved = [&](std::vector<mmr_copy_chunk>& table) {
      struct Key {
        uint64_t array, fraction, slot, off;
        uint32_t index;
      };
      std::vector<Key> keys(table.size());
      for (size_t i = 0; i < table.size(); ++i) {
        const mmr_copy_chunk& c = table[i];
        const SlotInfo& info = slot_info[c.dst_slot];
        const uint64_t fractions = std::max<int64_t>(1, info.shard_bytes / fraction_bytes);
        keys[i] = Key{static_cast<uint64_t>(info.array),
                      info.shard_bytes > 0 ? c.dst_off * fractions / static_cast<uint64_t>(info.shard_bytes) : 0, c.dst_slot,
                      c.dst_off, static_cast<uint32_t>(i)};
      }
      std::sort(keys.begin(), keys.end(), [](const Key& a, const Key& b) {
        return std::tie(a.array, a.fraction, a.slot, a.off, a.index) < std::tie(b.array, b.fraction, b.slot, b.off, b.index);
      });
      std::vector<mmr_copy_chunk> out(table.size());
      for (size_t i = 0; i < keys.size(); ++i) out[i] = table[keys[i].index];
      table.swap(out);
    };
    if (order == 4) sort_interleaved(plan->copy16);
    sort_interleaved(plan->generic);
  }
  if (order == 2 || order == 3 || order == 4) {
    // Tiles: by destination in blocks of 8 x 8 tiles rather than row after row, so the workgroups in flight
    // together cover a compact region with long contiguous pieces on the source side as well as on the
    // destination side (measured +10 % over plain destination order).
    auto tile_key = [](const mmr_transpose_chunk& c) {
      const uint64_t pitch = c.dst_xstride > 0 ? static_cast<uint64_t>(c.dst_xstride) : 1;
      uint32_t tx = 0, ty = 0;
      transpose_tile_extent(c.itemsize, &tx, &ty);
      const uint64_t x = c.dst_off / pitch, y = c.dst_off % pitch;  // destination row, byte within it
      return std::make_tuple(c.dst_slot, x / (8ull * tx), y / (8ull * ty * c.itemsize), x, y);
    };
    std::stable_sort(plan->transposes.begin(), plan->transposes.end(),
                     [&](const mmr_transpose_chunk& a, const mmr_transpose_chunk& b) {
                       return order != 3 ? tile_key(a) < tile_key(b)
                                         : std::make_pair(a.src_slot, a.src_off) < std::make_pair(b.src_slot, b.src_off);
                     });
  }
  // one launch per element width (a narrow type's kernel keeps its own register and LDS budget) and kind (tiles that
  // are 16-byte aligned with whole vectors on both sides run through a leaner kernel than ragged or misaligned
  // ones): runs of equal (itemsize, kind), the order above kept inside each run
  std::stable_sort(plan->transposes.begin(), plan->transposes.end(),
                   [](const mmr_transpose_chunk& a, const mmr_transpose_chunk& b) {
                     return std::make_pair(a.itemsize, !transpose_is_vector(a)) < std::make_pair(b.itemsize, !transpose_is_vector(b));
                   });
  plan->stats.order_used = options.order;
  plan->stats.interleave_kib = options.order == 4 ? (((options.flags >> 8) & 0xffffu) ? ((options.flags >> 8) & 0xffffu) : 64) : 0;
  plan->stats.n_arrays = n;
  plan->stats.n_copy16_chunks = static_cast<int64_t>(plan->copy16.size());
  plan->stats.n_copy_generic_chunks = static_cast<int64_t>(plan->generic.size());
  plan->stats.n_transpose_chunks = static_cast<int64_t>(plan->transposes.size());
  plan->stats.n_slots = plan->n_slots;
  plan->stats.table_bytes =
      static_cast<int64_t>((plan->copy16.size() + plan->generic.size()) * sizeof(mmr_copy_chunk) +
                           plan->transposes.size() * sizeof(mmr_transpose_chunk) + plan->n_slots * sizeof(void*));
  return MMR_OK;
}

}  // namespace mmr

using mmr::fail;

extern "C" {

int mmr_plan_create(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int32_t n_arrays,
                    const mmr_plan_options* options, mmr_plan** out) {
  if (!out) return fail(MMR_INVALID_ARGUMENT, "null output");
  mmr_plan_options opt{};
  if (options) opt = *options;
  mmr_plan* plan = new mmr_plan();
  if (int rc = mmr::build_plan(srcs, dsts, n_arrays, opt, plan)) {
    delete plan;
    return rc;
  }
  *out = plan;
  return MMR_OK;
}

void mmr_plan_destroy(mmr_plan* plan) { delete plan; }

int mmr_plan_get_stats(const mmr_plan* plan, mmr_plan_stats* out) {
  if (!plan || !out) return fail(MMR_INVALID_ARGUMENT, "null argument");
  *out = plan->stats;
  return MMR_OK;
}

int64_t mmr_plan_get_copy_chunks(const mmr_plan* plan, int32_t kind, mmr_copy_chunk* out, int64_t capacity) {
  if (!plan) return 0;
  const auto& v = kind == 0 ? plan->copy16 : plan->generic;
  int64_t n = std::min<int64_t>(capacity, static_cast<int64_t>(v.size()));
  if (out && n > 0) std::memcpy(out, v.data(), sizeof(mmr_copy_chunk) * n);
  return out ? n : static_cast<int64_t>(v.size());
}

int64_t mmr_plan_get_transpose_chunks(const mmr_plan* plan, mmr_transpose_chunk* out, int64_t capacity) {
  if (!plan) return 0;
  int64_t n = std::min<int64_t>(capacity, static_cast<int64_t>(plan->transposes.size()));
  if (out && n > 0) std::memcpy(out, plan->transposes.data(), sizeof(mmr_transpose_chunk) * n);
  return out ? n : static_cast<int64_t>(plan->transposes.size());
}

int64_t mmr_plan_get_slot_bases(const mmr_plan* plan, int64_t* out, int64_t capacity) {
  if (!plan) return 0;
  int64_t n = std::min<int64_t>(capacity, static_cast<int64_t>(plan->slot_bases.size()));
  if (out && n > 0) std::memcpy(out, plan->slot_bases.data(), sizeof(int64_t) * n);
  return out ? n : static_cast<int64_t>(plan->slot_bases.size());
}

}  // extern "C"
