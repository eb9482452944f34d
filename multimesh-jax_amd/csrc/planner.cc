// Shard-intersection planner (host only).
//
// For every destination tile the overlapping source tiles are found by
// per-dimension interval intersection; each overlap is an N-d box with a byte
// stride per dim on either side.  Boxes are canonicalised (extent-1 dims
// dropped, dims that are contiguous on both sides merged) and lowered to
// workgroup-sized chunks:
//   * copy chunks     - n2 x n1 rows of w contiguous bytes (minor dim kept),
//   * transpose chunks - <=64x64-element tiles staged through LDS (source and
//                        destination disagree on the minor dim),
//   * fill chunks      - copy chunks without a source, zeroing the pad of short
//                        edge tiles.
#include "planner.h"

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

class Builder {
 public:
  Builder(mmr_plan* plan, uint32_t chunk_bytes, bool force_generic)
      : plan_(plan), chunk_bytes_(chunk_bytes), force_generic_(force_generic) {}

  int64_t generic_chunk_bytes() const { return std::max<int64_t>(chunk_bytes_ / 2, 256); }

  // statistics of one source-tile x destination-tile overlap
  void count_box(const BoxDim* in, int rank, int itemsize) {
    int64_t volume = 1;
    for (int i = 0; i < rank; ++i) volume *= std::max<int64_t>(in[i].n, 0);
    plan_->stats.n_boxes += 1;
    plan_->stats.bytes_moved += volume * itemsize;
  }

  void add_span(const mmr_span_chunk& c, int itemsize) {
    (void)itemsize;
    for (uint32_t j = 0; j < c.n_pieces; ++j)
      if (c.pieces[j].src_slot == MMR_SLOT_FILL) plan_->stats.bytes_filled += static_cast<int64_t>(c.pieces[j].w) * c.n_rows;
    plan_->spans.push_back(c);
  }

  // count_box: false when the caller has already counted the overlap this box is (part of)
  void add_box(uint32_t src_slot, uint32_t dst_slot, int64_t src_off, int64_t dst_off, const BoxDim* in, int rank,
               int itemsize, bool count = true) {
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
    } else if (count) {
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

 public:
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

 private:
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
    const int64_t cb = aligned ? chunk_bytes_ : generic_chunk_bytes();
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
    const int64_t rows = std::max<int64_t>(1, cb / w);
    int i1 = pick_row_dim(outer, -1);
    if (i1 < 0) {
      emit_copy(src_slot, dst_slot, so, dof, w, 1, 1, 0, 0, 0, 0, fill);
      return;
    }
    const BoxDim dim1 = outer[i1];
    const int64_t n1 = std::min(dim1.n, rows);
    BoxDim dim2{1, 0, 0};
    int64_t n2 = 1;
    int i2 = -1;
    if (aligned && n1 == dim1.n && rows / n1 >= 2) {  // the generic kernel walks a single row dimension
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
    const int64_t tile = itemsize == 16 ? kTransposeTile / 2 : kTransposeTile;
    const BoxDim dx = dims[x], dy = dims[y];
    std::vector<BoxDim> outer;
    for (int i = 0; i < static_cast<int>(dims.size()); ++i)
      if (i != x && i != y) outer.push_back(dims[i]);
    int ib = pick_row_dim(outer, -1);
    BoxDim db{1, 0, 0};
    if (ib >= 0) {
      db = outer[ib];
      outer.erase(outer.begin() + ib);
    }
    const int64_t nb = std::max<int64_t>(1, std::min<int64_t>(db.n, chunk_bytes_ / (tile * tile * itemsize)));
    for_each_index(outer, [&](int64_t ds, int64_t dd) {
      for (int64_t b0 = 0; b0 < db.n; b0 += nb) {
        for (int64_t y0 = 0; y0 < dy.n; y0 += tile) {
          for (int64_t x0 = 0; x0 < dx.n; x0 += tile) {
            mmr_transpose_chunk c{};
            c.src_slot = src_slot;
            c.dst_slot = dst_slot;
            c.src_off = static_cast<uint64_t>(so + ds + b0 * db.s + y0 * dy.s + x0 * dx.s);
            c.dst_off = static_cast<uint64_t>(dof + dd + b0 * db.d + y0 * dy.d + x0 * dx.d);
            c.nx = static_cast<uint32_t>(std::min(tile, dx.n - x0));
            c.ny = static_cast<uint32_t>(std::min(tile, dy.n - y0));
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
  bool force_generic_;
};

// One source-tile x destination-tile overlap of the tile being planned.
struct TileBox {
  uint32_t src_slot;
  int64_t soff, doff;       // bytes: first element of the box in either buffer
  BoxDim dims[kMaxRank];    // logical dim order
  int64_t b_lo[kMaxRank];   // global index where the box starts
};

struct TileGeometry {
  int64_t lo[kMaxRank], hi[kMaxRank], valid[kMaxRank];
  int64_t t_lo[kMaxRank], t_n[kMaxRank];  // overlapping source tiles per dim
  int64_t cstride[kMaxRank];              // box index = sum (t - t_lo) * cstride
};

// Zero the pad of a short tile: one slab per padded dim, dims taken in `order`:
// the slab of a dim spans the valid extent of the dims before it and the whole
// (padded) extent of the dims after it.  `skip_last`: the last dim's pad is
// filled by other means (span chunks carry it as a piece without a source).
void fill_pad(Builder& b, const Side& D, const TileGeometry& g, uint32_t dslot, const int* order, bool skip_last) {
  const int rank = D.rank, item = D.itemsize;
  for (int oi = 0; oi < rank - (skip_last ? 1 : 0); ++oi) {
    const int i = order[oi];
    if (g.valid[i] == D.ext[i]) continue;
    BoxDim dims[kMaxRank];
    for (int oj = 0; oj < rank; ++oj) {
      const int j = order[oj];
      const int64_t n = oj < oi ? g.valid[j] : (oj == oi ? D.ext[i] - g.valid[i] : D.ext[j]);
      dims[j] = BoxDim{n, D.stride[j] * item, D.stride[j] * item};
    }
    b.add_box(MMR_SLOT_FILL, dslot, 0, g.valid[i] * D.stride[i] * item, dims, rank, item);
  }
}

// Ragged rows (some offset, stride or width not a multiple of 16 bytes): plan the
// tile as dense destination rows gathered from the source tiles that meet
// inside a row, so every destination line is written whole by one workgroup.
// Returns false when the tile does not fit the pattern; the caller then plans
// it box by box.
bool plan_tile_as_spans(Builder& b, const Side& S, const Side& D, const TileGeometry& g, uint32_t dslot,
                        const std::vector<TileBox>& boxes) {
  const int rank = S.rank, item = S.itemsize;
  if (rank == 0 || boxes.empty()) return false;
  int m = -1;
  for (int i = 0; i < rank; ++i)
    if (D.stride[i] == 1 && D.ext[i] > 1) m = i;
  if (m < 0 || S.stride[m] != 1) return false;
  // all aligned -> the aligned copy kernel is the better tool
  uint64_t bits = 0;
  for (const TileBox& bx : boxes) {
    bits |= static_cast<uint64_t>(bx.soff | bx.doff);
    for (int i = 0; i < rank; ++i) {
      if (i == m) bits |= static_cast<uint64_t>(bx.dims[i].n * item);
      else if (bx.dims[i].n > 1) bits |= static_cast<uint64_t>(bx.dims[i].s | bx.dims[i].d);
    }
  }
  if ((bits & 15u) == 0) return false;
  const bool pad_m = g.valid[m] < D.ext[m];
  const int64_t n_pieces = g.t_n[m] + (pad_m ? 1 : 0);
  if (n_pieces > MMR_SPAN_MAX_PIECES) return false;
  const int64_t row_bytes = D.ext[m] * item;
  const int64_t budget = b.generic_chunk_bytes();
  if (row_bytes > 4 * budget) return false;  // very wide rows: split columns instead
  int r = -1;  // the dim whose consecutive indices are consecutive destination rows
  for (int i = 0; i < rank; ++i)
    if (i != m && D.stride[i] == D.ext[m] && D.ext[i] > 1) r = i;
  const int64_t rows_per_chunk = std::max<int64_t>(1, budget / row_bytes);

  // pad of the other dims as whole-row slabs; the minor dim's pad rides in the spans
  int order[kMaxRank], k = 0;
  for (int i = 0; i < rank; ++i)
    if (i != m) order[k++] = i;
  order[k] = m;
  fill_pad(b, D, g, dslot, order, /*skip_last=*/true);

  // every combination of source tiles over the outer dims, every index of the outer dims but r
  int64_t outer_combos = 1;
  for (int i = 0; i < rank; ++i)
    if (i != m) outer_combos *= g.t_n[i];
  for (int64_t oc = 0; oc < outer_combos; ++oc) {
    int64_t rem = oc, first = 0;  // index of the piece-0 box of this outer combination
    for (int i = rank - 1; i >= 0; --i) {
      if (i == m) continue;
      first += (rem % g.t_n[i]) * g.cstride[i];
      rem /= g.t_n[i];
    }
    const TileBox& b0 = boxes[static_cast<size_t>(first)];
    std::vector<BoxDim> others;  // outer dims except r: every index is its own set of rows
    std::vector<int> other_dim;
    for (int i = 0; i < rank; ++i)
      if (i != m && i != r) {
        others.push_back(b0.dims[i]);
        other_dim.push_back(i);
      }
    const int64_t n_r = r >= 0 ? b0.dims[r].n : 1;
    const int64_t s_r = r >= 0 ? b0.dims[r].s : 0;
    const int64_t d_r = r >= 0 ? b0.dims[r].d : 0;
    Builder::for_each_index(others, [&](int64_t ds, int64_t dd) {
      for (int64_t r0 = 0; r0 < n_r; r0 += rows_per_chunk) {
        const int64_t n = std::min(rows_per_chunk, n_r - r0);
        mmr_span_chunk c{};
        c.dst_slot = dslot;
        c.dst_off = static_cast<uint64_t>(b0.doff + dd + r0 * d_r);
        c.row_bytes = static_cast<uint32_t>(row_bytes);
        c.n_rows = static_cast<uint32_t>(n);
        bool safe = true;
        int64_t total = 0;
        for (int64_t pj = 0; pj < g.t_n[m]; ++pj) {
          const TileBox& bx = boxes[static_cast<size_t>(first + pj * g.cstride[m])];
          mmr_span_piece& pc = c.pieces[c.n_pieces++];
          pc.src_slot = bx.src_slot;
          pc.w = static_cast<uint32_t>(bx.dims[m].n * item);
          pc.src_off = static_cast<uint64_t>(bx.soff + ds + r0 * s_r);
          pc.s1 = n > 1 ? s_r : 0;
          total += pc.w;
          // the kernel reads up to 15 bytes before and after every source run
          if (pc.src_off < 15 || static_cast<int64_t>(pc.src_off) + (n - 1) * s_r + pc.w + 15 > S.shard_bytes) safe = false;
        }
        if (pad_m) {
          mmr_span_piece& pc = c.pieces[c.n_pieces++];
          pc.src_slot = MMR_SLOT_FILL;
          pc.w = static_cast<uint32_t>((D.ext[m] - g.valid[m]) * item);
          total += pc.w;
        }
        if (total != row_bytes) safe = false;  // cannot happen; keeps a malformed chunk off the GPU
        if (safe) {
          b.add_span(c, item);
        } else {
          // rows at the very start or end of a source buffer: move them piece by piece
          for (uint32_t pj = 0; pj < c.n_pieces; ++pj) {
            const mmr_span_piece& pc = c.pieces[pj];
            int64_t col = 0;
            for (uint32_t q = 0; q < pj; ++q) col += c.pieces[q].w;
            BoxDim dims[2] = {BoxDim{n, pc.src_slot == MMR_SLOT_FILL ? row_bytes : s_r, row_bytes},
                              BoxDim{pc.w / item, item, item}};
            b.add_box(pc.src_slot, dslot, static_cast<int64_t>(pc.src_off), static_cast<int64_t>(c.dst_off) + col, dims, 2,
                      item, /*count_box=*/false);
          }
        }
      }
    });
  }
  return true;
}

int plan_one_array(Builder& b, const Side& S, const Side& D, uint32_t slot_base, bool allow_spans) {
  const int rank = S.rank;
  const int item = S.itemsize;
  for (int i = 0; i < rank; ++i)
    if (S.size[i] == 0) return MMR_OK;  // empty array: nothing to move, nothing to pad
  int natural_order[kMaxRank];
  for (int i = 0; i < rank; ++i) natural_order[i] = i;
  for (int64_t dd = 0; dd < D.dev_count; ++dd) {
    const uint32_t dslot = slot_base + static_cast<uint32_t>(S.dev_count + dd);
    TileGeometry g;
    bool padded = false, empty = false;
    for (int i = 0; i < rank; ++i) {
      const int64_t c = (dd / D.dev_stride[i]) % D.tiles[i];
      g.lo[i] = std::min(c * D.ext[i], D.size[i]);
      g.hi[i] = std::min(g.lo[i] + D.ext[i], D.size[i]);
      g.valid[i] = g.hi[i] - g.lo[i];
      padded |= g.valid[i] < D.ext[i];
      empty |= g.valid[i] == 0;
    }
    if (empty) {
      if (padded) fill_pad(b, D, g, dslot, natural_order, false);
      continue;
    }
    int64_t combos = 1;
    for (int i = rank - 1; i >= 0; --i) {
      g.t_lo[i] = g.lo[i] / S.ext[i];
      g.t_n[i] = (g.hi[i] - 1) / S.ext[i] - g.t_lo[i] + 1;
      g.cstride[i] = combos;
      combos *= g.t_n[i];
    }
    std::vector<TileBox> boxes(static_cast<size_t>(combos));
    for (int64_t c = 0; c < combos; ++c) {
      int64_t rem = c, sdev = 0;
      TileBox& bx = boxes[static_cast<size_t>(c)];
      bx.soff = bx.doff = 0;
      for (int i = rank - 1; i >= 0; --i) {
        const int64_t t = g.t_lo[i] + rem % g.t_n[i];
        rem /= g.t_n[i];
        const int64_t s_lo = t * S.ext[i];
        const int64_t b_lo = std::max(g.lo[i], s_lo);
        const int64_t b_hi = std::min(g.hi[i], std::min(s_lo + S.ext[i], S.size[i]));
        bx.dims[i] = BoxDim{b_hi - b_lo, S.stride[i] * item, D.stride[i] * item};
        bx.b_lo[i] = b_lo;
        bx.soff += (b_lo - s_lo) * S.stride[i] * item;
        bx.doff += (b_lo - g.lo[i]) * D.stride[i] * item;
        sdev += t * S.dev_stride[i];  // of R source replicas the lowest device id is read
      }
      bx.src_slot = slot_base + static_cast<uint32_t>(sdev);
      b.count_box(bx.dims, rank, item);
    }
    if (allow_spans && plan_tile_as_spans(b, S, D, g, dslot, boxes)) continue;
    if (padded) fill_pad(b, D, g, dslot, natural_order, false);
    for (const TileBox& bx : boxes) b.add_box(bx.src_slot, dslot, bx.soff, bx.doff, bx.dims, rank, item, false);
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
  Builder builder(plan, chunk_bytes, (options.flags & MMR_PLAN_ALL_GENERIC) != 0);
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
    if (int rc = plan_one_array(builder, S, D, static_cast<uint32_t>(plan->n_slots),
                                (options.flags & (MMR_PLAN_NO_SPANS | MMR_PLAN_ALL_GENERIC)) == 0))
      return rc;
    plan->n_slots += S.dev_count + D.dev_count;
  }
  const uint32_t order = options.order ? options.order : 2;
  if (order == 2 || order == 3) {
    auto key = [order](const mmr_copy_chunk& c) {
      return order == 2 ? std::make_pair(c.dst_slot, c.dst_off) : std::make_pair(c.src_slot, c.src_off);
    };
    auto cmp = [&](const mmr_copy_chunk& a, const mmr_copy_chunk& b) { return key(a) < key(b); };
    std::stable_sort(plan->copy16.begin(), plan->copy16.end(), cmp);
    std::stable_sort(plan->generic.begin(), plan->generic.end(), cmp);
    std::stable_sort(plan->spans.begin(), plan->spans.end(), [order](const mmr_span_chunk& a, const mmr_span_chunk& b) {
      return order == 2 ? std::make_pair(a.dst_slot, a.dst_off) < std::make_pair(b.dst_slot, b.dst_off)
                        : std::make_pair(a.pieces[0].src_slot, a.pieces[0].src_off) <
                              std::make_pair(b.pieces[0].src_slot, b.pieces[0].src_off);
    });
    std::stable_sort(plan->transposes.begin(), plan->transposes.end(),
                     [order](const mmr_transpose_chunk& a, const mmr_transpose_chunk& b) {
                       return order == 2 ? std::make_pair(a.dst_slot, a.dst_off) < std::make_pair(b.dst_slot, b.dst_off)
                                         : std::make_pair(a.src_slot, a.src_off) < std::make_pair(b.src_slot, b.src_off);
                     });
  }
  plan->stats.n_arrays = n;
  plan->stats.n_copy16_chunks = static_cast<int64_t>(plan->copy16.size());
  plan->stats.n_copy_generic_chunks = static_cast<int64_t>(plan->generic.size());
  plan->stats.n_transpose_chunks = static_cast<int64_t>(plan->transposes.size());
  plan->stats.n_span_chunks = static_cast<int64_t>(plan->spans.size());
  plan->stats.n_slots = plan->n_slots;
  plan->stats.table_bytes =
      static_cast<int64_t>((plan->copy16.size() + plan->generic.size()) * sizeof(mmr_copy_chunk) +
                           plan->transposes.size() * sizeof(mmr_transpose_chunk) +
                           plan->spans.size() * sizeof(mmr_span_chunk) + plan->n_slots * sizeof(void*));
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

int64_t mmr_plan_get_span_chunks(const mmr_plan* plan, mmr_span_chunk* out, int64_t capacity) {
  if (!plan) return 0;
  int64_t n = std::min<int64_t>(capacity, static_cast<int64_t>(plan->spans.size()));
  if (out && n > 0) std::memcpy(out, plan->spans.data(), sizeof(mmr_span_chunk) * n);
  return out ? n : static_cast<int64_t>(plan->spans.size());
}

int64_t mmr_plan_get_slot_bases(const mmr_plan* plan, int64_t* out, int64_t capacity) {
  if (!plan) return 0;
  int64_t n = std::min<int64_t>(capacity, static_cast<int64_t>(plan->slot_bases.size()));
  if (out && n > 0) std::memcpy(out, plan->slot_bases.data(), sizeof(int64_t) * n);
  return out ? n : static_cast<int64_t>(plan->slot_bases.size());
}

}  // extern "C"
