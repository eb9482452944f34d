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
#include <map>
#include <tuple>

namespace mmr {
namespace {

struct BoxDim {
  int64_t n;  // extent in elements
  int64_t s;  // source byte stride
  int64_t d;  // destination byte stride
};

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

constexpr int64_t kGenericMaxPairs = 768;  // (row, slot) pairs of one generic chunk

// A box in canonical form: extent-1 dims dropped, dims in destination-major order, neighbours that are contiguous
// on both sides merged, the run that is contiguous on both sides taken out as `w` bytes.
struct CanonBox {
  uint32_t src_slot, dst_slot;
  int64_t so, dof;
  std::vector<BoxDim> outer;
  int64_t w;
  bool fill;
};

// A group before the launch order is fixed.
struct ProtoCopy {
  CopyGroup g{};  // k, n1, n2, m1, m2, c1, d1, d2 set; the rest follows when the launch is assembled
  std::vector<CopyPiece> pieces;
  int array = 0;
  uint32_t ordinal = 0;      // position among the groups of its (array, destination buffer)
  uint64_t chunk_bytes = 0;  // destination bytes of one chunk of the widest piece
};
struct ProtoSpan {
  SpanGroup g{};  // W, band_bytes, n1, span, head, div_W, div_n1 set
  SpanMember m{};
  std::vector<SpanPiece> pieces;
  int array = 0;
  uint32_t ordinal = 0;
};

constexpr size_t kSpanMaxPieces = 64;  // pieces of one destination row beyond which the span kernel's piece search costs too much

class Builder {
 public:
  Builder(mmr_plan* plan, uint32_t chunk_bytes, uint32_t generic_chunk_bytes, uint32_t span_bytes, bool force_ragged,
          bool no_span)
      : plan_(plan), chunk_bytes_(chunk_bytes), generic_chunk_bytes_(generic_chunk_bytes), span_bytes_(span_bytes),
        force_ragged_(force_ragged), no_span_(no_span) {}

  std::vector<ProtoCopy> copies;
  std::vector<ProtoSpan> spans;

  void begin_array(int array) { array_ = array; }

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
      for (BoxDim& d : dims) d.s = d.d;  // a fill has no source side: let its dims merge by the destination alone
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
    CanonBox box{src_slot, dst_slot, fill ? 0 : src_off, dst_off, {}, itemsize, fill};
    if (run >= 0) {
      box.w = dims[run].n * itemsize;
      dims.erase(dims.begin() + run);
    }
    box.outer = std::move(dims);
    tile_.push_back(std::move(box));
  }

  // All boxes of one destination tile are in: lower them.  A tile whose boxes are all 16-byte aligned becomes copy
  // groups; otherwise the whole tile goes to the span kernel (every byte of a destination row must come through the
  // same workgroup for it to leave as whole lines), and what that kernel does not take becomes generic chunks.
  void finish_tile() {
    bool aligned = !force_ragged_;
    for (const CanonBox& b : tile_) {
      uint64_t bits = static_cast<uint64_t>(b.so | b.dof | b.w);
      for (const BoxDim& d : b.outer) bits |= static_cast<uint64_t>(d.s | d.d);
      aligned &= (bits & 15u) == 0;
    }
    if (aligned) {
      lower_copy_groups();
    } else {
      std::vector<CanonBox> rest;
      if (no_span_) rest = tile_;
      else lower_span_groups(&rest);
      for (CanonBox& b : rest) lower_generic(b.src_slot, b.dst_slot, b.so, b.dof, b.outer, b.w, b.fill);
    }
    tile_.clear();
    ordinal_ = 0;
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

  // Calls fn(index vector) for every index combination of `dims`.
  template <class Fn>
  static void for_each_combo(const std::vector<BoxDim>& dims, Fn&& fn) {
    std::vector<int64_t> idx(dims.size(), 0);
    while (true) {
      fn(idx);
      int k = static_cast<int>(dims.size()) - 1;
      for (; k >= 0; --k) {
        if (++idx[k] < dims[k].n) break;
        idx[k] = 0;
      }
      if (k < 0) break;
    }
  }

  // Calls fn(src_delta, dst_delta) for every index combination of `dims`.
  template <class Fn>
  static void for_each_index(const std::vector<BoxDim>& dims, Fn&& fn) {
    for_each_combo(dims, [&](const std::vector<int64_t>& idx) {
      int64_t so = 0, dof = 0;
      for (size_t i = 0; i < dims.size(); ++i) {
        so += idx[i] * dims[i].s;
        dof += idx[i] * dims[i].d;
      }
      fn(so, dof);
    });
  }

  // Boxes that lie side by side in the same destination rows: equal row dims on the destination side and the same
  // first row.  Returns index lists into tile_, each in ascending destination order.
  std::vector<std::vector<int>> row_mates() const {
    struct Key {
      std::vector<int64_t> dims;  // (n, d) of every outer dim
      int64_t origin;
      bool operator<(const Key& o) const { return origin != o.origin ? origin < o.origin : dims < o.dims; }
    };
    std::map<Key, std::vector<int>> sets;
    for (int i = 0; i < static_cast<int>(tile_.size()); ++i) {
      const CanonBox& b = tile_[i];
      Key key;
      for (const BoxDim& d : b.outer) {
        key.dims.push_back(d.n);
        key.dims.push_back(d.d);
      }
      // the box is contiguous in the destination over its run and the dims that continue it (a chain of chain_bytes);
      // its neighbours share the rows of the first dim above that chain
      int64_t chain_bytes = b.w, pitch = 0;
      for (int d = static_cast<int>(b.outer.size()) - 1; d >= 0; --d) {
        if (b.outer[d].d != chain_bytes) {
          pitch = b.outer[d].d;
          break;
        }
        chain_bytes *= b.outer[d].n;
      }
      // a chain that does not fit between two rows has no neighbours in its rows
      key.origin = pitch > 0 && b.dof % pitch + chain_bytes <= pitch ? b.dof - b.dof % pitch : b.dof;
      sets[key].push_back(i);
    }
    std::vector<std::vector<int>> out;
    for (auto& kv : sets) {
      std::sort(kv.second.begin(), kv.second.end(), [&](int a, int b) { return tile_[a].dof < tile_[b].dof; });
      out.push_back(std::move(kv.second));
    }
    std::sort(out.begin(), out.end(), [&](const std::vector<int>& a, const std::vector<int>& b) {
      return tile_[a[0]].dof < tile_[b[0]].dof;
    });
    return out;
  }

  // A run many chunks long (a box that is contiguous on both sides: a whole tile, a band of whole rows) becomes rows
  // of one chunk each under a row dim of its own, so that one piece record serves the box; cut into column segments
  // like a long row it would take one record per chunk (a 1 GiB tile: 131,072 records, 8 MB of tables).  What is
  // left over behind the last whole row stays a box of its own.
  void fold_long_runs() {
    const int64_t row = chunk_bytes_;  // a multiple of 256
    std::vector<CanonBox> tails;
    for (CanonBox& b : tile_) {
      if (b.outer.size() > 2 || b.w < 16 * row) continue;  // three row dims are blocked; more would multiply the groups
      const int64_t n = b.w / row, rem = b.w % row;
      if (rem) {
        CanonBox tail = b;
        tail.so = b.fill ? 0 : b.so + n * row;
        tail.dof = b.dof + n * row;
        tail.w = rem;
        tails.push_back(std::move(tail));
      }
      b.outer.push_back(BoxDim{n, row, row});  // innermost: its rows abut on both sides
      b.w = row;
    }
    for (CanonBox& t : tails) tile_.push_back(std::move(t));
  }

  void lower_copy_groups() {
    fold_long_runs();
    for (const std::vector<int>& mates : row_mates()) {
      const CanonBox& first = tile_[mates[0]];
      int64_t w_max = 0;
      for (int i : mates) w_max = std::max(w_max, tile_[i].w);
      const std::vector<BoxDim>& outer = first.outer;  // row structure; the mates share it on the destination side
      const int64_t cb = chunk_bytes_;
      // pieces: a box, or its column segments when its rows are longer than a chunk (near-equal segments on 256-byte
      // boundaries of the row)
      struct Seg {
        int box;
        int64_t c0, w;
      };
      std::vector<Seg> segs;
      for (int i : mates) {
        const int64_t w = tile_[i].w;
        if (w > cb) {
          const int64_t nseg = ceil_div(w, cb);
          const int64_t seg = ceil_div(ceil_div(w, nseg), 256) * 256;
          for (int64_t c0 = 0; c0 < w; c0 += seg) segs.push_back({i, c0, std::min(seg, w - c0)});
        } else {
          segs.push_back({i, 0, w});
        }
      }
      int i1 = -1, i2 = -1;
      int64_t m1 = 1, m2 = 1;
      if (w_max > cb) {
        i1 = pick_row_dim(outer, -1);  // one row per chunk
        if (i1 >= 0) i2 = pick_row_dim(outer, i1);
      } else {
        const int64_t rows = std::max<int64_t>(1, cb / w_max);
        i1 = pick_row_dim(outer, -1);
        if (i1 >= 0) {
          const BoxDim dim1 = outer[i1];
          m1 = std::min(dim1.n, rows);
          if (m1 < dim1.n && (dim1.d == w_max || dim1.s == w_max)) {
            // Rows that abut on one side, cut into several chunks along this dim: keep the cuts on 128-byte lines of
            // that side where a few rows less achieve it, so no line is shared by two workgroups (832-byte rows: 8 per
            // chunk instead of 9 measured +3 %).
            int64_t g = w_max, h = 128;
            while (h != 0) {
              const int64_t t = g % h;
              g = h;
              h = t;
            }
            const int64_t m = 128 / g;
            if (m1 > m) m1 = m1 / m * m;
          }
          // Rows that continue the run on the destination side along one dim (A) and on the source side along
          // another (B), as a fused layout permutation produces: take a 2-D block so both sides see runs of several
          // rows instead of one side seeing single rows at a large stride.
          int ia = -1, ib = -1;
          if (!first.fill && outer.size() >= 2) {
            for (int i = 0; i < static_cast<int>(outer.size()); ++i) {
              if (outer[i].d == w_max && outer[i].s != w_max) ia = i;
              if (outer[i].s == w_max && outer[i].d != w_max) ib = i;
            }
          }
          if (ia >= 0 && ib >= 0 && rows >= 4) {
            const BoxDim da = outer[ia], db = outer[ib];
            int64_t na = 1;
            while (na * 2 <= da.n && na * na * 4 <= rows) na *= 2;  // about sqrt(rows), a power of two
            if (da.n * da.n <= 4 * rows) na = da.n;                  // or the whole of a short dim
            i1 = ia;
            m1 = std::min(na, da.n);
            i2 = ib;
            m2 = std::max<int64_t>(1, std::min(db.n, rows / m1));
          } else {
            i2 = pick_row_dim(outer, i1);
            if (i2 >= 0) m2 = m1 == dim1.n ? std::max<int64_t>(1, std::min(outer[i2].n, rows / m1)) : 1;
          }
        }
      }
      const BoxDim dim1 = i1 >= 0 ? outer[i1] : BoxDim{1, 0, 0};
      const BoxDim dim2 = i2 >= 0 ? outer[i2] : BoxDim{1, 0, 0};
      // a third row dim rides along unblocked (the innermost of what is left); dims beyond it make groups of their own
      int i3 = -1;
      for (int i = static_cast<int>(outer.size()) - 1; i >= 0 && i3 < 0; --i)
        if (i != i1 && i != i2) i3 = i;
      const BoxDim dim3 = i3 >= 0 ? outer[i3] : BoxDim{1, 0, 0};
      std::vector<BoxDim> rest;
      std::vector<int> rest_index;
      for (int i = 0; i < static_cast<int>(outer.size()); ++i)
        if (i != i1 && i != i2 && i != i3) {
          rest.push_back(outer[i]);
          rest_index.push_back(i);
        }
      for_each_combo(rest, [&](const std::vector<int64_t>& idx) {
        ProtoCopy pg;
        pg.array = array_;
        pg.ordinal = ordinal_++;
        CopyGroup& g = pg.g;
        g.k = static_cast<uint32_t>(segs.size());
        g.n1 = static_cast<uint32_t>(dim1.n);
        g.n2 = static_cast<uint32_t>(dim2.n);
        g.n3 = static_cast<uint32_t>(dim3.n);
        g.m1 = static_cast<uint32_t>(m1);
        g.m2 = static_cast<uint32_t>(m2);
        g.c1 = static_cast<uint32_t>(ceil_div(dim1.n, m1));
        g.c12 = g.c1 * static_cast<uint32_t>(ceil_div(dim2.n, m2));
        g.d1 = dim1.n > 1 ? dim1.d : 0;
        g.d2 = dim2.n > 1 ? dim2.d : 0;
        g.d3 = dim3.n > 1 ? dim3.d : 0;
        pg.chunk_bytes = static_cast<uint64_t>(std::min(w_max, cb) * m1 * m2);
        for (const Seg& sg : segs) {
          const CanonBox& b = tile_[sg.box];
          int64_t so = b.so + sg.c0, dof = b.dof + sg.c0;
          for (size_t r = 0; r < rest.size(); ++r) {
            so += idx[r] * b.outer[rest_index[r]].s;
            dof += idx[r] * b.outer[rest_index[r]].d;
          }
          CopyPiece p{};
          p.src_slot = b.src_slot;
          p.dst_slot = b.dst_slot;
          p.src = b.fill ? 0 : static_cast<uint64_t>(so);
          p.dst = static_cast<uint64_t>(dof);
          p.s1 = (i1 >= 0 && dim1.n > 1 && !b.fill) ? b.outer[i1].s : 0;
          p.s2 = (i2 >= 0 && dim2.n > 1 && !b.fill) ? b.outer[i2].s : 0;
          p.s3 = (i3 >= 0 && dim3.n > 1 && !b.fill) ? b.outer[i3].s : 0;
          p.w = static_cast<uint32_t>(sg.w);
          p.div_wv = make_fastdiv(std::max<uint32_t>(p.w >> 4, 1));
          pg.pieces.push_back(p);
        }
        copies.push_back(std::move(pg));
      });
    }
  }

  // Ragged tile -> span groups.  Boxes the span kernel does not take are returned in *rest_out.
  void lower_span_groups(std::vector<CanonBox>* rest_out) {
    // Per box: the chain of dims over which it is contiguous in the destination (from the run outwards) and the head
    // dims above it.  With head dims, the destination row is the innermost head dim's pitch and the chain dims are
    // enumerated into pieces of that row (source-strided runs that abut in the destination); boxes with the same head
    // and the same first row share the row.  Without head dims the box is dense by itself: its rows are the row.
    struct Piece {
      SpanPiece p;
      std::vector<int64_t> row_s;  // source stride of every row dim of the band, innermost first
    };
    struct Band {
      std::vector<BoxDim> rows;  // destination side, innermost first
      int64_t W = 0, origin = 0;
      uint32_t dst_slot = 0;
      std::vector<Piece> pieces;
      std::vector<int> boxes;
      bool ok = true;
    };
    std::map<std::pair<int64_t, std::vector<int64_t>>, Band> bands;
    for (int bi = 0; bi < static_cast<int>(tile_.size()); ++bi) {
      const CanonBox& b = tile_[bi];
      int64_t chain_bytes = b.w;
      int head_n = static_cast<int>(b.outer.size());
      while (head_n > 0 && b.outer[head_n - 1].d == chain_bytes) {
        chain_bytes *= b.outer[head_n - 1].n;
        --head_n;
      }
      std::vector<BoxDim> chain(b.outer.begin() + head_n, b.outer.end()), rows;
      int64_t W, col;
      if (head_n == 0) {  // dense by itself: rows of w bytes
        W = b.w;
        col = 0;
        rows.assign(chain.rbegin(), chain.rend());
        chain.clear();
      } else {
        W = b.outer[head_n - 1].d;
        col = b.dof % W;
        rows.assign(b.outer.rend() - head_n, b.outer.rend());
      }
      std::vector<int64_t> key_dims;
      for (const BoxDim& d : rows) {
        key_dims.push_back(d.n);
        key_dims.push_back(d.d);
      }
      Band& band = bands[{b.dof - col, key_dims}];
      if (band.boxes.empty()) {
        band.rows = rows;
        band.W = W;
        band.origin = b.dof - col;
        band.dst_slot = b.dst_slot;
      }
      band.boxes.push_back(bi);
      size_t count = 1;
      for (const BoxDim& d : chain) count *= static_cast<size_t>(d.n);
      if (W > static_cast<int64_t>(kSpanMaxRowBytes) || band.pieces.size() + count > kSpanMaxPieces) {
        band.ok = false;
        continue;
      }
      for_each_index(chain, [&](int64_t ds, int64_t dd) {
        Piece pc;
        pc.p = SpanPiece{};
        pc.p.src_slot = b.src_slot;
        pc.p.src = b.fill ? 0 : static_cast<uint64_t>(b.so + ds);
        pc.p.col = static_cast<uint32_t>(col + dd);
        pc.p.w = static_cast<uint32_t>(b.w);
        for (const BoxDim& d : rows) pc.row_s.push_back(b.fill ? 0 : d.s);
        band.pieces.push_back(std::move(pc));
      });
    }
    for (auto& kv : bands) {
      Band& band = kv.second;
      std::sort(band.pieces.begin(), band.pieces.end(), [](const Piece& a, const Piece& b) { return a.p.col < b.p.col; });
      int64_t end = 0;
      for (const Piece& pc : band.pieces) {  // the pieces must tile the row
        band.ok &= pc.p.col == end;
        end += pc.p.w;
      }
      band.ok &= end == band.W;
      const BoxDim r1 = band.rows.empty() ? BoxDim{1, 0, 0} : band.rows[0];
      band.ok &= band.rows.empty() || r1.d == band.W;  // rows abut
      int64_t total_rows = 1;
      for (const BoxDim& d : band.rows) total_rows *= d.n;
      band.ok &= total_rows < (1ll << 31);
      if (!band.ok) {
        for (int bi : band.boxes) rest_out->push_back(tile_[bi]);
        continue;
      }
      // n1 rows along the innermost dim; a second dim rides along when the rows stay dense across it; the dims above
      // (and a second dim that is not dense) are enumerated, one band each
      const bool dense2 = band.rows.size() > 1 && band.rows[1].d == r1.n * band.W;
      const size_t skip = band.rows.empty() ? 0 : (dense2 ? 2 : 1);
      const std::vector<BoxDim> rest(band.rows.begin() + skip, band.rows.end());
      const int64_t n2 = dense2 ? band.rows[1].n : 1;
      for_each_combo(rest, [&](const std::vector<int64_t>& idx) {
        ProtoSpan ps;
        ps.array = array_;
        ps.ordinal = ordinal_++;
        int64_t dst_shift = 0;
        for (size_t r = 0; r < rest.size(); ++r) dst_shift += idx[r] * rest[r].d;
        SpanGroup& g = ps.g;
        g.W = static_cast<uint32_t>(band.W);
        g.n1 = static_cast<uint32_t>(r1.n);
        g.band_bytes = static_cast<uint64_t>(r1.n * n2 * band.W);
        g.span = span_bytes_;
        const uint64_t at = static_cast<uint64_t>(band.origin + dst_shift);
        g.head = span_bytes_ - static_cast<uint32_t>(at % span_bytes_);
        g.div_W = make_fastdiv(g.W);
        g.div_n1 = make_fastdiv(g.n1);
        ps.m.dst = at;
        ps.m.dst_slot = band.dst_slot;
        uint32_t wide = 0;
        for (const Piece& pc : band.pieces) {
          SpanPiece p = pc.p;
          int64_t src_shift = 0;
          for (size_t r = 0; r < rest.size(); ++r) src_shift += idx[r] * pc.row_s[skip + r];
          p.src += static_cast<uint64_t>(src_shift);
          p.s1 = pc.row_s.empty() ? 0 : pc.row_s[0];
          p.s2 = dense2 ? pc.row_s[1] : 0;
          p.wide_index = wide;
          if (p.w >= 16) ++wide;
          ps.pieces.push_back(p);
        }
        ps.m.k = static_cast<uint32_t>(ps.pieces.size());
        ps.m.wide = wide;
        ps.m.narrow = ps.m.k - wide;
        ps.m.div_k = make_fastdiv(std::max<uint32_t>(ps.m.k, 1));
        ps.m.div_wide = make_fastdiv(std::max<uint32_t>(wide, 1));
        spans.push_back(std::move(ps));
      });
    }
  }

  void emit_generic(uint32_t src_slot, uint32_t dst_slot, int64_t so, int64_t dof, int64_t w, int64_t n1, int64_t s1,
                    int64_t d1, bool fill) {
    mmr_copy_chunk c{};
    c.src_slot = src_slot;
    c.dst_slot = dst_slot;
    c.src_off = fill ? 0 : static_cast<uint64_t>(so);
    c.dst_off = static_cast<uint64_t>(dof);
    c.w = static_cast<uint32_t>(w);
    c.n1 = static_cast<uint32_t>(n1);
    c.n2 = 1;
    c.s1 = (n1 > 1 && !fill) ? s1 : 0;
    c.d1 = n1 > 1 ? d1 : 0;
    uint64_t bits = c.src_off | c.dst_off | c.w | static_cast<uint64_t>(c.s1) | static_cast<uint64_t>(c.d1);
    c.align = (bits & 15u) ? static_cast<uint32_t>(bits & (~bits + 1)) : 16u;
    if (fill) plan_->stats.n_fill_chunks += 1;
    plan_->generic.push_back(c);
  }

  // Generic chunks: rows of one box along a single row dim, the other dims enumerated.
  void lower_generic(uint32_t src_slot, uint32_t dst_slot, int64_t so, int64_t dof, const std::vector<BoxDim>& outer,
                     int64_t w, bool fill) {
    const int64_t cb = generic_chunk_bytes_;
    if (w > cb) {
      // long rows: split columns into near-equal segments on 256-byte boundaries of the row
      const int64_t nseg = ceil_div(w, cb);
      const int64_t seg = ceil_div(ceil_div(w, nseg), 256) * 256;
      for_each_index(outer, [&](int64_t ds, int64_t dd) {
        for (int64_t c0 = 0; c0 < w; c0 += seg)
          emit_generic(src_slot, dst_slot, so + ds + c0, dof + dd + c0, std::min(seg, w - c0), 1, 0, 0, fill);
      });
      return;
    }
    // The generic kernel spends one lane per (row, 16-byte slot) pair whatever the row holds: a chunk of very narrow
    // rows sized by bytes alone keeps its workgroup busy long after its neighbours have finished and becomes the tail
    // of the launch.  Bound the pairs per chunk (3 per lane of a 256-lane workgroup) as well as the bytes.
    const int64_t slots = (w + 15) / 16 + 1;
    const int64_t rows = std::max<int64_t>(1, std::min(std::max<int64_t>(1, cb / w), kGenericMaxPairs / slots));
    const int i1 = pick_row_dim(outer, -1);
    if (i1 < 0) {
      emit_generic(src_slot, dst_slot, so, dof, w, 1, 0, 0, fill);
      return;
    }
    const BoxDim dim1 = outer[i1];
    const int64_t n1 = std::min(dim1.n, rows);
    std::vector<BoxDim> rest;
    for (int i = 0; i < static_cast<int>(outer.size()); ++i)
      if (i != i1) rest.push_back(outer[i]);
    for_each_index(rest, [&](int64_t ds, int64_t dd) {
      for (int64_t b1 = 0; b1 < dim1.n; b1 += n1)
        emit_generic(src_slot, dst_slot, so + ds + b1 * dim1.s, dof + dd + b1 * dim1.d, w, std::min(n1, dim1.n - b1),
                     dim1.s, dim1.d, fill);
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
  uint32_t span_bytes_;
  bool force_ragged_;
  bool no_span_;
  int array_ = 0;
  uint32_t ordinal_ = 0;
  std::vector<CanonBox> tile_;
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
    if (empty) {
      b.finish_tile();
      continue;
    }
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
    b.finish_tile();
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

namespace {

bool congruent(const ProtoCopy& a, const ProtoCopy& b) {
  const CopyGroup &x = a.g, &y = b.g;
  if (a.array != b.array || a.ordinal != b.ordinal || x.k != y.k || x.n1 != y.n1 || x.n2 != y.n2 || x.n3 != y.n3 ||
      x.m1 != y.m1 || x.m2 != y.m2 || x.d1 != y.d1 || x.d2 != y.d2 || x.d3 != y.d3)
    return false;
  for (uint32_t j = 0; j < x.k; ++j)
    if (a.pieces[j].w != b.pieces[j].w || a.pieces[j].dst != b.pieces[j].dst) return false;
  return true;
}

bool congruent(const ProtoSpan& a, const ProtoSpan& b) {
  const SpanGroup &x = a.g, &y = b.g;
  return a.array == b.array && a.ordinal == b.ordinal && x.W == y.W && x.band_bytes == y.band_bytes && x.n1 == y.n1 &&
         x.span == y.span && x.head == y.head;
}

// Fixes the launch order of the copy groups and lays them out in the plan.
//   order 1: as generated; 2: by destination address; 3: by source address; 4: by destination, the tiles of an array
//   interleaved in rounds of `fraction_bytes` per tile.
void assemble_copies(std::vector<ProtoCopy>& protos, uint32_t order, int64_t fraction_bytes, mmr_plan* plan) {
  std::vector<size_t> at(protos.size());
  for (size_t i = 0; i < at.size(); ++i) at[i] = i;
  auto dst_key = [&](size_t i) { return std::make_tuple(protos[i].pieces[0].dst_slot, protos[i].pieces[0].dst, i); };
  if (order == 2) {
    std::sort(at.begin(), at.end(), [&](size_t a, size_t b) { return dst_key(a) < dst_key(b); });
  } else if (order == 3) {
    std::sort(at.begin(), at.end(), [&](size_t a, size_t b) {
      return std::make_tuple(protos[a].pieces[0].src_slot, protos[a].pieces[0].src, a) <
             std::make_tuple(protos[b].pieces[0].src_slot, protos[b].pieces[0].src, b);
    });
  } else if (order == 4) {
    std::sort(at.begin(), at.end(), [&](size_t a, size_t b) {
      return std::make_tuple(protos[a].array, protos[a].ordinal, dst_key(a)) <
             std::make_tuple(protos[b].array, protos[b].ordinal, dst_key(b));
    });
  }
  uint32_t next_chunk = 0;
  for (size_t i = 0; i < at.size();) {
    const ProtoCopy& first = protos[at[i]];
    size_t j = i + 1;
    if (order == 4)
      while (j < at.size() && congruent(first, protos[at[j]])) ++j;
    CopyGroup g = first.g;
    const uint32_t members = static_cast<uint32_t>(j - i);
    const uint32_t member_chunks = g.k * g.c12 * g.n3;
    // a round holds whole row blocks of all k pieces
    uint32_t fraction = member_chunks;
    if (members > 1) {
      const uint64_t per = std::max<uint64_t>(first.chunk_bytes, 1);
      fraction = static_cast<uint32_t>(std::max<uint64_t>(1, static_cast<uint64_t>(fraction_bytes) / per / g.k)) * g.k;
    }
    g.first_chunk = next_chunk;
    g.n_chunks = members * member_chunks;
    g.first_piece = static_cast<uint32_t>(plan->copy_pieces.size());
    g.div_k = make_fastdiv(g.k);
    g.div_c1 = make_fastdiv(g.c1);
    g.div_c12 = make_fastdiv(g.c12);
    g.div_m1 = make_fastdiv(g.m1);
    g.div_last1 = make_fastdiv(g.n1 % g.m1 ? g.n1 % g.m1 : g.m1);
    g.il = make_interleave(members, member_chunks, fraction);
    // the lean chunk code: one pass, offsets inside a chunk in 32 bits (24 bits per factor for the fast multiplies)
    uint64_t reach = 0, widest = 0, stride_bits = static_cast<uint64_t>(g.d1 | g.d2);
    for (size_t m = i; m < j; ++m)
      for (const CopyPiece& pc : protos[at[m]].pieces) {
        widest = std::max<uint64_t>(widest, pc.w);
        stride_bits |= static_cast<uint64_t>(pc.s1 | pc.s2);
        reach = std::max<uint64_t>(reach, static_cast<uint64_t>(g.m2 - 1) * static_cast<uint64_t>(std::max(pc.s2, g.d2)) +
                                              static_cast<uint64_t>(g.m1 - 1) * static_cast<uint64_t>(std::max(pc.s1, g.d1)) + pc.w);
      }
    g.lean = 0;
    if (static_cast<uint64_t>(g.m1) * g.m2 * (widest >> 4) <= kLeanVectors && reach < (1ull << 32) && g.d1 >= 0 && g.d2 >= 0)
      g.lean = stride_bits < (1ull << 24) ? 2 : 1;
    for (size_t m = i; m < j; ++m)
      for (const CopyPiece& pc : protos[at[m]].pieces) {
        if (pc.src_slot == MMR_SLOT_FILL) plan->stats.n_fill_chunks += member_chunks / g.k;
        plan->copy_pieces.push_back(pc);
      }
    plan->copy_groups.push_back(g);
    next_chunk += g.n_chunks;
    i = j;
  }
  plan->n_copy_chunks = next_chunk;
}

void assemble_spans(std::vector<ProtoSpan>& protos, uint32_t order, int64_t fraction_bytes, bool segment_tables,
                    mmr_plan* plan) {
  std::vector<size_t> at(protos.size());
  for (size_t i = 0; i < at.size(); ++i) at[i] = i;
  auto dst_key = [&](size_t i) { return std::make_tuple(protos[i].m.dst_slot, protos[i].m.dst, i); };
  if (order == 2 || order == 3) {
    std::sort(at.begin(), at.end(), [&](size_t a, size_t b) { return dst_key(a) < dst_key(b); });
  } else if (order == 4) {
    std::sort(at.begin(), at.end(), [&](size_t a, size_t b) {
      return std::make_tuple(protos[a].array, protos[a].ordinal, dst_key(a)) <
             std::make_tuple(protos[b].array, protos[b].ordinal, dst_key(b));
    });
  }
  uint32_t next_chunk = 0;
  for (size_t i = 0; i < at.size();) {
    const ProtoSpan& first = protos[at[i]];
    size_t j = i + 1;
    if (order == 4)
      while (j < at.size() && congruent(first, protos[at[j]])) ++j;
    SpanGroup g = first.g;
    const uint32_t members = static_cast<uint32_t>(j - i);
    const uint32_t member_chunks = span_chunks(g.band_bytes, g.head, g.span);
    const uint32_t fraction =
        members > 1 ? static_cast<uint32_t>(std::max<int64_t>(1, fraction_bytes / g.span)) : member_chunks;
    g.first_chunk = next_chunk;
    g.n_chunks = members * member_chunks;
    g.first_member = static_cast<uint32_t>(plan->span_members.size());
    g.il = make_interleave(members, member_chunks, fraction);
    // few pieces per row and few (row, piece) pairs per span: the span kernel tabulates the pairs, one per lane
    uint32_t most_pieces = 0;
    for (size_t m = i; m < j; ++m) most_pieces = std::max(most_pieces, protos[at[m]].m.k);
    const uint64_t rows_per_span = g.span / g.W + 2;
    g.table_mode = segment_tables && most_pieces <= kSpanTablePieces && rows_per_span * most_pieces <= kSpanLanes ? 1 : 0;
    for (size_t m = i; m < j; ++m) {
      SpanMember mem = protos[at[m]].m;
      mem.first_piece = static_cast<uint32_t>(plan->span_pieces.size());
      plan->span_pieces.insert(plan->span_pieces.end(), protos[at[m]].pieces.begin(), protos[at[m]].pieces.end());
      plan->span_members.push_back(mem);
    }
    plan->span_groups.push_back(g);
    next_chunk += g.n_chunks;
    i = j;
  }
  plan->n_span_chunks = next_chunk;
}

}  // namespace

mmr_copy_chunk decoded_copy_chunk(const mmr_plan& plan, uint32_t ci) {
  const uint32_t gi = find_group(plan.copy_groups.data(), static_cast<uint32_t>(plan.copy_groups.size()), nullptr, ci);
  const CopyGroup& g = plan.copy_groups[gi];
  const DecodedCopy d = decode_copy(g, ci - g.first_chunk);
  return copy_chunk_of(g, plan.copy_pieces[d.piece], d);
}

int build_plan(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int n, const mmr_plan_options& options,
               mmr_plan* plan) {
  if (n < 0 || (n > 0 && (!srcs || !dsts))) return fail(MMR_INVALID_ARGUMENT, "bad descriptor arrays");
  uint32_t chunk_bytes = options.chunk_bytes ? options.chunk_bytes : kDefaultChunkBytes;
  chunk_bytes = std::min<uint32_t>(std::max<uint32_t>(chunk_bytes, 256), 16u << 20) & ~255u;
  plan->options = options;
  // Generic chunks (ragged boxes the span kernel does not take) cost more instructions per byte: half the aligned
  // size when a size is asked for, 7 KiB by default, less for small plans so that they still make some 8,000 chunks.
  uint32_t generic_chunk_bytes = std::max<uint32_t>(chunk_bytes / 2, 256);
  // Span of destination bytes per workgroup of the span kernel: the chunk size asked for, rounded to 128-byte lines.
  uint32_t span_bytes = std::min<uint32_t>(std::max<uint32_t>(chunk_bytes & ~127u, 128), kSpanMaxBytes);
  if (options.chunk_bytes == 0) {
    int64_t payload = 0;
    for (int a = 0; a < n; ++a) {
      int64_t bytes = mmr_itemsize(srcs[a].dtype) > 0 ? mmr_itemsize(srcs[a].dtype) : 1;
      for (int i = 0; i < srcs[a].ndims && i < MMR_MAX_DIMS; ++i) bytes *= std::max<int64_t>(srcs[a].dims[i].size, 1);
      payload += bytes;
    }
    generic_chunk_bytes = static_cast<uint32_t>(std::min<int64_t>(std::max<int64_t>(payload / 8192, 2048), 7168)) & ~255u;
    span_bytes = kDefaultSpanBytes;
  }
  Builder builder(plan, chunk_bytes, generic_chunk_bytes, span_bytes, (options.flags & MMR_PLAN_ALL_GENERIC) != 0,
                  (options.flags & MMR_PLAN_NO_SPAN) != 0);
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
    builder.begin_array(a);
    if (int rc = plan_one_array(builder, S, D, static_cast<uint32_t>(plan->n_slots))) return rc;
    plan->n_slots += S.dev_count + D.dev_count;
  }
  // Launch order.  Copy groups: by destination address unless the options say otherwise.  Span groups (ragged rows):
  // by destination with the tiles of an array interleaved - chunks of neighbouring tiles that cover the same rows
  // read the same source lines at the edges of their column ranges, and runs of table neighbours share an XCD's L2.
  const int64_t fraction_kib = (options.flags >> 8) & 0xffffu;
  const uint32_t copy_order = options.order ? options.order : 2;
  const uint32_t span_order = options.order ? options.order : 4;
  assemble_copies(builder.copies, copy_order, (fraction_kib ? fraction_kib : 64) * 1024, plan);
  assemble_spans(builder.spans, span_order, (fraction_kib ? fraction_kib : kDefaultSpanFractionKib) * 1024,
                 (options.flags & MMR_PLAN_NO_SEGMENT_TABLES) == 0, plan);
  if (plan->n_copy_chunks > 0x7ff00000u || plan->n_span_chunks > 0x7ff00000u)
    return fail(MMR_INVALID_ARGUMENT, "plan of more than 2^31 chunks");
  const uint32_t order = options.order ? options.order : 2;
  if (order == 2 || order == 3 || order == 4) {
    auto sort_generic = [order](std::vector<mmr_copy_chunk>& table) {
      std::stable_sort(table.begin(), table.end(), [order](const mmr_copy_chunk& a, const mmr_copy_chunk& b) {
        return order == 3 ? std::tie(a.src_slot, a.src_off) < std::tie(b.src_slot, b.src_off)
                          : std::tie(a.dst_slot, a.dst_off) < std::tie(b.dst_slot, b.dst_off);
      });
    };
    sort_generic(plan->generic);
    // Tiles: in blocks of 8 x 8 tiles (long contiguous pieces on the source side as well as on the destination
    // side: +10 % over plain destination order), the blocks taken diagonal after diagonal - (block column + block
    // row + 3 * destination buffer) mod 8 - rather than column after column: the tiles in flight together then differ
    // in their source rows as well as in their destination rows.  With power-of-two pitches, rows one tile apart lie
    // a multiple of the memory channels' interleave apart, and a launch that walks one side in address order keeps
    // hitting the same few channels on the other side (measured +3 to +12 % on power-of-two transposes of 1-, 2- and
    // 4-byte elements in six shapes and splits, -3 % on a 6144 x 6144 one; other block shapes, moduli and key orders
    // won on some of them and lost more on others).
    auto tile_key = [](const mmr_transpose_chunk& c) {
      const uint64_t pitch = c.dst_xstride > 0 ? static_cast<uint64_t>(c.dst_xstride) : 1;
      uint32_t tx = 0, ty = 0;
      transpose_tile_extent(c.itemsize, &tx, &ty);
      const uint64_t x = c.dst_off / pitch, y = c.dst_off % pitch;  // destination row, byte within it
      const uint64_t bx = x / (8ull * tx), by = y / (8ull * ty * c.itemsize);
      return std::make_tuple((bx + by + 3ull * c.dst_slot) % 8ull, bx, c.dst_slot, x, y);
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
  plan->stats.interleave_kib = options.order == 4 ? (fraction_kib ? fraction_kib : 64) : 0;
  plan->stats.n_arrays = n;
  plan->stats.n_copy16_chunks = plan->n_copy_chunks;
  plan->stats.n_copy16_launches = copy_group_launches(plan->n_copy_chunks, options.xcd_mode == 0 ? 64 : options.xcd_mode);
  plan->stats.n_span_chunks = plan->n_span_chunks;
  plan->stats.n_copy_generic_chunks = static_cast<int64_t>(plan->generic.size());
  plan->stats.n_transpose_chunks = static_cast<int64_t>(plan->transposes.size());
  plan->stats.n_groups = static_cast<int64_t>(plan->copy_groups.size() + plan->span_groups.size());
  plan->stats.n_pieces = static_cast<int64_t>(plan->copy_pieces.size() + plan->span_pieces.size());
  plan->stats.n_slots = plan->n_slots;
  plan->stats.table_bytes = static_cast<int64_t>(
      plan->copy_groups.size() * sizeof(CopyGroup) + plan->copy_pieces.size() * sizeof(CopyPiece) +
      plan->span_groups.size() * sizeof(SpanGroup) + plan->span_members.size() * sizeof(SpanMember) +
      plan->span_pieces.size() * sizeof(SpanPiece) +
      (((plan->n_copy_chunks + 63) >> 6) + ((plan->n_span_chunks + 63) >> 6)) * sizeof(uint32_t) +
      plan->generic.size() * sizeof(mmr_copy_chunk) + plan->transposes.size() * sizeof(mmr_transpose_chunk) +
      ((plan->generic.empty() && plan->transposes.empty()) ? 0 : plan->n_slots * sizeof(void*)));
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
  if (kind == 0) {  // decoded from the group table, in launch order
    if (!out) return plan->n_copy_chunks;
    const int64_t n = std::min<int64_t>(capacity, plan->n_copy_chunks);
    for (int64_t i = 0; i < n; ++i) out[i] = mmr::decoded_copy_chunk(*plan, static_cast<uint32_t>(i));
    return n;
  }
  if (kind == 2) {  // the row pieces of the span groups, one record each: n2 x n1 rows of w bytes
    std::vector<mmr_copy_chunk> v;
    for (const mmr::SpanGroup& g : plan->span_groups)
      for (uint32_t t = 0; t < g.il.members; ++t) {
        const mmr::SpanMember& m = plan->span_members[g.first_member + t];
        for (uint32_t j = 0; j < m.k; ++j) {
          const mmr::SpanPiece& p = plan->span_pieces[m.first_piece + j];
          mmr_copy_chunk c{};
          c.src_slot = p.src_slot;
          c.dst_slot = m.dst_slot;
          c.src_off = p.src;
          c.dst_off = m.dst + p.col;
          c.w = p.w;
          c.n1 = g.n1;
          c.n2 = static_cast<uint32_t>(g.band_bytes / g.W / g.n1);
          c.align = 1;
          c.s1 = p.s1;
          c.d1 = g.W;
          c.s2 = p.s2;
          c.d2 = static_cast<int64_t>(g.W) * g.n1;
          v.push_back(c);
        }
      }
    if (!out) return static_cast<int64_t>(v.size());
    const int64_t n = std::min<int64_t>(capacity, static_cast<int64_t>(v.size()));
    if (n > 0) std::memcpy(out, v.data(), sizeof(mmr_copy_chunk) * n);
    return n;
  }
  const auto& v = plan->generic;
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
