// Per-chunk data movement, written once for two callers:
//   * kernels.hip instantiates it with a device memory policy (global address
//     space, nontemporal hints) - one workgroup per chunk, `tid` = threadIdx.x;
//   * the host emulation used by the tests instantiates it with a bounds-checked
//     host policy and calls it once per thread id, so every index computation
//     below can be checked on a CPU before it ever runs on a GPU.
// Nothing here synchronises threads: the transpose is split into a load phase
// and a store phase around the caller's barrier.
//
// A memory policy `M` provides
//   typedef ... cptr;  typedef ... ptr;          byte pointers (const / mutable)
//   static V16 load16(cptr), load16u(cptr);       16-byte load, aligned / any alignment
//   static V16 load16u_keep(cptr);                the same for bytes other workgroups read too (no streaming hint)
//   static void store16(ptr, V16);                16-byte aligned store
//   static T loadu<T>(cptr); static void storeu<T>(ptr, T);   1/2/4/8-byte, any alignment
//   static uintptr_t addr(ptr), caddr(cptr);      numeric address (for alignment math)
#ifndef MMR_CSRC_CHUNK_OPS_H_
#define MMR_CSRC_CHUNK_OPS_H_

#include <cstdint>

#include "mmreshard.h"

#if defined(__HIP__)
#define MMR_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define MMR_HD inline
#endif

namespace mmr {

struct alignas(16) V16 {
  uint32_t x, y, z, w;
};

constexpr uint32_t kXcds = 8;  // MI355X: 256 CUs in 8 XCDs, each with its own L2

// Workgroup -> table index.  The hardware deals consecutive workgroups
// round-robin over the XCDs.  With group = G > 1, runs of G consecutive chunks
// go to one XCD (runs dealt round-robin), so chunks that are neighbours in the
// address-sorted table, and may share cache lines at their edges, meet in one
// L2.  G = 1 is the hardware order; G >= n / 8 gives each XCD a contiguous
// eighth of the table.  The grid is padded to a multiple of 8 * G; padded
// workgroups map to indices >= n and do nothing.
MMR_HD uint32_t chunk_index(uint32_t block, uint32_t group) {
  if (group <= 1) return block;
  if (group == 64) return ((((block >> 9) << 3) + (block & 7u)) << 6) | ((block >> 3) & 63u);  // the usual case, no division
  const uint32_t xcd = block % kXcds, j = block / kXcds;
  return ((j / group) * kXcds + xcd) * group + (j % group);
}

inline uint32_t xcd_group_of(int64_t n, uint32_t mode) {
  if (mode == 2) return static_cast<uint32_t>((n + kXcds - 1) / kXcds);
  if (mode >= 16) return mode;
  return 1;
}

inline uint32_t grid_size(int64_t n, uint32_t group) {
  if (group <= 1) return static_cast<uint32_t>(n);
  const int64_t span = static_cast<int64_t>(group) * kXcds;
  return static_cast<uint32_t>((n + span - 1) / span * span);
}

// Very long tables leave in pieces.  The eight XCDs do not work through their shares of a launch at the same rate
// (0.5-1.5 % apart; start times of every workgroup of a 655,360-chunk launch, a probe build), so the workgroups in
// flight spread over the table: 2,000 table positions at the start, 11,000 (90 MB) at the end of that launch, and
// the rate falls with it: the hidden 8-way -> sequence 4-way split of bf16 [N, 4096, 8192] runs at 83 % of the 8
// TB/s peak in one launch for N = 8 to 24 (65,536 to 196,608 chunks), at 81-82 % for N = 40 to 64 and at 80 % for N
// = 80 (655,360 chunks, 10.7 GB).  A launch boundary brings the XCDs together again (the spread stays under 2,900
// positions with pieces of 131,072) and costs 3-6 us.  Measured on
// MI355X, pieces of 131,072 chunks (1 GiB read + 1 GiB written, ~0.33 ms) against one launch: N = 80 1.673 -> 1.641
// ms, N = 64 1.313 -> 1.300 ms, N = 48 0.985 -> 0.977 ms, N = 40 0.825 -> 0.818 ms, a batch of 195 arrays (650 k
// chunks) 1.706 -> 1.652 ms - within 1 % of what its arrays take one by one; 65,536 and 98,304 measure the same,
// 196,608 and more gain less; N = 32 loses (0.675 -> 0.685 ms) and N <= 24 is unchanged or slower, so tables of
// fewer than three pieces are launched whole.
#ifndef MMR_COPY_PIECE_CHUNKS
#define MMR_COPY_PIECE_CHUNKS 131072
#endif
#ifndef MMR_COPY_PIECES_MIN
#define MMR_COPY_PIECES_MIN 3
#endif

// Chunks per launch of a copy-group table of n chunks (n itself: one launch).
inline int64_t copy_piece_chunks(int64_t n, uint32_t xcd_mode) {
  // a whole number of XCD rounds per piece, so that every piece but the last fills its grid exactly
  const int64_t group = xcd_group_of(n, xcd_mode);
  const int64_t unit = (group > 1 ? group : 1) * kXcds;
  const int64_t piece = (static_cast<int64_t>(MMR_COPY_PIECE_CHUNKS) + unit - 1) / unit * unit;
  if (xcd_mode == 2 || n < piece * MMR_COPY_PIECES_MIN) return n > 1 ? n : 1;
  return piece;
}

inline int64_t copy_group_launches(int64_t n, uint32_t xcd_mode) {
  if (n <= 0) return 0;
  const int64_t piece = copy_piece_chunks(n, xcd_mode);
  return (n + piece - 1) / piece;
}

// ---------------------------------------------------------------------------
// Aligned copy: every offset, stride and row width is a multiple of 16 bytes.
// Rows of wv = w/16 vectors.  The (row, column) pairs of the chunk are numbered
// row after row and dealt to the lanes, UNROLL per lane and pass.  Branch-free:
// a lane whose number runs past the end of the chunk repeats the chunk's last
// vector (same load, same store as the rightful lane), so a pass is
// straight-line code - UNROLL loads, UNROLL stores, the next pass's loads
// issued while these stores are still in flight - where per-lane branches made
// the compiler wait for each access before issuing the next.  One division
// chain per thread; after that a lane's (r2, r1, column) advances by a fixed
// step with carries.
// ---------------------------------------------------------------------------
template <class M, int THREADS, int UNROLL, bool FILL>
MMR_HD void copy16_rows(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  const uint32_t wv = c.w >> 4, n1 = c.n1, n2 = c.n2;
  const uint32_t total = n1 * n2 * wv;
  const uint32_t step_col = THREADS % wv, rest = THREADS / wv, step_r1 = rest % n1, step_r2 = rest / n1;
  uint32_t row = tid / wv, col = tid - row * wv, r2 = row / n1, r1 = row - r2 * n1;
  for (uint32_t base = 0; base < total; base += THREADS * UNROLL) {
    V16 v[UNROLL];
    int64_t soff[UNROLL], doff[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const bool inside = base + tid + u * THREADS < total;
      const uint32_t q2 = inside ? r2 : n2 - 1, q1 = inside ? r1 : n1 - 1, qc = inside ? col : wv - 1;
      soff[u] = q2 * c.s2 + q1 * c.s1 + (static_cast<int64_t>(qc) << 4);
      doff[u] = q2 * c.d2 + q1 * c.d1 + (static_cast<int64_t>(qc) << 4);
      col += step_col;
      if (col >= wv) {
        col -= wv;
        r1 += 1;
      }
      r1 += step_r1;
      if (r1 >= n1) {
        r1 -= n1;
        r2 += 1;
      }
      r2 += step_r2;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = FILL ? V16{0, 0, 0, 0} : M::load16(src + soff[u]);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) M::store16(dst + doff[u], v[u]);
  }
}

template <class M, int THREADS, int UNROLL>
MMR_HD void copy16_chunk(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  // uniform over the workgroup; a chunk without a source writes zeros
  if (c.src_slot == MMR_SLOT_FILL) copy16_rows<M, THREADS, UNROLL, true>(c, src, dst, tid);
  else copy16_rows<M, THREADS, UNROLL, false>(c, src, dst, tid);
}

// ---------------------------------------------------------------------------
// Generic copy: n1 rows of any width at any byte alignment on either side
// (the planner emits generic chunks with n2 == 1).  Each row is cut at the
// 16-byte boundaries of its SOURCE (of its destination when the chunk fills):
// a lane owns one aligned 16-byte slot, loads it with one 16-byte load and
// writes the matching destination bytes with one 16-byte store at whatever
// alignment they have - measured on MI355X, a misaligned store costs less than
// a misaligned load (2-3 % of the kernel time on byte-misaligned rows).  A slot
// cut off by a row end (the first and the last slot of a row, in general)
// slides inwards until it lies inside the row: it still moves 16 bytes, now
// unaligned on both sides, and overlaps its neighbour, which writes the same
// values to the shared bytes.  So every lane runs the same two instructions
// and no access ever leaves its row (lanes with no pair of their own left
// repeat the last pair, see generic_slot).  Rows
// narrower than 16 bytes have no room to slide: their 1..15 bytes move as
// 8/4/2/1-byte pieces (binary decomposition of the length), carried in one V16:
// .x/.y the 8-byte piece, .z the 4-byte piece, .w the 2-byte piece (low half)
// and the 1-byte piece (bits 16-23).
// ---------------------------------------------------------------------------
template <class M>
MMR_HD V16 load_ragged(typename M::cptr s, uint32_t len) {
  V16 v{0, 0, 0, 0};
  const uint32_t o4 = len & 8, o2 = o4 + (len & 4), o1 = o2 + (len & 2);
  if (len & 8) {
    const uint64_t a = M::template loadu<uint64_t>(s);
    v.x = static_cast<uint32_t>(a);
    v.y = static_cast<uint32_t>(a >> 32);
  }
  if (len & 4) v.z = M::template loadu<uint32_t>(s + o4);
  if (len & 2) v.w = M::template loadu<uint16_t>(s + o2);
  if (len & 1) v.w |= static_cast<uint32_t>(M::template loadu<uint8_t>(s + o1)) << 16;
  return v;
}

template <class M>
MMR_HD void store_ragged(typename M::ptr d, uint32_t len, V16 v) {
  const uint32_t o4 = len & 8, o2 = o4 + (len & 4), o1 = o2 + (len & 2);
  if (len & 8) M::template storeu<uint64_t>(d, static_cast<uint64_t>(v.x) | (static_cast<uint64_t>(v.y) << 32));
  if (len & 4) M::template storeu<uint32_t>(d + o4, v.z);
  if (len & 2) M::template storeu<uint16_t>(d + o2, static_cast<uint16_t>(v.w));
  if (len & 1) M::template storeu<uint8_t>(d + o1, static_cast<uint8_t>(v.w >> 16));
}

// Rows of at least 16 bytes.  Branch-free: a (row, slot) pair past the end of its row or of the chunk repeats the
// last slot of that row (of the last row), i.e. loads the same 16 bytes and stores them to the same place as the
// rightful lane does.  With no lane predicated the loop body is straight-line code - UNROLL loads, one wait,
// UNROLL stores - where per-lane branches made the compiler wait for each access before issuing the next.
template <class M>
MMR_HD void generic_slot(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, bool fill, uint32_t row,
                         uint32_t slot, typename M::cptr* spos, typename M::ptr* dpos) {
  typename M::ptr drow = dst + row * c.d1;
  typename M::cptr srow = src + row * c.s1;
  const int32_t w = static_cast<int32_t>(c.w);
  const int32_t mis = static_cast<int32_t>((fill ? M::addr(drow) : M::caddr(srow)) & 15u);
  const int32_t rel = static_cast<int32_t>(slot << 4) - mis;  // row-relative byte where this aligned slot starts
  const int32_t lo = rel < 0 ? 0 : (rel + 16 > w ? w - 16 : rel);
  *spos = srow + lo;
  *dpos = drow + lo;
}

template <class M, int THREADS, int UNROLL, bool FILL>
MMR_HD void generic_wide_rows(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  constexpr bool fill = FILL;  // a chunk without a source writes zeros: its own instance, so neither loop branches
  const uint32_t slots = ((c.w + 15u) >> 4) + 1u;  // a row of w bytes touches at most this many aligned slots
  const uint32_t rows = c.n1;
  if (slots >= THREADS) {
    for (uint32_t row = 0; row < rows; ++row) {
      for (uint32_t s0 = 0; s0 < slots; s0 += THREADS * UNROLL) {
        V16 v[UNROLL];
        typename M::cptr spos[UNROLL];
        typename M::ptr dpos[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const uint32_t slot = s0 + tid + u * THREADS;
          generic_slot<M>(c, src, dst, fill, row, slot < slots ? slot : slots - 1, &spos[u], &dpos[u]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = fill ? V16{0, 0, 0, 0} : M::load16u(spos[u]);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) M::template storeu<V16>(dpos[u], v[u]);
      }
    }
    return;
  }
  // Rows narrower than the workgroup: the (row, slot) pairs of the chunk are numbered row after row and dealt to
  // the lanes without regard to row ends, so no lane idles while pairs are left.  One division per thread; after
  // that a lane's pair advances by THREADS pairs per step = (step_rows, step_slots) with a carry.
  const uint32_t total = rows * slots;
  const uint32_t step_rows = THREADS / slots, step_slots = THREADS - step_rows * slots;
  uint32_t row = tid / slots, slot = tid - row * slots;
  for (uint32_t base = 0; base < total; base += THREADS * UNROLL) {
    V16 v[UNROLL];
    typename M::cptr spos[UNROLL];
    typename M::ptr dpos[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const bool inside = base + tid + u * THREADS < total;
      generic_slot<M>(c, src, dst, fill, inside ? row : rows - 1, inside ? slot : slots - 1, &spos[u], &dpos[u]);
      row += step_rows;
      slot += step_slots;
      if (slot >= slots) {
        slot -= slots;
        row += 1;
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = fill ? V16{0, 0, 0, 0} : M::load16u(spos[u]);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) M::template storeu<V16>(dpos[u], v[u]);
  }
}

// Rows narrower than 16 bytes: one (row, slot) pair per lane and step, 8/4/2/1-byte pieces.
template <class M>
MMR_HD void generic_narrow_load(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, bool fill, uint32_t row,
                                uint32_t slot, V16* v, typename M::ptr* dpos, int32_t* len) {
  typename M::ptr drow = dst + row * c.d1;
  typename M::cptr srow = src + row * c.s1;
  const int32_t w = static_cast<int32_t>(c.w);
  const int32_t mis = static_cast<int32_t>((fill ? M::addr(drow) : M::caddr(srow)) & 15u);
  const int32_t rel = static_cast<int32_t>(slot << 4) - mis;  // row-relative byte where this aligned slot starts
  const int32_t lo = rel < 0 ? 0 : rel;
  const int32_t hi = rel + 16 < w ? rel + 16 : w;
  *len = hi - lo;
  *dpos = drow + lo;
  if (*len > 0) *v = fill ? V16{0, 0, 0, 0} : load_ragged<M>(srow + lo, static_cast<uint32_t>(*len));
}

template <class M, int THREADS, int UNROLL>
MMR_HD void generic_narrow_rows(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  const bool fill = c.src_slot == MMR_SLOT_FILL;
  const uint32_t slots = 2;  // a row of under 16 bytes touches at most two aligned slots
  const uint32_t total = c.n1 * slots;
  for (uint32_t i0 = tid; i0 < total; i0 += THREADS * UNROLL) {
    V16 v[UNROLL];
    typename M::ptr dpos[UNROLL];
    int32_t len[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      len[u] = 0;
      const uint32_t i = i0 + u * THREADS;
      if (i < total) generic_narrow_load<M>(c, src, dst, fill, i >> 1, i & 1u, &v[u], &dpos[u], &len[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
      if (len[u] > 0) store_ragged<M>(dpos[u], static_cast<uint32_t>(len[u]), v[u]);
  }
}

template <class M, int THREADS, int UNROLL>
MMR_HD void generic_chunk(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  // all three choices are uniform over the workgroup
  if (c.w < 16) generic_narrow_rows<M, THREADS, UNROLL>(c, src, dst, tid);
  else if (c.src_slot == MMR_SLOT_FILL) generic_wide_rows<M, THREADS, UNROLL, true>(c, src, dst, tid);
  else generic_wide_rows<M, THREADS, UNROLL, false>(c, src, dst, tid);
}

// ---------------------------------------------------------------------------
// Tile transpose: x is contiguous in the source, y in the destination.
//
// A workgroup owns a tile of kTileX x kTileY elements, its waves one
// kEX x kEY sub-tile each (kWX x kWY waves; for 1-byte elements all four waves
// share one sub-tile).
//
// Every wave works alone, on its own sub-tile and its own slice of LDS, so the
// only synchronisation is between the lanes of a wave (the caller puts a
// wave-level fence between the two phases; a workgroup barrier where waves
// share a sub-tile).  What a wave does with its sub-tile depends on the part of
// it that lies inside the tile (snx x sny elements):
//
// Vector path (chunk 16-byte aligned on both sides, snx and sny multiples of
// the vector width): every global access is an aligned 16-byte vector and every
// LDS access at least a dword.  A lane loads the same vector of kPack =
// 4 / itemsize adjacent source rows (one row for elements of 4 bytes and more),
// so for each of the vector's x it holds kPack consecutive y: one dword (or one
// element of 8 / 16 bytes), written to row x of an LDS tile laid out [x][y]
// without padding.  In the second phase a lane reads one 16-byte group of an
// LDS row = consecutive y of one x and stores it to destination row x.  All
// global loads of a lane are issued before its first LDS write.
//
// General path (any alignment, snx and sny at least one vector): the same with
// unaligned 16-byte global accesses.  A vector cut off by the edge of the tile
// slides inwards until it ends at the edge (it overlaps its neighbour, which
// moves the same values); a packed source row beyond the edge is replaced by
// the last row inside (its LDS cells are never read).  A destination vector
// that slid is gathered from LDS element by element.  No access leaves the
// tile.
//
// Element path (a sub-tile thinner than one vector): one element per lane and
// step, same LDS layout.
//
// LDS banks: rows are a multiple of 128 bytes apart, so the 16-byte groups of a
// row are permuted by XOR with a function of x whose low three bits differ
// between the 8 lanes that write the same y of 8 neighbouring vectors (and
// between any 8 consecutive x): the dword writes of 32 lanes then fall into 32
// different banks.  Reads are conflict-free by construction (8 consecutive
// lanes read the 8 groups of one 128-byte row segment).
// ---------------------------------------------------------------------------
template <int ITEM>
struct TransposeTile {
  // wave sub-tile: 128 bytes (or more) wide on both sides, so every access of 8 lanes is a full 128-byte line
  static constexpr int kEX = ITEM == 1 ? 128 : (ITEM == 2 || ITEM == 4 ? 64 : 32);
  static constexpr int kEY = ITEM == 1 || ITEM == 4 ? 128 : (ITEM == 16 ? 16 : (ITEM == 8 ? 32 : 64));
  // Sub-tiles per workgroup tile, and the threads that share one.  1-byte elements: the smallest sub-tile is
  // already 16 KiB, too many registers for one wave, so the four waves of the workgroup share a single sub-tile
  // (and synchronise with a workgroup barrier instead of a wave fence).  4-byte elements: the four waves share the
  // whole 64 x 128 tile too, whose rows are 256 and 512 bytes long, and 16 lanes take a 256-byte piece of a row
  // (measured 1.6 % faster than four 32 x 64 sub-tiles with 128-byte pieces; for 2-byte elements the same change
  // measured 0.5 % slower and was not made).
  static constexpr bool kShared = ITEM == 1 || ITEM == 4;
  static constexpr int kWX = kShared ? 1 : 2, kWY = kWX;
  static constexpr int kWaves = kWX * kWY;                   // number of sub-tiles
  static constexpr int kGroupThreads = kShared ? 256 : 64;   // threads per sub-tile
  static constexpr int kThreads = kGroupThreads * kWaves;
  static constexpr int kTileX = kEX * kWX, kTileY = kEY * kWY;
  static constexpr int kVec = 16 / ITEM;                     // elements per 16-byte vector
  static constexpr int kPack = ITEM >= 4 ? 1 : 4 / ITEM;     // source rows a lane packs into one LDS word
  static constexpr int kRowBytes = kEY * ITEM;               // bytes per LDS row (no padding)
  static constexpr int kSrcVecs = kEX / kVec;                // 16-byte groups per source row of a sub-tile
  static constexpr int kDstVecs = kEY / kVec;                // 16-byte groups per destination row of a sub-tile
  static constexpr int kSrcSeg = ITEM == 4 ? 16 : 8;         // lanes that share a row segment when loading ...
  static constexpr int kDstSeg = ITEM == 4 ? 16 : 8;         // ... and when storing (transpose_task)
  static constexpr int kRowPacks = kEY / kPack;              // packed source-row groups per sub-tile
  static constexpr int kWaveLdsBytes = kEX * kEY * ITEM;     // one sub-tile's slice
  static constexpr int kLdsBytes = kWaveLdsBytes * kWaves;
  static_assert(kSrcVecs % 8 == 0 && kDstVecs % 8 == 0, "sub-tile rows must be whole 128-byte lines");
  static_assert(kSrcVecs * kRowPacks % kGroupThreads == 0 && kEX * kDstVecs % kGroupThreads == 0,
                "sub-tile must divide over its threads");
};
constexpr int kTransposeLdsBytes = 32 * 1024;  // the largest TransposeTile<>::kLdsBytes

// Workgroup tile extents in elements for an element width (the planner cuts boxes into these).
inline void transpose_tile_extent(uint32_t itemsize, uint32_t* tile_x, uint32_t* tile_y) {
  switch (itemsize) {
    case 1: *tile_x = TransposeTile<1>::kTileX; *tile_y = TransposeTile<1>::kTileY; break;
    case 2: *tile_x = TransposeTile<2>::kTileX; *tile_y = TransposeTile<2>::kTileY; break;
    case 4: *tile_x = TransposeTile<4>::kTileX; *tile_y = TransposeTile<4>::kTileY; break;
    case 8: *tile_x = TransposeTile<8>::kTileX; *tile_y = TransposeTile<8>::kTileY; break;
    default: *tile_x = TransposeTile<16>::kTileX; *tile_y = TransposeTile<16>::kTileY; break;
  }
}

// What a wave does with its sub-tile (uniform over the threads that share the sub-tile).
enum TransposeMode { kTransposeNothing = 0, kTransposeVector = 1, kTransposeGeneral = 2, kTransposeElement = 3 };

MMR_HD bool transpose_is_aligned(const mmr_transpose_chunk& c) {
  const uint64_t bits = c.src_off | c.dst_off | static_cast<uint64_t>(c.src_ystride) | static_cast<uint64_t>(c.dst_xstride) |
                        static_cast<uint64_t>(c.src_bstride) | static_cast<uint64_t>(c.dst_bstride);
  return (bits & 15u) == 0;
}

// A chunk whose every sub-tile takes the vector path (or lies outside the tile).  Such chunks run through a kernel
// that holds nothing but the vector path: with the general and the element path compiled in, the kernel needs twice
// the registers and runs at half the occupancy.  The planner keeps the two kinds apart in the table.
MMR_HD bool transpose_is_vector(const mmr_transpose_chunk& c) {
  const uint32_t vec = 16u / c.itemsize;
  return transpose_is_aligned(c) && c.nx % vec == 0 && c.ny % vec == 0;
}

// XOR applied to the 16-byte group index of LDS row x.
template <int ITEM>
MMR_HD uint32_t transpose_swizzle(uint32_t x) {
  constexpr uint32_t vec = TransposeTile<ITEM>::kVec;
  return (vec == 1 ? x : (x ^ (x / vec))) & 7u;
}

template <typename T>
MMR_HD T element_of(const V16& v, int i) {
  // i is a compile-time constant after unrolling
  if constexpr (sizeof(T) == 16) {
    return v;
  } else if constexpr (sizeof(T) == 8) {
    return i == 0 ? (static_cast<uint64_t>(v.x) | (static_cast<uint64_t>(v.y) << 32))
                  : (static_cast<uint64_t>(v.z) | (static_cast<uint64_t>(v.w) << 32));
  } else {
    constexpr int per = 4 / static_cast<int>(sizeof(T));  // elements per dword
    const uint32_t d = i / per == 0 ? v.x : (i / per == 1 ? v.y : (i / per == 2 ? v.z : v.w));
    return static_cast<T>(d >> (8 * static_cast<int>(sizeof(T)) * (i % per)));
  }
}

// Task t of a wave's phase -> (row index, 16-byte group within the row).  `seg`
// consecutive lanes take the groups of one row segment of seg * 16 bytes (8:
// a 128-byte line; 16: two), the next `seg` lanes the same segment of the next
// row; wider rows are covered segment after segment.  `rows` is the number of
// rows in the phase.
MMR_HD void transpose_task(uint32_t t, uint32_t rows, uint32_t* row, uint32_t* group, uint32_t seg) {
  const uint32_t r = t / seg;
  *group = (t % seg) + (r / rows) * seg;
  *row = r % rows;
}

// Origin of the sub-tile of wave `wave` inside the workgroup tile, in elements.
template <int ITEM>
MMR_HD void transpose_subtile(uint32_t wave, uint32_t* x0, uint32_t* y0) {
  typedef TransposeTile<ITEM> G;
  *x0 = (wave % G::kWX) * G::kEX;
  *y0 = (wave / G::kWX) * G::kEY;
}

// The part of sub-tile `wave` that lies inside the tile, and what to do with it.
template <int ITEM>
MMR_HD TransposeMode transpose_mode(const mmr_transpose_chunk& c, uint32_t wave, uint32_t* x0, uint32_t* y0, uint32_t* snx,
                                    uint32_t* sny) {
  typedef TransposeTile<ITEM> G;
  transpose_subtile<ITEM>(wave, x0, y0);
  *snx = c.nx > *x0 ? (c.nx - *x0 < static_cast<uint32_t>(G::kEX) ? c.nx - *x0 : static_cast<uint32_t>(G::kEX)) : 0u;
  *sny = c.ny > *y0 ? (c.ny - *y0 < static_cast<uint32_t>(G::kEY) ? c.ny - *y0 : static_cast<uint32_t>(G::kEY)) : 0u;
  if (*snx == 0 || *sny == 0) return kTransposeNothing;
  if (*snx % G::kVec == 0 && *sny % G::kVec == 0 && transpose_is_aligned(c)) return kTransposeVector;
  if (*snx >= static_cast<uint32_t>(G::kVec) && *sny >= static_cast<uint32_t>(G::kVec)) return kTransposeGeneral;
  return kTransposeElement;
}

// LDS address of element (x, y) of a sub-tile slice: row x, 16-byte groups of the row permuted.
template <int ITEM>
MMR_HD uint32_t transpose_lds_offset(uint32_t x, uint32_t y) {
  const uint32_t ybyte = y * static_cast<uint32_t>(ITEM);
  return x * TransposeTile<ITEM>::kRowBytes + (((ybyte >> 4) ^ transpose_swizzle<ITEM>(x)) << 4) + (ybyte & 15u);
}

template <typename T>
MMR_HD void set_element(V16* v, int i, T e) {
  // i is a compile-time constant after unrolling; *v starts as zero
  if constexpr (sizeof(T) == 16) {
    *v = e;
  } else if constexpr (sizeof(T) == 8) {
    if (i == 0) {
      v->x = static_cast<uint32_t>(e);
      v->y = static_cast<uint32_t>(e >> 32);
    } else {
      v->z = static_cast<uint32_t>(e);
      v->w = static_cast<uint32_t>(e >> 32);
    }
  } else {
    constexpr int per = 4 / static_cast<int>(sizeof(T));
    const uint32_t bits = static_cast<uint32_t>(e) << (8 * static_cast<int>(sizeof(T)) * (i % per));
    if (i / per == 0) v->x |= bits;
    else if (i / per == 1) v->y |= bits;
    else if (i / per == 2) v->z |= bits;
    else v->w |= bits;
  }
}

// Vector path, phase 1: global -> registers -> this wave's LDS slice.  tid = thread of the workgroup.  The
// sub-tile must hold at least one vector (the callers skip sub-tiles outside the tile).  No lane is predicated: a
// task that falls outside the tile loads the sub-tile's first vector again and parks it in LDS cells that nobody
// reads (every task's cells lie inside the wave's slice), so the loads are straight-line code and all of them are
// in flight before the first LDS write.
template <class M, typename T>
MMR_HD void transpose_load_vec(const mmr_transpose_chunk& c, typename M::cptr src, uint32_t b, T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  constexpr int kTasks = G::kSrcVecs * G::kRowPacks / G::kGroupThreads;  // per lane
  const uint32_t wave = tid / G::kGroupThreads, lane = tid % G::kGroupThreads;
  uint32_t x0, y0;
  transpose_subtile<sizeof(T)>(wave, &x0, &y0);
  typename M::cptr s = src + (b * c.src_bstride + y0 * c.src_ystride + static_cast<int64_t>(x0) * static_cast<int64_t>(sizeof(T)));
  uint8_t* tile = reinterpret_cast<uint8_t*>(lds) + wave * G::kWaveLdsBytes;
  V16 v[kTasks][G::kPack];
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t yg, xv;
    transpose_task(lane + k * G::kGroupThreads, G::kRowPacks, &yg, &xv, G::kSrcSeg);
    const bool inside = y0 + yg * G::kPack < c.ny && x0 + xv * G::kVec < c.nx;
    const uint32_t yl = inside ? yg * G::kPack : 0u, xl = inside ? xv : 0u;
#pragma unroll
    for (int p = 0; p < G::kPack; ++p)
      v[k][p] = M::load16(s + ((yl + p) * c.src_ystride + static_cast<int64_t>(xl) * 16));
  }
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t yg, xv;
    transpose_task(lane + k * G::kGroupThreads, G::kRowPacks, &yg, &xv, G::kSrcSeg);
    const uint32_t ybyte = yg * G::kPack * static_cast<uint32_t>(sizeof(T));  // byte of y within LDS row x
#pragma unroll
    for (int i = 0; i < G::kVec; ++i) {
      const uint32_t x = xv * G::kVec + i;
      uint8_t* at = tile + x * G::kRowBytes + (((ybyte >> 4) ^ transpose_swizzle<sizeof(T)>(x)) << 4) + (ybyte & 15u);
      if constexpr (sizeof(T) >= 4) {
        *reinterpret_cast<T*>(at) = element_of<T>(v[k][0], i);
      } else {
        uint32_t word = 0;
#pragma unroll
        for (int p = 0; p < G::kPack; ++p)
          word |= static_cast<uint32_t>(element_of<T>(v[k][p], i)) << (8 * static_cast<int>(sizeof(T)) * p);
        *reinterpret_cast<uint32_t*>(at) = word;
      }
    }
  }
}

// Vector path, phase 2: this wave's LDS slice -> registers -> global.
template <class M, typename T>
MMR_HD void transpose_store_vec(const mmr_transpose_chunk& c, typename M::ptr dst, uint32_t b, const T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  constexpr int kTasks = G::kEX * G::kDstVecs / G::kGroupThreads;  // per lane
  const uint32_t wave = tid / G::kGroupThreads, lane = tid % G::kGroupThreads;
  uint32_t x0, y0;
  transpose_subtile<sizeof(T)>(wave, &x0, &y0);
  typename M::ptr d = dst + (b * c.dst_bstride + x0 * c.dst_xstride + static_cast<int64_t>(y0) * static_cast<int64_t>(sizeof(T)));
  const uint8_t* tile = reinterpret_cast<const uint8_t*>(lds) + wave * G::kWaveLdsBytes;
  V16 v[kTasks];
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t x, yv;
    transpose_task(lane + k * G::kGroupThreads, G::kEX, &x, &yv, G::kDstSeg);
    if (x0 + x < c.nx && y0 + yv * G::kVec < c.ny)
      v[k] = *reinterpret_cast<const V16*>(tile + x * G::kRowBytes + ((yv ^ transpose_swizzle<sizeof(T)>(x)) << 4));
  }
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t x, yv;
    transpose_task(lane + k * G::kGroupThreads, G::kEX, &x, &yv, G::kDstSeg);
    if (x0 + x < c.nx && y0 + yv * G::kVec < c.ny) M::store16(d + (x * c.dst_xstride + static_cast<int64_t>(yv) * 16), v[k]);
  }
}

// General path, phase 1.  (x0, y0) origin and snx x sny valid extent of this wave's sub-tile (at least one vector
// each way).  No lane is predicated here either: a vector beyond the edge becomes the last vector inside, a row
// beyond the edge the last row inside; what such a task writes to LDS either repeats what the rightful task writes
// to the same cells or lands in cells of rows y >= sny, which nobody reads.
template <class M, typename T>
MMR_HD void transpose_load_general(const mmr_transpose_chunk& c, typename M::cptr src, uint32_t b, T* lds, uint32_t tid,
                                   uint32_t x0, uint32_t y0, uint32_t snx, uint32_t sny) {
  typedef TransposeTile<sizeof(T)> G;
  constexpr int kTasks = G::kSrcVecs * G::kRowPacks / G::kGroupThreads;  // per lane
  const uint32_t wave = tid / G::kGroupThreads, lane = tid % G::kGroupThreads;
  typename M::cptr s = src + (b * c.src_bstride + y0 * c.src_ystride + static_cast<int64_t>(x0) * static_cast<int64_t>(sizeof(T)));
  uint8_t* tile = reinterpret_cast<uint8_t*>(lds) + wave * G::kWaveLdsBytes;
  V16 v[kTasks][G::kPack];
  uint32_t xs[kTasks];
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t yg, xv;
    transpose_task(lane + k * G::kGroupThreads, G::kRowPacks, &yg, &xv, G::kSrcSeg);
    xs[k] = xv * G::kVec + G::kVec > snx ? snx - G::kVec : xv * G::kVec;  // slides inwards, overlapping its neighbour
#pragma unroll
    for (int p = 0; p < G::kPack; ++p) {
      const uint32_t y = yg * G::kPack + p < sny ? yg * G::kPack + p : sny - 1;  // past the edge: the last row again
      v[k][p] = M::load16u(s + (y * c.src_ystride + static_cast<int64_t>(xs[k]) * static_cast<int64_t>(sizeof(T))));
    }
  }
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t yg, xv;
    transpose_task(lane + k * G::kGroupThreads, G::kRowPacks, &yg, &xv, G::kSrcSeg);
#pragma unroll
    for (int i = 0; i < G::kVec; ++i) {
      uint8_t* at = tile + transpose_lds_offset<sizeof(T)>(xs[k] + i, yg * G::kPack);
      if constexpr (sizeof(T) >= 4) {
        *reinterpret_cast<T*>(at) = element_of<T>(v[k][0], i);
      } else {
        uint32_t word = 0;
#pragma unroll
        for (int p = 0; p < G::kPack; ++p)
          word |= static_cast<uint32_t>(element_of<T>(v[k][p], i)) << (8 * static_cast<int>(sizeof(T)) * p);
        *reinterpret_cast<uint32_t*>(at) = word;
      }
    }
  }
}

// General path, phase 2.
template <class M, typename T>
MMR_HD void transpose_store_general(const mmr_transpose_chunk& c, typename M::ptr dst, uint32_t b, const T* lds, uint32_t tid,
                                    uint32_t x0, uint32_t y0, uint32_t snx, uint32_t sny) {
  typedef TransposeTile<sizeof(T)> G;
  constexpr int kTasks = G::kEX * G::kDstVecs / G::kGroupThreads;  // per lane
  const uint32_t wave = tid / G::kGroupThreads, lane = tid % G::kGroupThreads;
  typename M::ptr d = dst + (b * c.dst_bstride + x0 * c.dst_xstride + static_cast<int64_t>(y0) * static_cast<int64_t>(sizeof(T)));
  const uint8_t* tile = reinterpret_cast<const uint8_t*>(lds) + wave * G::kWaveLdsBytes;
  V16 v[kTasks];
  uint32_t ys[kTasks];
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t x, yv;
    transpose_task(lane + k * G::kGroupThreads, G::kEX, &x, &yv, G::kDstSeg);
    ys[k] = yv * G::kVec;
    if (x < snx && ys[k] < sny) {
      if (ys[k] + G::kVec <= sny) {
        v[k] = *reinterpret_cast<const V16*>(tile + x * G::kRowBytes + ((yv ^ transpose_swizzle<sizeof(T)>(x)) << 4));
      } else {  // cut off by the edge: slides inwards and is gathered element by element
        ys[k] = sny - G::kVec;
        v[k] = V16{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < G::kVec; ++i)
          set_element<T>(&v[k], i, *reinterpret_cast<const T*>(tile + transpose_lds_offset<sizeof(T)>(x, ys[k] + i)));
      }
    }
  }
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t x, yv;
    transpose_task(lane + k * G::kGroupThreads, G::kEX, &x, &yv, G::kDstSeg);
    if (x < snx && yv * G::kVec < sny)
      M::template storeu<V16>(d + (x * c.dst_xstride + static_cast<int64_t>(ys[k]) * static_cast<int64_t>(sizeof(T))), v[k]);
  }
}

// Element path, both phases: a sub-tile thinner than one vector, at most kTransposeThin elements per lane.  All
// loads of a lane are issued before its first LDS write; one division per phase, the (row, column) of a lane's
// next element follows by a fixed step with a carry.
constexpr int kTransposeThin = 8;

template <class M, typename T>
MMR_HD void transpose_load_element(const mmr_transpose_chunk& c, typename M::cptr src, uint32_t b, T* lds, uint32_t tid,
                                   uint32_t x0, uint32_t y0, uint32_t snx, uint32_t sny) {
  typedef TransposeTile<sizeof(T)> G;
  static_assert((G::kEX > G::kEY ? G::kEX : G::kEY) * (G::kVec - 1) <= kTransposeThin * G::kGroupThreads,
                "a thin sub-tile must fit the unrolled element path");
  const uint32_t wave = tid / G::kGroupThreads, lane = tid % G::kGroupThreads;
  typename M::cptr s = src + (b * c.src_bstride + y0 * c.src_ystride + static_cast<int64_t>(x0) * static_cast<int64_t>(sizeof(T)));
  uint8_t* tile = reinterpret_cast<uint8_t*>(lds) + wave * G::kWaveLdsBytes;
  const uint32_t n = snx * sny;
  const uint32_t step_y = G::kGroupThreads / snx, step_x = G::kGroupThreads - step_y * snx;
  uint32_t y = lane / snx, x = lane - y * snx;
  T e[kTransposeThin];
  uint32_t at[kTransposeThin];
#pragma unroll
  for (int k = 0; k < kTransposeThin; ++k) {
    if (lane + k * G::kGroupThreads < n) {
      e[k] = M::template loadu<T>(s + (y * c.src_ystride + static_cast<int64_t>(x) * static_cast<int64_t>(sizeof(T))));
      at[k] = transpose_lds_offset<sizeof(T)>(x, y);
    }
    x += step_x;
    y += step_y;
    if (x >= snx) {
      x -= snx;
      y += 1;
    }
  }
#pragma unroll
  for (int k = 0; k < kTransposeThin; ++k)
    if (lane + k * G::kGroupThreads < n) *reinterpret_cast<T*>(tile + at[k]) = e[k];
}

template <class M, typename T>
MMR_HD void transpose_store_element(const mmr_transpose_chunk& c, typename M::ptr dst, uint32_t b, const T* lds, uint32_t tid,
                                    uint32_t x0, uint32_t y0, uint32_t snx, uint32_t sny) {
  typedef TransposeTile<sizeof(T)> G;
  const uint32_t wave = tid / G::kGroupThreads, lane = tid % G::kGroupThreads;
  typename M::ptr d = dst + (b * c.dst_bstride + x0 * c.dst_xstride + static_cast<int64_t>(y0) * static_cast<int64_t>(sizeof(T)));
  const uint8_t* tile = reinterpret_cast<const uint8_t*>(lds) + wave * G::kWaveLdsBytes;
  const uint32_t n = snx * sny;
  const uint32_t step_x = G::kGroupThreads / sny, step_y = G::kGroupThreads - step_x * sny;
  uint32_t x = lane / sny, y = lane - x * sny;
#pragma unroll
  for (int k = 0; k < kTransposeThin; ++k) {
    if (lane + k * G::kGroupThreads < n)
      M::template storeu<T>(d + (x * c.dst_xstride + static_cast<int64_t>(y) * static_cast<int64_t>(sizeof(T))),
                            *reinterpret_cast<const T*>(tile + transpose_lds_offset<sizeof(T)>(x, y)));
    y += step_y;
    x += step_x;
    if (y >= sny) {
      y -= sny;
      x += 1;
    }
  }
}

// Thin path: a chunk whose tile is thinner than one vector one way (a small dimension moving into or out of the
// minor position).  Its batch entries together fill at most the workgroup's LDS (the planner sizes nb so), so the
// whole chunk moves in two phases around ONE workgroup barrier: every thread loads elements in source order
// (batch entry, y, x: consecutive lanes read consecutive source elements) and parks them in LDS in destination
// order (batch entry, x, y), then stores them in destination order (consecutive lanes write consecutive elements
// of a destination row, and of the next row where the rows abut).  kTransposeThinUnroll loads of a lane are in
// flight before its first LDS write; one division chain per phase, after that a lane's next element follows by a
// fixed step with carries.
constexpr int kTransposeThinUnroll = 8;

MMR_HD bool transpose_is_thin(const mmr_transpose_chunk& c) {
  const uint32_t vec = 16u / c.itemsize;
  return c.nx < vec || c.ny < vec;
}

template <class M, typename T>
MMR_HD void transpose_thin_load(const mmr_transpose_chunk& c, typename M::cptr src, T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  const uint32_t nx = c.nx, ny = c.ny, tile = nx * ny, n = c.nb * tile;
  const uint32_t step_x = G::kThreads % nx, rest = G::kThreads / nx, step_y = rest % ny, step_b = rest / ny;
  uint32_t bb = tid / tile, y = (tid - bb * tile) / nx, x = tid - bb * tile - y * nx;
  uint8_t* cells = reinterpret_cast<uint8_t*>(lds);
  for (uint32_t base = tid; base < n; base += G::kThreads * kTransposeThinUnroll) {
    T e[kTransposeThinUnroll];
    uint32_t at[kTransposeThinUnroll];
#pragma unroll
    for (int k = 0; k < kTransposeThinUnroll; ++k) {
      if (base + k * G::kThreads < n) {
        e[k] = M::template loadu<T>(src + (bb * c.src_bstride + y * c.src_ystride +
                                           static_cast<int64_t>(x) * static_cast<int64_t>(sizeof(T))));
        at[k] = ((bb * nx + x) * ny + y) * static_cast<uint32_t>(sizeof(T));
      }
      x += step_x;
      if (x >= nx) {
        x -= nx;
        y += 1;
      }
      y += step_y;
      if (y >= ny) {
        y -= ny;
        bb += 1;
      }
      bb += step_b;
    }
#pragma unroll
    for (int k = 0; k < kTransposeThinUnroll; ++k)
      if (base + k * G::kThreads < n) *reinterpret_cast<T*>(cells + at[k]) = e[k];
  }
}

template <class M, typename T>
MMR_HD void transpose_thin_store(const mmr_transpose_chunk& c, typename M::ptr dst, const T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  const uint32_t nx = c.nx, ny = c.ny, tile = nx * ny, n = c.nb * tile;
  const uint32_t step_y = G::kThreads % ny, rest = G::kThreads / ny, step_x = rest % nx, step_b = rest / nx;
  uint32_t bb = tid / tile, x = (tid - bb * tile) / ny, y = tid - bb * tile - x * ny;
  for (uint32_t i = tid; i < n; i += G::kThreads) {
    M::template storeu<T>(dst + (bb * c.dst_bstride + x * c.dst_xstride + static_cast<int64_t>(y) * static_cast<int64_t>(sizeof(T))),
                          lds[i]);
    y += step_y;
    if (y >= ny) {
      y -= ny;
      x += 1;
    }
    x += step_x;
    if (x >= nx) {
      x -= nx;
      bb += 1;
    }
    bb += step_b;
  }
}

// Phase 1 / phase 2 of batch entry b for thread tid, whatever its sub-tile needs; `wave` = tid / kGroupThreads.
// This is how the host emulation walks a chunk.  The kernel makes the same choice once per chunk and wave and then
// runs a batch loop of its own for the chosen path (see transpose_tiles in kernels.hip for why).
template <class M, typename T>
MMR_HD void transpose_load_any(const mmr_transpose_chunk& c, typename M::cptr src, uint32_t b, T* lds, uint32_t tid,
                               uint32_t wave) {
  uint32_t x0, y0, snx, sny;
  switch (transpose_mode<sizeof(T)>(c, wave, &x0, &y0, &snx, &sny)) {
    case kTransposeVector: transpose_load_vec<M, T>(c, src, b, lds, tid); break;
    case kTransposeGeneral: transpose_load_general<M, T>(c, src, b, lds, tid, x0, y0, snx, sny); break;
    case kTransposeElement: transpose_load_element<M, T>(c, src, b, lds, tid, x0, y0, snx, sny); break;
    default: break;
  }
}

template <class M, typename T>
MMR_HD void transpose_store_any(const mmr_transpose_chunk& c, typename M::ptr dst, uint32_t b, const T* lds, uint32_t tid,
                                uint32_t wave) {
  uint32_t x0, y0, snx, sny;
  switch (transpose_mode<sizeof(T)>(c, wave, &x0, &y0, &snx, &sny)) {
    case kTransposeVector: transpose_store_vec<M, T>(c, dst, b, lds, tid); break;
    case kTransposeGeneral: transpose_store_general<M, T>(c, dst, b, lds, tid, x0, y0, snx, sny); break;
    case kTransposeElement: transpose_store_element<M, T>(c, dst, b, lds, tid, x0, y0, snx, sny); break;
    default: break;
  }
}

}  // namespace mmr

#endif  // MMR_CSRC_CHUNK_OPS_H_
