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

// ---------------------------------------------------------------------------
// Aligned copy: every offset, stride and row width is a multiple of 16 bytes.
// Rows of wv = w/16 vectors.  No division in the loops: a thread fixes its
// column (and, for rows narrower than the workgroup, its sub-row) once, then
// steps through rows.  UNROLL loads are issued before the first store.
// ---------------------------------------------------------------------------
template <class M, int THREADS, int UNROLL>
MMR_HD void copy16_chunk(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  const bool fill = c.src_slot == MMR_SLOT_FILL;
  const uint32_t wv = c.w >> 4;
  const uint32_t rows = c.n1 * c.n2;
  if (wv >= THREADS) {
    // wide rows: the whole workgroup walks one row at a time
    for (uint32_t r2 = 0; r2 < c.n2; ++r2) {
      for (uint32_t r1 = 0; r1 < c.n1; ++r1) {
        typename M::cptr srow = src + (r2 * c.s2 + r1 * c.s1);
        typename M::ptr drow = dst + (r2 * c.d2 + r1 * c.d1);
        for (uint32_t c0 = tid; c0 < wv; c0 += THREADS * UNROLL) {
          V16 v[UNROLL];
#pragma unroll
          for (int u = 0; u < UNROLL; ++u) {
            const uint32_t col = c0 + u * THREADS;
            if (col < wv) v[u] = fill ? V16{0, 0, 0, 0} : M::load16(srow + (static_cast<int64_t>(col) << 4));
          }
#pragma unroll
          for (int u = 0; u < UNROLL; ++u) {
            const uint32_t col = c0 + u * THREADS;
            if (col < wv) M::store16(drow + (static_cast<int64_t>(col) << 4), v[u]);
          }
        }
      }
    }
    return;
  }
  // narrow rows: R = THREADS / wv rows per pass; thread = (sub-row, column), fixed
  const uint32_t R = THREADS / wv;
  const uint32_t sub = tid / wv;
  const uint32_t col = tid - sub * wv;
  if (sub >= R) return;
  const int64_t cb = static_cast<int64_t>(col) << 4;
  // (r2, r1) of this thread's first row and the per-pass step, so the loop needs no division
  uint32_t r2 = sub / c.n1, r1 = sub - r2 * c.n1;
  const uint32_t step2 = R / c.n1, step1 = R - step2 * c.n1;
  for (uint32_t row0 = sub; row0 < rows; row0 += R * UNROLL) {
    V16 v[UNROLL];
    int64_t doff[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (row0 + u * R < rows) {
        doff[u] = r2 * c.d2 + r1 * c.d1 + cb;
        v[u] = fill ? V16{0, 0, 0, 0} : M::load16(src + (r2 * c.s2 + r1 * c.s1 + cb));
      }
      r1 += step1;
      r2 += step2;
      if (r1 >= c.n1) {
        r1 -= c.n1;
        r2 += 1;
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      if (row0 + u * R < rows) M::store16(dst + doff[u], v[u]);
    }
  }
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
// and no access ever leaves its row.  Rows
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

// One (row, slot) of a generic chunk: phase 1 (all loads).  WIDE: rows of at least 16 bytes.
template <class M, bool WIDE>
MMR_HD void generic_load(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, bool fill, uint32_t row,
                         uint32_t slot, V16* v, typename M::ptr* dpos, int32_t* len) {
  typename M::ptr drow = dst + row * c.d1;
  typename M::cptr srow = src + row * c.s1;
  const int32_t w = static_cast<int32_t>(c.w);
  const int32_t mis = static_cast<int32_t>((fill ? M::addr(drow) : M::caddr(srow)) & 15u);
  const int32_t rel = static_cast<int32_t>(slot << 4) - mis;  // row-relative byte where this aligned slot starts
  if constexpr (WIDE) {
    if (rel >= w) {
      *len = 0;
      return;
    }
    const int32_t lo = rel < 0 ? 0 : (rel + 16 > w ? w - 16 : rel);
    *len = 16;
    *dpos = drow + lo;
    *v = fill ? V16{0, 0, 0, 0} : M::load16u(srow + lo);
  } else {
    const int32_t lo = rel < 0 ? 0 : rel;
    const int32_t hi = rel + 16 < w ? rel + 16 : w;
    *len = hi - lo;
    *dpos = drow + lo;
    if (*len > 0) *v = fill ? V16{0, 0, 0, 0} : load_ragged<M>(srow + lo, static_cast<uint32_t>(*len));
  }
}

template <class M, bool WIDE>
MMR_HD void generic_store(typename M::ptr dpos, int32_t len, V16 v) {
  if constexpr (WIDE) {
    if (len != 0) M::template storeu<V16>(dpos, v);
  } else {
    if (len > 0) store_ragged<M>(dpos, static_cast<uint32_t>(len), v);
  }
}

template <class M, int THREADS, int UNROLL, bool WIDE>
MMR_HD void generic_rows(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  const bool fill = c.src_slot == MMR_SLOT_FILL;
  const uint32_t slots = ((c.w + 15u) >> 4) + 1u;  // a row of w bytes touches at most this many aligned slots
  const uint32_t rows = c.n1;
  if (slots >= THREADS) {
    for (uint32_t row = 0; row < rows; ++row) {
      for (uint32_t s0 = tid; s0 < slots; s0 += THREADS * UNROLL) {
        V16 v[UNROLL];
        typename M::ptr dpos[UNROLL];
        int32_t len[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          len[u] = 0;
          const uint32_t slot = s0 + u * THREADS;
          if (slot < slots) generic_load<M, WIDE>(c, src, dst, fill, row, slot, &v[u], &dpos[u], &len[u]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) generic_store<M, WIDE>(dpos[u], len[u], v[u]);
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
  for (uint32_t i0 = tid; i0 < total; i0 += THREADS * UNROLL) {
    V16 v[UNROLL];
    typename M::ptr dpos[UNROLL];
    int32_t len[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      len[u] = 0;
      if (i0 + u * THREADS < total) generic_load<M, WIDE>(c, src, dst, fill, row, slot, &v[u], &dpos[u], &len[u]);
      row += step_rows;
      slot += step_slots;
      if (slot >= slots) {
        slot -= slots;
        row += 1;
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) generic_store<M, WIDE>(dpos[u], len[u], v[u]);
  }
}

template <class M, int THREADS, int UNROLL>
MMR_HD void generic_chunk(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  if (c.w >= 16) generic_rows<M, THREADS, UNROLL, true>(c, src, dst, tid);  // uniform over the workgroup
  else generic_rows<M, THREADS, UNROLL, false>(c, src, dst, tid);
}

// ---------------------------------------------------------------------------
// Tile transpose: x is contiguous in the source, y in the destination.
//
// A workgroup owns a tile of kTileX x kTileY elements, its waves one
// kEX x kEY sub-tile each (kWX x kWY waves; for 1-byte elements all four waves
// share one sub-tile).
//
// Vector path (tile 16-byte aligned on both sides, extents multiples of the
// vector width): every wave works alone, on its own slice of LDS, so the only
// synchronisation is between the lanes of a wave (the caller puts a wave-level
// fence between the two phases; a workgroup barrier where waves share a
// sub-tile).  Every global
// access is a 16-byte vector and every LDS access at least a dword.  A lane
// loads the same vector of kPack = 4 / itemsize adjacent source rows (one row
// for elements of 4 bytes and more), so for each of the vector's x it holds
// kPack consecutive y: one dword (or one element of 8 / 16 bytes), written to
// row x of an LDS tile laid out [x][y] without padding.  In the second phase a
// lane reads one 16-byte group of an LDS row = consecutive y of one x and
// stores it to destination row x.  All global loads of a lane are issued before
// its first LDS write.
//
// LDS banks: rows are a multiple of 128 bytes apart, so the 16-byte groups of a
// row are permuted by XOR with a function of x whose low three bits differ
// between the 8 lanes that write the same y of 8 neighbouring vectors (and
// between any 8 consecutive x): the dword writes of 32 lanes then fall into 32
// different banks.  Reads are conflict-free by construction (8 consecutive
// lanes read the 8 groups of one 128-byte row segment).
//
// Element path (anything else, e.g. ragged edge tiles): the whole workgroup
// walks the sub-tiles one after the other, one element per lane, LDS laid out
// [y][x] with pitch kEX + 1; the caller puts a workgroup barrier after each
// phase.
// ---------------------------------------------------------------------------
template <int ITEM>
struct TransposeTile {
  // wave sub-tile: 128 bytes (or more) wide on both sides, so every access of 8 lanes is a full 128-byte line
  static constexpr int kEX = ITEM == 1 ? 128 : (ITEM == 2 ? 64 : 32);
  static constexpr int kEY = ITEM == 1 ? 128 : (ITEM == 16 ? 16 : (ITEM == 8 ? 32 : 64));
  // Sub-tiles per workgroup tile, and the threads that share one.  1-byte elements: the smallest sub-tile is
  // already 16 KiB, too many registers for one wave, so the four waves of the workgroup share a single sub-tile
  // (and synchronise with a workgroup barrier instead of a wave fence).
  static constexpr int kWX = ITEM == 1 ? 1 : 2, kWY = kWX;
  static constexpr int kWaves = kWX * kWY;                   // number of sub-tiles
  static constexpr int kGroupThreads = ITEM == 1 ? 256 : 64; // threads per sub-tile
  static constexpr int kThreads = kGroupThreads * kWaves;
  static constexpr int kTileX = kEX * kWX, kTileY = kEY * kWY;
  static constexpr int kVec = 16 / ITEM;                     // elements per 16-byte vector
  static constexpr int kPack = ITEM >= 4 ? 1 : 4 / ITEM;     // source rows a lane packs into one LDS word
  static constexpr int kRowBytes = kEY * ITEM;               // vector path: bytes per LDS row (no padding)
  static constexpr int kSrcVecs = kEX / kVec;                // 16-byte groups per source row of a sub-tile
  static constexpr int kDstVecs = kEY / kVec;                // 16-byte groups per destination row of a sub-tile
  static constexpr int kRowPacks = kEY / kPack;              // packed source-row groups per sub-tile
  static constexpr int kWaveLdsBytes = kEX * kEY * ITEM;     // vector path: one wave's slice
  static constexpr int kPitch1 = kEX + 1;                    // element path, elements
  static constexpr int kLdsBytes =
      kWaveLdsBytes * kWaves > kEY * kPitch1 * ITEM ? kWaveLdsBytes * kWaves : kEY * kPitch1 * ITEM;
  static_assert(kSrcVecs % 8 == 0 && kDstVecs % 8 == 0, "sub-tile rows must be whole 128-byte lines");
  static_assert(kSrcVecs * kRowPacks % kGroupThreads == 0 && kEX * kDstVecs % kGroupThreads == 0,
                "sub-tile must divide over its threads");
};
constexpr int kTransposeLdsBytes = 32 * 1024 + 1024;  // at least the largest TransposeTile<>::kLdsBytes

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

MMR_HD bool transpose_is_vector(const mmr_transpose_chunk& c) {
  const uint32_t vec = 16u / c.itemsize;
  const uint64_t bits = c.src_off | c.dst_off | static_cast<uint64_t>(c.src_ystride) | static_cast<uint64_t>(c.dst_xstride) |
                        static_cast<uint64_t>(c.src_bstride) | static_cast<uint64_t>(c.dst_bstride);
  return (bits & 15u) == 0 && c.nx % vec == 0 && c.ny % vec == 0;
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

// Task t of a wave's phase -> (row index, 16-byte group within the row).  8
// consecutive lanes take the 8 groups of one 128-byte row segment, the next 8
// lanes the same segment of the next row; rows wider than 128 bytes are covered
// segment after segment.  `rows` is the number of rows in the phase.
MMR_HD void transpose_task(uint32_t t, uint32_t rows, uint32_t* row, uint32_t* group) {
  const uint32_t r = t >> 3;
  *group = (t & 7u) + ((r / rows) << 3);
  *row = r % rows;
}

// Origin of the sub-tile of wave `wave` inside the workgroup tile, in elements.
template <int ITEM>
MMR_HD void transpose_subtile(uint32_t wave, uint32_t* x0, uint32_t* y0) {
  typedef TransposeTile<ITEM> G;
  *x0 = (wave % G::kWX) * G::kEX;
  *y0 = (wave / G::kWX) * G::kEY;
}

// Vector path, phase 1: global -> registers -> this wave's LDS slice.  tid = thread of the workgroup.
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
    transpose_task(lane + k * G::kGroupThreads, G::kRowPacks, &yg, &xv);
    if (y0 + yg * G::kPack < c.ny && x0 + xv * G::kVec < c.nx) {
#pragma unroll
      for (int p = 0; p < G::kPack; ++p)
        v[k][p] = M::load16(s + ((yg * G::kPack + p) * c.src_ystride + static_cast<int64_t>(xv) * 16));
    }
  }
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t yg, xv;
    transpose_task(lane + k * G::kGroupThreads, G::kRowPacks, &yg, &xv);
    if (y0 + yg * G::kPack < c.ny && x0 + xv * G::kVec < c.nx) {
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
    transpose_task(lane + k * G::kGroupThreads, G::kEX, &x, &yv);
    if (x0 + x < c.nx && y0 + yv * G::kVec < c.ny)
      v[k] = *reinterpret_cast<const V16*>(tile + x * G::kRowBytes + ((yv ^ transpose_swizzle<sizeof(T)>(x)) << 4));
  }
#pragma unroll
  for (int k = 0; k < kTasks; ++k) {
    uint32_t x, yv;
    transpose_task(lane + k * G::kGroupThreads, G::kEX, &x, &yv);
    if (x0 + x < c.nx && y0 + yv * G::kVec < c.ny) M::store16(d + (x * c.dst_xstride + static_cast<int64_t>(yv) * 16), v[k]);
  }
}

// Element path: sub-tile `sub` of the workgroup tile, all threads of the workgroup.
template <class M, typename T>
MMR_HD void transpose_load(const mmr_transpose_chunk& c, typename M::cptr src, uint32_t b, uint32_t sub, T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  uint32_t x0, y0;
  transpose_subtile<sizeof(T)>(sub, &x0, &y0);
  if (x0 >= c.nx || y0 >= c.ny) return;
  const uint32_t nx = c.nx - x0 < G::kEX ? c.nx - x0 : G::kEX, ny = c.ny - y0 < G::kEY ? c.ny - y0 : G::kEY;
  typename M::cptr s = src + (b * c.src_bstride + y0 * c.src_ystride + static_cast<int64_t>(x0) * static_cast<int64_t>(sizeof(T)));
  const uint32_t n = nx * ny;
  for (uint32_t i = tid; i < n; i += G::kThreads) {
    const uint32_t y = i / nx, x = i - y * nx;
    lds[y * G::kPitch1 + x] =
        M::template loadu<T>(s + (y * c.src_ystride + static_cast<int64_t>(x) * static_cast<int64_t>(sizeof(T))));
  }
}

template <class M, typename T>
MMR_HD void transpose_store(const mmr_transpose_chunk& c, typename M::ptr dst, uint32_t b, uint32_t sub, const T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  uint32_t x0, y0;
  transpose_subtile<sizeof(T)>(sub, &x0, &y0);
  if (x0 >= c.nx || y0 >= c.ny) return;
  const uint32_t nx = c.nx - x0 < G::kEX ? c.nx - x0 : G::kEX, ny = c.ny - y0 < G::kEY ? c.ny - y0 : G::kEY;
  typename M::ptr d = dst + (b * c.dst_bstride + x0 * c.dst_xstride + static_cast<int64_t>(y0) * static_cast<int64_t>(sizeof(T)));
  const uint32_t n = nx * ny;
  for (uint32_t i = tid; i < n; i += G::kThreads) {
    const uint32_t x = i / ny, y = i - x * ny;
    M::template storeu<T>(d + (x * c.dst_xstride + static_cast<int64_t>(y) * static_cast<int64_t>(sizeof(T))),
                          lds[y * G::kPitch1 + x]);
  }
}

}  // namespace mmr

#endif  // MMR_CSRC_CHUNK_OPS_H_
