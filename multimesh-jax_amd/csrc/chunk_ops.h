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
//   static uintptr_t addr(ptr);                   numeric address (for alignment math)
#ifndef MMR_CSRC_CHUNK_OPS_H_
#define MMR_CSRC_CHUNK_OPS_H_

#include <cstdint>

#include "mmreshard.h"

#if defined(__HIPCC__) || defined(__CUDACC__)
#define MMR_HD __host__ __device__ __forceinline__
#else
#define MMR_HD inline
#endif

namespace mmr {

struct V16 {
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
// 16-byte boundaries of its DESTINATION: a lane owns one aligned 16-byte slot,
// loads the matching source bytes with one unaligned 16-byte load and writes
// one aligned 16-byte store.  The at most two ragged slots at the ends of a row
// hold 1..15 bytes, moved as 8/4/2/1-byte pieces (binary decomposition of the
// length).  The pieces travel in one V16: .x/.y the 8-byte piece, .z the 4-byte
// piece, .w the 2-byte piece (low half) and the 1-byte piece (bits 16-23).
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

// One (row, slot) of a generic chunk: phase 1 (all loads).
template <class M>
MMR_HD void generic_load(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, bool fill, uint32_t row,
                         uint32_t slot, V16* v, typename M::ptr* dpos, int32_t* len) {
  typename M::ptr drow = dst + row * c.d1;
  typename M::cptr srow = src + row * c.s1;
  const int32_t w = static_cast<int32_t>(c.w);
  const int32_t mis = static_cast<int32_t>(M::addr(drow) & 15u);
  const int32_t rel = static_cast<int32_t>(slot << 4) - mis;  // row-relative byte where this aligned slot starts
  const int32_t lo = rel < 0 ? 0 : rel;
  const int32_t hi = rel + 16 < w ? rel + 16 : w;
  *len = hi - lo;
  *dpos = drow + lo;
  if (*len == 16) {
    *v = fill ? V16{0, 0, 0, 0} : M::load16u(srow + lo);
  } else if (*len > 0) {
    *v = fill ? V16{0, 0, 0, 0} : load_ragged<M>(srow + lo, static_cast<uint32_t>(*len));
  }
}

template <class M>
MMR_HD void generic_store(typename M::ptr dpos, int32_t len, V16 v) {
  if (len == 16) {
    M::store16(dpos, v);
  } else if (len > 0) {
    store_ragged<M>(dpos, static_cast<uint32_t>(len), v);
  }
}

template <class M, int THREADS, int UNROLL>
MMR_HD void generic_chunk(const mmr_copy_chunk& c, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
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
          if (slot < slots) generic_load<M>(c, src, dst, fill, row, slot, &v[u], &dpos[u], &len[u]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) generic_store<M>(dpos[u], len[u], v[u]);
      }
    }
    return;
  }
  const uint32_t R = THREADS / slots;
  const uint32_t sub = tid / slots;
  const uint32_t slot = tid - sub * slots;
  if (sub >= R) return;
  for (uint32_t row0 = sub; row0 < rows; row0 += R * UNROLL) {
    V16 v[UNROLL];
    typename M::ptr dpos[UNROLL];
    int32_t len[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      len[u] = 0;
      const uint32_t row = row0 + u * R;
      if (row < rows) generic_load<M>(c, src, dst, fill, row, slot, &v[u], &dpos[u], &len[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) generic_store<M>(dpos[u], len[u], v[u]);
  }
}

// ---------------------------------------------------------------------------
// Tile transpose: x is contiguous in the source, y in the destination.  The
// caller puts a workgroup barrier between the load and the store phase and
// after the store phase.  Tile edge in elements: 128 for 1-byte, 64 for 2/4/8-
// byte, 32 for 16-byte elements.
//
// Vector path (tile 16-byte aligned on both sides, extents multiples of the
// vector width): every global access is a 16-byte vector.  A lane loads one
// vector of a source row, scatters its elements into LDS laid out [x][y] (row
// pitch EDGE + elements-per-vector, so rows stay 16-byte aligned), and after the
// barrier reads one 16-byte vector of an LDS row = consecutive y of one x and
// stores it to the destination row x.  All loads of a thread are issued before
// its first LDS write.
//
// Element path (anything else, e.g. ragged edge tiles): one element per lane,
// LDS laid out [y][x] with pitch EDGE + 1.
// ---------------------------------------------------------------------------
template <int ITEM>
struct TransposeTile {
  static constexpr int kEdge = ITEM == 1 ? 128 : (ITEM == 16 ? 32 : 64);
  static constexpr int kVec = 16 / ITEM;           // elements per 16-byte vector
  static constexpr int kPitch = kEdge + kVec;      // vector path, elements
  static constexpr int kPitch1 = kEdge + 1;        // element path, elements
  static constexpr int kLdsBytes = kEdge * kPitch * ITEM;
};
constexpr int kTransposeLdsBytes = 64 * 66 * 8;  // the largest of TransposeTile<>::kLdsBytes (8-byte elements)

MMR_HD bool transpose_is_vector(const mmr_transpose_chunk& c) {
  const uint32_t vec = 16u / c.itemsize;
  const uint64_t bits = c.src_off | c.dst_off | static_cast<uint64_t>(c.src_ystride) | static_cast<uint64_t>(c.dst_xstride) |
                        static_cast<uint64_t>(c.src_bstride) | static_cast<uint64_t>(c.dst_bstride);
  return (bits & 15u) == 0 && c.nx % vec == 0 && c.ny % vec == 0;
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

template <class M, typename T, int THREADS>
MMR_HD void transpose_load_vec(const mmr_transpose_chunk& c, typename M::cptr src, uint32_t b, T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  constexpr int kRowVecs = G::kEdge / G::kVec;                // vectors per full source row of the tile
  constexpr int kPerThread = G::kEdge * kRowVecs / THREADS;   // vectors per thread
  typename M::cptr s = src + b * c.src_bstride;
  V16 v[kPerThread];
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const uint32_t vi = tid + k * THREADS;
    const uint32_t y = vi / kRowVecs, xv = vi % kRowVecs;
    if (y < c.ny && xv * G::kVec < c.nx) v[k] = M::load16(s + (y * c.src_ystride + static_cast<int64_t>(xv) * 16));
  }
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const uint32_t vi = tid + k * THREADS;
    const uint32_t y = vi / kRowVecs, xv = vi % kRowVecs;
    if (y < c.ny && xv * G::kVec < c.nx) {
#pragma unroll
      for (int i = 0; i < G::kVec; ++i) lds[(xv * G::kVec + i) * G::kPitch + y] = element_of<T>(v[k], i);
    }
  }
}

template <class M, typename T, int THREADS>
MMR_HD void transpose_store_vec(const mmr_transpose_chunk& c, typename M::ptr dst, uint32_t b, const T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  constexpr int kRowVecs = G::kEdge / G::kVec;  // vectors per full destination row of the tile
  constexpr int kPerThread = G::kEdge * kRowVecs / THREADS;
  typename M::ptr d = dst + b * c.dst_bstride;
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    const uint32_t vi = tid + k * THREADS;
    const uint32_t x = vi / kRowVecs, yv = vi % kRowVecs;
    if (x < c.nx && yv * G::kVec < c.ny) {
      const V16 v = *reinterpret_cast<const V16*>(&lds[x * G::kPitch + yv * G::kVec]);  // 16-byte aligned by construction
      M::store16(d + (x * c.dst_xstride + static_cast<int64_t>(yv) * 16), v);
    }
  }
}

template <class M, typename T, int THREADS>
MMR_HD void transpose_load(const mmr_transpose_chunk& c, typename M::cptr src, uint32_t b, T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  typename M::cptr s = src + b * c.src_bstride;
  const uint32_t n = c.nx * c.ny;
  for (uint32_t i = tid; i < n; i += THREADS) {
    const uint32_t y = i / c.nx, x = i - y * c.nx;
    lds[y * G::kPitch1 + x] =
        M::template loadu<T>(s + (y * c.src_ystride + static_cast<int64_t>(x) * static_cast<int64_t>(sizeof(T))));
  }
}

template <class M, typename T, int THREADS>
MMR_HD void transpose_store(const mmr_transpose_chunk& c, typename M::ptr dst, uint32_t b, const T* lds, uint32_t tid) {
  typedef TransposeTile<sizeof(T)> G;
  typename M::ptr d = dst + b * c.dst_bstride;
  const uint32_t n = c.nx * c.ny;
  for (uint32_t i = tid; i < n; i += THREADS) {
    const uint32_t x = i / c.ny, y = i - x * c.ny;
    M::template storeu<T>(d + (x * c.dst_xstride + static_cast<int64_t>(y) * static_cast<int64_t>(sizeof(T))),
                          lds[y * G::kPitch1 + x]);
  }
}

}  // namespace mmr

#endif  // MMR_CSRC_CHUNK_OPS_H_
