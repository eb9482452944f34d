// gfx950 (CDNA4) data-movement kernels of the reshard path.
//
// Pure byte movement: nothing is ever typed as a float, so NaN payloads, FP8
// and integer data all come through bit-exact.  Every kernel is bound by HBM
// bandwidth; there is no MFMA work on this path.
//
// Work distribution: one workgroup per chunk of the plan's table.  The chunk
// record and the two base pointers are wave-uniform and come in through scalar
// loads; lanes then move 16 bytes each, consecutive lanes covering consecutive
// 16-byte vectors of a row so every wavefront touches whole 128-byte lines.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdlib>

#include "kernels.h"

namespace mmr {
namespace {

constexpr int kXcds = 8;  // MI355X: 256 CUs in 8 XCDs, each with its own L2

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Shard buffers are always device (global) memory.  Pointers read from the
// pointer table would otherwise be generic and compile to flat_* accesses;
// address space 1 makes every access a global_* instruction.
#define MMR_GLOBAL __attribute__((address_space(1)))
typedef MMR_GLOBAL char gchar;
typedef MMR_GLOBAL const char gcchar;

struct alignas(16) u128 {
  uint64_t lo, hi;
};

// Streaming accesses: every byte is touched exactly once, so keep it out of
// the way of the caches' replacement policy (nontemporal).  ALIGN is what the
// caller promises about the address; gfx950 under the HSA runtime runs with
// unaligned global access enabled, so ALIGN = 1 still compiles to one access.
template <typename T, int ALIGN = alignof(T)>
__device__ __forceinline__ T stream_load(gcchar* p) {
  typedef MMR_GLOBAL const T __attribute__((aligned(ALIGN))) gt;
  return __builtin_nontemporal_load(reinterpret_cast<gt*>(p));
}
template <typename T, int ALIGN = alignof(T)>
__device__ __forceinline__ void stream_store(gchar* p, T v) {
  typedef MMR_GLOBAL T __attribute__((aligned(ALIGN))) gt;
  __builtin_nontemporal_store(v, reinterpret_cast<gt*>(p));
}
template <>
__device__ __forceinline__ u128 stream_load<u128, 16>(gcchar* p) {
  u32x4 v = stream_load<u32x4>(p);
  u128 r;
  r.lo = static_cast<uint64_t>(v.x) | (static_cast<uint64_t>(v.y) << 32);
  r.hi = static_cast<uint64_t>(v.z) | (static_cast<uint64_t>(v.w) << 32);
  return r;
}
template <>
__device__ __forceinline__ void stream_store<u128, 16>(gchar* p, u128 r) {
  u32x4 v;
  v.x = static_cast<uint32_t>(r.lo);
  v.y = static_cast<uint32_t>(r.lo >> 32);
  v.z = static_cast<uint32_t>(r.hi);
  v.w = static_cast<uint32_t>(r.hi >> 32);
  stream_store<u32x4>(p, v);
}

// Plain (cacheable) accesses for rows whose ragged ends share cache lines with
// a neighbouring row or chunk: the L2 can then merge the pieces of a line.
template <typename T, int ALIGN = alignof(T)>
__device__ __forceinline__ T cached_load(gcchar* p) {
  typedef MMR_GLOBAL const T __attribute__((aligned(ALIGN))) gt;
  return *reinterpret_cast<gt*>(p);
}
template <typename T, int ALIGN = alignof(T)>
__device__ __forceinline__ void cached_store(gchar* p, T v) {
  typedef MMR_GLOBAL T __attribute__((aligned(ALIGN))) gt;
  *reinterpret_cast<gt*>(p) = v;
}
template <typename T, int ALIGN, bool NT>
__device__ __forceinline__ T ld(gcchar* p) {
  if constexpr (NT) return stream_load<T, ALIGN>(p);
  else return cached_load<T, ALIGN>(p);
}
template <typename T, int ALIGN, bool NT>
__device__ __forceinline__ void st(gchar* p, T v) {
  if constexpr (NT) stream_store<T, ALIGN>(p, v);
  else cached_store<T, ALIGN>(p, v);
}

__device__ __forceinline__ gchar* slot_base(void* const* __restrict__ ptrs, uint32_t slot, uint64_t off) {
  return (gchar*)(static_cast<char*>(ptrs[slot])) + off;
}

// Table index of this workgroup.  The hardware deals consecutive workgroups
// round-robin over the XCDs; with xcd_split each XCD instead walks a contiguous
// eighth of the table, so chunks that are neighbours in the (address-sorted)
// table, and may share cache lines at their edges, meet in the same L2.
__device__ __forceinline__ bool chunk_index(uint32_t n, bool xcd_split, uint32_t* index) {
  uint32_t b = blockIdx.x;
  if (xcd_split) {
    const uint32_t per = (n + kXcds - 1) / kXcds;
    b = (b % kXcds) * per + b / kXcds;
  }
  *index = b;
  return b < n;
}

uint32_t grid_size(int64_t n, bool xcd_split) {
  return xcd_split ? static_cast<uint32_t>((n + kXcds - 1) / kXcds * kXcds) : static_cast<uint32_t>(n);
}

// ---------------------------------------------------------------------------
// Aligned copy: every offset, stride and row width is a multiple of 16 bytes.
// Moves (or zero-fills) the n2 x n1 x (w / 16) vectors of one chunk.  UNROLL
// loads are issued before the first store so each lane keeps several requests
// in flight.
// ---------------------------------------------------------------------------
template <int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void mmr_copy16_kernel(const mmr_copy_chunk* __restrict__ chunks, uint32_t n,
                                                             void* const* __restrict__ ptrs, bool xcd_split) {
  uint32_t ci;
  if (!chunk_index(n, xcd_split, &ci)) return;
  const mmr_copy_chunk c = chunks[ci];
  gchar* __restrict__ dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  const bool fill = c.src_slot == MMR_SLOT_FILL;
  gcchar* __restrict__ src = fill ? dst : slot_base(ptrs, c.src_slot, c.src_off);  // never read when filling
  const uint32_t wv = c.w >> 4;
  const uint32_t total = wv * c.n1 * c.n2;
  for (uint32_t base = threadIdx.x; base < total; base += THREADS * UNROLL) {
    u32x4 v[UNROLL];
    int64_t doff[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
      const uint32_t idx = base + k * THREADS;
      if (idx < total) {
        const uint32_t row = idx / wv;
        const uint32_t col = idx - row * wv;
        const uint32_t r2 = row / c.n1;
        const uint32_t r1 = row - r2 * c.n1;
        const int64_t cb = static_cast<int64_t>(col) << 4;
        doff[k] = r2 * c.d2 + r1 * c.d1 + cb;
        v[k] = fill ? u32x4{0, 0, 0, 0} : stream_load<u32x4>(src + (r2 * c.s2 + r1 * c.s1 + cb));
      }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
      const uint32_t idx = base + k * THREADS;
      if (idx < total) stream_store<u32x4>(dst + doff[k], v[k]);
    }
  }
}

// ---------------------------------------------------------------------------
// Generic copy: rows of any width at any byte alignment on either side
// (non-divisible shardings of 1- and 4-byte types).  Each row is cut at the
// 16-byte boundaries of its DESTINATION: a lane owns one aligned 16-byte slot,
// loads the matching source bytes with one unaligned 16-byte load and writes
// one aligned 16-byte store.  The at most two ragged slots at the ends of a
// row are moved as 8/4/2/1-byte pieces.
// ---------------------------------------------------------------------------
// A ragged slot holds 1..15 bytes: moved as 8/4/2/1-byte pieces (binary
// decomposition of the length), every piece independent of the others.  The
// pieces travel in the lanes of one u32x4: .xy the 8-byte piece, .z the 4-byte
// piece, .w the 2-byte piece (low half) and the 1-byte piece (bits 16-23).
template <bool NT>
__device__ __forceinline__ u32x4 load_ragged(gcchar* __restrict__ s, uint32_t len) {
  u32x4 v = {0, 0, 0, 0};
  const uint32_t o4 = len & 8, o2 = o4 + (len & 4), o1 = o2 + (len & 2);
  if (len & 8) {
    const uint64_t a = ld<uint64_t, 1, NT>(s);
    v.x = static_cast<uint32_t>(a);
    v.y = static_cast<uint32_t>(a >> 32);
  }
  if (len & 4) v.z = ld<uint32_t, 1, NT>(s + o4);
  if (len & 2) v.w = ld<uint16_t, 1, NT>(s + o2);
  if (len & 1) v.w |= static_cast<uint32_t>(ld<uint8_t, 1, NT>(s + o1)) << 16;
  return v;
}
template <bool NT>
__device__ __forceinline__ void store_ragged(gchar* __restrict__ d, uint32_t len, u32x4 v) {
  const uint32_t o4 = len & 8, o2 = o4 + (len & 4), o1 = o2 + (len & 2);
  if (len & 8) st<uint64_t, 1, NT>(d, static_cast<uint64_t>(v.x) | (static_cast<uint64_t>(v.y) << 32));
  if (len & 4) st<uint32_t, 1, NT>(d + o4, v.z);
  if (len & 2) st<uint16_t, 1, NT>(d + o2, static_cast<uint16_t>(v.w));
  if (len & 1) st<uint8_t, 1, NT>(d + o1, static_cast<uint8_t>(v.w >> 16));
}

template <int THREADS, int UNROLL, bool NTL, bool NTS>
__global__ __launch_bounds__(THREADS) void mmr_copy_generic_kernel(const mmr_copy_chunk* __restrict__ chunks, uint32_t n,
                                                                   void* const* __restrict__ ptrs, bool xcd_split) {
  uint32_t ci;
  if (!chunk_index(n, xcd_split, &ci)) return;
  const mmr_copy_chunk c = chunks[ci];
  gchar* __restrict__ dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  const bool fill = c.src_slot == MMR_SLOT_FILL;
  gcchar* __restrict__ src = fill ? dst : slot_base(ptrs, c.src_slot, c.src_off);  // never read when filling
  const int32_t w = static_cast<int32_t>(c.w);
  const uint32_t slots = ((c.w + 15u) >> 4) + 1u;  // a row of w bytes touches at most this many aligned slots
  const uint32_t total = slots * c.n1 * c.n2;
  for (uint32_t base = threadIdx.x; base < total; base += THREADS * UNROLL) {
    u32x4 v[UNROLL];
    gchar* dpos[UNROLL];   // first destination byte this lane writes
    int32_t len[UNROLL];   // bytes this lane moves: 16 (aligned slot), 1..15 (ragged end), <= 0 (nothing)
    // phase 1: every load of the iteration, ragged pieces included, before any store
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
      const uint32_t idx = base + k * THREADS;
      len[k] = 0;
      if (idx < total) {
        const uint32_t row = idx / slots;
        const uint32_t slot = idx - row * slots;
        const uint32_t r2 = row / c.n1;
        const uint32_t r1 = row - r2 * c.n1;
        gchar* drow = dst + (r2 * c.d2 + r1 * c.d1);
        gcchar* srow = src + (r2 * c.s2 + r1 * c.s1);
        const int32_t mis = static_cast<int32_t>(reinterpret_cast<uintptr_t>(drow) & 15u);
        const int32_t rel = static_cast<int32_t>(slot << 4) - mis;  // row-relative byte where this aligned slot starts
        const int32_t lo = rel < 0 ? 0 : rel;
        const int32_t hi = rel + 16 < w ? rel + 16 : w;
        len[k] = hi - lo;
        dpos[k] = drow + lo;
        if (len[k] == 16) {
          v[k] = fill ? u32x4{0, 0, 0, 0} : ld<u32x4, 1, NTL>(srow + lo);
        } else if (len[k] > 0) {
          v[k] = fill ? u32x4{0, 0, 0, 0} : load_ragged<NTL>(srow + lo, static_cast<uint32_t>(len[k]));
        }
      }
    }
    // phase 2: stores
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
      if (len[k] == 16) {
        st<u32x4, 16, NTS>(dpos[k], v[k]);
      } else if (len[k] > 0) {
        store_ragged<NTS>(dpos[k], static_cast<uint32_t>(len[k]), v[k]);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Tile transpose through LDS, for source/destination pairs that disagree on the
// minor-most dim.  One batch of tiles per workgroup: x is contiguous in the
// source, y in the destination.  Rows of the tile are read along x, parked in
// LDS (row pitch TILE + 1 elements to spread the column reads over the banks),
// and written along y.
// ---------------------------------------------------------------------------
constexpr int kTransposeThreads = 256;

template <typename T, int TILE>
__device__ __forceinline__ void transpose_tiles(const mmr_transpose_chunk& c, gcchar* __restrict__ src,
                                                gchar* __restrict__ dst, void* lds_raw) {
  T(*tile)[TILE + 1] = reinterpret_cast<T(*)[TILE + 1]>(lds_raw);
  const uint32_t n = c.nx * c.ny;
  for (uint32_t b = 0; b < c.nb; ++b) {
    gcchar* s = src + b * c.src_bstride;
    gchar* d = dst + b * c.dst_bstride;
    for (uint32_t i = threadIdx.x; i < n; i += kTransposeThreads) {
      const uint32_t y = i / c.nx, x = i - y * c.nx;
      tile[y][x] = stream_load<T>(s + y * c.src_ystride + static_cast<int64_t>(x) * sizeof(T));
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < n; i += kTransposeThreads) {
      const uint32_t x = i / c.ny, y = i - x * c.ny;
      stream_store<T>(d + x * c.dst_xstride + static_cast<int64_t>(y) * sizeof(T), tile[y][x]);
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(kTransposeThreads) void mmr_transpose_kernel(const mmr_transpose_chunk* __restrict__ chunks,
                                                                          uint32_t n, void* const* __restrict__ ptrs,
                                                                          bool xcd_split) {
  // 64 x 65 eight-byte elements is the largest tile (33,280 bytes); sixteen-byte
  // elements use 32 x 33 tiles (16,896 bytes).
  __shared__ alignas(16) uint64_t lds[64 * 65];
  uint32_t ci;
  if (!chunk_index(n, xcd_split, &ci)) return;  // uniform over the workgroup: no barrier is skipped by part of it
  const mmr_transpose_chunk c = chunks[ci];
  gcchar* src = slot_base(ptrs, c.src_slot, c.src_off);
  gchar* dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  switch (c.itemsize) {  // wave-uniform
    case 1: transpose_tiles<uint8_t, 64>(c, src, dst, lds); break;
    case 2: transpose_tiles<uint16_t, 64>(c, src, dst, lds); break;
    case 4: transpose_tiles<uint32_t, 64>(c, src, dst, lds); break;
    case 8: transpose_tiles<uint64_t, 64>(c, src, dst, lds); break;
    default: transpose_tiles<u128, 32>(c, src, dst, lds); break;
  }
}

hipError_t check_grid(int64_t n) { return (n < 0 || n > 0x7ffffff0LL) ? hipErrorInvalidValue : hipSuccess; }

}  // namespace

hipError_t launch_copy16(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, bool xcd_split,
                         hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  static const int variant = getenv("MMR_COPY16_VARIANT") ? atoi(getenv("MMR_COPY16_VARIANT")) : 0;
  const dim3 grid(grid_size(n, xcd_split));
  const uint32_t count = static_cast<uint32_t>(n);
#define MMR_V(T, U) \
  hipLaunchKernelGGL((mmr_copy16_kernel<T, U>), grid, dim3(T), 0, stream, d_chunks, count, d_ptrs, xcd_split)
  switch (variant) {
    case 1: MMR_V(256, 4); break;
    case 2: MMR_V(256, 2); break;
    case 3: MMR_V(128, 4); break;
    case 4: MMR_V(128, 8); break;
    case 5: MMR_V(64, 8); break;
    case 6: MMR_V(512, 2); break;
    case 7: MMR_V(1024, 1); break;
    case 8: MMR_V(128, 2); break;
    case 9: MMR_V(64, 4); break;
    case 10: MMR_V(512, 1); break;
    case 11: MMR_V(256, 1); break;
    default: MMR_V(256, 8); break;
  }
#undef MMR_V
  return hipGetLastError();
}

hipError_t launch_copy_generic(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, bool xcd_split,
                               hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  static const int variant = getenv("MMR_GENERIC_VARIANT") ? atoi(getenv("MMR_GENERIC_VARIANT")) : 0;
  const dim3 grid(grid_size(n, xcd_split));
  const uint32_t count = static_cast<uint32_t>(n);
  static const int nt = getenv("MMR_GENERIC_NT") ? atoi(getenv("MMR_GENERIC_NT")) : 2;
#define MMR_V(T, U)                                                                                                  \
  do {                                                                                                               \
    if (nt == 3)                                                                                                     \
      hipLaunchKernelGGL((mmr_copy_generic_kernel<T, U, true, true>), grid, dim3(T), 0, stream, d_chunks, count,     \
                         d_ptrs, xcd_split);                                                                         \
    else if (nt == 1)                                                                                                \
      hipLaunchKernelGGL((mmr_copy_generic_kernel<T, U, true, false>), grid, dim3(T), 0, stream, d_chunks, count,    \
                         d_ptrs, xcd_split);                                                                         \
    else if (nt == 2)                                                                                                \
      hipLaunchKernelGGL((mmr_copy_generic_kernel<T, U, false, true>), grid, dim3(T), 0, stream, d_chunks, count,    \
                         d_ptrs, xcd_split);                                                                         \
    else                                                                                                             \
      hipLaunchKernelGGL((mmr_copy_generic_kernel<T, U, false, false>), grid, dim3(T), 0, stream, d_chunks, count,   \
                         d_ptrs, xcd_split);                                                                         \
  } while (0)
  switch (variant) {
    case 1: MMR_V(256, 4); break;
    case 2: MMR_V(256, 1); break;
    case 3: MMR_V(128, 4); break;
    case 4: MMR_V(128, 2); break;
    default: MMR_V(256, 2); break;
  }
#undef MMR_V
  return hipGetLastError();
}

hipError_t launch_transpose(const mmr_transpose_chunk* d_chunks, int64_t n, void* const* d_ptrs, bool xcd_split,
                            hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  hipLaunchKernelGGL(mmr_transpose_kernel, dim3(grid_size(n, xcd_split)), dim3(kTransposeThreads), 0, stream, d_chunks,
                     static_cast<uint32_t>(n), d_ptrs, xcd_split);
  return hipGetLastError();
}

}  // namespace mmr
