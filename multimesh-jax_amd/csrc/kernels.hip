// gfx950 (CDNA4) data-movement kernels of the reshard path.
//
// Pure byte movement: nothing is ever typed as a float, so NaN payloads, FP8
// and integer data all come through bit-exact.  Every kernel is bound by HBM
// bandwidth; there is no MFMA work on this path.
//
// Work distribution: one 256-thread workgroup (4 wavefronts of 64) per chunk of
// the plan's table.  The chunk record and the two base pointers are wave-uniform
// and come in through scalar loads; lanes then move 16 bytes each, consecutive
// lanes covering consecutive 16-byte vectors of a row so every wavefront touches
// whole 128-byte lines.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernels.h"

namespace mmr {
namespace {

constexpr int kThreads = 256;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct alignas(16) u128 {
  uint64_t lo, hi;
};

// Streaming accesses: every byte is touched exactly once, so keep it out of
// the way of the caches' replacement policy.
template <typename T>
__device__ __forceinline__ T stream_load(const void* p) {
  return __builtin_nontemporal_load(static_cast<const T*>(p));
}
template <typename T>
__device__ __forceinline__ void stream_store(void* p, T v) {
  __builtin_nontemporal_store(v, static_cast<T*>(p));
}
template <>
__device__ __forceinline__ u128 stream_load<u128>(const void* p) {
  u32x4 v = __builtin_nontemporal_load(static_cast<const u32x4*>(p));
  u128 r;
  r.lo = static_cast<uint64_t>(v.x) | (static_cast<uint64_t>(v.y) << 32);
  r.hi = static_cast<uint64_t>(v.z) | (static_cast<uint64_t>(v.w) << 32);
  return r;
}
template <>
__device__ __forceinline__ void stream_store<u128>(void* p, u128 r) {
  u32x4 v;
  v.x = static_cast<uint32_t>(r.lo);
  v.y = static_cast<uint32_t>(r.lo >> 32);
  v.z = static_cast<uint32_t>(r.hi);
  v.w = static_cast<uint32_t>(r.hi >> 32);
  __builtin_nontemporal_store(v, static_cast<u32x4*>(p));
}

// Moves (or zero-fills) the n2 x n1 x (w / sizeof(T)) elements of one chunk.
// UNROLL loads are issued before the first store so each lane keeps several
// requests in flight.
template <typename T, int UNROLL>
__device__ __forceinline__ void move_chunk(const mmr_copy_chunk& c, const char* __restrict__ src,
                                           char* __restrict__ dst) {
  const uint32_t wv = c.w / static_cast<uint32_t>(sizeof(T));
  const uint32_t total = wv * c.n1 * c.n2;
  const bool fill = c.src_slot == MMR_SLOT_FILL;
  for (uint32_t base = threadIdx.x; base < total; base += kThreads * UNROLL) {
    T v[UNROLL];
    int64_t doff[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
      const uint32_t idx = base + k * kThreads;
      if (idx < total) {
        const uint32_t row = idx / wv;
        const uint32_t col = idx - row * wv;
        const uint32_t r2 = row / c.n1;
        const uint32_t r1 = row - r2 * c.n1;
        const int64_t cb = static_cast<int64_t>(col) * static_cast<int64_t>(sizeof(T));
        doff[k] = r2 * c.d2 + r1 * c.d1 + cb;
        if (fill) {
          v[k] = T{};
        } else {
          v[k] = stream_load<T>(src + (r2 * c.s2 + r1 * c.s1 + cb));
        }
      }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
      const uint32_t idx = base + k * kThreads;
      if (idx < total) stream_store<T>(dst + doff[k], v[k]);
    }
  }
}

__global__ __launch_bounds__(kThreads) void mmr_copy16_kernel(const mmr_copy_chunk* __restrict__ chunks,
                                                              void* const* __restrict__ ptrs) {
  const mmr_copy_chunk c = chunks[blockIdx.x];
  char* dst = static_cast<char*>(ptrs[c.dst_slot]) + c.dst_off;
  const char* src = c.src_slot == MMR_SLOT_FILL ? nullptr : static_cast<const char*>(ptrs[c.src_slot]) + c.src_off;
  move_chunk<u32x4, 8>(c, src, dst);
}

__global__ __launch_bounds__(kThreads) void mmr_copy_generic_kernel(const mmr_copy_chunk* __restrict__ chunks,
                                                                    void* const* __restrict__ ptrs) {
  const mmr_copy_chunk c = chunks[blockIdx.x];
  char* dst = static_cast<char*>(ptrs[c.dst_slot]) + c.dst_off;
  const char* src = c.src_slot == MMR_SLOT_FILL ? nullptr : static_cast<const char*>(ptrs[c.src_slot]) + c.src_off;
  switch (c.align) {  // wave-uniform
    case 16: move_chunk<u32x4, 4>(c, src, dst); break;
    case 8: move_chunk<uint64_t, 4>(c, src, dst); break;
    case 4: move_chunk<uint32_t, 4>(c, src, dst); break;
    case 2: move_chunk<uint16_t, 4>(c, src, dst); break;
    default: move_chunk<uint8_t, 4>(c, src, dst); break;
  }
}

// One batch of tiles: x is contiguous in the source, y in the destination.
// Rows of the tile are read along x, parked in LDS (row pitch TILE + 1 elements
// to spread the column reads over the banks), and written along y.
template <typename T, int TILE>
__device__ __forceinline__ void transpose_tiles(const mmr_transpose_chunk& c, const char* __restrict__ src,
                                                char* __restrict__ dst, void* lds_raw) {
  T(*tile)[TILE + 1] = reinterpret_cast<T(*)[TILE + 1]>(lds_raw);
  const uint32_t n = c.nx * c.ny;
  for (uint32_t b = 0; b < c.nb; ++b) {
    const char* s = src + b * c.src_bstride;
    char* d = dst + b * c.dst_bstride;
    for (uint32_t i = threadIdx.x; i < n; i += kThreads) {
      const uint32_t y = i / c.nx, x = i - y * c.nx;
      tile[y][x] = stream_load<T>(s + y * c.src_ystride + static_cast<int64_t>(x) * sizeof(T));
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < n; i += kThreads) {
      const uint32_t x = i / c.ny, y = i - x * c.ny;
      stream_store<T>(d + x * c.dst_xstride + static_cast<int64_t>(y) * sizeof(T), tile[y][x]);
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(kThreads) void mmr_transpose_kernel(const mmr_transpose_chunk* __restrict__ chunks,
                                                                 void* const* __restrict__ ptrs) {
  // 64 x 65 eight-byte elements is the largest tile (33,280 bytes); sixteen-byte
  // elements use 32 x 33 tiles (16,896 bytes).
  __shared__ alignas(16) uint64_t lds[64 * 65];
  const mmr_transpose_chunk c = chunks[blockIdx.x];
  const char* src = static_cast<const char*>(ptrs[c.src_slot]) + c.src_off;
  char* dst = static_cast<char*>(ptrs[c.dst_slot]) + c.dst_off;
  switch (c.itemsize) {  // wave-uniform
    case 1: transpose_tiles<uint8_t, 64>(c, src, dst, lds); break;
    case 2: transpose_tiles<uint16_t, 64>(c, src, dst, lds); break;
    case 4: transpose_tiles<uint32_t, 64>(c, src, dst, lds); break;
    case 8: transpose_tiles<uint64_t, 64>(c, src, dst, lds); break;
    default: transpose_tiles<u128, 32>(c, src, dst, lds); break;
  }
}

hipError_t check_grid(int64_t n) { return (n < 0 || n > 0x7fffffffLL) ? hipErrorInvalidValue : hipSuccess; }

}  // namespace

hipError_t launch_copy16(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  hipLaunchKernelGGL(mmr_copy16_kernel, dim3(static_cast<uint32_t>(n)), dim3(kThreads), 0, stream, d_chunks, d_ptrs);
  return hipGetLastError();
}

hipError_t launch_copy_generic(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  hipLaunchKernelGGL(mmr_copy_generic_kernel, dim3(static_cast<uint32_t>(n)), dim3(kThreads), 0, stream, d_chunks,
                     d_ptrs);
  return hipGetLastError();
}

hipError_t launch_transpose(const mmr_transpose_chunk* d_chunks, int64_t n, void* const* d_ptrs, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  hipLaunchKernelGGL(mmr_transpose_kernel, dim3(static_cast<uint32_t>(n)), dim3(kThreads), 0, stream, d_chunks, d_ptrs);
  return hipGetLastError();
}

}  // namespace mmr
