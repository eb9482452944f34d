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
// The per-chunk index arithmetic lives in chunk_ops.h, shared with the host
// emulation the tests run.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "chunk_ops.h"
#include "kernels.h"

namespace mmr {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Shard buffers are always device (global) memory.  Pointers read from the
// pointer table would otherwise be generic and compile to flat_* accesses;
// address space 1 makes every access a global_* instruction.
#define MMR_GLOBAL __attribute__((address_space(1)))
typedef MMR_GLOBAL char gchar;
typedef MMR_GLOBAL const char gcchar;

// Device memory policy for chunk_ops.h.  NTL / NTS: nontemporal loads / stores
// (every byte is touched exactly once, keep it out of the caches' way), or
// plain cacheable ones (ragged rows: a line shared by two rows or two chunks
// is fetched once and its pieces merge in the L2).  gfx950 under the HSA
// runtime runs with unaligned global access enabled and the compiler emits a
// single access for the aligned(1) types below.
template <bool NTL, bool NTS>
struct DeviceMem {
  typedef gcchar* cptr;
  typedef gchar* ptr;

  template <typename T, int ALIGN>
  static __device__ __forceinline__ T ld(cptr p) {
    typedef MMR_GLOBAL const T __attribute__((aligned(ALIGN))) gt;
    if constexpr (NTL) return __builtin_nontemporal_load(reinterpret_cast<gt*>(p));
    else return *reinterpret_cast<gt*>(p);
  }
  template <typename T, int ALIGN>
  static __device__ __forceinline__ void st(ptr p, T v) {
    typedef MMR_GLOBAL T __attribute__((aligned(ALIGN))) gt;
    if constexpr (NTS) __builtin_nontemporal_store(v, reinterpret_cast<gt*>(p));
    else *reinterpret_cast<gt*>(p) = v;
  }
  static __device__ __forceinline__ V16 pack(u32x4 v) { return V16{v.x, v.y, v.z, v.w}; }
  static __device__ __forceinline__ u32x4 unpack(V16 v) { return u32x4{v.x, v.y, v.z, v.w}; }

  static __device__ __forceinline__ V16 load16(cptr p) { return pack(ld<u32x4, 16>(p)); }
  static __device__ __forceinline__ V16 load16u(cptr p) { return pack(ld<u32x4, 1>(p)); }
  static __device__ __forceinline__ void store16(ptr p, V16 v) { st<u32x4, 16>(p, unpack(v)); }
  template <typename T>
  static __device__ __forceinline__ T loadu(cptr p) {
    if constexpr (sizeof(T) == 16) return load16u(p);
    else return ld<T, 1>(p);
  }
  template <typename T>
  static __device__ __forceinline__ void storeu(ptr p, T v) {
    if constexpr (sizeof(T) == 16) st<u32x4, 1>(p, unpack(v));
    else st<T, 1>(p, v);
  }
  static __device__ __forceinline__ uintptr_t addr(ptr p) { return reinterpret_cast<uintptr_t>(p); }
};

__device__ __forceinline__ gchar* slot_base(void* const* __restrict__ ptrs, uint32_t slot, uint64_t off) {
  return (gchar*)(static_cast<char*>(ptrs[slot])) + off;
}

constexpr int kThreads = 256;  // every chunk class runs 256-thread workgroups (4 wavefronts)

// Launch shapes are the measured optimum on MI355X for 8 KiB (aligned) and
// 4 KiB (generic, span) chunks: up to 8 (aligned) or 2 (generic) 16-byte
// accesses in flight per lane before the first store.
__device__ __forceinline__ void run_copy16(const mmr_copy_chunk* __restrict__ chunks, uint32_t ci,
                                           void* const* __restrict__ ptrs) {
  const mmr_copy_chunk c = chunks[ci];
  gchar* dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  gcchar* src = c.src_slot == MMR_SLOT_FILL ? dst : slot_base(ptrs, c.src_slot, c.src_off);  // never read when filling
  copy16_chunk<DeviceMem<true, true>, kThreads, 8>(c, src, dst, threadIdx.x);
}

__device__ __forceinline__ void run_generic(const mmr_copy_chunk* __restrict__ chunks, uint32_t ci,
                                            void* const* __restrict__ ptrs) {
  const mmr_copy_chunk c = chunks[ci];
  gchar* dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  gcchar* src = c.src_slot == MMR_SLOT_FILL ? dst : slot_base(ptrs, c.src_slot, c.src_off);
  // cacheable loads (a source line shared by two chunks is fetched once), nontemporal stores
  generic_chunk<DeviceMem<false, true>, kThreads, 2>(c, src, dst, threadIdx.x);
}

__device__ __forceinline__ void run_span(const mmr_span_chunk* __restrict__ chunks, uint32_t ci,
                                         void* const* __restrict__ ptrs) {
  typedef DeviceMem<false, true> M;  // cacheable loads: neighbouring slots and rows share source lines
  const mmr_span_chunk c = chunks[ci];
  gchar* dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  SpanSources<M> srcs;
#pragma unroll
  for (uint32_t j = 0; j < MMR_SPAN_MAX_PIECES; ++j) {
    const bool live = j < c.n_pieces && c.pieces[j].src_slot != MMR_SLOT_FILL;
    srcs.base[j] = live ? slot_base(ptrs, c.pieces[j].src_slot, c.pieces[j].src_off) : dst;  // never read when not live
  }
  span_chunk<M, kThreads>(c, srcs, dst, threadIdx.x);
}

template <typename T, int TILE>
__device__ __forceinline__ void transpose_tiles(const mmr_transpose_chunk& c, gcchar* src, gchar* dst, void* lds_raw) {
  typedef DeviceMem<true, true> M;
  T(*tile)[TILE + 1] = reinterpret_cast<T(*)[TILE + 1]>(lds_raw);
  for (uint32_t b = 0; b < c.nb; ++b) {
    transpose_load<M, T, TILE, kThreads>(c, src, b, tile, threadIdx.x);
    __syncthreads();
    transpose_store<M, T, TILE, kThreads>(c, dst, b, tile, threadIdx.x);
    __syncthreads();
  }
}

__device__ __forceinline__ void run_transpose(const mmr_transpose_chunk* __restrict__ chunks, uint32_t ci,
                                              void* const* __restrict__ ptrs, void* lds) {
  const mmr_transpose_chunk c = chunks[ci];
  gcchar* src = slot_base(ptrs, c.src_slot, c.src_off);
  gchar* dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  switch (c.itemsize) {  // wave-uniform
    case 1: transpose_tiles<uint8_t, 64>(c, src, dst, lds); break;
    case 2: transpose_tiles<uint16_t, 64>(c, src, dst, lds); break;
    case 4: transpose_tiles<uint32_t, 64>(c, src, dst, lds); break;
    case 8: transpose_tiles<uint64_t, 64>(c, src, dst, lds); break;
    default: transpose_tiles<V16, 32>(c, src, dst, lds); break;
  }
}

// One launch per plan: the grid is the four chunk tables back to back (each
// padded to its XCD grouping); a workgroup finds its table by its block index
// (wave-uniform branches) and runs one chunk of it.
__global__ __launch_bounds__(kThreads) void mmr_reshard_kernel(PlanTables t, void* const* __restrict__ ptrs) {
  // LDS is only allocated (at launch) when the plan has transpose chunks:
  // 64 x 65 eight-byte elements is the largest tile (33,280 bytes).
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  uint32_t b = blockIdx.x;
  if (b < t.copy16.grid) {
    const uint32_t ci = chunk_index(b, t.copy16.group);
    if (ci < t.copy16.n) run_copy16(static_cast<const mmr_copy_chunk*>(t.copy16.chunks), ci, ptrs);
    return;
  }
  b -= t.copy16.grid;
  if (b < t.span.grid) {
    const uint32_t ci = chunk_index(b, t.span.group);
    if (ci < t.span.n) run_span(static_cast<const mmr_span_chunk*>(t.span.chunks), ci, ptrs);
    return;
  }
  b -= t.span.grid;
  if (b < t.generic.grid) {
    const uint32_t ci = chunk_index(b, t.generic.group);
    if (ci < t.generic.n) run_generic(static_cast<const mmr_copy_chunk*>(t.generic.chunks), ci, ptrs);
    return;
  }
  b -= t.generic.grid;
  const uint32_t ci = chunk_index(b, t.transpose.group);
  if (ci < t.transpose.n)  // uniform over the workgroup: no barrier is skipped by part of it
    run_transpose(static_cast<const mmr_transpose_chunk*>(t.transpose.chunks), ci, ptrs, lds);
}

}  // namespace

void set_table(PlanTables::Table* t, const void* d_chunks, int64_t n, uint32_t xcd_mode) {
  t->chunks = d_chunks;
  t->n = static_cast<uint32_t>(n);
  t->group = xcd_group_of(n, xcd_mode);
  t->grid = n == 0 ? 0u : grid_size(n, t->group);
}

hipError_t launch_plan(const PlanTables& t, void* const* d_ptrs, hipStream_t stream) {
  const uint64_t grid = static_cast<uint64_t>(t.copy16.grid) + t.span.grid + t.generic.grid + t.transpose.grid;
  if (grid == 0) return hipSuccess;
  if (grid > 0x7ff00000ULL) return hipErrorInvalidValue;
  const size_t lds = t.transpose.n ? 64 * 65 * 8 : 0;
  hipLaunchKernelGGL(mmr_reshard_kernel, dim3(static_cast<uint32_t>(grid)), dim3(kThreads), lds, stream, t, d_ptrs);
  return hipGetLastError();
}

}  // namespace mmr
