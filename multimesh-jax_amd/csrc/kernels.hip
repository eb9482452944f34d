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

#include <algorithm>
#include <cstdint>
#include <mutex>

#include "chunk_ops.h"
#include "group_ops.h"
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
  // 16 bytes at any alignment that other workgroups read too: an ordinary cacheable load whatever NTL says
  static __device__ __forceinline__ V16 load16u_keep(cptr p) {
    typedef MMR_GLOBAL const u32x4 __attribute__((aligned(1))) gt;
    return pack(*reinterpret_cast<gt*>(p));
  }
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
  static __device__ __forceinline__ uintptr_t caddr(cptr p) { return reinterpret_cast<uintptr_t>(p); }
};

// LDS accesses of the span kernel.  gfx950 takes a 16-byte LDS access at any byte address (the compiler emits a single
// ds_write_b128 for the aligned(1) type below).
struct DeviceLds {
  static __device__ __forceinline__ void store16u(uint8_t* p, V16 v) {
    typedef u32x4 __attribute__((aligned(1))) u4u;
    *reinterpret_cast<u4u*>(p) = u32x4{v.x, v.y, v.z, v.w};
  }
  static __device__ __forceinline__ void store8(uint8_t* p, uint8_t v) { *p = v; }
  static __device__ __forceinline__ V16 load16(const uint8_t* p) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(p);
    return V16{v.x, v.y, v.z, v.w};
  }
  static __device__ __forceinline__ uint8_t load8(const uint8_t* p) { return *p; }
};

__device__ __forceinline__ gchar* slot_base(void* const* __restrict__ ptrs, uint32_t slot, uint64_t off) {
  return (gchar*)(static_cast<char*>(ptrs[slot])) + off;
}

// Launch shape of the aligned kernel: 256 threads, 2 vectors each (8 KiB per workgroup), nontemporal both ways.
// Measured against it on MI355X (bf16 [8,4096,8192] hidden 8-way -> sequence 4-way, 160.6 us): 512 threads x 1 vector
// 222 us - every wave decodes its chunk on the scalar unit (some 200 scalar instructions), and with twice the waves
// per byte the scalar unit, 53 % busy at 256 x 2, is the bound; 128 threads x 4 vectors 169 us.  A stand-alone copy of
// the same access pattern whose chunk falls out of three shifts runs in 169 us at 256 x 2 and 160-162 us at 512 x 1.
#ifndef MMR_COPY16_THREADS
#define MMR_COPY16_THREADS 256
#endif
#ifndef MMR_COPY16_UNROLL
#define MMR_COPY16_UNROLL 2
#endif
constexpr int kCopy16Threads = MMR_COPY16_THREADS;
constexpr int kCopy16Unroll = MMR_COPY16_UNROLL;
constexpr bool kCopy16NtLoads = true;

// Translation prefetch.  A launch streams through its buffers once, so every 2 MiB page is new when the first
// workgroup reaches it, and thousands of waves then wait for the same page walk.  Every kPrefetchEvery-th workgroup
// therefore also touches the source and the destination of the chunk kPrefetchAhead places further down the table
// (one 4-byte load each by one lane, results unused; the value read from the destination may be in the middle of
// being written by another workgroup, which does not matter): by the time that chunk runs, its translations are
// in the TLBs.  Measured on MI355X: bf16 [8,4096,8192] hidden 8-way -> sequence 4-way 162.3 -> 160.8 us (three
// alternating pairs), the same split of a four times larger array 684.7 -> 675.0 us; 4,096, 8,192 and 16,384 chunks
// ahead and every 13th or 37th workgroup all measure the same; small arrays (64 MiB per side) neither gain nor lose.
#ifndef MMR_PREFETCH_AHEAD
#define MMR_PREFETCH_AHEAD 8192
#endif
#ifndef MMR_PREFETCH_EVERY
#define MMR_PREFETCH_EVERY 37
#endif
constexpr uint32_t kPrefetchAhead = MMR_PREFETCH_AHEAD;  // chunks; 0 = off
constexpr uint32_t kPrefetchEvery = MMR_PREFETCH_EVERY;  // a prime, so that every piece of a row block gets its turn

// Copy groups: the workgroup works its chunk out from the group table (bound: absolute addresses).  `groups` and
// `pieces` are wave-uniform reads (scalar loads); the records are taken by value so that their loads leave together.
template <int THREADS, int UNROLL, class FindGroup>
__device__ __forceinline__ void copy_group_chunk(const CopyGroup* __restrict__ groups, const CopyPiece* __restrict__ pieces,
                                                 uint32_t gi, uint32_t ci, uint32_t n, FindGroup find) {
  const CopyGroup g = groups[gi];
  const DecodedCopy d = decode_copy(g, ci - g.first_chunk);
  const CopyPiece p = pieces[d.piece];
  const mmr_copy_chunk c = copy_chunk_of(g, p, d);
  gchar* dst = (gchar*)(c.dst_off);
  gcchar* src = c.src_slot == MMR_SLOT_FILL ? dst : (gcchar*)(c.src_off);  // never read when filling
  uint32_t touched = 0;
  bool touching = false;
  if constexpr (kPrefetchAhead != 0) {
    const uint32_t ahead = ci + kPrefetchAhead;
    touching = ci % kPrefetchEvery == 0 && ahead < n;  // uniform over the workgroup
    if (touching && threadIdx.x == 0) {
      const CopyGroup g2 = groups[find(ahead)];
      const DecodedCopy d2 = decode_copy(g2, ahead - g2.first_chunk);
      const CopyPiece p2 = pieces[d2.piece];
      const mmr_copy_chunk c2 = copy_chunk_of(g2, p2, d2);
      typedef MMR_GLOBAL const uint32_t gu32;
      touched = *reinterpret_cast<gu32*>(c2.dst_off);
      if (c2.src_slot != MMR_SLOT_FILL) touched ^= *reinterpret_cast<gu32*>(c2.src_off);
    }
  }
  copy_group_rows<DeviceMem<kCopy16NtLoads, true>, THREADS, UNROLL>(g, p, c, src, dst, threadIdx.x);
  if constexpr (kPrefetchAhead != 0) {
    // the loaded words are used, so that the loads stay: a pause nobody notices if they happen to spell this number
    if (touching && touched == 0x9e3779b9u) __builtin_amdgcn_s_sleep(1);
  }
}

// DIRECT: the table has at most kMaxDirectGroups groups and `starts` holds their first chunks (no hint lookup).
template <int THREADS, int UNROLL, bool DIRECT>
__global__ __launch_bounds__(THREADS) void mmr_copy16_kernel(const CopyGroup* __restrict__ groups, uint32_t n_groups,
                                                             const CopyPiece* __restrict__ pieces,
                                                             const uint32_t* __restrict__ hints, uint32_t n,
                                                             uint32_t xcd_group, const GroupStarts starts, uint32_t first) {
  const uint32_t ci = first + chunk_index(blockIdx.x, xcd_group);  // first: where this launch's piece of the table begins
  if (ci >= n) return;
  auto find = [&](uint32_t at) { return DIRECT ? find_group_direct(starts, at) : find_group(groups, n_groups, hints, at); };
  copy_group_chunk<THREADS, UNROLL>(groups, pieces, find(ci), ci, n, find);
}

// The same with the whole table in the kernel's argument block (nothing in device memory to look up or to keep alive).
template <int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void mmr_copy16_inline_kernel(const InlineCopyTable table, uint32_t xcd_group,
                                                                    uint32_t first) {
  const uint32_t ci = first + chunk_index(blockIdx.x, xcd_group);
  if (ci >= table.n_chunks) return;
  auto find = [&](uint32_t at) { return find_group(table.groups, table.n_groups, nullptr, at); };
  copy_group_chunk<THREADS, UNROLL>(table.groups, table.pieces, find(ci), ci, table.n_chunks, find);
}

// 16 readable bytes for the loads of span items that need none.
__device__ __align__(16) const uint32_t span_safe_bytes[4] = {0, 0, 0, 0};

template <int THREADS, int UNROLL>
__device__ __forceinline__ void span_chunk(const SpanGroup* __restrict__ groups, uint32_t n_groups,
                                           const SpanMember* __restrict__ members, const SpanPiece* __restrict__ pieces,
                                           const uint32_t* __restrict__ hints, uint32_t ci, uint8_t* lds) {
  typedef DeviceMem<true, true> M;  // nontemporal both ways: measured no more HBM reads than cacheable loads, and faster
  const uint32_t gi = find_group(groups, n_groups, hints, ci);
  const SpanGroup g = groups[gi];
  uint32_t member, lm;
  deinterleave(g.il, ci - g.first_chunk, &member, &lm);
  const SpanMember m = members[g.first_member + member];
  uint64_t x0;
  uint32_t len;
  span_range(g, lm, &x0, &len);
  gchar* dst = (gchar*)(m.dst + x0);
  const uint32_t a = static_cast<uint32_t>(m.dst + x0) & 15u;
  gcchar* safe = (gcchar*)(reinterpret_cast<uintptr_t>(&span_safe_bytes[0]));
  // one wavefront per workgroup: the barriers only order its LDS writes before its LDS reads
  if (g.table_mode) {
    const SpanPiece* pc = pieces + m.first_piece;
    const SpanPieces4 pcs = span_pieces4(pc, m.k);
    uint8_t* table = lds + kSpanStageBytes;
    const SpanRowEnds<M> b = span_table_build<M, DeviceLds, THREADS>(g, m, pcs, safe, x0, len, a, table, threadIdx.x);
    __syncthreads();
    span_table_gather<M, DeviceLds, THREADS, UNROLL>(g, m, pc, pcs, safe, x0, len, a, lds, table, b, threadIdx.x);
  } else {
    span_gather<M, DeviceLds, THREADS, UNROLL>(g, m, pieces, safe, x0, len, a, lds, threadIdx.x);
  }
  __syncthreads();
  span_write<M, DeviceLds, THREADS, UNROLL>(dst, len, a, lds, threadIdx.x);
}

template <int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void mmr_span_kernel(const SpanGroup* __restrict__ groups, uint32_t n_groups,
                                                           const SpanMember* __restrict__ members,
                                                           const SpanPiece* __restrict__ pieces,
                                                           const uint32_t* __restrict__ hints, uint32_t n,
                                                           uint32_t xcd_group) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[kSpanLdsBytes];
  const uint32_t ci = chunk_index(blockIdx.x, xcd_group);
  if (ci >= n) return;  // uniform over the workgroup: no barrier is skipped by part of it
  span_chunk<THREADS, UNROLL>(groups, n_groups, members, pieces, hints, ci, lds);
}

template <int THREADS, int UNROLL>
__global__ __launch_bounds__(THREADS) void mmr_span_inline_kernel(const InlineSpanTable table, uint32_t xcd_group) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[kSpanLdsBytes];
  const uint32_t ci = chunk_index(blockIdx.x, xcd_group);
  if (ci >= table.n_chunks) return;
  span_chunk<THREADS, UNROLL>(table.groups, table.n_groups, table.members, table.pieces, nullptr, ci, lds);
}

template <int THREADS, int UNROLL, bool NTL, bool NTS>
__global__ __launch_bounds__(THREADS) void mmr_copy_generic_kernel(const mmr_copy_chunk* __restrict__ chunks, uint32_t n,
                                                                   void* const* __restrict__ ptrs, uint32_t xcd_group) {
  const uint32_t ci = chunk_index(blockIdx.x, xcd_group);
  if (ci >= n) return;
  const mmr_copy_chunk c = chunks[ci];
  gchar* dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  gcchar* src = c.src_slot == MMR_SLOT_FILL ? dst : slot_base(ptrs, c.src_slot, c.src_off);  // never read when filling
  generic_chunk<DeviceMem<NTL, NTS>, THREADS, UNROLL>(c, src, dst, threadIdx.x);
}

// Launch shape of the generic kernel; cacheable loads (a source line shared by two chunks is fetched once).
constexpr int kGenericThreads = 256;
constexpr int kGenericUnroll = 2;
constexpr bool kGenericNtLoads = false;

// Orders the LDS accesses of the lanes of one wave: what a lane wrote before is visible to the others after.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T>
__device__ __forceinline__ void transpose_sync() {  // between the phases of the threads that share a sub-tile
  if constexpr (TransposeTile<sizeof(T)>::kGroupThreads == 64) wave_sync(); else __syncthreads();
}

// VECTOR_ONLY: every chunk of the launch satisfies transpose_is_vector (the caller launches the two kinds apart).
template <typename T, bool VECTOR_ONLY>
__device__ __forceinline__ void transpose_tiles(const mmr_transpose_chunk& c, gcchar* src, gchar* dst, void* lds_raw) {
  typedef DeviceMem<true, true> M;
  typedef TransposeTile<sizeof(T)> G;
  T* lds = static_cast<T*>(lds_raw);
  const uint32_t tid = threadIdx.x;
  // The threads that share a sub-tile take the same path, chosen by the part of the sub-tile that lies inside the
  // tile; waves with sub-tiles of their own run independently (a sub-tile outside the tile: nothing to do).
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / G::kGroupThreads);
  uint32_t x0, y0, snx, sny;
  const TransposeMode mode = transpose_mode<sizeof(T)>(c, wave, &x0, &y0, &snx, &sny);
  if constexpr (VECTOR_ONLY) {
    if (mode == kTransposeNothing) return;
    for (uint32_t b = 0; b < c.nb; ++b) {
      transpose_load_vec<M, T>(c, src, b, lds, tid);
      transpose_sync<T>();
      transpose_store_vec<M, T>(c, dst, b, lds, tid);
      transpose_sync<T>();
    }
    return;
  }
  if (transpose_is_thin(c)) {  // uniform over the workgroup: the whole chunk in two phases around one barrier
    transpose_thin_load<M, T>(c, src, lds, tid);
    __syncthreads();
    transpose_thin_store<M, T>(c, dst, lds, tid);
    return;
  }
  // One batch loop per path: with the choice inside a common loop the compiler hoists every path's loop-invariant
  // addresses out of it and the register need is the sum over the paths instead of the maximum.
  switch (mode) {
    case kTransposeVector:
      for (uint32_t b = 0; b < c.nb; ++b) {
        transpose_load_vec<M, T>(c, src, b, lds, tid);
        transpose_sync<T>();
        transpose_store_vec<M, T>(c, dst, b, lds, tid);
        transpose_sync<T>();
      }
      break;
    case kTransposeGeneral:
      for (uint32_t b = 0; b < c.nb; ++b) {
        transpose_load_general<M, T>(c, src, b, lds, tid, x0, y0, snx, sny);
        transpose_sync<T>();
        transpose_store_general<M, T>(c, dst, b, lds, tid, x0, y0, snx, sny);
        transpose_sync<T>();
      }
      break;
    case kTransposeElement:
      for (uint32_t b = 0; b < c.nb; ++b) {
        transpose_load_element<M, T>(c, src, b, lds, tid, x0, y0, snx, sny);
        transpose_sync<T>();
        transpose_store_element<M, T>(c, dst, b, lds, tid, x0, y0, snx, sny);
        transpose_sync<T>();
      }
      break;
    default:  // the sub-tile lies outside the tile (never the case where the whole workgroup shares one sub-tile)
      break;
  }
}

// Waves per SIMD the register allocation of the general kernel aims at (0 = the compiler's choice): three where the
// widest path fits 168 registers without spilling; the 2-byte instance needs 170 and stays at two.
template <typename T>
constexpr int transpose_general_waves() { return sizeof(T) == 2 || sizeof(T) >= 8 ? 0 : 3; }

template <typename T, bool VECTOR_ONLY>
__global__ __launch_bounds__(TransposeTile<sizeof(T)>::kThreads, VECTOR_ONLY ? 0 : transpose_general_waves<T>())
void mmr_transpose_kernel(
    const mmr_transpose_chunk* __restrict__ chunks, uint32_t n, void* const* __restrict__ ptrs, uint32_t xcd_group) {
  // one instance per element width, each with the register and LDS budget of its own tile; the general kernel
  // also takes thin chunks, which park up to kTransposeLdsBytes at once
  __shared__ __attribute__((aligned(16))) uint8_t lds[VECTOR_ONLY ? TransposeTile<sizeof(T)>::kLdsBytes : kTransposeLdsBytes];
  const uint32_t ci = chunk_index(blockIdx.x, xcd_group);
  if (ci >= n) return;  // uniform over the workgroup: no barrier is skipped by part of it
  const mmr_transpose_chunk c = chunks[ci];
  gcchar* src = slot_base(ptrs, c.src_slot, c.src_off);
  gchar* dst = slot_base(ptrs, c.dst_slot, c.dst_off);
  transpose_tiles<T, VECTOR_ONLY>(c, src, dst, lds);
}

// Flat copy of `vectors` 16-byte vectors: workgroup i moves the i-th block of kFlatVectors vectors, all loads of a
// lane before its first store.  AssembleShards of a device-resident shard (one flat copy of the shard's bytes).
constexpr uint32_t kFlatVectors = 512;  // 8 KiB per workgroup, like the plan's chunks

__global__ __launch_bounds__(256) void mmr_flat_copy_kernel(const void* __restrict__ src_, void* __restrict__ dst_,
                                                            uint64_t vectors) {
  typedef DeviceMem<true, true> M;
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * kFlatVectors;
  gcchar* src = (gcchar*)(static_cast<const char*>(src_)) + (base << 4);
  gchar* dst = (gchar*)(static_cast<char*>(dst_)) + (base << 4);
  const uint64_t left = vectors - base;
  const uint32_t n = left < kFlatVectors ? static_cast<uint32_t>(left) : kFlatVectors;
  V16 v[kFlatVectors / 256];
#pragma unroll
  for (uint32_t u = 0; u < kFlatVectors / 256; ++u) {
    const uint32_t i = threadIdx.x + u * 256;
    if (i < n) v[u] = M::load16(src + (static_cast<int64_t>(i) << 4));
  }
#pragma unroll
  for (uint32_t u = 0; u < kFlatVectors / 256; ++u) {
    const uint32_t i = threadIdx.x + u * 256;
    if (i < n) M::store16(dst + (static_cast<int64_t>(i) << 4), v[u]);
  }
}

// Device memory that exists without any allocation call: the tables of a launch issued by callers that may not
// allocate (the static entry point of the C ABI).  One copy per GPU, held until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; the device address it yields is what launches and copies use.
static __device__ __align__(256) unsigned char scratch[MMR_STATIC_SCRATCH_BYTES];

hipError_t check_grid(int64_t n) { return (n < 0 || n > 0x7ff00000LL) ? hipErrorInvalidValue : hipSuccess; }

}  // namespace

// Launch shapes are the measured optimum on MI355X: 256 threads and 2 16-byte
// accesses in flight per lane for 8 KiB (aligned) and 7 KiB (generic) chunks,
// one wavefront and 4 + 1 accesses per lane for 4 KiB spans; one workgroup per
// chunk (persistent workgroups that loop over the table, 4 to 16 per CU, with
// the next chunk record prefetched, were 2-18 % slower on every configuration).
hipError_t static_scratch_address(int device, void** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* address[kMaxDevices] = {};
  if (!out || device < 0 || device >= kMaxDevices) return hipErrorInvalidValue;
  std::lock_guard<std::mutex> lock(mu);
  if (!address[device]) {
    int current = -1;
    if (hipError_t e = hipGetDevice(&current)) return e;
    if (current != device) return hipErrorInvalidDevice;  // every GPU holds its own copy of the array at its own address
    void* ptr = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))) return e;
    if (!ptr) return hipErrorInvalidSymbol;
    address[device] = ptr;
  }
  *out = address[device];
  return hipSuccess;
}

hipError_t launch_flat_copy(const void* src, void* dst, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | bytes) & 15u) return hipErrorInvalidValue;
  const uint64_t vectors = bytes >> 4;
  const uint64_t blocks = (vectors + kFlatVectors - 1) / kFlatVectors;
  if (hipError_t e = check_grid(static_cast<int64_t>(blocks))) return e;
  hipLaunchKernelGGL(mmr_flat_copy_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream, src, dst, vectors);
  return hipGetLastError();
}

hipError_t launch_copy_groups(const CopyGroup* d_groups, uint32_t n_groups, const CopyPiece* d_pieces,
                              const uint32_t* d_hints, const uint32_t* starts, int64_t n, uint32_t xcd_mode,
                              hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  const uint32_t group = xcd_group_of(n, xcd_mode);
  GroupStarts s;
  for (uint32_t i = 0; i < kMaxDirectGroups; ++i) s.first[i] = starts && i < n_groups ? starts[i] : 0xffffffffu;
  const int64_t piece = copy_piece_chunks(n, xcd_mode);  // long tables leave in pieces (chunk_ops.h says why)
  for (int64_t first = 0; first < n; first += piece) {
    const uint32_t grid = grid_size(std::min(piece, n - first), group);
    if (starts && n_groups <= kMaxDirectGroups)
      hipLaunchKernelGGL((mmr_copy16_kernel<kCopy16Threads, kCopy16Unroll, true>), dim3(grid), dim3(kCopy16Threads), 0, stream, d_groups,
                         n_groups, d_pieces, d_hints, static_cast<uint32_t>(n), group, s, static_cast<uint32_t>(first));
    else
      hipLaunchKernelGGL((mmr_copy16_kernel<kCopy16Threads, kCopy16Unroll, false>), dim3(grid), dim3(kCopy16Threads), 0, stream, d_groups,
                         n_groups, d_pieces, d_hints, static_cast<uint32_t>(n), group, s, static_cast<uint32_t>(first));
  }
  return hipGetLastError();
}

hipError_t launch_copy_groups_inline(const InlineCopyTable& table, uint32_t xcd_mode, hipStream_t stream) {
  const int64_t n = table.n_chunks;
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  if (table.n_groups > kInlineCopyGroups) return hipErrorInvalidValue;
  const uint32_t group = xcd_group_of(n, xcd_mode);
  const int64_t piece = copy_piece_chunks(n, xcd_mode);
  for (int64_t first = 0; first < n; first += piece)
    hipLaunchKernelGGL((mmr_copy16_inline_kernel<kCopy16Threads, kCopy16Unroll>), dim3(grid_size(std::min(piece, n - first), group)),
                       dim3(kCopy16Threads), 0, stream, table, group, static_cast<uint32_t>(first));
  return hipGetLastError();
}

hipError_t launch_spans(const SpanGroup* d_groups, uint32_t n_groups, const SpanMember* d_members,
                        const SpanPiece* d_pieces, const uint32_t* d_hints, int64_t n, uint32_t xcd_mode,
                        hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  const uint32_t group = xcd_group_of(n, xcd_mode);
  hipLaunchKernelGGL((mmr_span_kernel<kSpanLanes, kSpanDepth>), dim3(grid_size(n, group)), dim3(kSpanLanes), 0, stream, d_groups,
                     n_groups, d_members, d_pieces, d_hints, static_cast<uint32_t>(n), group);
  return hipGetLastError();
}

hipError_t launch_spans_inline(const InlineSpanTable& table, uint32_t xcd_mode, hipStream_t stream) {
  const int64_t n = table.n_chunks;
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  if (table.n_groups > kInlineSpanGroups) return hipErrorInvalidValue;
  const uint32_t group = xcd_group_of(n, xcd_mode);
  hipLaunchKernelGGL((mmr_span_inline_kernel<kSpanLanes, kSpanDepth>), dim3(grid_size(n, group)), dim3(kSpanLanes), 0, stream, table,
                     group);
  return hipGetLastError();
}

hipError_t launch_copy_generic(const mmr_copy_chunk* d_chunks, int64_t n, void* const* d_ptrs, uint32_t xcd_mode,
                               hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  const uint32_t group = xcd_group_of(n, xcd_mode);
  // cacheable loads (a source line shared by two chunks is fetched once), nontemporal stores
  hipLaunchKernelGGL((mmr_copy_generic_kernel<kGenericThreads, kGenericUnroll, kGenericNtLoads, true>),
                     dim3(grid_size(n, group)), dim3(kGenericThreads), 0, stream, d_chunks, static_cast<uint32_t>(n), d_ptrs,
                     group);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_transpose_of(const mmr_transpose_chunk* d_chunks, int64_t n, void* const* d_ptrs, uint32_t xcd_mode,
                               bool vector_only, hipStream_t stream) {
  const uint32_t group = xcd_group_of(n, xcd_mode);
  const dim3 grid(grid_size(n, group)), block(TransposeTile<sizeof(T)>::kThreads);
  if (vector_only)
    hipLaunchKernelGGL((mmr_transpose_kernel<T, true>), grid, block, 0, stream, d_chunks, static_cast<uint32_t>(n), d_ptrs, group);
  else
    hipLaunchKernelGGL((mmr_transpose_kernel<T, false>), grid, block, 0, stream, d_chunks, static_cast<uint32_t>(n), d_ptrs, group);
  return hipGetLastError();
}

hipError_t launch_transpose(const mmr_transpose_chunk* d_chunks, int64_t n, void* const* d_ptrs, uint32_t xcd_mode,
                            uint32_t itemsize, bool vector_only, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  if (hipError_t e = check_grid(n)) return e;
  switch (itemsize) {
    case 1: return launch_transpose_of<uint8_t>(d_chunks, n, d_ptrs, xcd_mode, vector_only, stream);
    case 2: return launch_transpose_of<uint16_t>(d_chunks, n, d_ptrs, xcd_mode, vector_only, stream);
    case 4: return launch_transpose_of<uint32_t>(d_chunks, n, d_ptrs, xcd_mode, vector_only, stream);
    case 8: return launch_transpose_of<uint64_t>(d_chunks, n, d_ptrs, xcd_mode, vector_only, stream);
    case 16: return launch_transpose_of<V16>(d_chunks, n, d_ptrs, xcd_mode, vector_only, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace mmr
