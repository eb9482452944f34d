// Host emulation of the GPU kernels, for tests only.
//
// Runs a plan's chunk tables through the SAME per-chunk routines the kernels
// use (multimesh-jax_amd/csrc/chunk_ops.h), one call per thread id, with a
// memory policy that checks every access: it must lie inside one of the
// registered shard buffers, and "aligned" accesses must be aligned.  This is
// how index arithmetic is validated on a CPU before a kernel runs on the GPU;
// it is never a fallback of the library.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "chunk_ops.h"
#include "group_ops.h"
#include "mmreshard.h"
#include "planner.h"

namespace {

struct Range {
  uintptr_t lo, hi;
};
thread_local std::vector<Range> g_ranges;
thread_local std::string g_error;
thread_local uint64_t g_loaded, g_stored;

void violation(const char* what, uintptr_t p, size_t n) {
  if (!g_error.empty()) return;
  char buf[256];
  std::snprintf(buf, sizeof(buf), "%s of %zu bytes at %#zx", what, n, static_cast<size_t>(p));
  g_error = buf;
}

bool inside(uintptr_t p, size_t n) {
  for (const Range& r : g_ranges)
    if (p >= r.lo && p + n <= r.hi) return true;
  return false;
}

struct HostMem {
  typedef const uint8_t* cptr;
  typedef uint8_t* ptr;

  template <typename T>
  static T get(cptr p, size_t align, const char* what) {
    T v{};
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    if (!inside(a, sizeof(T))) {
      violation(what, a, sizeof(T));
      return v;
    }
    if (a % align) violation("misaligned aligned-load", a, sizeof(T));
    std::memcpy(&v, p, sizeof(T));
    g_loaded += sizeof(T);
    return v;
  }
  template <typename T>
  static void put(ptr p, T v, size_t align, const char* what) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    if (!inside(a, sizeof(T))) {
      violation(what, a, sizeof(T));
      return;
    }
    if (a % align) violation("misaligned aligned-store", a, sizeof(T));
    std::memcpy(p, &v, sizeof(T));
    g_stored += sizeof(T);
  }
  static mmr::V16 load16(cptr p) { return get<mmr::V16>(p, 16, "out-of-bounds load"); }
  static mmr::V16 load16u(cptr p) { return get<mmr::V16>(p, 1, "out-of-bounds load"); }
  static mmr::V16 load16u_keep(cptr p) { return get<mmr::V16>(p, 1, "out-of-bounds load"); }
  static void store16(ptr p, mmr::V16 v) { put<mmr::V16>(p, v, 16, "out-of-bounds store"); }
  template <typename T>
  static T loadu(cptr p) { return get<T>(p, 1, "out-of-bounds load"); }
  template <typename T>
  static void storeu(ptr p, T v) { put<T>(p, v, 1, "out-of-bounds store"); }
  static uintptr_t addr(ptr p) { return reinterpret_cast<uintptr_t>(p); }
  static uintptr_t caddr(cptr p) { return reinterpret_cast<uintptr_t>(p); }
};

// LDS of the span kernel: a host array; a cell read before it is written shows up as wrong bytes (poison).
thread_local const uint8_t* g_lds_lo = nullptr;
thread_local const uint8_t* g_lds_hi = nullptr;
struct HostLds {
  static bool ok(const uint8_t* p, size_t n) {
    if (p >= g_lds_lo && p + n <= g_lds_hi) return true;
    violation("LDS access outside the staging array", reinterpret_cast<uintptr_t>(p), n);
    return false;
  }
  static void store16u(uint8_t* p, mmr::V16 v) {
    if (ok(p, 16)) std::memcpy(p, &v, 16);
  }
  static void store8(uint8_t* p, uint8_t v) {
    if (ok(p, 1)) *p = v;
  }
  static mmr::V16 load16(const uint8_t* p) {
    mmr::V16 v{};
    if (reinterpret_cast<uintptr_t>(p) % 16) violation("misaligned LDS vector load", reinterpret_cast<uintptr_t>(p), 16);
    if (ok(p, 16)) std::memcpy(&v, p, 16);
    return v;
  }
  static uint8_t load8(const uint8_t* p) { return ok(p, 1) ? *p : 0; }
};

template <typename T>
void run_transpose(const mmr_transpose_chunk& c, const uint8_t* src, uint8_t* dst) {
  typedef mmr::TransposeTile<sizeof(T)> G;
  constexpr uint32_t kThreads = G::kThreads;
  alignas(16) static thread_local uint8_t lds_raw[mmr::kTransposeLdsBytes];
  static_assert(G::kLdsBytes <= mmr::kTransposeLdsBytes, "LDS tile too large");
  T* lds = reinterpret_cast<T*>(lds_raw);
  // a phase runs for every thread before the next one starts: what the wave fence (or the workgroup barrier
  // where the waves share a sub-tile) guarantees on the device
  if (!mmr::transpose_is_vector(c) && mmr::transpose_is_thin(c)) {  // as the general kernel decides
    std::memset(lds_raw, 0xA5, sizeof(lds_raw));
    if (static_cast<uint64_t>(c.nb) * c.nx * c.ny * sizeof(T) > sizeof(lds_raw)) {
      g_error = "thin transpose chunk larger than the workgroup's LDS";
      return;
    }
    for (uint32_t tid = 0; tid < kThreads; ++tid) mmr::transpose_thin_load<HostMem, T>(c, src, lds, tid);
    for (uint32_t tid = 0; tid < kThreads; ++tid) mmr::transpose_thin_store<HostMem, T>(c, dst, lds, tid);
    return;
  }
  for (uint32_t b = 0; b < c.nb; ++b) {
    std::memset(lds_raw, 0xA5 ^ static_cast<int>(b & 0x3f), sizeof(lds_raw));  // a cell read before it is written shows up as wrong bytes
    for (uint32_t tid = 0; tid < kThreads; ++tid)
      mmr::transpose_load_any<HostMem, T>(c, src, b, lds, tid, tid / G::kGroupThreads);
    for (uint32_t tid = 0; tid < kThreads; ++tid)
      mmr::transpose_store_any<HostMem, T>(c, dst, b, lds, tid, tid / G::kGroupThreads);
  }
}

// Visits every workgroup of the launch grid exactly like the kernels do.
template <class Fn>
bool for_each_chunk(int64_t n, uint32_t xcd_mode, Fn&& fn) {
  const uint32_t group = mmr::xcd_group_of(n, xcd_mode);
  const uint32_t grid = mmr::grid_size(n, group);
  std::vector<uint8_t> seen(static_cast<size_t>(n), 0);
  for (uint32_t block = 0; block < grid; ++block) {
    const uint32_t ci = mmr::chunk_index(block, group);
    if (ci >= n) continue;
    if (seen[ci]++) {
      g_error = "chunk " + std::to_string(ci) + " visited twice by the workgroup mapping";
      return false;
    }
    fn(ci);
  }
  for (int64_t i = 0; i < n; ++i)
    if (!seen[i]) {
      g_error = "chunk " + std::to_string(i) + " never visited by the workgroup mapping";
      return false;
    }
  return true;
}

template <int THREADS, int UNROLL>
void run_copy16(const mmr_copy_chunk& c, const uint8_t* src, uint8_t* dst) {
  for (uint32_t tid = 0; tid < THREADS; ++tid) mmr::copy16_chunk<HostMem, THREADS, UNROLL>(c, src, dst, tid);
}
template <int THREADS, int UNROLL>
void run_generic(const mmr_copy_chunk& c, const uint8_t* src, uint8_t* dst) {
  for (uint32_t tid = 0; tid < THREADS; ++tid) mmr::generic_chunk<HostMem, THREADS, UNROLL>(c, src, dst, tid);
}

}  // namespace

extern "C" {

// slot_ptrs[i] / slot_bytes[i]: host buffer standing in for the shard buffer of
// slot i (16-byte aligned).  shape: 0 = the kernels' default (threads, unroll),
// other values pick the alternative instantiations.  Returns 0, or -1 with a
// message in err.
int mmr_emulate_plan(const mmr_plan* plan, void* const* slot_ptrs, const size_t* slot_bytes, int64_t n_slots,
                     uint32_t xcd_mode, int shape, uint64_t* bytes_loaded, uint64_t* bytes_stored, char* err,
                     size_t err_len) {
  g_ranges.clear();
  g_error.clear();
  g_loaded = g_stored = 0;
  for (int64_t i = 0; i < n_slots; ++i) {
    const uintptr_t p = reinterpret_cast<uintptr_t>(slot_ptrs[i]);
    if (p % 16) g_error = "slot buffer is not 16-byte aligned";
    g_ranges.push_back(Range{p, p + slot_bytes[i]});
  }
  auto base = [&](uint32_t slot, uint64_t off) { return static_cast<uint8_t*>(slot_ptrs[slot]) + off; };
  for (const mmr::CopyPiece& pc : plan->copy_pieces)
    if (pc.dst_slot >= n_slots || (pc.src_slot != MMR_SLOT_FILL && pc.src_slot >= n_slots))
      g_error = "piece names a slot outside the pointer table";
  for (const mmr::SpanMember& m : plan->span_members)
    if (m.dst_slot >= n_slots) g_error = "span member names a slot outside the pointer table";
  for (const mmr::SpanPiece& pc : plan->span_pieces)
    if (pc.src_slot != MMR_SLOT_FILL && pc.src_slot >= n_slots) g_error = "span piece names a slot outside the pointer table";
  const uint32_t mode = xcd_mode == 0 ? 64 : xcd_mode;
  if (g_error.empty() && plan->n_copy_chunks) {
    // the copy-group launch as the kernel runs it: the table bound to addresses, every workgroup decoding its chunk
    std::vector<mmr::CopyPiece> pieces = plan->copy_pieces;
    for (mmr::CopyPiece& pc : pieces) {
      pc.dst = reinterpret_cast<uint64_t>(base(pc.dst_slot, pc.dst));
      pc.src = pc.src_slot == MMR_SLOT_FILL ? 0 : reinterpret_cast<uint64_t>(base(pc.src_slot, pc.src));
    }
    const std::vector<uint32_t> hints = mmr::group_hints(plan->copy_groups, plan->n_copy_chunks);
    for_each_chunk(plan->n_copy_chunks, mode, [&](uint32_t ci) {
      const uint32_t gi = mmr::find_group(plan->copy_groups.data(), static_cast<uint32_t>(plan->copy_groups.size()),
                                          (shape & 1) ? nullptr : hints.data(), ci);
      const mmr::CopyGroup& g = plan->copy_groups[gi];
      if (ci < g.first_chunk || ci - g.first_chunk >= g.n_chunks) {
        g_error = "chunk " + std::to_string(ci) + " resolved to the wrong group";
        return;
      }
      const mmr::DecodedCopy d = mmr::decode_copy(g, ci - g.first_chunk);
      if (d.piece >= pieces.size() || d.n1 == 0 || d.n2 == 0) {
        g_error = "chunk " + std::to_string(ci) + " decodes to nothing";
        return;
      }
      const mmr::CopyPiece& pc = pieces[d.piece];
      const mmr_copy_chunk c = mmr::copy_chunk_of(g, pc, d);
      uint8_t* dst = reinterpret_cast<uint8_t*>(c.dst_off);
      const uint8_t* src = c.src_slot == MMR_SLOT_FILL ? dst : reinterpret_cast<const uint8_t*>(c.src_off);
      switch (shape) {  // 0 and 2 run the lean chunk code where the group allows it, 1 and 3 always the general one
        case 1: run_copy16<128, 4>(c, src, dst); break;
        case 2:
          for (uint32_t tid = 0; tid < 512; ++tid) mmr::copy_group_rows<HostMem, 512, 1>(g, pc, c, src, dst, tid);
          break;
        case 3: run_copy16<64, 8>(c, src, dst); break;
        default:
          for (uint32_t tid = 0; tid < 256; ++tid) mmr::copy_group_rows<HostMem, 256, 2>(g, pc, c, src, dst, tid);
          break;
      }
    });
  }
  if (g_error.empty() && plan->n_span_chunks) {
    std::vector<mmr::SpanMember> members = plan->span_members;
    std::vector<mmr::SpanPiece> pieces = plan->span_pieces;
    for (mmr::SpanMember& m : members) m.dst = reinterpret_cast<uint64_t>(base(m.dst_slot, m.dst));
    for (mmr::SpanPiece& pc : pieces)
      pc.src = pc.src_slot == MMR_SLOT_FILL ? 0 : reinterpret_cast<uint64_t>(base(pc.src_slot, pc.src));
    alignas(16) static thread_local uint8_t safe[16];
    g_ranges.push_back(Range{reinterpret_cast<uintptr_t>(safe), reinterpret_cast<uintptr_t>(safe) + 16});
    alignas(16) static thread_local uint8_t lds[mmr::kSpanLdsBytes];
    g_lds_lo = lds;
    g_lds_hi = lds + sizeof(lds);
    const std::vector<uint32_t> hints = mmr::group_hints(plan->span_groups, plan->n_span_chunks);
    for_each_chunk(plan->n_span_chunks, mode, [&](uint32_t ci) {
      const uint32_t gi = mmr::find_group(plan->span_groups.data(), static_cast<uint32_t>(plan->span_groups.size()),
                                          (shape & 1) ? nullptr : hints.data(), ci);
      const mmr::SpanGroup& g = plan->span_groups[gi];
      if (ci < g.first_chunk || ci - g.first_chunk >= g.n_chunks) {
        g_error = "span chunk " + std::to_string(ci) + " resolved to the wrong group";
        return;
      }
      uint32_t member, lm;
      mmr::deinterleave(g.il, ci - g.first_chunk, &member, &lm);
      if (member >= g.il.members || lm >= g.il.member_chunks) {
        g_error = "span chunk " + std::to_string(ci) + " decodes outside its group";
        return;
      }
      const mmr::SpanMember& m = members[g.first_member + member];
      uint64_t x0;
      uint32_t len;
      mmr::span_range(g, lm, &x0, &len);
      if (len == 0 || len > g.span || x0 + len > g.band_bytes) {
        g_error = "span chunk " + std::to_string(ci) + " covers a bad range";
        return;
      }
      uint8_t* dst = reinterpret_cast<uint8_t*>(m.dst + x0);
      const uint32_t a = static_cast<uint32_t>(m.dst + x0) & 15u;
      std::memset(lds, 0xA5 ^ static_cast<int>(ci & 0x3f), sizeof(lds));
      // a phase runs for every thread before the next one starts: the workgroup barrier
      // shape 0 is the kernel's own launch shape; 1 runs the vector-by-vector gather on every group, also those the
      // kernel uses a segment table for; 2 and 3 are other widths and depths of both
      const mmr::SpanPiece* pc = pieces.data() + m.first_piece;
      uint8_t* table = lds + mmr::kSpanStageBytes;
      auto with_table = [&](auto lanes_c, auto depth_c) {
        constexpr int LANES = decltype(lanes_c)::value, DEPTH = decltype(depth_c)::value;
        const mmr::SpanPieces4 pcs = mmr::span_pieces4(pc, m.k);
        std::vector<mmr::SpanRowEnds<HostMem>> starts(LANES);
        for (uint32_t tid = 0; tid < LANES; ++tid)
          starts[tid] = mmr::span_table_build<HostMem, HostLds, LANES>(g, m, pcs, safe, x0, len, a, table, tid);
        for (uint32_t tid = 0; tid < LANES; ++tid)
          mmr::span_table_gather<HostMem, HostLds, LANES, DEPTH>(g, m, pc, pcs, safe, x0, len, a, lds, table, starts[tid], tid);
        for (uint32_t tid = 0; tid < LANES; ++tid) mmr::span_write<HostMem, HostLds, LANES, DEPTH>(dst, len, a, lds, tid);
      };
      auto without = [&](auto threads_c, auto unroll_c) {
        constexpr int THREADS = decltype(threads_c)::value, UNROLL = decltype(unroll_c)::value;
        for (uint32_t tid = 0; tid < THREADS; ++tid)
          mmr::span_gather<HostMem, HostLds, THREADS, UNROLL>(g, m, pieces.data(), safe, x0, len, a, lds, tid);
        for (uint32_t tid = 0; tid < THREADS; ++tid) mmr::span_write<HostMem, HostLds, THREADS, UNROLL>(dst, len, a, lds, tid);
      };
      using std::integral_constant;
      switch (shape) {
        case 1:
          without(integral_constant<int, 128>{}, integral_constant<int, 4>{});
          break;
        case 2:
          if (g.table_mode) with_table(integral_constant<int, 64>{}, integral_constant<int, 5>{});
          else without(integral_constant<int, 256>{}, integral_constant<int, 1>{});
          break;
        case 3:
          if (g.table_mode) with_table(integral_constant<int, 64>{}, integral_constant<int, 8>{});
          else without(integral_constant<int, 32>{}, integral_constant<int, 3>{});
          break;
        default:
          if (g.table_mode) with_table(integral_constant<int, mmr::kSpanLanes>{}, integral_constant<int, mmr::kSpanDepth>{});
          else without(integral_constant<int, mmr::kSpanLanes>{}, integral_constant<int, mmr::kSpanDepth>{});
          break;
      }
    });
  }
  if (g_error.empty()) {
    const int64_t n = mmr_plan_get_copy_chunks(plan, 1, nullptr, 0);
    std::vector<mmr_copy_chunk> chunks(static_cast<size_t>(n));
    mmr_plan_get_copy_chunks(plan, 1, chunks.data(), n);
    for_each_chunk(n, mode, [&](uint32_t ci) {
      const mmr_copy_chunk& c = chunks[ci];
      if (c.dst_slot >= n_slots || (c.src_slot != MMR_SLOT_FILL && c.src_slot >= n_slots)) {
        g_error = "chunk names a slot outside the pointer table";
        return;
      }
      uint8_t* dst = base(c.dst_slot, c.dst_off);
      const uint8_t* src = c.src_slot == MMR_SLOT_FILL ? dst : base(c.src_slot, c.src_off);
      if (c.n2 != 1) g_error = "generic chunk with n2 != 1";
      switch (shape) {
        case 1: run_generic<128, 4>(c, src, dst); break;
        case 2: run_generic<256, 1>(c, src, dst); break;
        case 3: run_generic<256, 4>(c, src, dst); break;
        default: run_generic<256, 2>(c, src, dst); break;
      }
    });
  }
  if (g_error.empty()) {
    const int64_t n = mmr_plan_get_transpose_chunks(plan, nullptr, 0);
    std::vector<mmr_transpose_chunk> chunks(static_cast<size_t>(n));
    mmr_plan_get_transpose_chunks(plan, chunks.data(), n);
    for_each_chunk(n, xcd_mode, [&](uint32_t ci) {
      const mmr_transpose_chunk& c = chunks[ci];
      if (c.dst_slot >= n_slots || c.src_slot >= n_slots) {
        g_error = "chunk names a slot outside the pointer table";
        return;
      }
      const uint8_t* src = base(c.src_slot, c.src_off);
      uint8_t* dst = base(c.dst_slot, c.dst_off);
      uint32_t tile_x = 0, tile_y = 0;
      mmr::transpose_tile_extent(c.itemsize, &tile_x, &tile_y);
      if (!mmr::transpose_is_thin(c) && (c.nx > tile_x || c.ny > tile_y)) {  // thin chunks: checked against LDS below
        g_error = "transpose tile larger than the LDS tile";
        return;
      }
      switch (c.itemsize) {
        case 1: run_transpose<uint8_t>(c, src, dst); break;
        case 2: run_transpose<uint16_t>(c, src, dst); break;
        case 4: run_transpose<uint32_t>(c, src, dst); break;
        case 8: run_transpose<uint64_t>(c, src, dst); break;
        default: run_transpose<mmr::V16>(c, src, dst); break;
      }
    });
  }
  if (bytes_loaded) *bytes_loaded = g_loaded;
  if (bytes_stored) *bytes_stored = g_stored;
  if (!g_error.empty()) {
    if (err && err_len) std::snprintf(err, err_len, "%s", g_error.c_str());
    return -1;
  }
  return 0;
}

}  // extern "C"
