// Group tables: the plan of a launch as a handful of records, decoded by arithmetic.
//
// A reshard is a set of boxes (source tile x destination tile overlaps).  Boxes
// that lie side by side in the same destination rows form a GROUP: k pieces that
// share their row structure.  A launch is a short table of groups plus their
// pieces; workgroup i finds its group from the table's prefix of chunk counts
// and works out its piece and its rows from i alone.  The table of a 1 GiB
// reshard is a few KiB (it used to be one 72-byte record per 8 KiB of payload),
// small enough to ride in the kernel's argument block, and it holds absolute
// addresses once it is bound to a set of shard buffers, so a workgroup reaches
// its first global load without a chain of dependent table loads.
//
// Two kinds of group:
//   * copy groups - every offset, stride and width a multiple of 16 bytes; a
//     chunk is a block of rows of ONE piece (copy16_rows of chunk_ops.h);
//   * span groups - ragged rows.  The destination tile is dense, so a chunk is
//     a SPAN of destination bytes cut at multiples of the span size counted from
//     the buffer's base: the workgroup gathers the pieces of every row that
//     touches the span into LDS, laid out as the destination is (16-byte global
//     loads and LDS writes at any byte alignment), and then writes the span out as whole
//     aligned 16-byte vectors - no partial line ever reaches memory from the
//     middle of a tile.
// The same code runs on the GPU (kernels.hip) and, with a bounds-checking
// memory policy, on the host (the tests' kernel emulation).
#ifndef MMR_CSRC_GROUP_OPS_H_
#define MMR_CSRC_GROUP_OPS_H_

#include <cstdint>

#include "chunk_ops.h"

namespace mmr {

// n / d for n < 2^31 as a multiplication: mulhi(2 n, mul) >> shift (one multiply-high, two shifts).
struct FastDiv {
  uint32_t mul;
  uint32_t shift;
};

inline FastDiv make_fastdiv(uint32_t d) {  // d >= 1
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;
  // mul = ceil(2^(31+l) / d) < 2^32 because 2^(l-1) < d; (n * mul) >> (31 + l) is exact for every n < 2^31
  // (Granlund & Montgomery, N = 31), and (2 n * mul) >> 32 >> l is the same number
  const uint64_t m = ((1ull << (31 + l)) + d - 1) / d;
  return FastDiv{static_cast<uint32_t>(m), l};
}

MMR_HD uint32_t mulhi32(uint32_t a, uint32_t b) { return static_cast<uint32_t>((static_cast<uint64_t>(a) * b) >> 32); }

// a * b for a, b < 2^24 (full rate on the vector ALU, where a 32-bit multiply takes four times as long)
MMR_HD uint32_t mul24(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__) && __has_builtin(__builtin_amdgcn_mul_u24)
  return __builtin_amdgcn_mul_u24(a, b);
#else
  return a * b;
#endif
}

MMR_HD uint32_t fdiv(uint32_t n, FastDiv f) { return mulhi32(n << 1, f.mul) >> f.shift; }

// How the chunks of `members` congruent destination tiles are interleaved in a launch: rounds of `fraction` chunks
// of every member in turn (the last round may be shorter).  members = 1 is plain order.
struct Interleave {
  uint32_t members;
  uint32_t fraction;       // chunks of one member per round
  uint32_t member_chunks;  // chunks of one member
  uint32_t full_rounds;    // member_chunks / fraction
  uint32_t last_fraction;  // member_chunks % fraction (0: no short round)
  FastDiv div_round;       // by members * fraction
  FastDiv div_fraction;
  FastDiv div_last;        // by last_fraction (or 1)
};

inline Interleave make_interleave(uint32_t members, uint32_t member_chunks, uint32_t fraction) {
  Interleave il{};
  il.members = members;
  il.member_chunks = member_chunks;
  il.fraction = fraction < 1 ? 1 : (fraction > member_chunks ? member_chunks : fraction);
  if (members == 1) il.fraction = member_chunks;
  il.full_rounds = member_chunks / il.fraction;
  il.last_fraction = member_chunks % il.fraction;
  il.div_round = make_fastdiv(members * il.fraction);
  il.div_fraction = make_fastdiv(il.fraction);
  il.div_last = make_fastdiv(il.last_fraction ? il.last_fraction : 1);
  return il;
}

// Chunk `local` of an interleaved group -> (member, chunk of that member).  Branch-free: both kinds of round are
// worked out and one is kept, so that a kernel's table reads stay in one basic block and leave together.
MMR_HD void deinterleave(const Interleave& il, uint32_t local, uint32_t* member, uint32_t* member_chunk) {
  const uint32_t round = fdiv(local, il.div_round);
  const uint32_t rem = local - round * il.members * il.fraction;
  const bool full = round < il.full_rounds;
  const uint32_t t_full = fdiv(rem, il.div_fraction), t_last = fdiv(rem, il.div_last);
  const uint32_t t = full ? t_full : t_last;
  const uint32_t i = rem - t * (full ? il.fraction : il.last_fraction);
  *member = t;
  *member_chunk = round * il.fraction + i;
}

// ---------------------------------------------------------------------------
// Copy groups
// ---------------------------------------------------------------------------
struct CopyPiece {
  uint64_t src;       // plan: byte offset inside the source slot's buffer; bound table: absolute address
  uint64_t dst;       // the same for the destination
  uint32_t src_slot;  // MMR_SLOT_FILL: the piece writes zeros (pad of a short edge tile)
  uint32_t dst_slot;
  int64_t s1, s2, s3;  // source byte strides of the group's row dims
  uint32_t w;          // contiguous bytes per row
  uint32_t reserved;
  FastDiv div_wv;      // by w / 16
};

struct CopyGroup {
  uint32_t first_chunk;  // index of the group's first chunk in its launch
  uint32_t n_chunks;
  uint32_t first_piece;  // pieces [first_piece, first_piece + members * k), member after member
  uint32_t k;            // pieces per member: boxes side by side in the same destination rows
  uint32_t n1, n2, n3;   // rows along the fast, the slow and the outermost row dim
  uint32_t m1, m2;       // rows per chunk along the first two (one index of the third per chunk)
  uint32_t c1;           // chunks along the fast row dim = ceil(n1 / m1)
  uint32_t c12;          // chunks per index of the outermost dim = c1 * ceil(n2 / m2)
  uint32_t lean;         // 0: general chunk code; 1: every chunk of the group is one pass of kLeanVectors vectors at
                         // most and every offset inside a chunk fits 32 bits; 2: and all strides fit 24 bits
  FastDiv div_m1, div_last1;  // by the rows of a chunk along the fast dim: m1, or what is left in the last block
  int64_t d1, d2, d3;    // destination byte strides of the row dims
  FastDiv div_k, div_c1, div_c12;
  Interleave il;
};

struct DecodedCopy {
  uint32_t piece;   // index into the launch's piece table
  uint32_t r1, r2, r3;  // first row of the chunk along each row dim
  uint32_t n1, n2;      // rows of this chunk along the first two
};

// Chunk `local` of group g: the chunks of a member run row block after row block, the k pieces of a row block side by
// side (destination address order).
MMR_HD DecodedCopy decode_copy(const CopyGroup& g, uint32_t local) {
  uint32_t member, lm;
  deinterleave(g.il, local, &member, &lm);
  const uint32_t rb = fdiv(lm, g.div_k), j = lm - rb * g.k;
  const uint32_t b3 = fdiv(rb, g.div_c12), rb12 = rb - b3 * g.c12;
  const uint32_t b2 = fdiv(rb12, g.div_c1), b1 = rb12 - b2 * g.c1;
  DecodedCopy d;
  d.piece = g.first_piece + member * g.k + j;
  d.r1 = b1 * g.m1;
  d.r2 = b2 * g.m2;
  d.r3 = b3;
  d.n1 = g.n1 - d.r1 < g.m1 ? g.n1 - d.r1 : g.m1;
  d.n2 = g.n2 - d.r2 < g.m2 ? g.n2 - d.r2 : g.m2;
  return d;
}

constexpr uint32_t kLeanVectors = 512;  // 256 lanes x 2 vectors: the kernel's launch shape

// Lean chunk code for the common case (CopyGroup::lean): one pass, no loop, 32-bit offsets from the chunk's first
// byte, divisions by multiplication.  A lane past the end repeats the chunk's last vector.  SMALL: strides < 2^24.
template <class M, int THREADS, int UNROLL, bool FILL, bool SMALL>
MMR_HD void copy16_lean(uint32_t wv, FastDiv div_wv, uint32_t n1c, FastDiv div_n1c, uint32_t n2c, uint32_t s1, uint32_t d1,
                        uint32_t s2, uint32_t d2, typename M::cptr src, typename M::ptr dst, uint32_t tid) {
  const uint32_t total = n1c * n2c * wv;
  V16 v[UNROLL];
  uint32_t soff[UNROLL], doff[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    uint32_t idx = tid + u * THREADS;
    idx = idx < total ? idx : total - 1;
    const uint32_t row = fdiv(idx, div_wv);
    const uint32_t col = idx - (SMALL ? mul24(row, wv) : row * wv);
    uint32_t r1 = row, r2 = 0;
    if (n2c > 1) {  // uniform
      r2 = fdiv(row, div_n1c);
      r1 = row - (SMALL ? mul24(r2, n1c) : r2 * n1c);
    }
    soff[u] = (SMALL ? mul24(r2, s2) + mul24(r1, s1) : r2 * s2 + r1 * s1) + (col << 4);
    doff[u] = (SMALL ? mul24(r2, d2) + mul24(r1, d1) : r2 * d2 + r1 * d1) + (col << 4);
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) v[u] = FILL ? V16{0, 0, 0, 0} : M::load16(src + soff[u]);
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) M::store16(dst + doff[u], v[u]);
}

// One chunk of a copy group, by whichever code the group allows.  c: the decoded chunk (its offsets count from src /
// dst); lean_ok: the caller's launch shape is the one CopyGroup::lean was worked out for.
template <class M, int THREADS, int UNROLL>
MMR_HD void copy_group_rows(const CopyGroup& g, const CopyPiece& p, const mmr_copy_chunk& c, typename M::cptr src,
                            typename M::ptr dst, uint32_t tid) {
  const bool fill = c.src_slot == MMR_SLOT_FILL;  // uniform over the workgroup, like everything below
  if (g.lean != 0 && THREADS * UNROLL == kLeanVectors) {
    const uint32_t wv = c.w >> 4;
    const FastDiv div_n1c = c.n1 == g.m1 ? g.div_m1 : g.div_last1;
    const uint32_t s1 = static_cast<uint32_t>(c.s1), d1 = static_cast<uint32_t>(c.d1);
    const uint32_t s2 = static_cast<uint32_t>(c.s2), d2 = static_cast<uint32_t>(c.d2);
    if (g.lean == 2) {
      if (fill) copy16_lean<M, THREADS, UNROLL, true, true>(wv, p.div_wv, c.n1, div_n1c, c.n2, s1, d1, s2, d2, src, dst, tid);
      else copy16_lean<M, THREADS, UNROLL, false, true>(wv, p.div_wv, c.n1, div_n1c, c.n2, s1, d1, s2, d2, src, dst, tid);
    } else {
      if (fill) copy16_lean<M, THREADS, UNROLL, true, false>(wv, p.div_wv, c.n1, div_n1c, c.n2, s1, d1, s2, d2, src, dst, tid);
      else copy16_lean<M, THREADS, UNROLL, false, false>(wv, p.div_wv, c.n1, div_n1c, c.n2, s1, d1, s2, d2, src, dst, tid);
    }
    return;
  }
  copy16_chunk<M, THREADS, UNROLL>(c, src, dst, tid);
}

// The chunk record copy16_rows takes, from a decoded chunk and its piece: src_off / dst_off count from the piece's
// src / dst (slot-relative offsets in a plan, absolute addresses in a bound table).
MMR_HD mmr_copy_chunk copy_chunk_of(const CopyGroup& g, const CopyPiece& p, const DecodedCopy& d) {
  mmr_copy_chunk c;
  c.src_slot = p.src_slot;
  c.dst_slot = p.dst_slot;
  c.src_off = p.src_slot == MMR_SLOT_FILL ? 0 : p.src + static_cast<uint64_t>(d.r3 * p.s3 + d.r2 * p.s2 + d.r1 * p.s1);
  c.dst_off = p.dst + static_cast<uint64_t>(d.r3 * g.d3 + d.r2 * g.d2 + d.r1 * g.d1);
  c.w = p.w;
  c.n1 = d.n1;
  c.n2 = d.n2;
  c.align = 16;
  c.s1 = p.s1;
  c.d1 = g.d1;
  c.s2 = p.s2;
  c.d2 = g.d2;
  return c;
}

// ---------------------------------------------------------------------------
// Span groups
// ---------------------------------------------------------------------------
constexpr uint32_t kSpanMaxBytes = 4 * 1024;           // largest span a workgroup (one wavefront) stages in LDS
constexpr uint32_t kSpanLanes = 64, kSpanDepth = 4;     // the span kernel's launch shape: lanes x 16-byte vectors each
constexpr uint32_t kSpanTablePieces = 4;                // most pieces per row of a group whose spans use a segment table
constexpr uint32_t kSpanStageBytes = kSpanMaxBytes + 64;  // 16 spare bytes in front, up to 15 of phase, 16 + 16 spare behind
constexpr uint32_t kSpanLdsBytes = kSpanStageBytes + kSpanLanes * 16;  // and a 16-byte segment record per lane
constexpr uint32_t kSpanMaxRowBytes = 1u << 28;

struct SpanPiece {
  uint64_t src;         // plan: byte offset of the piece's first row inside the source slot's buffer; bound: address
  uint32_t src_slot;    // MMR_SLOT_FILL: zeros
  uint32_t col;         // first byte of the piece within the destination row; the pieces of a member tile [0, W)
  int64_t s1, s2;       // source byte strides of row % n1 and row / n1
  uint32_t w;           // bytes per row; "wide" pieces have w >= 16
  uint32_t wide_index;  // wide pieces: how many wide pieces of the member come before this one
};

struct SpanMember {   // one destination tile's band
  uint64_t dst;       // plan: byte offset of the band inside the destination slot's buffer; bound: address
  uint32_t dst_slot;
  uint32_t first_piece, k;  // pieces in ascending col order
  uint32_t wide;            // how many of them are wide
  FastDiv div_wide;         // by max(wide, 1)
  uint32_t narrow;          // ... and how many narrower than 16 bytes
  uint32_t reserved;
  FastDiv div_k;
};

struct SpanGroup {
  uint32_t first_chunk, n_chunks;
  uint32_t first_member;
  uint32_t W;           // bytes per destination row; rows abut (the band is dense)
  uint64_t band_bytes;  // rows * W
  uint32_t n1;          // rows per index of the slow row dim
  uint32_t span;        // bytes per chunk, a multiple of 128
  uint32_t head;        // bytes of the first chunk: the later ones start at multiples of `span` from the buffer's base
  uint32_t table_mode;  // 1: at most kSpanTablePieces pieces per row and at most kSpanLanes (row, piece) pairs touch a
                        // span: the lanes work those pairs out once, one each (span_table_build / span_table_gather)
  FastDiv div_W, div_n1;
  Interleave il;
};

// Byte range [*x0, *x0 + *len) of a member's band covered by chunk lm.
MMR_HD void span_range(const SpanGroup& g, uint32_t lm, uint64_t* x0, uint32_t* len) {
  if (lm == 0) {
    *x0 = 0;
    *len = g.band_bytes < g.head ? static_cast<uint32_t>(g.band_bytes) : g.head;
    return;
  }
  *x0 = g.head + static_cast<uint64_t>(lm - 1) * g.span;
  const uint64_t left = g.band_bytes - *x0;
  *len = left < g.span ? static_cast<uint32_t>(left) : g.span;
}

inline uint32_t span_chunks(uint64_t band_bytes, uint32_t head, uint32_t span) {
  if (band_bytes <= head) return 1;
  return 1 + static_cast<uint32_t>((band_bytes - head + span - 1) / span);
}

// An LDS policy `L` provides (pointers are byte pointers into the workgroup's staging array)
//   static void store16u(uint8_t*, V16);  16-byte store at any alignment
//   static void store8(uint8_t*, uint8_t);
//   static V16 load16(const uint8_t*);    16-byte aligned load
//   static uint8_t load8(const uint8_t*);

// Phase 1 of a span chunk: the span's bytes are gathered into LDS, laid out as the destination has them.
// `a` = (address of the span's first destination byte) & 15; LDS offset 16 + a + i holds span byte i, so the 16-byte
// vectors of the destination are 16-byte aligned in LDS as well.  Two kinds of item:
//   A  one per aligned destination vector of the span: the 16 source bytes that start where the vector's first byte
//      comes from; if the row piece ends before the vector does, the load slides back to end with the piece (it then
//      lands in LDS at an odd offset and overlaps its neighbour, same values).  A vector that begins in a piece
//      narrower than 16 bytes or in a pad loads nothing.
//   B  one per (row that touches the span, wide piece): the first 16 bytes of the row piece - the bytes a vector of
//      kind A that began in the previous piece (or row) could not bring.
// Then the narrow pieces, byte by byte.  Every byte of the span is written by at least one item because the pieces
// tile the row.  Items that lie outside the span land in the spare bytes around it.  `safe` is any address 16 bytes
// can be read from (the load of an item that needs none goes there: loads are never predicated, so they leave
// back to back; the LDS writes of lanes without an item are).
// The fields of the piece a lane's item falls into, gathered by per-lane selects over the (uniform) piece list.
struct SpanPick {
  uint64_t src = 0;
  int64_t s1 = 0, s2 = 0;
  uint32_t pcol = 0, w = 0, src_slot = MMR_SLOT_FILL;
  MMR_HD void take(bool yes, const SpanPiece& c) {
    src = yes ? c.src : src;
    s1 = yes ? c.s1 : s1;
    s2 = yes ? c.s2 : s2;
    pcol = yes ? c.col : pcol;
    w = yes ? c.w : w;
    src_slot = yes ? c.src_slot : src_slot;
  }
};

// Where an item loads from (`from`; `zero`: it loads nothing and stores zeros) and where its 16 bytes go in LDS.
// rr: row of the span (0 = the row the span starts in), pos: first byte wanted within the piece's row.
template <class M>
MMR_HD void span_item(const SpanGroup& g, const SpanPick& pk, uint32_t r0, uint32_t rr, uint32_t pos, uint32_t o0,
                      int32_t ilen, uint32_t a, typename M::cptr safe, typename M::cptr* from, bool* zero, uint32_t* at) {
  const bool wide = pk.w >= 16;
  const uint32_t lo = wide ? (pos + 16 > pk.w ? pk.w - 16 : pos) : 0u;  // slides back to end with the row piece
  const uint32_t row = r0 + rr;
  const uint32_t r2 = fdiv(row, g.div_n1), r1 = row - r2 * g.n1;
  const bool no_load = !wide || pk.src_slot == MMR_SLOT_FILL;
  *from = no_load ? safe : reinterpret_cast<typename M::cptr>(pk.src) + (r2 * pk.s2 + r1 * pk.s1 + static_cast<int64_t>(lo));
  *zero = no_load;
  int32_t drel = static_cast<int32_t>(rr * g.W + pk.pcol + lo) - static_cast<int32_t>(o0);  // relative to the span
  drel = !wide || drel < -16 ? -16 : (drel > ilen ? ilen : drel);  // outside the span: into the spare bytes
  *at = static_cast<uint32_t>(16 + static_cast<int32_t>(a) + drel);
}

// The pieces narrower than 16 bytes of the rows that touch the span (uniform loop over the pieces): one byte per item.
template <class M, class L, int THREADS>
MMR_HD void span_gather_narrow(const SpanGroup& g, const SpanPiece* pc, uint32_t k, uint32_t nrows, uint32_t r0,
                               uint32_t o0, int32_t ilen, uint32_t a, uint8_t* lds, uint32_t tid) {
  for (uint32_t p = 0; p < k; ++p) {
    const SpanPiece& c = pc[p];
    if (c.w >= 16) continue;
    const uint32_t total_n = nrows * c.w;
    for (uint32_t i = tid; i < total_n; i += THREADS) {
      const uint32_t r = i / c.w, b = i - r * c.w;
      const int32_t drel = static_cast<int32_t>(r * g.W + c.col + b) - static_cast<int32_t>(o0);
      if (drel < 0 || drel >= ilen) continue;
      uint8_t value = 0;
      if (c.src_slot != MMR_SLOT_FILL) {
        const uint32_t row = r0 + r;
        const uint32_t r2 = fdiv(row, g.div_n1), r1 = row - r2 * g.n1;
        value = M::template loadu<uint8_t>(reinterpret_cast<typename M::cptr>(c.src) + (r2 * c.s2 + r1 * c.s1 + static_cast<int64_t>(b)));
      }
      L::store8(lds + 16 + a + static_cast<uint32_t>(drel), value);
    }
  }
}

template <class M, class L, int THREADS, int UNROLL>
MMR_HD void span_gather(const SpanGroup& g, const SpanMember& m, const SpanPiece* pieces, typename M::cptr safe,
                        uint64_t x0, uint32_t len, uint32_t a, uint8_t* lds, uint32_t tid) {
  const uint32_t W = g.W;
  // row the span starts in: one division per workgroup (by multiplication while the offset allows it)
  const uint64_t row0 = x0 < (1ull << 31) ? fdiv(static_cast<uint32_t>(x0), g.div_W) : x0 / W;
  const uint32_t o0 = static_cast<uint32_t>(x0 - row0 * W);
  const uint32_t nrows = fdiv(o0 + len + W - 1, g.div_W);
  const uint32_t r0 = static_cast<uint32_t>(row0);
  const SpanPiece* pc = pieces + m.first_piece;
  const uint32_t k = m.k, kw = m.wide;
  const int32_t ilen = static_cast<int32_t>(len);
  const uint32_t n_a = (len + a + 15) >> 4;  // aligned destination vectors that overlap the span
  const uint32_t n_b = nrows * kw;           // (row, wide piece) pairs
  // Kind A in passes of UNROLL per lane, kind B one per lane and pass; the first pass of both is issued together, so
  // a span of up to THREADS * UNROLL vectors whose rows hold up to THREADS pieces waits for memory once.
  for (uint32_t base_a = 0, base_b = 0; base_a < n_a || base_b < n_b; base_a += THREADS * UNROLL, base_b += THREADS) {
    uint32_t rr[UNROLL + 1], pos[UNROLL + 1], key[UNROLL + 1];
    bool live[UNROLL + 1];
    SpanPick pk[UNROLL + 1];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {  // the row piece the vector's first in-span byte comes from
      const uint32_t i = base_a + tid + u * THREADS;
      live[u] = i < n_a;
      const uint32_t v16 = i << 4;
      const uint32_t y = o0 + (!live[u] || v16 < a ? 0u : v16 - a);
      rr[u] = fdiv(y, g.div_W);
      key[u] = y - rr[u] * W;  // column
    }
    {
      const uint32_t t = base_b + tid;
      live[UNROLL] = t < n_b;
      rr[UNROLL] = live[UNROLL] ? fdiv(t, m.div_wide) : 0u;
      key[UNROLL] = live[UNROLL] ? t - rr[UNROLL] * kw : 0u;  // index among the wide pieces
    }
    for (uint32_t p = 0; p < k; ++p) {  // uniform loop; the pieces are in ascending col order
      const SpanPiece c = pc[p];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) pk[u].take(key[u] >= c.col, c);
      pk[UNROLL].take(c.w >= 16 && key[UNROLL] >= c.wide_index, c);
    }
    V16 v[UNROLL + 1];
    uint32_t at[UNROLL + 1];
    bool zero[UNROLL + 1];
    typename M::cptr from[UNROLL + 1];
#pragma unroll
    for (int u = 0; u <= UNROLL; ++u) {
      pos[u] = u < UNROLL ? key[u] - pk[u].pcol : 0u;
      span_item<M>(g, pk[u], r0, rr[u], pos[u], o0, ilen, a, safe, &from[u], &zero[u], &at[u]);
      from[u] = live[u] ? from[u] : safe;
    }
#pragma unroll
    for (int u = 0; u <= UNROLL; ++u) v[u] = M::load16u(from[u]);
#pragma unroll
    for (int u = 0; u <= UNROLL; ++u)
      if (live[u]) L::store16u(lds + at[u], zero[u] ? V16{0, 0, 0, 0} : v[u]);
  }
  if (m.narrow) span_gather_narrow<M, L, THREADS>(g, pc, k, nrows, r0, o0, ilen, a, lds, tid);
}

// Phase 1 with a segment table (SpanGroup::table_mode).  span_gather finds the row and the piece of every
// destination vector and works out its source address lane by lane, some 150 vector instructions per 16 bytes.  Here
// the (row, piece) pairs that touch the span - its SEGMENTS, at most one per lane - are worked out once, lane s
// taking segment s, and left in LDS as 16-byte records; an item then needs one division for its row, a few compares
// for its piece, one LDS read and an add.
//
// Items of a span in table mode:
//   A  one per aligned destination vector of the span, belonging to the segment the vector's first in-span byte
//      lies in: the 16 source bytes that start where that byte comes from (an unaligned load); if the piece row ends
//      before the vector does, the load slides back to end with the row.
//   B  one per segment: the first 16 bytes of the piece row (what a vector that began in the previous segment
//      could not bring).
// Two variations are kept as build options.  Both do what they were made for and neither makes the kernel faster
// (3-way -> 5-way rows of 4,099 bytes on MI355X: 20.4 us as shipped, 20.8-21.4 us with either or both):
//   MMR_SPAN_ALIGNED_LOADS  A items load the ALIGNED 16-byte vector of the source that holds their first byte
//      (clamped to the piece row; all A items of a segment are shifted by the same amount, so they tile its
//      middle), and a third kind of item, C, brings the last 16 bytes of the piece row or of its part inside the
//      span.  A third fewer accesses in the vector L1 (3.19 M against 4.77 M per launch).
//   MMR_SPAN_KEEP_EDGES  loads that touch the first or the last 128-byte line of their piece row - the lines that
//      also hold bytes of the neighbouring piece, which the span of the neighbouring destination tile reads at
//      about the same time - go through the caches in the ordinary way (M::load16u_keep), everything in between
//      keeps the streaming hint.  Memory reads fall from 1.085 x to 1.013 x the source bytes.
#ifndef MMR_SPAN_ALIGNED_LOADS
#define MMR_SPAN_ALIGNED_LOADS 0
#endif
#ifndef MMR_SPAN_KEEP_EDGES
#define MMR_SPAN_KEEP_EDGES 0
#endif
constexpr bool kSpanAlignedLoads = MMR_SPAN_ALIGNED_LOADS != 0;
constexpr bool kSpanKeepEdges = MMR_SPAN_KEEP_EDGES != 0;

struct SpanSegment {   // 16 bytes in LDS
  uint32_t d_lo, d_hi;  // (address of the piece row's first byte) - start, so that destination position y reads at d + y
  uint32_t w_flags;     // bits 0-29: bytes of the piece row; bits 30-31: 0 load, 1 the piece is a pad (zeros),
                        // 2 narrower than 16 bytes (gathered byte by byte)
  int32_t end16;        // start + w - 16: the last position a 16-byte vector of this piece row may begin at
};
// The items of kind B and C a lane brings from span_table_build to span_table_gather.
template <class M>
struct SpanRowEnds {
  typename M::cptr from_b, from_c;
  uint32_t at_b, at_c;
  bool on, zero;
};

struct SpanPieces4 {  // the first pieces of a member, read once by the wavefront (uniform)
  SpanPiece c0, c1, c2, c3;
};
MMR_HD SpanPieces4 span_pieces4(const SpanPiece* pc, uint32_t k) {
  return SpanPieces4{pc[0], pc[k > 1 ? 1 : 0], pc[k > 2 ? 2 : 0], pc[k > 3 ? 3 : 0]};
}

template <class M, class L, int LANES>
MMR_HD SpanRowEnds<M> span_table_build(const SpanGroup& g, const SpanMember& m, const SpanPieces4& pcs,
                                       typename M::cptr safe, uint64_t x0, uint32_t len, uint32_t a, uint8_t* table,
                                       uint32_t lane) {
  const uint32_t W = g.W;
  const uint64_t row0 = x0 < (1ull << 31) ? fdiv(static_cast<uint32_t>(x0), g.div_W) : x0 / W;
  const uint32_t o0 = static_cast<uint32_t>(x0 - row0 * W);
  const uint32_t nrows = fdiv(o0 + len + W - 1, g.div_W);
  const uint32_t r0 = static_cast<uint32_t>(row0);
  const uint32_t k = m.k;
  const int32_t ilen = static_cast<int32_t>(len);
  const bool on = lane < nrows * k;  // planner: nrows * k <= LANES in table mode
  const uint32_t s = on ? lane : 0u;
  const uint32_t rr = fdiv(s, m.div_k), p = s - rr * k;
  SpanPick pk;
  pk.take(true, pcs.c0);
  if (k > 1) pk.take(p >= 1, pcs.c1);
  if (k > 2) pk.take(p >= 2, pcs.c2);
  if (k > 3) pk.take(p >= 3, pcs.c3);
  const uint32_t row = r0 + rr;
  const uint32_t r2 = fdiv(row, g.div_n1), r1 = row - r2 * g.n1;
  const uint64_t src_row = pk.src + static_cast<uint64_t>(r2 * pk.s2 + r1 * pk.s1);
  const int32_t start = static_cast<int32_t>(rr * W + pk.pcol) - static_cast<int32_t>(o0);
  const bool wide = pk.w >= 16, fill = pk.src_slot == MMR_SLOT_FILL;
  SpanSegment seg;
  const uint64_t d = src_row - static_cast<uint64_t>(static_cast<int64_t>(start));
  seg.d_lo = static_cast<uint32_t>(d);
  seg.d_hi = static_cast<uint32_t>(d >> 32);
  seg.w_flags = pk.w | ((!wide ? 2u : (fill ? 1u : 0u)) << 30);  // planner: w <= kSpanMaxRowBytes < 2^30
  seg.end16 = wide ? start + static_cast<int32_t>(pk.w) - 16 : -16;  // narrow: its vectors land in the spare bytes
  if (on) L::store16u(table + (s << 4), V16{seg.d_lo, seg.d_hi, seg.w_flags, static_cast<uint32_t>(seg.end16)});
  SpanRowEnds<M> b;
  b.on = on && wide;
  b.zero = fill;
  const bool loads = b.on && !fill;
  // C begins where the piece row's last 16 bytes do, or the span's if the row runs on, and never before the row
  int32_t c = seg.end16 < ilen - 16 ? seg.end16 : ilen - 16;
  c = c < start ? start : c;
  b.from_b = loads ? reinterpret_cast<typename M::cptr>(src_row) : safe;
  b.from_c = loads ? reinterpret_cast<typename M::cptr>(src_row + static_cast<uint64_t>(static_cast<int64_t>(c - start))) : safe;
  // outside the span: into the spare bytes around it
  const int32_t drel_b = start < -16 ? -16 : (start > ilen ? ilen : start);
  const int32_t drel_c = c < -16 ? -16 : (c > ilen ? ilen : c);
  b.at_b = static_cast<uint32_t>(static_cast<int32_t>(16 + a) + drel_b);
  b.at_c = static_cast<uint32_t>(static_cast<int32_t>(16 + a) + drel_c);
  return b;
}

template <class M, class L, int LANES, int DEPTH>
MMR_HD void span_table_gather(const SpanGroup& g, const SpanMember& m, const SpanPiece* pc, const SpanPieces4& pcs,
                              typename M::cptr safe, uint64_t x0, uint32_t len, uint32_t a, uint8_t* lds,
                              const uint8_t* table, const SpanRowEnds<M>& b, uint32_t lane) {
  const uint32_t W = g.W;
  const uint64_t row0 = x0 < (1ull << 31) ? fdiv(static_cast<uint32_t>(x0), g.div_W) : x0 / W;
  const uint32_t o0 = static_cast<uint32_t>(x0 - row0 * W);
  const uint32_t k = m.k;
  const uint32_t n_a = (len + a + 15) >> 4;  // aligned destination vectors that overlap the span
  constexpr int ITEMS = DEPTH + (kSpanAlignedLoads ? 2 : 1);
  // one pass unless the span is a full one in a buffer that is not 16-byte aligned (one vector more than LANES * DEPTH)
  for (uint32_t base = 0; base < n_a; base += LANES * DEPTH) {
    constexpr int SLOTS = DEPTH + 2;  // ITEMS of them are used
    V16 v[SLOTS];
    uint32_t at[SLOTS];
    bool live[SLOTS], zero[SLOTS], keep[SLOTS];
    typename M::cptr from[SLOTS];
#pragma unroll
    for (int u = 0; u < DEPTH; ++u) {
      const uint32_t i = base + lane + u * LANES;
      live[u] = i < n_a;
      const uint32_t v16 = i << 4;
      const uint32_t y = !live[u] || v16 < a ? 0u : v16 - a;  // the vector's first byte inside the span
      const uint32_t rr = fdiv(o0 + y, g.div_W), col = o0 + y - rr * W;
      uint32_t p = 0;
      if (k > 1) p += col >= pcs.c1.col ? 1u : 0u;
      if (k > 2) p += col >= pcs.c2.col ? 1u : 0u;
      if (k > 3) p += col >= pcs.c3.col ? 1u : 0u;
      const V16 rec = L::load16(table + ((rr * k + p) << 4));
      const int32_t end16 = static_cast<int32_t>(rec.w);
      const uint32_t w = rec.z & 0x3fffffffu;
      const int32_t start = end16 + 16 - static_cast<int32_t>(w);
      int32_t yy = static_cast<int32_t>(y);
      if (kSpanAlignedLoads) {
        yy -= static_cast<int32_t>((rec.x + y) & 15u);  // back to the 16-byte boundary of the source
        yy = yy < start ? start : yy;                   // ... but not before the piece row begins
      }
      yy = yy < end16 ? yy : end16;  // slides back to end with the piece row
      const uint64_t d = (static_cast<uint64_t>(rec.y) << 32) | rec.x;
      zero[u] = (rec.z >> 30) != 0;
      from[u] = live[u] && !zero[u] ? reinterpret_cast<typename M::cptr>(d + static_cast<uint64_t>(static_cast<int64_t>(yy))) : safe;
      at[u] = static_cast<uint32_t>(static_cast<int32_t>(16 + a) + yy);
      // first or last 128-byte line of the piece row (low address bits suffice: the row is shorter than 4 GiB)
      const uint32_t row_lo = rec.x + static_cast<uint32_t>(start), lo = rec.x + static_cast<uint32_t>(yy);
      keep[u] = (lo >> 7) == (row_lo >> 7) || ((lo + 15u) >> 7) == ((row_lo + w - 1u) >> 7);
    }
    live[DEPTH] = b.on && base == 0;
    zero[DEPTH] = b.zero;
    from[DEPTH] = base == 0 ? b.from_b : safe;
    at[DEPTH] = b.at_b;
    keep[DEPTH] = true;
    if (kSpanAlignedLoads) {
      live[DEPTH + 1] = live[DEPTH];
      zero[DEPTH + 1] = b.zero;
      from[DEPTH + 1] = base == 0 ? b.from_c : safe;
      at[DEPTH + 1] = b.at_c;
      keep[DEPTH + 1] = true;
    }
#pragma unroll
    for (int u = 0; u < ITEMS; ++u) {
      if (kSpanKeepEdges && u >= DEPTH) v[u] = M::load16u_keep(from[u]);
      else if (kSpanKeepEdges) v[u] = keep[u] ? M::load16u_keep(from[u]) : M::load16u(from[u]);
      else v[u] = M::load16u(from[u]);
    }
#pragma unroll
    for (int u = 0; u < ITEMS; ++u)
      if (live[u]) L::store16u(lds + at[u], zero[u] ? V16{0, 0, 0, 0} : v[u]);
  }
  if (m.narrow) {
    const uint32_t nrows = fdiv(o0 + len + W - 1, g.div_W);
    span_gather_narrow<M, L, LANES>(g, pc, k, nrows, static_cast<uint32_t>(row0), o0, static_cast<int32_t>(len), a, lds, lane);
  }
}

// Phase 2 (after a workgroup barrier): the span leaves LDS as aligned 16-byte vectors; the bytes before the first and
// after the last whole vector (only at the ends of a band whose ends are not 16-byte aligned) go out one by one.
template <class M, class L, int THREADS, int UNROLL>
MMR_HD void span_write(typename M::ptr dst, uint32_t len, uint32_t a, const uint8_t* lds, uint32_t tid) {
  const uint32_t head = a ? (16 - a < len ? 16 - a : len) : 0;
  const uint32_t nvec = (len - head) >> 4;
  const uint32_t tail0 = head + (nvec << 4);
  const uint8_t* body = lds + 16 + a + head;  // 16-byte aligned: a + head is 0 or 16
  for (uint32_t base = 0; base < nvec; base += THREADS * UNROLL) {
    V16 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      uint32_t i = base + tid + u * THREADS;
      i = i < nvec ? i : nvec - 1;
      v[u] = L::load16(body + (i << 4));
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      uint32_t i = base + tid + u * THREADS;
      i = i < nvec ? i : nvec - 1;
      M::store16(dst + (head + (static_cast<int64_t>(i) << 4)), v[u]);
    }
  }
  if (tid < head) M::template storeu<uint8_t>(dst + tid, L::load8(lds + 16 + a + tid));
  if (tid < len - tail0) M::template storeu<uint8_t>(dst + (tail0 + tid), L::load8(lds + 16 + a + tail0 + tid));
}

// ---------------------------------------------------------------------------
// Tables of a launch
// ---------------------------------------------------------------------------
constexpr uint32_t kHintShift = 6;  // one hint per 64 chunks

// Group that holds chunk ci: start from the hint for ci's block of 64 chunks (the group of the block's first
// chunk) and walk forward.  `Groups` is indexable and its elements have first_chunk.
template <class G>
MMR_HD uint32_t find_group(const G* groups, uint32_t n_groups, const uint32_t* hints, uint32_t ci) {
  uint32_t g = hints ? hints[ci >> kHintShift] : 0;
  while (g + 1 < n_groups && groups[g + 1].first_chunk <= ci) ++g;
  return g;
}

// The first chunk of every group of a small table, handed to the kernel by value: the group of a chunk is then found
// without touching memory.  Unused entries hold 0xffffffff.
constexpr uint32_t kMaxDirectGroups = 16;
struct GroupStarts {
  uint32_t first[kMaxDirectGroups];
};

MMR_HD uint32_t find_group_direct(const GroupStarts& starts, uint32_t ci) {
  uint32_t g = 0;
#pragma unroll
  for (uint32_t i = 1; i < kMaxDirectGroups; ++i) g += starts.first[i] <= ci ? 1u : 0u;
  return g;
}

// Small plans travel in the kernel's argument block (no device table, nothing to upload or to keep alive).
constexpr uint32_t kInlineCopyGroups = 8, kInlineCopyPieces = 32;
struct InlineCopyTable {
  uint32_t n_groups, n_chunks;
  CopyGroup groups[kInlineCopyGroups];
  CopyPiece pieces[kInlineCopyPieces];
};
constexpr uint32_t kInlineSpanGroups = 4, kInlineSpanMembers = 12, kInlineSpanPieces = 32;
struct InlineSpanTable {
  uint32_t n_groups, n_chunks;
  SpanGroup groups[kInlineSpanGroups];
  SpanMember members[kInlineSpanMembers];
  SpanPiece pieces[kInlineSpanPieces];
};
static_assert(sizeof(InlineCopyTable) <= 3900 && sizeof(InlineSpanTable) <= 3900, "must fit the kernel argument block");

}  // namespace mmr

#endif  // MMR_CSRC_GROUP_OPS_H_
