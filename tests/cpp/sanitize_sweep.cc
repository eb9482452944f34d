// Host-side sanitizer sweep, for tests only (CPU, no GPU call anywhere).
//
// Built with -fsanitize=address,undefined together with the planner, the
// descriptor geometry and the host emulation of the kernels.  Draws seeded
// random (source sharding, destination sharding) pairs - ragged extents, empty
// edge tiles, replication, permuted device order, physical layouts, every
// element width - plans them, runs the plan through the kernels' per-chunk code
// and checks every destination byte against an element-by-element owner
// computation written here from the descriptor fields alone.  Any overflow,
// out-of-bounds host access or wrong byte fails the run.
//
// usage: sanitize_sweep <cases> <seed>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "mmreshard.h"

extern "C" int mmr_emulate_plan(const mmr_plan* plan, void* const* slot_ptrs, const size_t* slot_bytes, int64_t n_slots,
                                uint32_t xcd_mode, int shape, uint64_t* bytes_loaded, uint64_t* bytes_stored, char* err,
                                size_t err_len);

namespace {

struct SideDesc {
  mmr_sharded_shape shape{};
  int rank = 0;
  int64_t ext[MMR_MAX_DIMS] = {};     // tile extent per tensor dim
  int64_t stride[MMR_MAX_DIMS] = {};  // element stride of each logical dim inside a shard buffer
  int64_t dev_stride[MMR_MAX_DIMS] = {};
  int64_t shard_elems = 1;
  int64_t replication = 1;
};

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Fills geometry from the descriptor: tile extent ceil(size / tiles); device id = start + sum over entries of
// coordinate x stride, an entry's stride being the product of the tile counts of all less significant entries
// (larger permutation value = less significant); buffers dense in minor_to_major order (row-major by default).
void derive(SideDesc* s) {
  const mmr_sharded_shape& d = s->shape;
  const bool repl = d.ndims > 0 && d.ndims > s->rank;
  s->replication = repl ? d.dims[d.ndims - 1].sharding : 1;
  for (int i = 0; i < d.ndims; ++i) {
    int64_t st = 1;
    for (int j = 0; j < d.ndims; ++j)
      if (d.dims[j].permutation > d.dims[i].permutation) st *= d.dims[j].sharding;
    s->dev_stride[i] = st;
  }
  s->shard_elems = 1;
  for (int i = 0; i < s->rank; ++i) {
    s->ext[i] = ceil_div(d.dims[i].size, d.dims[i].sharding);
    s->shard_elems *= s->ext[i];
  }
  int64_t st = 1;
  for (int k = 0; k < s->rank; ++k) {
    const int dim = d.has_layout ? d.minor_to_major[k] : s->rank - 1 - k;
    s->stride[dim] = st;
    st *= s->ext[dim];
  }
}

SideDesc random_side(std::mt19937_64& rng, int32_t dtype, const std::vector<int64_t>& sizes, int64_t dev_start,
                     bool allow_layout) {
  SideDesc s;
  s.rank = static_cast<int>(sizes.size());
  s.shape.dtype = dtype;
  std::vector<int64_t> tiles(s.rank);
  int64_t count = 1;
  for (int i = 0; i < s.rank; ++i) {
    const int64_t choices[] = {1, 1, 2, 3, 4, 5};
    int64_t t = choices[rng() % 6];
    if (count * t > 12 || sizes[i] == 1) t = 1;  // {size 1, sharding > 1} in last place would read as a replication entry
    tiles[i] = t;
    count *= t;
  }
  int64_t repl = (rng() % 4 == 0 && count <= 6) ? 2 : 1;
  s.shape.ndims = s.rank + (repl > 1 ? 1 : 0);
  std::vector<int> perm(s.shape.ndims);
  for (int i = 0; i < s.shape.ndims; ++i) perm[i] = i;
  for (int i = s.shape.ndims - 1; i > 0; --i) std::swap(perm[i], perm[rng() % (i + 1)]);
  for (int i = 0; i < s.rank; ++i) s.shape.dims[i] = mmr_sharding_dim{sizes[i], tiles[i], perm[i]};
  if (repl > 1) s.shape.dims[s.rank] = mmr_sharding_dim{1, repl, perm[s.rank]};
  s.shape.dev_start = dev_start;
  s.shape.dev_count = count * repl;
  if (allow_layout && s.rank >= 2 && rng() % 3 == 0) {
    s.shape.has_layout = 1;
    std::vector<int> m(s.rank);
    for (int i = 0; i < s.rank; ++i) m[i] = s.rank - 1 - i;
    for (int i = s.rank - 1; i > 0; --i) std::swap(m[i], m[rng() % (i + 1)]);
    for (int i = 0; i < s.rank; ++i) s.shape.minor_to_major[i] = m[i];
  }
  derive(&s);
  return s;
}

// Device (relative to dev_start, lowest replica) and element offset holding global coordinate `g`.
void locate(const SideDesc& s, const int64_t* g, int64_t replica, int64_t* dev, int64_t* off) {
  int64_t d = 0, o = 0;
  for (int i = 0; i < s.rank; ++i) {
    const int64_t t = g[i] / s.ext[i];
    d += t * s.dev_stride[i];
    o += (g[i] - t * s.ext[i]) * s.stride[i];
  }
  if (s.replication > 1) d += replica * s.dev_stride[s.rank];
  *dev = d;
  *off = o;
}

int64_t g_aligned = 0, g_generic = 0, g_tiles = 0, g_fills = 0;

int run_case(std::mt19937_64& rng, int index) {
  const int32_t dtypes[] = {MMR_U8, MMR_BF16, MMR_F32, MMR_F64, MMR_C128};
  const int items[] = {1, 2, 4, 8, 16};
  const int ti = static_cast<int>(rng() % 5);
  const int item = items[ti];
  const int rank = static_cast<int>(rng() % 4);  // 0..3
  std::vector<int64_t> sizes(rank);
  int64_t total = 1;
  for (int i = 0; i < rank; ++i) {
    const int64_t pool[] = {1, 2, 3, 5, 7, 8, 13, 16, 17, 31, 33, 64, 70, 129, 257, 1030};
    sizes[i] = pool[rng() % 16];
    if (total * sizes[i] > 60000) sizes[i] = 1 + rng() % 4;
    total *= sizes[i];
  }
  SideDesc S = random_side(rng, dtypes[ti], sizes, static_cast<int64_t>(rng() % 3), true);
  SideDesc D = random_side(rng, dtypes[ti], sizes, S.shape.dev_start + S.shape.dev_count, true);

  mmr_plan_options opt{};
  const uint32_t chunk_choices[] = {0, 256, 1024, 4096, 65536};
  opt.chunk_bytes = chunk_choices[rng() % 5];
  opt.order = static_cast<uint32_t>(rng() % 5);
  mmr_plan* plan = nullptr;
  if (mmr_plan_create(&S.shape, &D.shape, 1, &opt, &plan) != MMR_OK) {
    std::fprintf(stderr, "case %d: plan failed: %s\n", index, mmr_last_error());
    return 1;
  }
  mmr_plan_stats st{};
  mmr_plan_get_stats(plan, &st);
  g_aligned += st.n_copy16_chunks;
  g_generic += st.n_copy_generic_chunks;
  g_tiles += st.n_transpose_chunks;
  g_fills += st.n_fill_chunks;
  const int64_t ns = S.shape.dev_count, nd = D.shape.dev_count;
  const size_t sbytes = static_cast<size_t>(S.shard_elems) * item, dbytes = static_cast<size_t>(D.shard_elems) * item;
  // exact-size heap blocks: the address sanitizer sees any access past a shard buffer, on top of the emulation's checks
  std::vector<uint8_t*> bufs;
  std::vector<size_t> sizes_b;
  auto alloc16 = [](size_t n) { return static_cast<uint8_t*>(std::aligned_alloc(16, (n + 15) / 16 * 16 + 16)); };
  // every source replica carries the same data: fill by global coordinate
  std::vector<uint8_t> global(static_cast<size_t>(total) * item);
  for (auto& b : global) b = static_cast<uint8_t>(rng());
  for (int64_t k = 0; k < ns; ++k) {
    bufs.push_back(alloc16(sbytes));
    sizes_b.push_back(sbytes);
    std::memset(bufs.back(), 0xEE, sbytes);
  }
  for (int64_t k = 0; k < nd; ++k) {
    bufs.push_back(alloc16(dbytes));
    sizes_b.push_back(dbytes);
    std::memset(bufs.back(), 0x5A, dbytes);
  }
  std::vector<int64_t> g(rank > 0 ? rank : 1, 0);
  for (int64_t lin = 0; lin < total; ++lin) {
    int64_t r = lin;
    for (int i = rank - 1; i >= 0; --i) {
      g[i] = r % sizes[i];
      r /= sizes[i];
    }
    for (int64_t rep = 0; rep < S.replication; ++rep) {
      int64_t dev, off;
      locate(S, g.data(), rep, &dev, &off);
      std::memcpy(bufs[dev] + off * item, &global[static_cast<size_t>(lin) * item], item);
    }
  }
  char err[512] = {0};
  uint64_t loaded = 0, stored = 0;
  std::vector<void*> ptrs(bufs.begin(), bufs.end());
  int rc = mmr_emulate_plan(plan, ptrs.data(), sizes_b.data(), static_cast<int64_t>(bufs.size()),
                            static_cast<uint32_t>(rng() % 3 == 0 ? 16 : 0), static_cast<int>(rng() % 4), &loaded, &stored, err,
                            sizeof(err));
  int bad = 0;
  if (rc != 0) {
    std::fprintf(stderr, "case %d: emulation: %s\n", index, err);
    bad = 1;
  }
  // expected destination buffers: zero (pad), then every element at its place in every replica
  for (int64_t k = 0; k < nd && !bad; ++k) {
    std::vector<uint8_t> expect(dbytes, 0);
    bool any = false;
    for (int64_t lin = 0; lin < total; ++lin) {
      int64_t r = lin;
      for (int i = rank - 1; i >= 0; --i) {
        g[i] = r % sizes[i];
        r /= sizes[i];
      }
      for (int64_t rep = 0; rep < D.replication; ++rep) {
        int64_t dev, off;
        locate(D, g.data(), rep, &dev, &off);
        if (dev == k) {
          std::memcpy(&expect[static_cast<size_t>(off) * item], &global[static_cast<size_t>(lin) * item], item);
          any = true;
        }
      }
    }
    (void)any;
    if (std::memcmp(expect.data(), bufs[ns + k], dbytes) != 0) {
      std::fprintf(stderr, "case %d: destination device %lld differs (rank %d, item %d, order %u, chunk %u)\n", index,
                   static_cast<long long>(D.shape.dev_start + k), rank, item, opt.order, opt.chunk_bytes);
      bad = 1;
    }
  }
  for (uint8_t* b : bufs) std::free(b);
  mmr_plan_destroy(plan);
  return bad;
}

}  // namespace

int main(int argc, char** argv) {
  const int cases = argc > 1 ? std::atoi(argv[1]) : 200;
  const uint64_t seed = argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 1;
  std::mt19937_64 rng(seed);
  int failures = 0;
  for (int i = 0; i < cases; ++i) failures += run_case(rng, i);
  if (failures) {
    std::fprintf(stderr, "%d of %d cases failed\n", failures, cases);
    return 1;
  }
  std::printf("%d cases OK (%lld aligned, %lld generic, %lld transpose, %lld fill chunks)\n", cases,
              static_cast<long long>(g_aligned), static_cast<long long>(g_generic), static_cast<long long>(g_tiles),
              static_cast<long long>(g_fills));
  return 0;
}
