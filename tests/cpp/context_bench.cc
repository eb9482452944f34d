// Times the reshard path behind the reference-shaped interface: a ReshardSchedule executed through
// HipExecuteContext the way MultiMeshPjRtExecutable::Execute drives the reference's context
// (mm_pjrt_executable.cc:362-364 bracket, :495-498 fresh root stores, :616-658 one Reshard call per op and local
// device, :704-706 closing bracket), over 12 local devices.
//
//   context_bench <configuration 2|4> [executions=50] [warmup=9]
//
// Prints one JSON line: wall milliseconds per execution (back to back, the host free to run ahead until the window
// limit holds it), host milliseconds until Execute returns (measured with the device idle at every call, so no
// back-pressure is in it), algorithmic GB/s.  Sampled elements of the last execution's outputs are checked against
// the closed form (destination tile = slice of the global array); the full comparisons with the CPU restatement are
// in hip_execute_context_test.cc.
//
// Needs a GPU.
#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "hip_execute_context.h"

using namespace mmr;
using Clock = std::chrono::steady_clock;

namespace {

struct ArraySpec {
  std::string name;
  std::vector<int64_t> shape;
  int src_dim, src_tiles, dst_dim, dst_tiles;  // the one sharded dim of each side
};

double ms_since(Clock::time_point t0) { return std::chrono::duration<double, std::milli>(Clock::now() - t0).count(); }

ShardedShape make_shape(SupportedType type, const std::vector<int64_t>& shape, int dim, int tiles, int64_t dev_start) {
  ShardedShape s;
  s.type = type;
  for (size_t i = 0; i < shape.size(); ++i)
    s.sharding.dims.push_back(ShardingDim{shape[i], static_cast<int>(i) == dim ? tiles : 1, static_cast<int64_t>(i)});
  s.sharding.devices = DeviceList::Create(dev_start, tiles);
  return s;
}

// the value of global element `linear` of array `a`: any function that tells elements and arrays apart
template <class T>
T value_of(size_t a, int64_t linear) {
  uint64_t h = (static_cast<uint64_t>(linear) + 0x9e3779b97f4a7c15ull * (a + 1)) * 0xbf58476d1ce4e5b9ull;
  return static_cast<T>(h >> 40);
}

int64_t linear_index(const std::vector<int64_t>& shape, const std::vector<int64_t>& idx) {
  int64_t l = 0;
  for (size_t i = 0; i < shape.size(); ++i) l = l * shape[i] + idx[i];
  return l;
}

// shard k of `spec` sharded `tiles` ways along `dim`, dense row-major, filled from value_of
template <class T>
void fill_shard(size_t a, const ArraySpec& spec, int dim, int tiles, int k, std::vector<T>* out) {
  std::vector<int64_t> local = spec.shape;
  local[static_cast<size_t>(dim)] /= tiles;
  const int rank = static_cast<int>(local.size());
  int64_t n = 1;
  for (int64_t e : local) n *= e;
  out->resize(static_cast<size_t>(n));
  const int64_t row = local[static_cast<size_t>(rank - 1)];
  std::vector<int64_t> idx(local.size(), 0), g(local.size(), 0);
  T* dst = out->data();
  for (int64_t at = 0; at < n; at += row) {  // one row of the shard = one contiguous run of the global array
    g = idx;
    g[static_cast<size_t>(dim)] += k * local[static_cast<size_t>(dim)];
    const int64_t base = linear_index(spec.shape, g);
    for (int64_t j = 0; j < row; ++j) dst[at + j] = value_of<T>(a, base + j);
    for (int d = rank - 2; d >= 0; --d) {
      if (++idx[static_cast<size_t>(d)] < local[static_cast<size_t>(d)]) break;
      idx[static_cast<size_t>(d)] = 0;
    }
  }
}

template <class T>
int run(int config, int executions, int warmup, SupportedType type) {
  const int kLocal = 12;
  std::vector<ArraySpec> specs;
  int64_t src_start = 0, dst_start = 0;
  if (config == 2) {  // bf16 [8, 4096, 8192]: hidden 8-way on devices 0-7 -> sequence 4-way on devices 8-11
    specs.push_back({"c2", {8, 4096, 8192}, 2, 8, 1, 4});
    src_start = 0;
    dst_start = 8;
  } else {  // the 195 f32 arrays of a 24-layer decoder: last dim 4-way on devices 0-3 -> first dim 8-way on devices 4-11
    const int64_t d_model = 2048, ffn = 8192, vocab = 32000;
    auto add = [&](std::string name, std::vector<int64_t> shape) {
      const int last = static_cast<int>(shape.size()) - 1;
      specs.push_back({std::move(name), std::move(shape), last, 4, 0, 8});
    };
    for (int layer = 0; layer < 24; ++layer) {
      const std::string p = "layer" + std::to_string(layer) + ".";
      add(p + "ln1", {d_model});
      for (const char* w : {"wq", "wk", "wv", "wo"}) add(p + w, {d_model, d_model});
      add(p + "ln2", {d_model});
      add(p + "w_in", {d_model, ffn});
      add(p + "w_out", {ffn, d_model});
    }
    add("embed", {vocab, d_model});
    add("final_ln", {d_model});
    add("lm_head", {d_model, vocab});
    src_start = 0;
    dst_start = 4;
  }
  std::set<int> local;
  for (int d = 0; d < kLocal; ++d) local.insert(d);
  auto ctx = HipExecuteContext::Create(local);

  ReshardSchedule schedule(config == 2 ? "c2_hidden_to_sequence" : "c4_pytree");
  std::vector<ShardedShape> src_shapes, dst_shapes;
  int64_t algorithmic = 0;
  for (size_t a = 0; a < specs.size(); ++a) {
    src_shapes.push_back(make_shape(type, specs[a].shape, specs[a].src_dim, specs[a].src_tiles, src_start));
    dst_shapes.push_back(make_shape(type, specs[a].shape, specs[a].dst_dim, specs[a].dst_tiles, dst_start));
    Store in = schedule.AddStore(Store::Type::PARAM, specs[a].name, src_shapes[a]);
    Store out = schedule.AddStore(Store::Type::ROOT, specs[a].name + ".resharded", dst_shapes[a]);
    schedule.AddReshardTask(in, out);
    int64_t n = 1;
    for (int64_t e : specs[a].shape) n *= e;
    algorithmic += 2 * n * static_cast<int64_t>(sizeof(T));
  }

  // parameter sets: enough of them that no read of an execution can come out of the 256 MB last-level cache
  const int sets = config == 2 ? 3 : 1;
  std::vector<std::vector<std::vector<StoreHandle>>> params(
      static_cast<size_t>(sets), std::vector<std::vector<StoreHandle>>(kLocal, std::vector<StoreHandle>(specs.size())));
  {
    // AssembleShards is issued by every local device once per array and set: member devices copy their shard
    for (size_t a = 0; a < specs.size(); ++a) {
      const int tiles = specs[a].src_tiles;
      std::vector<std::vector<T>> shards(static_cast<size_t>(tiles));
      for (int k = 0; k < tiles; ++k) fill_shard<T>(a, specs[a], specs[a].src_dim, tiles, k, &shards[static_cast<size_t>(k)]);
      for (int s = 0; s < sets; ++s)
        for (int d = 0; d < kLocal; ++d) {
          const int k = d - static_cast<int>(src_start);
          const bool member = k >= 0 && k < tiles;
          Shard sh{member ? shards[static_cast<size_t>(k)].data() : nullptr, d,
                   member ? shards[static_cast<size_t>(k)].size() * sizeof(T) : 0};
          params[static_cast<size_t>(s)][static_cast<size_t>(d)][a] = ctx->AssembleShards(d, d, src_shapes[a], sh);
        }
    }
  }
  if (mmr_sync(ctx->raw()) != MMR_OK) return 1;

  // the last results stay alive for two more executions, so destination buffers rotate too
  std::vector<std::vector<std::vector<StoreHandle>>> keep(3);
  int turn = 0;
  auto execute = [&] {
    auto roots = schedule.Execute(*ctx, params[static_cast<size_t>(turn % sets)]);
    keep[static_cast<size_t>(turn % 3)] = std::move(roots);
    ++turn;
  };
  for (int i = 0; i < warmup; ++i) execute();
  if (mmr_sync(ctx->raw()) != MMR_OK) return 1;

  // (1) host cost of one Execute with the device idle
  std::vector<double> host_ms;
  for (int i = 0; i < executions; ++i) {
    const auto t0 = Clock::now();
    execute();
    host_ms.push_back(ms_since(t0));
    if (mmr_sync(ctx->raw()) != MMR_OK) return 1;
  }
  std::sort(host_ms.begin(), host_ms.end());
  double host_mean = 0;
  for (double v : host_ms) host_mean += v;
  host_mean /= static_cast<double>(host_ms.size());

  // (2) back to back
  const mmr_context_stats s0 = ctx->Stats();
  if (mmr_sync(ctx->raw()) != MMR_OK) return 1;
  const auto t0 = Clock::now();
  for (int i = 0; i < executions; ++i) execute();
  const double issue_ms = ms_since(t0);
  if (mmr_sync(ctx->raw()) != MMR_OK) return 1;
  const double wall_ms = ms_since(t0) / executions;
  const mmr_context_stats s1 = ctx->Stats();
  int64_t timers_done = 0;
  const double timer_ms = ctx->LastTimerMilliseconds(schedule.name(), &timers_done);

  // sampled check of the newest outputs against the closed form
  int64_t checked = 0, wrong = 0;
  const auto& newest = keep[static_cast<size_t>((turn - 1) % 3)];
  std::vector<T> got;
  for (size_t a = 0; a < specs.size(); a += std::max<size_t>(1, specs.size() / 7)) {
    const ArraySpec& sp = specs[a];
    const int tiles = sp.dst_tiles;
    std::vector<int64_t> localshape = sp.shape;
    localshape[static_cast<size_t>(sp.dst_dim)] /= tiles;
    int64_t n = 1;
    for (int64_t e : localshape) n *= e;
    for (int k : {0, tiles - 1}) {
      const int d = static_cast<int>(dst_start) + k;
      const StoreHandle& h = newest[static_cast<size_t>(d)][a];
      got.resize(static_cast<size_t>(n));
      ctx->CopyShardToHost(h, got.data(), got.size() * sizeof(T));
      const int64_t step = std::max<int64_t>(1, n / 4099);
      for (int64_t i = 0; i < n; i += step) {
        std::vector<int64_t> idx(localshape.size());
        int64_t rem = i;
        for (int q = static_cast<int>(localshape.size()) - 1; q >= 0; --q) {
          idx[static_cast<size_t>(q)] = rem % localshape[static_cast<size_t>(q)];
          rem /= localshape[static_cast<size_t>(q)];
        }
        idx[static_cast<size_t>(sp.dst_dim)] += k * localshape[static_cast<size_t>(sp.dst_dim)];
        wrong += got[static_cast<size_t>(i)] != value_of<T>(a, linear_index(sp.shape, idx));
        ++checked;
      }
    }
  }

  std::printf(
      "{\"configuration\": %d, \"interface\": \"ReshardSchedule::Execute over HipExecuteContext, %d local devices\", "
      "\"arrays\": %zu, \"reshard_calls_issued_per_execution\": %zu, \"executions\": %d, \"warmup\": %d, "
      "\"algorithmic_bytes\": %lld, \"wall_ms_per_execution\": %.5f, \"GB/s\": %.1f, "
      "\"host_ms_per_execute_mean\": %.5f, \"host_ms_per_execute_median\": %.5f, \"host_ms_per_execute_p90\": %.5f, "
      "\"issue_ms_per_execution_back_to_back\": %.5f, \"device_ms_named_timer_last\": %.5f, \"named_timers_completed\": %lld, "
      "\"batched_reshards_per_execution\": %.2f, \"kernel_launches_per_execution\": %.2f, "
      "\"host_blocking_syncs_back_to_back\": %lld, \"window_waits_back_to_back\": %lld, "
      "\"device_allocations_back_to_back\": %lld, \"bindings_built_back_to_back\": %lld, \"plans_built_back_to_back\": %lld, "
      "\"elements_checked\": %lld, \"elements_wrong\": %lld}\n",
      config, kLocal, specs.size(), specs.size() * kLocal, executions, warmup, static_cast<long long>(algorithmic), wall_ms,
      static_cast<double>(algorithmic) / (wall_ms * 1e-3) / 1e9, host_mean, host_ms[host_ms.size() / 2],
      host_ms[host_ms.size() * 9 / 10], issue_ms / executions, timer_ms, static_cast<long long>(timers_done),
      static_cast<double>(s1.reshard_calls - s0.reshard_calls) / executions,
      static_cast<double>(s1.kernel_launches - s0.kernel_launches) / executions,
      static_cast<long long>(s1.host_blocking_syncs - s0.host_blocking_syncs),
      static_cast<long long>(s1.window_waits - s0.window_waits),
      static_cast<long long>(s1.device_allocations - s0.device_allocations),
      static_cast<long long>(s1.bindings_built - s0.bindings_built), static_cast<long long>(s1.plans_built - s0.plans_built),
      static_cast<long long>(checked), static_cast<long long>(wrong));
  return wrong == 0 ? 0 : 3;
}

}  // namespace

int main(int argc, char** argv) {
  const int config = argc > 1 ? std::atoi(argv[1]) : 2;
  const int executions = argc > 2 ? std::atoi(argv[2]) : 50;
  const int warmup = argc > 3 ? std::atoi(argv[3]) : 9;
  if ((config != 2 && config != 4) || executions < 1 || warmup < 0) {
    std::fprintf(stderr, "usage: context_bench <2|4> [executions] [warmup]\n");
    return 2;
  }
  try {
    return config == 2 ? run<uint16_t>(2, executions, warmup, SupportedType::BF16)
                       : run<uint32_t>(4, executions, warmup, SupportedType::F32);
  } catch (const std::exception& e) {
    std::fprintf(stderr, "ERROR: %s\n", e.what());
    return 2;
  }
}
