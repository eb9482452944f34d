// Drives HipExecuteContext the way MultiMeshPjRtExecutable::Execute drives the
// reference's ZukuExecuteContext (mm_pjrt_executable.cc:391-431 parameter stores,
// :495-498 root stores, :616-658 schedule loop, mm_pjrt_buffer.cc:84-95 read-back):
// every local device issues every call.  Results are compared with the C
// restatement of the reshard (oracle/reshard_cpu.c), bit for bit.
//
// Needs a GPU.  Prints "OK" and exits 0 on success.
#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "hip_execute_context.h"
#include "shard_buffer.h"

extern "C" {
// oracle/reshard_cpu.c
struct orc_desc {
  int32_t itemsize;
  int32_t ndims;
  int64_t size[9];
  int64_t sharding[9];
  int64_t permutation[9];
  int64_t dev_start;
  int64_t dev_count;
  int32_t has_layout;
  int32_t minor_to_major[9];
};
int orc_reshard(const orc_desc* src, const void* const* src_bufs, const orc_desc* dst, void* const* dst_bufs,
                int nthreads);
}

using namespace mmr;

#define EXPECT(cond)                                                              \
  do {                                                                            \
    if (!(cond)) {                                                                \
      std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
      return 1;                                                                   \
    }                                                                             \
  } while (0)

static orc_desc to_orc(const ShardedShape& s, int itemsize) {
  orc_desc d{};
  d.itemsize = itemsize;
  d.ndims = static_cast<int32_t>(s.sharding.dims.size());
  for (int i = 0; i < d.ndims; ++i) {
    d.size[i] = s.sharding.dims[i].size;
    d.sharding[i] = s.sharding.dims[i].sharding;
    d.permutation[i] = s.sharding.dims[i].permutation;
  }
  d.dev_start = s.sharding.devices.start();
  d.dev_count = s.sharding.devices.size();
  return d;
}

template <class Fn>
static bool throws(Fn&& fn, const char* needle) {
  try {
    fn();
  } catch (const std::runtime_error& e) {
    return std::strstr(e.what(), needle) != nullptr;
  }
  return false;
}

static int run() {
  const int kLocal = 12;
  std::set<int> local;
  for (int d = 0; d < kLocal; ++d) local.insert(d);
  auto ctx = HipExecuteContext::Create(local);
  std::printf("context created\n");
  std::fflush(stdout);

  // bf16 [4, 64, 256]: hidden 8-way on devices 0-7 -> sequence 4-way on devices 8-11
  ShardedShape src{SupportedType::BF16, {{{4, 1, 0}, {64, 1, 1}, {256, 8, 2}}, DeviceList::Create(0, 8)}, {}};
  ShardedShape dst{SupportedType::BF16, {{{4, 1, 0}, {64, 4, 1}, {256, 1, 2}}, DeviceList::Create(8, 4)}, {}};
  EXPECT(ShardSize(src) == 4 * 64 * 32 * 2);
  EXPECT(ShardSize(dst) == 4 * 16 * 256 * 2);

  // native shards of the parameter, one per source device
  std::vector<std::vector<uint16_t>> shards(8, std::vector<uint16_t>(4 * 64 * 32));
  uint32_t lcg = 12345;
  for (auto& s : shards)
    for (auto& v : s) {
      lcg = lcg * 1664525u + 1013904223u;
      v = static_cast<uint16_t>(lcg >> 13);
    }

  // parameter stores: every local device wraps "its" native buffer (members copy, the rest attach)
  std::vector<StoreHandle> param(kLocal), root(kLocal);
  for (int d = 0; d < kLocal; ++d) {
    Shard shard{d < 8 ? shards[d].data() : nullptr, d, d < 8 ? shards[d].size() * 2 : 0};
    param[d] = ctx->AssembleShards(d, d, src, shard);
  }
  for (int d = 1; d < kLocal; ++d) EXPECT(param[d].unique_id == param[0].unique_id);
  // root store of the reshard's output, created by every local device
  for (int d = 0; d < kLocal; ++d) root[d] = ctx->CreateStore(d, d, dst, {.name = "reshard.out"});
  for (int d = 1; d < kLocal; ++d) EXPECT(root[d].unique_id == root[0].unique_id);
  EXPECT(root[0].unique_id != param[0].unique_id);
  EXPECT(ctx->Stats().stores_live == 2);
  EXPECT(ctx->GetStoreShardedShape(root[3]) == dst);
  for (int d = 0; d < kLocal; ++d) {
    EXPECT(ctx->HasLocalShard(param[d]) == (d < 8));
    EXPECT(ctx->HasLocalShard(root[d]) == (d >= 8));
  }

  // schedule loop: the Reshard op, issued by every local device, inside two named timers that overlap
  // (zuku_execute_context_impl.cc:462-486: any number pending, keyed by name, neither call waits)
  {
    const int64_t syncs0 = ctx->Stats().host_blocking_syncs;
    ctx->StartTimer("execute");
    ctx->StartTimer("execute+readback");
    ctx->StartTimer("execute");  // already running: stays as it is (pending_timers_.emplace)
    for (int d = 0; d < kLocal; ++d) ctx->Reshard(d, d, param[d], root[d]);
    ctx->StopTimer("execute");
    ctx->StopTimer("no such timer");  // a warning, as in the reference
    EXPECT(ctx->Stats().reshard_calls == 1);  // the copy ran once, not twelve times
    EXPECT(ctx->Stats().plans_built == 1);
    std::vector<uint16_t> scratch(4 * 16 * 256);
    EXPECT(ctx->Stats().host_blocking_syncs == syncs0);  // none of the timer calls waited
    ctx->CopyShardToHost(root[8], scratch.data(), scratch.size() * 2);  // device work inside the outer timer only
    ctx->StopTimer("execute+readback");
    int64_t done = 0;
    const double inner = ctx->WaitTimerMilliseconds("execute");
    const double outer = ctx->WaitTimerMilliseconds("execute+readback");
    EXPECT(inner > 0.0 && inner < 1000.0);
    EXPECT(outer >= inner && outer < 1000.0);
    EXPECT(ctx->LastTimerMilliseconds("execute", &done) == inner && done == 1);
    EXPECT(ctx->LastTimerMilliseconds("no such timer", &done) == 0.0 && done == 0);
    ctx->MarkProfile("after the first execution");
    EXPECT(ctx->Stats().profile_marks == 1);
    EXPECT(ctx->Stats().timers_resolved == 2);
  }

  // expectation from the CPU restatement
  std::vector<std::vector<uint16_t>> expect(4, std::vector<uint16_t>(4 * 16 * 256, 0xDEAD));
  {
    orc_desc so = to_orc(src, 2), dd = to_orc(dst, 2);
    const void* sp[8];
    void* dp[4];
    for (int k = 0; k < 8; ++k) sp[k] = shards[k].data();
    for (int k = 0; k < 4; ++k) dp[k] = expect[k].data();
    EXPECT(orc_reshard(&so, sp, &dd, dp, 2) == 0);
  }
  for (int d = 8; d < kLocal; ++d) {
    void* ptr = ctx->SliceLocalShard(d, root[d]);  // blocking, as in the reference
    EXPECT(ptr != nullptr);
    std::vector<uint16_t> got(expect[d - 8].size());
    ctx->CopyShardToHost(root[d], got.data(), got.size() * 2);
    EXPECT(std::memcmp(got.data(), expect[d - 8].data(), got.size() * 2) == 0);
  }
  // RunAfterAllTasks: the callback runs once the stream has drained, the call does not wait (a second reshard is
  // queued right behind it)
  {
    std::atomic<int> fired{0};
    ctx->RunAfterAllTasks(0, [&fired] { fired.fetch_add(1); });
    ctx->RunAfterAllTasks(0, nullptr);  // no callback: nothing to do (zuku_execute_context_impl.cc:349)
    EXPECT(mmr_sync(ctx->raw()) == MMR_OK);
    EXPECT(fired.load() == 1);
    // The reference's callback completes a future whose continuations drop buffers (mm_pjrt_executable.cc:373-375):
    // a callback may use the context.  This one lets go of the last handles of a store (its memory returns to the
    // pool), creates another one and reads the context's statistics; it runs on a thread the context owns.
    std::vector<StoreHandle> doomed(kLocal);
    for (int d = 0; d < kLocal; ++d) doomed[d] = ctx->CreateStore(d, d, dst, {.name = "dropped by a callback"});
    const int64_t live = ctx->Stats().stores_live;
    std::atomic<int64_t> seen_live{-1};
    std::atomic<bool> on_other_thread{false};
    const std::thread::id caller = std::this_thread::get_id();
    auto held = std::make_shared<std::vector<StoreHandle>>(std::move(doomed));
    ctx->RunAfterAllTasks(0, [&, held]() mutable {
      on_other_thread.store(std::this_thread::get_id() != caller);
      for (StoreHandle& h : *held) ctx->Destroy(h);
      seen_live.store(ctx->Stats().stores_live);
      StoreHandle again = ctx->CreateStore(0, 0, src, {.name = "made by a callback"});
      for (int d = 1; d < kLocal; ++d) (void)ctx->CreateStore(d, d, src, {.name = "made by a callback"});
      (void)again;
    });
    held.reset();
    EXPECT(mmr_sync(ctx->raw()) == MMR_OK);  // also waits for the callbacks whose turn has come
    EXPECT(on_other_thread.load());
    EXPECT(seen_live.load() == live - 1);
    EXPECT(ctx->Stats().stores_live == live - 1);  // the callback's own store went when it returned
  }
  // Destroy drops one reference (zuku_execute_context_impl.cc:356-361): a copy of the handle - what a zero-copy view
  // of the tile holds, mm_pjrt_buffer.cc:27-36 - keeps working after the buffer that made it destroyed its own
  {
    std::vector<StoreHandle> owner(kLocal), view(kLocal);
    for (int d = 0; d < kLocal; ++d) owner[d] = ctx->CreateStore(d, d, dst, {.name = "viewed"});
    for (int d = 0; d < kLocal; ++d) view[d] = owner[d];  // shares the impl
    const int64_t live = ctx->Stats().stores_live;
    for (int d = 0; d < kLocal; ++d) ctx->Destroy(owner[d]);
    EXPECT(ctx->Stats().stores_live == live);
    EXPECT(ctx->SliceLocalShard(9, view[9]) != nullptr);
    EXPECT(ctx->HasLocalShard(view[9]) && !ctx->HasLocalShard(owner[9]));
    for (int d = 0; d < kLocal; ++d) ctx->Destroy(view[d]);
    EXPECT(ctx->Stats().stores_live == live - 1);
  }
  // a device outside the store's device list has no shard to slice
  EXPECT(throws([&] { ctx->SliceLocalShard(0, root[0]); }, "holds no shard"));

  // later executions over the same stores reuse the plan; the second builds the device tables, the third finds them
  for (int rep = 0; rep < 2; ++rep) {
    for (int d = 0; d < kLocal; ++d) ctx->Reshard(d, d, param[d], root[d]);
    ctx->Flush();
  }
  EXPECT(ctx->Stats().reshard_calls == 3);
  EXPECT(ctx->Stats().plans_built == 1);
  EXPECT(ctx->Stats().inline_launches == 1);
  EXPECT(ctx->Stats().bindings_built == 1);
  EXPECT(ctx->Stats().binding_cache_hits == 1);

  // offload to the pinned host cache and back, issued by every local device like any other op; the host never waits
  {
    const mmr_context_stats before = ctx->Stats();
    for (int d = 0; d < kLocal; ++d) ctx->OffloadDtoH(d, {root[d]}, {param[d]}, "task");
    EXPECT(ctx->Stats().host_bytes_allocated > before.host_bytes_allocated);
    // the mock's invariant: an offloaded store cannot take part in device work
    EXPECT(throws([&] { ctx->Reshard(0, 0, param[0], root[0]); }, "offloaded"));  // consumes no position
    for (int d = 0; d < kLocal; ++d) ctx->OffloadHtoD(d, {root[d]}, "task");
    EXPECT(ctx->Stats().host_blocking_syncs == before.host_blocking_syncs);
    EXPECT(ctx->Stats().device_allocations == before.device_allocations);  // the tile came back out of the device cache
    for (int d = 0; d < kLocal; ++d) ctx->OffloadDtoH(d, {root[d]}, {}, "task");  // pinned buffer from the host cache
    for (int d = 0; d < kLocal; ++d) ctx->OffloadHtoD(d, {root[d]}, "task");
    EXPECT(ctx->Stats().host_cache_hits == before.host_cache_hits + 1);
    EXPECT(ctx->Stats().host_bytes_allocated == before.host_bytes_allocated + 4 * ShardSize(dst));  // still one pinned buffer
    std::vector<uint16_t> got(expect[0].size());
    ctx->CopyShardToHost(root[8], got.data(), got.size() * 2);
    EXPECT(std::memcmp(got.data(), expect[0].data(), got.size() * 2) == 0);
  }

  // control replication broken: device 1 describes the k-th store differently from device 0
  {
    StoreHandle a = ctx->CreateStore(0, 0, dst);
    EXPECT(throws([&] { ctx->CreateStore(1, 1, src); }, "control replication"));
    (void)a;
  }
  // ... or reshards different stores than device 0 did in the same position
  {
    ctx->Reshard(0, 0, param[0], root[0]);
    EXPECT(throws([&] { ctx->Reshard(1, 1, root[1], param[1]); }, "control replication"));
  }

  // A schedule window of many Reshard ops (a pytree crossing a task boundary, mm_pjrt_executable.cc:616-658):
  // op by op, device by device, exactly as Execute issues them.  They leave as one batch: one plan, one launch.
  {
    auto win = HipExecuteContext::Create(local);
    const int kArrays = 9;
    std::vector<ShardedShape> ws(kArrays), wd(kArrays);
    std::vector<std::vector<std::vector<float>>> wshards(kArrays);
    std::vector<std::vector<StoreHandle>> wparam(kArrays, std::vector<StoreHandle>(kLocal)),
        wroot(kArrays, std::vector<StoreHandle>(kLocal));
    for (int a = 0; a < kArrays; ++a) {
      const int64_t rows = 64 * (1 + a % 3), cols = 128 * (1 + a % 2);
      ws[a] = ShardedShape{SupportedType::F32, {{{rows, 1, 0}, {cols, 4, 1}}, DeviceList::Create(0, 4)}, {}};
      wd[a] = ShardedShape{SupportedType::F32, {{{rows, 8, 0}, {cols, 1, 1}}, DeviceList::Create(4, 8)}, {}};
      wshards[a].assign(4, std::vector<float>(rows * cols / 4));
      for (auto& sh : wshards[a])
        for (auto& v : sh) {
          lcg = lcg * 1664525u + 1013904223u;
          v = static_cast<float>(lcg >> 8);
        }
      for (int d = 0; d < kLocal; ++d) {
        Shard shard{d < 4 ? wshards[a][d].data() : nullptr, d, d < 4 ? wshards[a][d].size() * 4 : 0};
        wparam[a][d] = win->AssembleShards(d, d, ws[a], shard);
      }
      for (int d = 0; d < kLocal; ++d) wroot[a][d] = win->CreateStore(d, d, wd[a]);
    }
    const mmr_context_stats before = win->Stats();
    for (int a = 0; a < kArrays; ++a)
      for (int d = 0; d < kLocal; ++d) win->Reshard(d, d, wparam[a][d], wroot[a][d]);
    const mmr_context_stats after = win->Stats();  // flushes the window
    EXPECT(after.reshard_calls - before.reshard_calls == 1);
    EXPECT(after.kernel_launches - before.kernel_launches == 1);
    EXPECT(after.plans_built - before.plans_built == 1);
    for (int a = 0; a < kArrays; ++a) {
      const size_t n = static_cast<size_t>(ShardSize(wd[a])) / 4;
      std::vector<std::vector<float>> want(8, std::vector<float>(n));
      orc_desc so = to_orc(ws[a], 4), dd = to_orc(wd[a], 4);
      const void* sp[4];
      void* dp[8];
      for (int k = 0; k < 4; ++k) sp[k] = wshards[a][k].data();
      for (int k = 0; k < 8; ++k) dp[k] = want[k].data();
      EXPECT(orc_reshard(&so, sp, &dd, dp, 1) == 0);
      for (int d = 4; d < kLocal; ++d) {
        std::vector<float> got(n);
        win->CopyShardToHost(wroot[a][d], got.data(), n * 4);
        EXPECT(std::memcmp(got.data(), want[d - 4].data(), n * 4) == 0);
      }
    }
    // a chain inside one window (B := reshard(A), then A2 := reshard(B)) is split where it depends on itself
    std::vector<StoreHandle> back(kLocal);
    for (int d = 0; d < kLocal; ++d) back[d] = win->CreateStore(d, d, ws[0]);
    const mmr_context_stats b2 = win->Stats();
    for (int d = 0; d < kLocal; ++d) win->Reshard(d, d, wparam[0][d], wroot[0][d]);
    for (int d = 0; d < kLocal; ++d) win->Reshard(d, d, wroot[0][d], back[d]);
    const mmr_context_stats a2 = win->Stats();
    EXPECT(a2.reshard_calls - b2.reshard_calls == 2);
    for (int d = 0; d < 4; ++d) {
      std::vector<float> got(wshards[0][d].size());
      win->CopyShardToHost(back[d], got.data(), got.size() * 4);
      EXPECT(std::memcmp(got.data(), wshards[0][d].data(), got.size() * 4) == 0);  // round trip restores the source
    }
    // a bad call is reported by the call itself, not when the window is flushed
    EXPECT(throws([&] { win->Reshard(0, 0, wparam[0][0], wroot[1][0]); }, "in the source and"));
    // without deferral every op launches on its own
    win->SetDeferReshards(false);
    const mmr_context_stats b3 = win->Stats();
    for (int a = 0; a < 3; ++a)
      for (int d = 0; d < kLocal; ++d) win->Reshard(d, d, wparam[a][d], wroot[a][d]);
    EXPECT(win->Stats().reshard_calls - b3.reshard_calls == 3);
  }

  // The schedule mirror: stores and reshard tasks registered as the scheduler does, executed as Execute does.
  {
    auto sc = HipExecuteContext::Create(local);
    ShardedShape a{SupportedType::F32, {{{96, 1, 0}, {128, 4, 1}}, DeviceList::Create(0, 4)}, {}};
    ShardedShape b{SupportedType::F32, {{{96, 8, 0}, {128, 1, 1}}, DeviceList::Create(4, 8)}, {}};
    ShardedShape c{SupportedType::F32, {{{96, 2, 0}, {128, 2, 1}}, DeviceList::Create(0, 4)}, {}};
    ReshardSchedule schedule;
    Store p0 = schedule.AddStore(Store::Type::PARAM, "p0", a);
    Store p1 = schedule.AddStore(Store::Type::PARAM, "p1", a);
    Store t0 = schedule.AddStore(Store::Type::TEMP, "t0", b);
    Store r0 = schedule.AddStore(Store::Type::ROOT, "r0", c);
    Store r1 = schedule.AddStore(Store::Type::ROOT, "r1", b);
    schedule.AddReshardTask(p0, t0);
    schedule.AddReshardTask(t0, r0);  // depends on the first: the window splits here
    schedule.AddReshardTask(p1, r1);
    schedule.AddReshardTask(p1, r1);  // scheduled once
    EXPECT(schedule.schedule().size() == 3 && schedule.num_parameters() == 2 && schedule.num_roots() == 2);
    std::vector<std::vector<float>> data0(4, std::vector<float>(96 * 32)), data1 = data0;
    for (auto* set : {&data0, &data1})
      for (auto& sh : *set)
        for (auto& v : sh) {
          lcg = lcg * 1664525u + 1013904223u;
          v = static_cast<float>(lcg >> 9);
        }
    std::vector<std::vector<StoreHandle>> params(kLocal, std::vector<StoreHandle>(2));
    for (int d = 0; d < kLocal; ++d) {
      params[d][0] = sc->AssembleShards(d, d, a, Shard{d < 4 ? data0[d].data() : nullptr, d, d < 4 ? data0[d].size() * 4 : 0});
      params[d][1] = sc->AssembleShards(d, d, a, Shard{d < 4 ? data1[d].data() : nullptr, d, d < 4 ? data1[d].size() * 4 : 0});
    }
    auto expect_for = [&](const std::vector<std::vector<float>>& in, const ShardedShape& to, int devs) {
      std::vector<std::vector<float>> out(devs, std::vector<float>(static_cast<size_t>(ShardSize(to)) / 4));
      orc_desc so = to_orc(a, 4), dd = to_orc(to, 4);
      const void* sp[4];
      void* dp[8];
      for (int k = 0; k < 4; ++k) sp[k] = in[k].data();
      for (int k = 0; k < devs; ++k) dp[k] = out[k].data();
      if (orc_reshard(&so, sp, &dd, dp, 1) != 0) out.clear();
      return out;
    };
    const auto want_r0 = expect_for(data0, c, 4), want_r1 = expect_for(data1, b, 8);
    EXPECT(!want_r0.empty() && !want_r1.empty());
    int64_t first_root = -1;
    const int64_t stores_before = sc->Stats().stores_live;
    for (int run_index = 0; run_index < 2; ++run_index) {
      const mmr_context_stats s0 = sc->Stats();
      auto roots = schedule.Execute(*sc, params);
      const mmr_context_stats s1 = sc->Stats();
      EXPECT(s1.reshard_calls - s0.reshard_calls == 2);  // {p0->t0} | {t0->r0, p1->r1}
      for (int d = 0; d < 4; ++d) {
        std::vector<float> got(want_r0[d].size());
        sc->CopyShardToHost(roots[d][0], got.data(), got.size() * 4);
        EXPECT(std::memcmp(got.data(), want_r0[d].data(), got.size() * 4) == 0);
      }
      for (int d = 4; d < kLocal; ++d) {
        std::vector<float> got(want_r1[d - 4].size());
        sc->CopyShardToHost(roots[d][1], got.data(), got.size() * 4);
        EXPECT(std::memcmp(got.data(), want_r1[d - 4].data(), got.size() * 4) == 0);
      }
      // roots are new stores per execution, the temporary is created once
      if (run_index == 0) first_root = roots[0][0].unique_id;
      else EXPECT(roots[0][0].unique_id != first_root);
      EXPECT(sc->Stats().stores_live == stores_before + 1 + 2);  // t0 + this run's two roots (last run's are gone)
    }
    // Steady state of a training loop: fresh ROOT stores every execution, yet no allocation, no table upload and no
    // wait on the device from the third execution on (the roots' memory comes back through the allocator's pool at
    // the same addresses, so the device tables bound to them are found again).
    for (int warm = 0; warm < 2; ++warm) schedule.Execute(*sc, params);
    const mmr_context_stats steady0 = sc->Stats();
    for (int step = 0; step < 5; ++step) schedule.Execute(*sc, params);
    const mmr_context_stats steady1 = sc->Stats();
    EXPECT(steady1.reshard_calls - steady0.reshard_calls == 10);
    EXPECT(steady1.device_allocations == steady0.device_allocations);
    EXPECT(steady1.bindings_built == steady0.bindings_built);
    EXPECT(steady1.plans_built == steady0.plans_built);
    // ... with the bracket every execution carries (OpenWindow, StartTimer, MarkProfile ... StopTimer, CloseWindow,
    // MarkProfile): the only wait it may cause is the window limit's
    EXPECT(steady1.host_blocking_syncs - steady1.window_waits == steady0.host_blocking_syncs - steady0.window_waits);
    EXPECT(steady1.windows_opened - steady0.windows_opened == 5);
    EXPECT(steady1.profile_marks - steady0.profile_marks == 10);
    // StopTimer, CloseWindow and the next execution's StartTimer mark the same point of the stream: one event
    EXPECT(steady1.events_recorded - steady0.events_recorded == 5);
    EXPECT(steady1.pool_hits - steady0.pool_hits == 10);
    int64_t timed = 0;
    const double last = sc->WaitTimerMilliseconds(schedule.name());
    (void)sc->LastTimerMilliseconds(schedule.name(), &timed);
    EXPECT(timed == 9 && last > 0.0 && last < 1000.0);  // one interval per execution so far
    // the compute callbacks of an execution (mm_pjrt_executable.cc:369-377, 660-667): one per local device
    std::atomic<int> fired{0};
    std::vector<std::function<void()>> on_done;
    for (int d = 0; d < kLocal; ++d) on_done.push_back([&fired] { fired.fetch_add(1); });
    schedule.Execute(*sc, params, &on_done);
    EXPECT(mmr_sync(sc->raw()) == MMR_OK);
    EXPECT(fired.load() == kLocal);
  }

  // Window back-pressure (zuku_execute_context_impl.cc:46, 128-136): with 8 windows still running on the device the
  // ninth OpenWindow waits for the oldest, the eighth does not.  The device is held at a host function on the
  // context's stream (no kernel waits for anything), released by this test; it lets go by itself after 20 s.
  {
    auto wc = HipExecuteContext::Create({0});
    void* stream = nullptr;
    EXPECT(mmr_context_stream(wc->raw(), &stream) == MMR_OK);
    static std::atomic<bool> gate_open{false};
    gate_open.store(false);
    EXPECT(hipLaunchHostFunc(static_cast<hipStream_t>(stream),
                             [](void*) {
                               const auto until = std::chrono::steady_clock::now() + std::chrono::seconds(20);
                               while (!gate_open.load() && std::chrono::steady_clock::now() < until)
                                 std::this_thread::sleep_for(std::chrono::milliseconds(1));
                             },
                             nullptr) == hipSuccess);
    const mmr_context_stats w0 = wc->Stats();
    for (int w = 0; w < 8; ++w) {
      wc->OpenWindow();
      wc->CloseWindow();
    }
    const mmr_context_stats w1 = wc->Stats();
    EXPECT(w1.windows_opened - w0.windows_opened == 8);
    EXPECT(w1.window_waits == w0.window_waits && w1.host_blocking_syncs == w0.host_blocking_syncs);
    std::atomic<bool> ninth_returned{false};
    std::thread ninth([&] {
      wc->OpenWindow();
      ninth_returned.store(true);
    });
    std::this_thread::sleep_for(std::chrono::milliseconds(200));
    const bool blocked = !ninth_returned.load();
    gate_open.store(true);
    ninth.join();
    EXPECT(blocked);
    wc->CloseWindow();
    const mmr_context_stats w2 = wc->Stats();
    EXPECT(w2.window_waits - w1.window_waits == 1);
    EXPECT(w2.host_blocking_syncs - w1.host_blocking_syncs == 1);
    // a higher limit: nothing waits
    wc->SetMaxOpenWindows(64);
    for (int w = 0; w < 20; ++w) {
      wc->OpenWindow();
      wc->CloseWindow();
    }
    EXPECT(wc->Stats().window_waits == w2.window_waits);
  }

  // Free(keep_in_cache) + CreateStore(allocate_from_cache) on a fresh context
  auto ctx2 = HipExecuteContext::Create({0, 1});
  ShardedShape small{SupportedType::F32, {{{16, 2, 0}}, DeviceList::Create(0, 2)}, {}};
  StoreHandle h0 = ctx2->CreateStore(0, 0, small), h1 = ctx2->CreateStore(1, 1, small);
  const int64_t bytes = ctx2->Stats().bytes_allocated;
  ctx2->Free(0, h0, /*keep_in_cache=*/true);
  EXPECT(ctx2->Stats().stores_live == 1);  // device 1 still holds it
  ctx2->Free(1, h1, /*keep_in_cache=*/true);
  EXPECT(ctx2->Stats().stores_live == 0);
  EXPECT(throws([&] { ctx2->SliceLocalShard(0, h0); }, "was freed"));  // the caller's copy of the handle is dead too
  StoreHandle h2 = ctx2->CreateStore(0, 0, small, {.allocate_from_cache = true});
  StoreHandle h3 = ctx2->CreateStore(1, 1, small, {.allocate_from_cache = true});
  EXPECT(ctx2->Stats().cache_hits == 1);
  EXPECT(ctx2->Stats().bytes_allocated == bytes);
  // unsupported element type and bad descriptors surface as exceptions, not aborts
  ShardedShape bad = small;
  bad.sharding.dims[0].permutation = 3;
  EXPECT(throws([&] { ctx2->CreateStore(0, 0, bad); }, "permutation"));
  // the failed call consumed no position: both devices can go on in step
  StoreHandle h4 = ctx2->CreateStore(0, 0, small), h5 = ctx2->CreateStore(1, 1, small);
  EXPECT(h4.unique_id == h5.unique_id);
  ctx2->Destroy(h2);
  ctx2->Destroy(h3);
  // Free without keep_in_cache only drops the copy it is given (zuku_execute_context_impl.cc:513-514): every other
  // copy of the handle still works, and the store lives until the last one goes
  {
    StoreHandle k0 = ctx2->CreateStore(0, 0, small), k1 = ctx2->CreateStore(1, 1, small);
    const int64_t live = ctx2->Stats().stores_live;
    ctx2->Free(0, k0, /*keep_in_cache=*/false);
    EXPECT(ctx2->Stats().stores_live == live);
    EXPECT(ctx2->SliceLocalShard(0, k0) != nullptr);
    ctx2->Destroy(k0);
    ctx2->Destroy(k1);
    EXPECT(ctx2->Stats().stores_live == live - 1);
  }
  // CreateStoreConfig::min_cache_size: the cache of the descriptor is filled to that many buffers at once
  {
    ShardedShape other{SupportedType::F32, {{{6000, 2, 0}}, DeviceList::Create(0, 2)}, {}};  // a size nothing has freed yet
    const mmr_context_stats b = ctx2->Stats();
    StoreHandle m0 = ctx2->CreateStore(0, 0, other, {.allocate_from_cache = true, .min_cache_size = 3});
    StoreHandle m1 = ctx2->CreateStore(1, 1, other, {.allocate_from_cache = true, .min_cache_size = 3});
    EXPECT(ctx2->Stats().device_allocations == b.device_allocations + 3);
    StoreHandle n0 = ctx2->CreateStore(0, 0, other, {.allocate_from_cache = true});
    StoreHandle n1 = ctx2->CreateStore(1, 1, other, {.allocate_from_cache = true});
    StoreHandle o0 = ctx2->CreateStore(0, 0, other, {.allocate_from_cache = true});
    StoreHandle o1 = ctx2->CreateStore(1, 1, other, {.allocate_from_cache = true});
    EXPECT(ctx2->Stats().device_allocations == b.device_allocations + 3);
    EXPECT(ctx2->Stats().cache_hits == b.cache_hits + 2);
    EXPECT(m0.unique_id == m1.unique_id && n0.unique_id != m0.unique_id && o1.unique_id != n1.unique_id);
  }

  // The buffer wrapper (MultiMeshPjRtBuffer): native shards -> store, store -> zero-copy view that pins the store.
  {
    auto bc = HipExecuteContext::Create(local);
    hipStream_t producer = nullptr;
    EXPECT(hipStreamCreateWithFlags(&producer, hipStreamNonBlocking) == hipSuccess);
    auto producer_stream = std::make_shared<MultiMeshStream>(producer);
    // native shards in device memory, written by work on the producer's stream that nobody waits for on the host
    std::vector<void*> device_shards(8, nullptr);
    std::vector<std::unique_ptr<ShardBuffer>> natives(kLocal);
    for (int d = 0; d < 8; ++d) {
      EXPECT(hipMalloc(&device_shards[d], shards[d].size() * 2) == hipSuccess);
      EXPECT(hipMemcpyAsync(device_shards[d], shards[d].data(), shards[d].size() * 2, hipMemcpyHostToDevice, producer) ==
             hipSuccess);
    }
    const mmr_context_stats b0 = bc->Stats();
    std::vector<StoreHandle> as_store(kLocal);
    for (int d = 0; d < kLocal; ++d) {
      auto native = std::make_shared<NativeBuffer>(d < 8 ? device_shards[d] : nullptr, d < 8 ? shards[d].size() * 2 : 0);
      natives[d] = std::make_unique<ShardBuffer>(native, std::vector<int64_t>{4, 64, 256}, std::vector<int64_t>{4, 64, 32},
                                                 SupportedType::BF16, bc, d, d, "param");
      EXPECT(natives[d]->has_native_buffer() && natives[d]->HasValidShard());
      as_store[d] = natives[d]->ToStore(src, producer_stream);
    }
    EXPECT(bc->Stats().host_blocking_syncs == b0.host_blocking_syncs);  // ordered by an event, not by the host
    // output buffers backed by a store, as Execute hands them out (mm_pjrt_executable.cc:684-689)
    std::vector<std::unique_ptr<ShardBuffer>> outs(kLocal);
    {
      std::vector<StoreHandle> r(kLocal);
      for (int d = 0; d < kLocal; ++d) r[d] = bc->CreateStore(d, d, dst, {.name = "out"});
      for (int d = 0; d < kLocal; ++d) bc->Reshard(d, d, as_store[d], r[d]);
      for (int d = 0; d < kLocal; ++d)
        outs[d] = std::make_unique<ShardBuffer>(r[d], std::vector<int64_t>{4, 64, 256}, std::vector<int64_t>{4, 16, 256},
                                                SupportedType::BF16, bc, d, d, "out");
    }  // the executable's own handles are gone: the buffers hold the store now
    for (int d = 0; d < kLocal; ++d) {
      EXPECT(outs[d]->has_store());
      EXPECT(outs[d]->HasValidShard() == (d >= 8));
      EXPECT(outs[d]->GetOnDeviceSizeInBytes() == static_cast<size_t>(ShardSize(dst)));
      EXPECT(outs[d]->ToStore(dst, producer_stream).unique_id == outs[d]->store().unique_id);  // already a store
    }
    // a view of device 9's tile, then every buffer and handle of the store goes
    std::unique_ptr<ShardBuffer> view = outs[9]->SliceLocalShard();
    EXPECT(view->has_native_buffer() && view->name() == "out.sliced");
    ShardBuffer::ExternalReference ext = outs[10]->AcquireExternalReference();
    EXPECT(ext.data != nullptr && ext.store.has_value());
    const int64_t live_before = bc->Stats().stores_live;
    outs.clear();
    EXPECT(bc->Stats().stores_live == live_before);  // the view and the external reference pin it
    // other work reuses freed memory if it can: a reshard into a new store of the same descriptor
    {
      std::vector<StoreHandle> r2(kLocal);
      for (int d = 0; d < kLocal; ++d) r2[d] = bc->CreateStore(d, d, dst);
      std::vector<std::vector<uint16_t>> other(8, std::vector<uint16_t>(4 * 64 * 32, 0x5A5A));
      std::vector<StoreHandle> p2(kLocal);
      for (int d = 0; d < kLocal; ++d)
        p2[d] = bc->AssembleShards(d, d, src, Shard{d < 8 ? other[d].data() : nullptr, d, d < 8 ? other[d].size() * 2 : 0});
      for (int d = 0; d < kLocal; ++d) bc->Reshard(d, d, p2[d], r2[d]);
      bc->Flush();
    }
    std::vector<uint16_t> got(expect[1].size());
    view->ToLiteral(got.data(), got.size() * 2);
    EXPECT(std::memcmp(got.data(), expect[1].data(), got.size() * 2) == 0);  // device 9 = second destination tile
    EXPECT(hipMemcpy(got.data(), ext.data, got.size() * 2, hipMemcpyDeviceToHost) == hipSuccess);
    EXPECT(std::memcmp(got.data(), expect[2].data(), got.size() * 2) == 0);
    view.reset();
    ext = ShardBuffer::ExternalReference{};
    EXPECT(bc->Stats().stores_live == live_before - 1);  // now it is gone
    natives.clear();
    as_store.clear();
    bc.reset();
    for (void* p : device_shards) EXPECT(hipFree(p) == hipSuccess);
    EXPECT(hipStreamDestroy(producer) == hipSuccess);
  }

  // Checking mode kept from the reference's mock: the same schedule hashes the same on every run, a different one does
  // not; every reshard operand is checked for a tile on each of its devices.
  {
    auto run_schedule = [&](bool swap) -> int64_t {
      auto hc = HipExecuteContext::Create({0, 1, 2, 3});
      hc->SetCheckInvariants(true);
      ShardedShape a{SupportedType::F32, {{{32, 2, 0}, {16, 1, 1}}, DeviceList::Create(0, 2)}, {}};
      ShardedShape b{SupportedType::F32, {{{32, 1, 0}, {16, 2, 1}}, DeviceList::Create(2, 2)}, {}};
      std::vector<StoreHandle> x(4), y(4);
      for (int d = 0; d < 4; ++d) x[d] = hc->CreateStore(d, d, swap ? b : a);
      for (int d = 0; d < 4; ++d) y[d] = hc->CreateStore(d, d, swap ? a : b);
      for (int d = 0; d < 4; ++d) hc->Reshard(d, d, x[d], y[d]);
      const mmr_context_stats st = hc->Stats();
      return st.invariant_checks > 0 ? st.operation_hash : 0;
    };
    const int64_t h1 = run_schedule(false), h2 = run_schedule(false), h3 = run_schedule(true);
    EXPECT(h1 != 0 && h1 == h2 && h1 != h3);
  }

  // Output stores that come round in a longer cycle (the caller holds the results of the last three executions, the
  // parameters alternate between three sets: 12 combinations of buffers): every combination gets its device tables
  // the second time it is seen, after which no launch carries its tables in the kernel's argument block any more.
  {
    auto rc = HipExecuteContext::Create(local);
    ReshardSchedule rotating("rotating");
    const Store p = rotating.AddStore(Store::Type::PARAM, "p", src);
    const Store r = rotating.AddStore(Store::Type::ROOT, "r", dst);
    rotating.AddReshardTask(p, r);
    std::vector<std::vector<std::vector<StoreHandle>>> sets(
        3, std::vector<std::vector<StoreHandle>>(kLocal, std::vector<StoreHandle>(1)));
    for (auto& set : sets)
      for (int d = 0; d < kLocal; ++d) set[d][0] = rc->CreateStore(d, d, src);
    std::vector<std::vector<std::vector<StoreHandle>>> keep(3);
    int turn = 0;
    auto execute = [&] {
      auto roots = rotating.Execute(*rc, sets[turn % 3]);
      keep[turn % 3] = std::move(roots);
      ++turn;
    };
    for (int i = 0; i < 36; ++i) execute();
    const mmr_context_stats r0 = rc->Stats();
    for (int i = 0; i < 24; ++i) execute();
    const mmr_context_stats r1 = rc->Stats();
    EXPECT(r1.reshard_calls - r0.reshard_calls == 24);
    EXPECT(r1.inline_launches == r0.inline_launches);
    EXPECT(r1.bindings_built == r0.bindings_built);
    EXPECT(r1.binding_cache_hits - r0.binding_cache_hits == 24);
    EXPECT(r1.device_allocations == r0.device_allocations);
  }

  // A context that goes away with callbacks still waiting runs them all first - also the one a callback queued in
  // its turn, behind a reshard it issued.
  {
    std::atomic<int> ran{0};
    {
      auto dc = HipExecuteContext::Create({0, 1});
      ShardedShape a{SupportedType::F32, {{{64, 2, 0}, {32, 1, 1}}, DeviceList::Create(0, 2)}, {}};
      ShardedShape b{SupportedType::F32, {{{64, 1, 0}, {32, 2, 1}}, DeviceList::Create(0, 2)}, {}};
      std::vector<StoreHandle> x(2), y(2);
      for (int d = 0; d < 2; ++d) x[d] = dc->CreateStore(d, d, a);
      for (int d = 0; d < 2; ++d) y[d] = dc->CreateStore(d, d, b);
      for (int d = 0; d < 2; ++d) dc->Reshard(d, d, x[d], y[d]);
      HipExecuteContext* raw = dc.get();
      dc->RunAfterAllTasks(0, [&ran, raw, x, y] {
        ran.fetch_add(1);
        for (int d = 0; d < 2; ++d) raw->Reshard(d, d, x[d], y[d]);
        raw->RunAfterAllTasks(0, [&ran] { ran.fetch_add(10); });
      });
    }
    EXPECT(ran.load() == 11);
  }

  std::printf("OK\n");
  return 0;
}

int main() {
  try {
    return run();
  } catch (const std::exception& e) {
    std::fprintf(stderr, "ERROR: %s\n", e.what());
    return 2;
  }
}
