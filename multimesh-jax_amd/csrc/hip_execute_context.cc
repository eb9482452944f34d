// See hip_execute_context.h.
#include "hip_execute_context.h"

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <stdexcept>

namespace mmr {

namespace {
[[noreturn]] void raise(const std::string& what) { throw std::runtime_error(what); }
void require_live(const StoreHandle& h, const char* where);
void check(int status, const char* where) {
  if (status != MMR_OK) raise(std::string(where) + ": " + mmr_last_error());
}
}  // namespace

mmr_sharded_shape ShardedShape::ToPod() const {
  mmr_sharded_shape p{};
  if (sharding.dims.size() > MMR_MAX_DIMS) raise("ShardedShape has more than MMR_MAX_DIMS entries");
  p.dtype = static_cast<int32_t>(type);
  p.ndims = static_cast<int32_t>(sharding.dims.size());
  for (int i = 0; i < p.ndims; ++i)
    p.dims[i] = mmr_sharding_dim{sharding.dims[i].size, sharding.dims[i].sharding, sharding.dims[i].permutation};
  p.dev_start = sharding.devices.start();
  p.dev_count = sharding.devices.size();
  if (!minor_to_major.empty()) {
    p.has_layout = 1;
    for (size_t i = 0; i < minor_to_major.size() && i < MMR_MAX_DIMS; ++i) p.minor_to_major[i] = minor_to_major[i];
  }
  return p;
}

ShardedShape ShardedShape::FromPod(const mmr_sharded_shape& p) {
  ShardedShape s;
  s.type = static_cast<SupportedType>(p.dtype);
  for (int i = 0; i < p.ndims; ++i)
    s.sharding.dims.push_back(ShardingDim{p.dims[i].size, p.dims[i].sharding, p.dims[i].permutation});
  s.sharding.devices = DeviceList::Create(p.dev_start, p.dev_count);
  if (p.has_layout) {
    int32_t rank = 0;
    int64_t ext[MMR_MAX_DIMS];
    check(mmr_shard_extents(&p, ext, &rank), "ShardedShape::FromPod");
    s.minor_to_major.assign(p.minor_to_major, p.minor_to_major + rank);
  }
  return s;
}

int64_t ShardSize(const ShardedShape& shape) {
  mmr_sharded_shape p = shape.ToPod();
  int64_t bytes = 0;
  check(mmr_shard_bytes(&p, &bytes), "ShardSize");
  return bytes;
}

MultiMeshStream::~MultiMeshStream() {
  if (event_) (void)hipEventDestroy(static_cast<hipEvent_t>(event_));
}

void* MultiMeshStream::RecordEvent() {
  if (!event_) {
    hipEvent_t e = nullptr;
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) raise("MultiMeshStream: hipEventCreate failed");
    event_ = e;
  }
  if (hipEventRecord(static_cast<hipEvent_t>(event_), static_cast<hipStream_t>(stream_)) != hipSuccess)
    raise("MultiMeshStream: hipEventRecord failed");
  return event_;
}

// One sharded array; freed when the last handle of the last device lets go.
struct HipExecuteContext::SharedStore {
  mmr_context* ctx{nullptr};
  std::shared_ptr<std::atomic<bool>> ctx_alive;
  mmr_store* store{nullptr};
  ShardedShape shape;
  bool keep_in_cache{false};
  ~SharedStore() {
    // a handle may outlive its context (shutdown order); the context then took the buffers with it
    if (store && ctx_alive && ctx_alive->load()) mmr_store_free(ctx, store, keep_in_cache ? 1 : 0);
  }
};

struct StoreHandleImpl {
  std::shared_ptr<HipExecuteContext::SharedStore> array;
  std::string name;
  int64_t local_device_id{-1};
  int64_t global_device_id{-1};
};

namespace {
void require_live(const StoreHandle& h, const char* where) {
  if (!h.impl) raise(std::string(where) + ": empty store handle");
  if (!h.impl->array) raise(std::string(where) + ": store " + std::to_string(h.unique_id) + " was freed");
}
}  // namespace

std::shared_ptr<HipExecuteContext> HipExecuteContext::Create(std::set<int> local_devices, int hip_device) {
  std::shared_ptr<HipExecuteContext> c(new HipExecuteContext());
  if (local_devices.empty()) raise("HipExecuteContext::Create: no local devices");
  if (*local_devices.begin() < 0) raise("HipExecuteContext::Create: negative local device id");
  c->local_devices_ = std::move(local_devices);
  c->position_of_.assign(static_cast<size_t>(*c->local_devices_.rbegin()) + 1, -1);
  int32_t position = 0;
  for (int d : c->local_devices_) c->position_of_[static_cast<size_t>(d)] = position++;
  for (OpStream& s : c->streams_) s.next_seq.assign(c->local_devices_.size(), 0);
  check(mmr_context_create(hip_device, nullptr, &c->ctx_), "HipExecuteContext::Create");
  return c;
}

HipExecuteContext::~HipExecuteContext() {
  pending_.clear();  // work nobody waited for
  for (OpStream& s : streams_) s.ops.clear();  // drops the stores still attached to half-arrived ops
  // Handles may outlive the context (Python shutdown order in the reference,
  // zuku_execute_context_impl.cc:64-71); their stores die with the context.
  alive_->store(false);
  if (ctx_) mmr_context_destroy(ctx_);  // runs the callbacks of RunAfterAllTasks that are still waiting
}

namespace {
const char* const kOpNames[] = {"CreateStore", "Reshard", "OffloadDtoH", "OffloadHtoD"};
}

HipExecuteContext::ReplicatedOp& HipExecuteContext::Arrive(OpKind kind, int64_t local_device_id, bool* first, int64_t* seq) {
  if (local_device_id < 0 || local_device_id >= static_cast<int64_t>(position_of_.size()) ||
      position_of_[static_cast<size_t>(local_device_id)] < 0)
    raise(std::string(kOpNames[kind]) + ": device " + std::to_string(local_device_id) + " is not a local device");
  OpStream& s = streams_[kind];
  *seq = s.next_seq[static_cast<size_t>(position_of_[static_cast<size_t>(local_device_id)])]++;
  const int64_t at = *seq - s.first_seq;  // >= 0: an op leaves the front only after every device has issued it
  *first = at == static_cast<int64_t>(s.ops.size());
  if (at > static_cast<int64_t>(s.ops.size()))
    raise(std::string(kOpNames[kind]) + ": call order between local devices is inconsistent");
  if (*first) s.ops.emplace_back();
  ReplicatedOp& op = s.ops[static_cast<size_t>(at)];
  op.arrivals += 1;
  return op;
}

void HipExecuteContext::Leave(OpKind kind) {
  OpStream& s = streams_[kind];
  const int n = static_cast<int>(local_devices_.size());
  while (!s.ops.empty() && s.ops.front().arrivals == n) {
    s.ops.pop_front();
    s.first_seq += 1;
  }
}

void HipExecuteContext::Retract(OpKind kind, int64_t local_device_id) {
  OpStream& s = streams_[kind];
  s.ops.pop_back();
  s.next_seq[static_cast<size_t>(position_of_[static_cast<size_t>(local_device_id)])]--;
}

StoreHandle HipExecuteContext::CreateStore(int64_t local_device_id, int64_t global_device_id, ShardedShape shape,
                                           CreateStoreConfig config) {
  std::lock_guard<std::mutex> lock(mu_);
  bool first = false;
  int64_t seq = 0;
  ReplicatedOp& op = Arrive(kCreateStore, local_device_id, &first, &seq);
  if (first) {
    auto shared = std::make_shared<SharedStore>();
    shared->ctx = ctx_;
    shared->ctx_alive = alive_;
    shared->shape = shape;
    mmr_sharded_shape pod = shape.ToPod();
    const char* name = config.name.has_value() ? config.name->c_str() : nullptr;
    const uint32_t flags = (config.allocate_from_cache ? MMR_STORE_FROM_CACHE : 0u) |
                           (config.uninitialized ? MMR_STORE_UNINITIALIZED : 0u);
    int rc = mmr_store_create_ex(ctx_, &pod, name, flags, config.min_cache_size.value_or(1), &shared->store);
    if (rc != MMR_OK) {
      Retract(kCreateStore, local_device_id);
      check(rc, "CreateStore");
    }
    op.store = shared;
  } else if (!(op.store->shape == shape)) {
    raise("CreateStore: device " + std::to_string(local_device_id) + " describes store #" + std::to_string(seq) +
          " differently from the device that created it (control replication broken)");
  }
  StoreHandle handle;
  handle.impl = std::make_shared<StoreHandleImpl>();
  handle.impl->array = op.store;
  handle.impl->name = config.name.value_or("anonymous");
  handle.impl->local_device_id = local_device_id;
  handle.impl->global_device_id = global_device_id;
  handle.unique_id = mmr_store_id(op.store->store);
  Leave(kCreateStore);
  return handle;
}

StoreHandle HipExecuteContext::AssembleShards(int64_t local_device_id, int64_t global_device_id, ShardedShape shape,
                                              Shard shard, std::shared_ptr<MultiMeshStream> stream,
                                              std::optional<StoreHandle> existing_store) {
  StoreHandle output =
      existing_store.has_value() ? *std::move(existing_store) : CreateStore(local_device_id, global_device_id, shape);
  require_live(output, "AssembleShards");
  std::lock_guard<std::mutex> lock(mu_);
  FlushLocked();
  // across(shape.sharding.devices).if_on(p): only a member device copies its shard
  if (shape.sharding.devices.Contains(global_device_id)) {
    // behind the producer of the native shard, on the device (zuku_execute_context_impl.cc:410-414 issues the copy on
    // the producer's own stream)
    if (stream && stream->hip_stream()) check(mmr_context_wait_event(ctx_, stream->RecordEvent()), "AssembleShards");
    check(mmr_store_assemble(ctx_, output.impl->array->store, global_device_id, shard.data, shard.size, 2),
          "AssembleShards");
  }
  return output;
}

void HipExecuteContext::Reshard(int64_t local_device_id, int64_t global_device_id, const StoreHandle& src,
                                const StoreHandle& dst) {
  (void)global_device_id;
  require_live(src, "Reshard");
  require_live(dst, "Reshard");
  std::lock_guard<std::mutex> lock(mu_);
  bool first = false;
  int64_t seq = 0;
  ReplicatedOp& op = Arrive(kReshard, local_device_id, &first, &seq);
  const int64_t s = src.unique_id, d = dst.unique_id;
  if (first) {
    op.a = s;
    op.b = d;
    // the whole copy runs once, for the first arriving device's call; it is queued so that the reshards of one
    // schedule window leave in one batch
    std::shared_ptr<SharedStore> sa = src.impl->array, da = dst.impl->array;
    int rc = mmr_reshard_validate(ctx_, sa->store, da->store);
    if (rc == MMR_OK && defer_reshards_) {
      // reads or overwrites a queued result, or overwrites a queued input
      const bool depends = pending_dsts_.count(sa.get()) || pending_dsts_.count(da.get()) || pending_srcs_.count(da.get());
      try {
        if (depends) FlushLocked();
      } catch (...) {
        Retract(kReshard, local_device_id);
        throw;
      }
      pending_srcs_.insert(sa.get());
      pending_dsts_.insert(da.get());
      pending_.emplace_back(std::move(sa), std::move(da));
    } else if (rc == MMR_OK) {
      rc = mmr_reshard(ctx_, sa->store, da->store);
    }
    if (rc != MMR_OK) {
      Retract(kReshard, local_device_id);
      check(rc, "Reshard");
    }
  } else if (op.a != s || op.b != d) {
    raise("Reshard: device " + std::to_string(local_device_id) + " issues reshard #" + std::to_string(seq) +
          " on different stores than the device that started it (control replication broken)");
  }
  Leave(kReshard);
}

void HipExecuteContext::FlushLocked() {
  if (pending_.empty()) return;
  flush_srcs_.clear();
  flush_dsts_.clear();
  for (const auto& q : pending_) {
    flush_srcs_.push_back(q.first->store);
    flush_dsts_.push_back(q.second->store);
  }
  auto keep = std::move(pending_);  // the stores stay alive until the launches are issued; a failure is not retried
  pending_.clear();
  pending_srcs_.clear();
  pending_dsts_.clear();
  (void)mmr_profile_range_push(ctx_, "HipExecuteContext: reshards of a window");  // the named region of a task
  const int rc = flush_srcs_.size() == 1
                     ? mmr_reshard(ctx_, flush_srcs_[0], flush_dsts_[0])
                     : mmr_reshard_batch(ctx_, flush_srcs_.data(), flush_dsts_.data(), static_cast<int32_t>(flush_srcs_.size()));
  (void)mmr_profile_range_pop(ctx_);
  check(rc, "Reshard");
}

void HipExecuteContext::Flush() {
  std::lock_guard<std::mutex> lock(mu_);
  FlushLocked();
}

void HipExecuteContext::SetCheckInvariants(bool on) {
  std::lock_guard<std::mutex> lock(mu_);
  FlushLocked();
  check(mmr_context_set_flags(ctx_, on ? MMR_CHECK_INVARIANTS : 0u), "SetCheckInvariants");
}

void HipExecuteContext::SetDeferReshards(bool defer) {
  std::lock_guard<std::mutex> lock(mu_);
  FlushLocked();
  defer_reshards_ = defer;
}

void* HipExecuteContext::SliceLocalShard(int64_t local_device_id, const StoreHandle& handle) {
  (void)local_device_id;
  require_live(handle, "SliceLocalShard");
  Flush();
  void* ptr = nullptr;
  check(mmr_store_shard_ptr(ctx_, handle.impl->array->store, handle.impl->global_device_id, &ptr), "SliceLocalShard");
  return ptr;
}

void* HipExecuteContext::TilePointer(const StoreHandle& handle) {
  require_live(handle, "TilePointer");
  Flush();
  void* ptr = nullptr;
  check(mmr_store_shard_ptr_async(ctx_, handle.impl->array->store, handle.impl->global_device_id, &ptr), "TilePointer");
  return ptr;
}

void HipExecuteContext::CopyShardToHost(const StoreHandle& handle, void* host_dst, size_t size) {
  require_live(handle, "CopyShardToHost");
  Flush();
  check(mmr_store_read_shard(ctx_, handle.impl->array->store, handle.impl->global_device_id, host_dst, size),
        "CopyShardToHost");
}

ShardedShape HipExecuteContext::GetStoreShardedShape(const StoreHandle& handle) {
  require_live(handle, "GetStoreShardedShape");
  return handle.impl->array->shape;
}

bool HipExecuteContext::HasLocalShard(const StoreHandle& handle) {
  if (!handle.impl || !handle.impl->array) return false;
  return handle.impl->array->shape.sharding.devices.Contains(handle.impl->global_device_id);
}

void HipExecuteContext::Free(int64_t local_device_id, StoreHandle handle, bool keep_in_cache) {
  (void)local_device_id;
  if (!handle.impl) return;
  std::lock_guard<std::mutex> lock(mu_);
  if (!handle.impl->array) return;  // already freed through another copy of this handle
  // As in the reference (zuku_execute_context_impl.cc:504-515): with keep_in_cache the array is moved out of the shared
  // impl into the cache, so every copy of this device's handle lets go (the buffers are parked once the last device has
  // freed); without it only the copy passed by value is dropped and the array lives on for every other copy.
  if (!keep_in_cache) return;
  handle.impl->array->keep_in_cache = true;
  handle.impl->array.reset();
}

void HipExecuteContext::Destroy(StoreHandle& store) { store.impl = nullptr; }

void HipExecuteContext::ClearStoreCache(int64_t local_device_id) {
  (void)local_device_id;
  check(mmr_clear_store_cache(ctx_), "ClearStoreCache");
}

void HipExecuteContext::Rename(StoreHandle& handle, std::string name) {
  if (handle.impl) handle.impl->name = std::move(name);
}

void HipExecuteContext::OffloadDtoH(int64_t local_device_id, const std::vector<StoreHandle>& to_offload,
                                    const std::vector<StoreHandle>& pipelined, const std::string& task_name) {
  (void)pipelined;
  (void)task_name;
  std::lock_guard<std::mutex> lock(mu_);
  bool first = false;
  int64_t seq = 0;
  (void)Arrive(kOffloadDtoH, local_device_id, &first, &seq);
  if (first) {
    try {
      FlushLocked();
      for (const StoreHandle& h : to_offload) {
        require_live(h, "OffloadDtoH");
        check(mmr_store_offload(ctx_, h.impl->array->store), "OffloadDtoH");
      }
    } catch (...) {
      Retract(kOffloadDtoH, local_device_id);  // the failed call consumed no position: the devices stay in step
      throw;
    }
  }
  Leave(kOffloadDtoH);
}

void HipExecuteContext::OffloadHtoD(int64_t local_device_id, const std::vector<StoreHandle>& to_offload,
                                    const std::string& task_name) {
  (void)task_name;
  std::lock_guard<std::mutex> lock(mu_);
  bool first = false;
  int64_t seq = 0;
  (void)Arrive(kOffloadHtoD, local_device_id, &first, &seq);
  if (first) {
    try {
      FlushLocked();
      for (const StoreHandle& h : to_offload) {
        require_live(h, "OffloadHtoD");
        check(mmr_store_reload(ctx_, h.impl->array->store), "OffloadHtoD");
      }
    } catch (...) {
      Retract(kOffloadHtoD, local_device_id);  // the failed call consumed no position: the devices stay in step
      throw;
    }
  }
  Leave(kOffloadHtoD);
}

void HipExecuteContext::OpenWindow() { check(mmr_window_open(ctx_), "OpenWindow"); }

void HipExecuteContext::CloseWindow() {
  Flush();
  check(mmr_window_close(ctx_), "CloseWindow");
}

void HipExecuteContext::SetMaxOpenWindows(int n) { check(mmr_context_set_max_open_windows(ctx_, n), "SetMaxOpenWindows"); }

void HipExecuteContext::RunAfterAllTasks(int64_t local_device_id, std::function<void()> on_done) {
  (void)local_device_id;
  if (!on_done) return;  // zuku_execute_context_impl.cc:349
  Flush();
  // deferred behind everything queued so far, like after(last_execute_events_[...]).defer(callback); the caller
  // does not wait
  auto* boxed = new std::function<void()>(std::move(on_done));
  const int rc = mmr_context_run_after(
      ctx_,
      [](void* p) {
        std::unique_ptr<std::function<void()>> fn(static_cast<std::function<void()>*>(p));
        (*fn)();
      },
      boxed);
  if (rc != MMR_OK) {
    delete boxed;
    check(rc, "RunAfterAllTasks");
  }
}

void HipExecuteContext::MarkProfile(const std::string& name) { check(mmr_profile_mark(ctx_, name.c_str()), "MarkProfile"); }

void HipExecuteContext::StartTimer(const std::string& name) {
  Flush();  // the timer starts behind the work issued so far
  check(mmr_timer_begin(ctx_, name.c_str()), "StartTimer");
}

void HipExecuteContext::StopTimer(const std::string& name) {
  Flush();
  const int rc = mmr_timer_end(ctx_, name.c_str());
  if (rc == MMR_NOT_FOUND) {  // zuku_execute_context_impl.cc:471-474: a warning, not an error
    std::fprintf(stderr, "warning: %s\n", mmr_last_error());
    return;
  }
  check(rc, "StopTimer");
}

double HipExecuteContext::LastTimerMilliseconds(const std::string& name, int64_t* completed) {
  float ms = 0;
  int64_t n = 0;
  check(mmr_timer_poll(ctx_, name.c_str(), &ms, &n), "LastTimerMilliseconds");
  if (completed) *completed = n;
  return ms;
}

double HipExecuteContext::WaitTimerMilliseconds(const std::string& name) {
  float ms = 0;
  check(mmr_timer_wait(ctx_, name.c_str(), &ms, nullptr), "WaitTimerMilliseconds");
  return ms;
}

mmr_context_stats HipExecuteContext::Stats() {
  Flush();
  mmr_context_stats s{};
  check(mmr_context_get_stats(ctx_, &s), "Stats");
  return s;
}

Store ReshardSchedule::AddStore(Store::Type type, std::string name, ShardedShape shape) {
  Store store;
  store.type = type;
  store.name = std::move(name);
  store.sharded_shape = std::move(shape);
  switch (type) {
    case Store::Type::PARAM: store.index = num_params_++; break;
    case Store::Type::ROOT: store.index = num_roots_++; break;
    case Store::Type::TEMP:
      store.index = static_cast<int64_t>(temporaries_.size());
      temporaries_.push_back(store);
      break;
  }
  return store;
}

void ReshardSchedule::AddReshardTask(const Store& input, const Store& output) {
  if (output.type == Store::Type::PARAM) raise("AddReshardTask: a parameter store cannot be a reshard's output");
  if (!already_scheduled_.emplace(input.name, output.name).second) return;
  schedule_.push_back(MpmdOperation{Reshard{input, output}});
}

std::vector<std::vector<StoreHandle>> ReshardSchedule::Execute(
    HipExecuteContext& ctx, const std::vector<std::vector<StoreHandle>>& parameter_stores,
    std::vector<std::function<void()>>* on_done) {
  const std::set<int> local = ctx.GetLocalDevices();
  const std::vector<int> devices(local.begin(), local.end());
  const size_t n = devices.size();
  if (parameter_stores.size() != n) raise("Execute: one list of parameter stores per local device is required");
  for (const auto& p : parameter_stores)
    if (static_cast<int64_t>(p.size()) != num_params_) raise("Execute: wrong number of parameter stores");
  if (on_done && !on_done->empty() && on_done->size() != n) raise("Execute: one callback per local device is required");
  if (start_mark_.empty()) {
    start_mark_ = "start " + name_;
    finish_mark_ = "finish " + name_;
  }
  // mm_pjrt_executable.cc:362-364
  ctx.OpenWindow();
  ctx.StartTimer(name_);
  ctx.MarkProfile(start_mark_);
  std::vector<std::vector<StoreHandle>> root_stores(n, std::vector<StoreHandle>(static_cast<size_t>(num_roots_)));
  for (const MpmdOperation& op : schedule_) {  // add_root_store: once per root, for every local device
    const Store& out = op.op.output;
    if (out.type != Store::Type::ROOT || root_stores[0][out.index].impl) continue;
    for (size_t i = 0; i < n; ++i)
      // written entirely by the reshard that produces it (pad included): no zero fill
      root_stores[i][out.index] =
          ctx.CreateStore(devices[i], devices[i], out.sharded_shape, {.name = out.name, .uninitialized = true});
  }
  if (cached_temporary_stores_.empty()) {
    cached_temporary_stores_.resize(n);
    for (size_t i = 0; i < n; ++i)
      for (const Store& t : temporaries_)
        cached_temporary_stores_[i].push_back(ctx.CreateStore(devices[i], devices[i], t.sharded_shape, {.name = t.name}));
  }
  auto handle_of = [&](size_t i, const Store& store) -> const StoreHandle& {
    switch (store.type) {
      case Store::Type::PARAM: return parameter_stores[i][store.index];
      case Store::Type::ROOT: return root_stores[i][store.index];
      default: return cached_temporary_stores_[i][store.index];
    }
  };
  for (const MpmdOperation& op : schedule_)
    for (size_t i = 0; i < n; ++i)
      ctx.Reshard(devices[i], devices[i], handle_of(i, op.op.input), handle_of(i, op.op.output));
  if (on_done && !on_done->empty())  // :660-667
    for (size_t i = 0; i < n; ++i) ctx.RunAfterAllTasks(devices[i], std::move((*on_done)[i]));
  // :704-706
  ctx.StopTimer(name_);
  ctx.CloseWindow();
  ctx.MarkProfile(finish_mark_);
  return root_stores;
}

}  // namespace mmr
