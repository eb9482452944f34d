// C++ host-side mirror of the store/reshard subset of xla::ZukuExecuteContext
// (reference: src/pjrt_client/zuku_execute_context.h:38-133), implemented on the
// C ABI of mmreshard.h.  Same method names, argument order and meaning, so the
// plugin's callers (mm_pjrt_executable.cc:391-431, 495-498, 548-561, 616-658;
// mm_pjrt_buffer.cc:141-142, 175-183) read the same against it.
//
// The zuku:: types the reference signatures use are mirrored here as plain
// structs with the fields and accessors the plugin touches (mm_sharding.cc:
// 53-61, 345-372, 638-668; mpmd_utils.cc:151-175).
//
// Control replication.  The plugin drives the context SPMD-style: every local
// device issues the same calls in the same order ("for local_device in
// num_local_devices", mm_pjrt_executable.cc:618-619).  Here all logical devices
// live in one GPU, so the k-th CreateStore / Reshard / Free of every device
// refers to the same sharded array / copy; the first arriving call does the
// work and the others attach to it.  Diverging arguments between devices are
// an invariant violation and throw.
//
// Errors: the reference's methods return void and abort on invariant
// violations (zuku_execute_context_impl.cc:271-290); the mock throws
// std::runtime_error.  This class throws std::runtime_error carrying
// mmr_last_error(); a caller that wants the reference's behaviour aborts.
#ifndef MMR_CSRC_HIP_EXECUTE_CONTEXT_H_
#define MMR_CSRC_HIP_EXECUTE_CONTEXT_H_

#include <atomic>
#include <cstdint>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <optional>
#include <set>
#include <string>
#include <unordered_set>
#include <vector>

#include "mmreshard.h"

namespace mmr {

// zuku::SupportedType: the fifteen types mm_sharding.cc:376-425 maps to.
enum class SupportedType : int32_t {
  PRED = MMR_PRED, F16 = MMR_F16, BF16 = MMR_BF16, F32 = MMR_F32, F64 = MMR_F64,
  S8 = MMR_S8, S16 = MMR_S16, S32 = MMR_S32, S64 = MMR_S64,
  U8 = MMR_U8, U16 = MMR_U16, U32 = MMR_U32, U64 = MMR_U64, C64 = MMR_C64, C128 = MMR_C128,
  F8E4M3FN = MMR_F8E4M3FN, F8E5M2 = MMR_F8E5M2,  // extensions
};

// zuku::ShardingDim
struct ShardingDim {
  int64_t size{1};
  int64_t sharding{1};
  int64_t permutation{0};
  bool operator==(const ShardingDim& o) const {
    return size == o.size && sharding == o.sharding && permutation == o.permutation;
  }
};

// zuku::DeviceList: a contiguous range of global device ids.
class DeviceList {
 public:
  struct Range {
    int64_t start{0};
    int64_t num_devices{0};
  };
  DeviceList() = default;
  DeviceList(Range r) : range_(r) {}  // NOLINT: the reference writes DeviceList{{.start=, .num_devices=}}
  static DeviceList Create(int64_t start, int64_t num_devices) { return DeviceList(Range{start, num_devices}); }
  int64_t start() const { return range_.start; }
  int64_t stop() const { return range_.start + range_.num_devices; }
  int64_t size() const { return range_.num_devices; }
  int64_t operator[](int64_t i) const { return range_.start + i; }
  bool Contains(int64_t device) const { return device >= start() && device < stop(); }
  bool Contains(const DeviceList& o) const { return o.start() >= start() && o.stop() <= stop(); }
  bool operator==(const DeviceList& o) const { return start() == o.start() && size() == o.size(); }
  bool operator!=(const DeviceList& o) const { return !(*this == o); }

 private:
  Range range_;
};

// zuku::ShardedShape {type, sharding{dims, devices}}
struct ShardedShape {
  SupportedType type{SupportedType::F32};
  struct Sharding {
    std::vector<ShardingDim> dims;
    DeviceList devices;
  } sharding;
  std::vector<int32_t> minor_to_major;  // extension; empty = row-major shards like the reference

  bool operator==(const ShardedShape& o) const {
    return type == o.type && sharding.dims == o.sharding.dims && sharding.devices == o.sharding.devices &&
           minor_to_major == o.minor_to_major;
  }
  mmr_sharded_shape ToPod() const;
  static ShardedShape FromPod(const mmr_sharded_shape& pod);
};

// zuku::ShardSize(shape): bytes of one shard buffer (mm_mock_mm_xla.cc:75).
int64_t ShardSize(const ShardedShape& shape);

// zuku_execute_context.h:20-30
struct Shard {
  const void* data;
  int64_t local_device_id;
  size_t size;
};
struct CreateStoreConfig {
  std::optional<std::string> name{std::nullopt};
  bool allocate_from_cache{false};
  std::optional<int64_t> min_cache_size{std::nullopt};  // -> mmr_store_create_ex
  bool uninitialized{false};  // extension: skip the zero fill (the store is a reshard's output: every byte is written)
};

// MultiMeshStream (mm_computation.h:131-149): the stream a native shard's producer runs on.  The reference issues the
// assemble copy on it (zuku_execute_context_impl.cc:405-415); here the copy runs on the context's stream and is ordered
// behind the producer's work by an event, without blocking the host.
class MultiMeshStream {
 public:
  explicit MultiMeshStream(void* hip_stream) : stream_(hip_stream) {}
  ~MultiMeshStream();
  void* hip_stream() const { return stream_; }
  // Records the producer's progress so far; returns the hipEvent_t (owned by this object).
  void* RecordEvent();

 private:
  void* stream_;
  void* event_{nullptr};
};

// store_handle_fwd.h:15-19, store_handle.h:16-20
struct StoreHandleImpl;
struct StoreHandle {
  std::shared_ptr<StoreHandleImpl> impl{nullptr};
  int64_t unique_id{-1};
};

// mpmd_store.h:16-25 and mpmd_partition.h:40-43, without the XLA members.
struct Store {
  enum class Type { PARAM, ROOT, TEMP };
  Type type{Type::TEMP};
  int64_t index{-1};
  std::string name;
  bool scalar{false};
  ShardedShape sharded_shape;
};
struct Reshard {
  Store input;
  Store output;
};

class HipExecuteContext {
 public:
  // ZukuExecuteContextImpl::Create (zuku_execute_context_impl.cc:559-577).
  // local_devices: the logical devices this process drives (all of them here).
  static std::shared_ptr<HipExecuteContext> Create(std::set<int> local_devices, int hip_device = 0);
  ~HipExecuteContext();

  StoreHandle CreateStore(int64_t local_device_id, int64_t global_device_id, ShardedShape shape,
                          CreateStoreConfig config = {});
  // Shard.data: device or host memory (the runtime tells which).  stream: where the shard's producer runs (may be
  // null: the shard is ready); the copy is ordered behind it on the device, the host does not wait.
  StoreHandle AssembleShards(int64_t local_device_id, int64_t global_device_id, ShardedShape shape, Shard shard,
                             std::shared_ptr<MultiMeshStream> stream = nullptr,
                             std::optional<StoreHandle> existing_store = std::nullopt);
  void Reshard(int64_t local_device_id, int64_t global_device_id, const StoreHandle& src, const StoreHandle& dst);
  void* SliceLocalShard(int64_t local_device_id, const StoreHandle& handle);
  // The same pointer without waiting, for work that stays on the context's stream (an adapter that launches compute
  // tasks there); queued reshards are issued first.
  void* TilePointer(const StoreHandle& handle);
  ShardedShape GetStoreShardedShape(const StoreHandle& handle);
  bool HasLocalShard(const StoreHandle& handle);
  void Free(int64_t local_device_id, StoreHandle handle, bool keep_in_cache);
  void Destroy(StoreHandle& store);
  void ClearStoreCache(int64_t local_device_id);
  void Rename(StoreHandle& handle, std::string name);
  // zuku_execute_context.h:61-68.  `pipelined` stores must have been produced
  // before the offload starts; on one stream that already holds.
  void OffloadDtoH(int64_t local_device_id, const std::vector<StoreHandle>& to_offload,
                   const std::vector<StoreHandle>& pipelined, const std::string& task_name);
  void OffloadHtoD(int64_t local_device_id, const std::vector<StoreHandle>& to_offload, const std::string& task_name);

  // zuku_execute_context_impl.cc:128-143: one window per execution; OpenWindow waits for the oldest window once
  // kMaxOpenWindows (8, :46) are still running on the device, CloseWindow marks the end of this one.
  void OpenWindow();
  void CloseWindow();
  // :347-354.  on_done runs on a thread the context owns, once everything issued so far is done; it may use the
  // context (drop buffers, issue work).  The call does not wait.
  void RunAfterAllTasks(int64_t local_device_id, std::function<void()> on_done);
  // :458-460: a named mark in the profile (a roctx marker).
  void MarkProfile(const std::string& name);
  // :462-486: named timers, any number pending, neither call waits for the device.  A second StartTimer of a running
  // name changes nothing; StopTimer of an unknown name prints the reference's warning and returns.
  void StartTimer(const std::string& name);
  void StopTimer(const std::string& name);
  std::set<int> GetLocalDevices() { return local_devices_; }
  bool IsGpu() { return true; }

  // Reshard calls are queued and issued together - one plan, one launch per kernel class for a whole schedule
  // window (the reference's Execute loop issues one Reshard per array, mm_pjrt_executable.cc:616-658; a pytree of
  // 195 arrays is 195 calls).  The queue is flushed by every other entry point that touches device memory or
  // time (AssembleShards, SliceLocalShard, CopyShardToHost, offloads, timers, RunAfterAllTasks, CloseWindow),
  // by a Reshard that depends on a queued one, and by Flush().  An adapter that also runs compute tasks calls
  // Flush() before it enqueues a task.  Argument errors are still raised by the Reshard call that causes them.
  void Flush();
  void SetDeferReshards(bool defer);
  // The reference's mock keeps invariants every C++ test of the plugin runs under (mm_mock_mm_xla.cc:259-262 rolling
  // hash of the operation stream, :347-369 every operand has a tile on each of its devices): kept here as a
  // checking mode; Stats().operation_hash is equal between two runs that issue the same operations.
  void SetCheckInvariants(bool on);

  // Not part of the reference interface: inspection for tests and benchmarks (both flush first).
  mmr_context* raw() {
    Flush();
    return ctx_;
  }
  // What ToLiteral does through SliceLocalShard (mm_pjrt_buffer.cc:84-95): blocking copy of the handle's shard.
  void CopyShardToHost(const StoreHandle& handle, void* host_dst, size_t size);
  mmr_context_stats Stats();
  // The most recent completed interval of the timer `name` (what the reference logs as "<name> finished in ...");
  // never waits: 0 until the device has passed the first StopTimer.  *completed: intervals completed so far.
  double LastTimerMilliseconds(const std::string& name, int64_t* completed = nullptr);
  // The same after waiting for every stopped interval of `name` (a host wait, counted as one).
  double WaitTimerMilliseconds(const std::string& name);
  void SetMaxOpenWindows(int n);

 private:
  struct SharedStore;  // one sharded array, shared by the handles of all local devices
  enum OpKind { kCreateStore = 0, kReshard, kOffloadDtoH, kOffloadHtoD, kNumOpKinds };
  struct ReplicatedOp {
    int64_t a{-1}, b{-1};
    std::shared_ptr<SharedStore> store;
    int arrivals{0};
  };
  // The ops of one kind that some but not all local devices have issued, oldest first: ops[k] is call number
  // first_seq + k of every device.
  struct OpStream {
    std::vector<int64_t> next_seq;  // by device position: calls so far
    std::deque<ReplicatedOp> ops;
    int64_t first_seq{0};
  };
  HipExecuteContext() = default;
  // k-th call of `kind` on this device -> the op all devices share; *seq = k
  ReplicatedOp& Arrive(OpKind kind, int64_t local_device_id, bool* first, int64_t* seq);
  void Leave(OpKind kind);
  void Retract(OpKind kind, int64_t local_device_id);  // the first arrival failed: it consumed no position

  void FlushLocked();

  mmr_context* ctx_{nullptr};
  bool defer_reshards_{true};
  std::vector<std::pair<std::shared_ptr<SharedStore>, std::shared_ptr<SharedStore>>> pending_;  // queued (src, dst)
  std::unordered_set<const SharedStore*> pending_srcs_, pending_dsts_;
  std::vector<mmr_store*> flush_srcs_, flush_dsts_;
  std::shared_ptr<std::atomic<bool>> alive_{std::make_shared<std::atomic<bool>>(true)};
  std::set<int> local_devices_;
  std::vector<int32_t> position_of_;  // local device id -> position in local_devices_, -1 = not local
  std::mutex mu_;
  OpStream streams_[kNumOpKinds];
  friend struct StoreHandleImpl;
};

// mpmd_partition.h:40-55 without the compute task: what a schedule holds on this path.
struct MpmdOperation {
  Reshard op;
};

// The reshard part of a compiled schedule and of its execution:
//   * AddStore / AddReshardTask as MpmdScheduler does (mpmd_partition.cc:250-323, 340-351): stores are named,
//     typed PARAM / ROOT / TEMP and indexed per type; a reshard is scheduled once;
//   * Execute as MultiMeshPjRtExecutable::Execute does (mm_pjrt_executable.cc:470-561 store set-up, 592-658 loop):
//     a fresh ROOT store per reshard output of type ROOT and execution, TEMP stores created on the first execution
//     and reused afterwards (cached_temporary_stores_), then every op issued by every local device in turn.
// Compute tasks are not part of it; the reshards of the whole schedule leave as one window.
class ReshardSchedule {
 public:
  explicit ReshardSchedule(std::string name = "reshard_schedule") : name_(std::move(name)) {}
  const std::string& name() const { return name_; }
  Store AddStore(Store::Type type, std::string name, ShardedShape shape);
  void AddReshardTask(const Store& input, const Store& output);
  const std::vector<MpmdOperation>& schedule() const { return schedule_; }
  int64_t num_parameters() const { return num_params_; }
  int64_t num_roots() const { return num_roots_; }
  // parameter_stores[local device position][parameter index] -> root_stores[local device position][root index];
  // positions follow the order of ctx.GetLocalDevices().
  // Every execution is bracketed exactly as the reference's (mm_pjrt_executable.cc:362-364 and :704-706):
  // OpenWindow, StartTimer(name), MarkProfile("start <name>") ... StopTimer(name), CloseWindow,
  // MarkProfile("finish <name>"); none of them waits for the device in the steady state.  on_done (optional, one
  // per local device position) are the compute callbacks of :369-377, handed to RunAfterAllTasks as at :660-667.
  std::vector<std::vector<StoreHandle>> Execute(HipExecuteContext& ctx,
                                                const std::vector<std::vector<StoreHandle>>& parameter_stores,
                                                std::vector<std::function<void()>>* on_done = nullptr);

 private:
  std::string name_;
  std::string start_mark_, finish_mark_;  // "start <name>" / "finish <name>", built once
  std::vector<MpmdOperation> schedule_;
  std::set<std::pair<std::string, std::string>> already_scheduled_;
  std::vector<Store> temporaries_;
  int64_t num_params_{0}, num_roots_{0};
  std::vector<std::vector<StoreHandle>> cached_temporary_stores_;  // [local device position][temp index]
};

}  // namespace mmr

#endif  // MMR_CSRC_HIP_EXECUTE_CONTEXT_H_
