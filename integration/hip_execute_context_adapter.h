// HipExecuteContextAdapter: the reference's runtime seam, xla::ZukuExecuteContext
// (src/pjrt_client/zuku_execute_context.h:38-133), implemented on the MI355X reshard
// library.  A maintainer adds this file to the plugin's sources and creates the
// adapter where the reference creates ZukuExecuteContextImpl
// (src/pjrt_client/mm_c_api_client.cc:82); mm_pjrt_executable.cc and
// mm_pjrt_buffer.cc stay as they are.
//
// NOT COMPILED IN THIS REPOSITORY.  It includes the reference's own headers
// (zuku_execute_context.h and, through it, the XLA tree and Zuku's type headers for
// zuku::ShardedShape, zuku::DeviceList, zuku::Future, zuku::ArrayTile), none of which
// exist here; no stand-ins for them are provided.  Everything it calls on this side
// (mmr::HipExecuteContext, the mmr_* C ABI) is compiled and tested in this repository;
// tests/cpp/hip_execute_context_test.cc drives HipExecuteContext through the same
// sequence of calls the plugin issues.
//
// Every pure virtual of the interface is overridden.  The store / reshard subset is
// served by the library.  Running XLA executables is not part of the reshard path:
// CreateExecuteTask, CreateCompileTask, CreateBuffer and FenceCompilation forward to a
// HipTaskRunner the plugin supplies (whatever launches its compiled executables on a
// HIP stream); its interface is declared below.
#ifndef XLA_PJRT_MULTIMESH_HIP_EXECUTE_CONTEXT_ADAPTER_H_
#define XLA_PJRT_MULTIMESH_HIP_EXECUTE_CONTEXT_ADAPTER_H_

#include <cstdlib>
#include <functional>
#include <iostream>
#include <map>
#include <memory>
#include <mutex>
#include <optional>
#include <set>
#include <string>
#include <utility>
#include <vector>

#include "xla/pjrt/multimesh/zuku_execute_context.h"  // the reference interface (also brings Shard, CreateStoreConfig)

#include "hip_execute_context.h"  // multimesh-jax_amd/csrc, this repository
#include "mmreshard.h"            // include/, this repository

namespace xla {

// store_handle.h:16-20 in the reference holds {name, zuku::Store<ShardedArray> array}; with this adapter it holds the
// library's handle instead.  (StoreHandle itself, store_handle_fwd.h:15-19, is unchanged: shared_ptr<impl> + unique_id.)
struct StoreHandleImpl {
  std::string name;
  mmr::StoreHandle inner;
};

// What the plugin has to bring for the calls that run XLA executables (out of the reshard path).  `stream` is the
// context's HIP stream: work enqueued on it is ordered with the reshards, assembles and offloads of the context.
class HipTaskRunner {
 public:
  virtual ~HipTaskRunner() = default;
  // Loads and compiles `compiler`'s module for the device (zuku_execute_context_impl.cc:213-230).
  virtual void Compile(int64_t local_device_id, std::shared_ptr<MultiMeshCompiler> compiler) = 0;
  // Blocks until every Compile issued so far is done (FenceCompilation).
  virtual void FenceCompilation() = 0;
  // Runs the compiled executable with these tile base pointers (inputs read, outputs written) on `stream`
  // (RunExecutable, zuku_execute_context_impl.cc:316-334).  Pointers of devices outside a store's device list are null.
  virtual void Execute(void* stream, int64_t run_id, int64_t local_device_id, int64_t global_device_id,
                       zuku::DeviceList mesh, std::shared_ptr<MultiMeshCompiler> compiler,
                       const std::vector<ScalarArgument>& scalars, const std::vector<void*>& inputs,
                       const std::vector<void*>& outputs, zuku::Future<zuku::ArrayTile>& temp_buffer,
                       const MultiMeshExecuteOptions& options) = 0;
  // A temporary buffer of `size` bytes on the device (CreateBuffer, zuku_execute_context_impl.cc:488-502).
  virtual zuku::Future<zuku::ArrayTile> CreateBuffer(int64_t local_device_id, int64_t global_device_id, int64_t size) = 0;
};

class HipExecuteContextAdapter : public ZukuExecuteContext {
 public:
  HipExecuteContextAdapter(std::set<int> local_devices, std::shared_ptr<HipTaskRunner> tasks, int hip_device = 0)
      : ctx_(mmr::HipExecuteContext::Create(std::move(local_devices), hip_device)), tasks_(std::move(tasks)) {}

  // ---- the reshard path ---------------------------------------------------------------------------------------
  void Reshard(int64_t local_device_id, int64_t global_device_id, const StoreHandle& src,
               const StoreHandle& dst) override {
    Guard([&] { ctx_->Reshard(local_device_id, global_device_id, Inner(src), Inner(dst)); });
  }

  void* SliceLocalShard(int64_t local_device_id, const StoreHandle& handle) override {
    void* tile = nullptr;
    Guard([&] { tile = ctx_->SliceLocalShard(local_device_id, Inner(handle)); });
    return tile;
  }

  zuku::ShardedShape GetStoreShardedShape(const StoreHandle& handle) override {
    zuku::ShardedShape shape;
    Guard([&] { shape = ToZuku(ctx_->GetStoreShardedShape(Inner(handle))); });
    return shape;
  }

  bool HasLocalShard(const StoreHandle& handle) override {
    return handle.impl != nullptr && ctx_->HasLocalShard(handle.impl->inner);
  }

  void Free(int64_t local_device_id, StoreHandle handle, bool keep_in_cache) override {
    if (handle.impl == nullptr) return;
    Guard([&] { ctx_->Free(local_device_id, handle.impl->inner, keep_in_cache); });
    if (!keep_in_cache) handle.impl = nullptr;  // release the handle (zuku_execute_context_impl.cc:512-514)
  }

  void Destroy(StoreHandle& store) override {
    // Drops the caller's reference only (zuku_execute_context_impl.cc:356-361).  The impl is shared by every copy of
    // the handle - ~MultiMeshPjRtBuffer calls Destroy while a StoreExternalReference (mm_pjrt_buffer.cc:27-36) may
    // still hold a copy to keep the tile of a zero-copy view alive - so the library's handle inside it is released
    // only when the last copy goes.
    store.impl = nullptr;
  }

  void ClearStoreCache(int64_t local_device_id) override {
    Guard([&] { ctx_->ClearStoreCache(local_device_id); });
  }

  void Rename(StoreHandle& handle, std::string name) override {
    if (handle.impl == nullptr) return;
    handle.impl->name = name;
    ctx_->Rename(handle.impl->inner, std::move(name));
  }

  void OffloadDtoH(int64_t local_device_id, const std::vector<StoreHandle>& to_offload,
                   const std::vector<StoreHandle>& pipelined, const std::string& task_name) override {
    Guard([&] { ctx_->OffloadDtoH(local_device_id, Inners(to_offload), Inners(pipelined), task_name); });
  }

  void OffloadHtoD(int64_t local_device_id, const std::vector<StoreHandle>& to_offload,
                   const std::string& task_name) override {
    Guard([&] { ctx_->OffloadHtoD(local_device_id, Inners(to_offload), task_name); });
  }

  // ---- windows, ordering, profiling ---------------------------------------------------------------------------
  void OpenWindow() override {
    Guard([&] { ctx_->OpenWindow(); });  // waits only while 8 earlier windows are still running on the device
  }
  void CloseWindow() override {
    Guard([&] { ctx_->CloseWindow(); });  // the reshards queued for the window leave here at the latest
  }
  void RunAfterAllTasks(int64_t local_device_id, std::function<void()> on_done) override {
    // on_done runs on a thread the library owns, never on a HIP runtime thread: it may complete a PjRtFuture whose
    // continuations drop buffers and so call back into this context (mm_pjrt_executable.cc:373-375)
    Guard([&] { ctx_->RunAfterAllTasks(local_device_id, std::move(on_done)); });
  }
  void MarkProfile(const std::string& name) override {
    Guard([&] { ctx_->MarkProfile(name); });
  }
  void StartTimer(const std::string& name) override {
    Guard([&] { ctx_->StartTimer(name); });
  }
  void StopTimer(const std::string& name) override {
    Guard([&] { ctx_->StopTimer(name); });
  }
  std::set<int> GetLocalDevices() override { return ctx_->GetLocalDevices(); }
  bool IsGpu() override { return true; }

  // ---- running executables: outside the reshard path, forwarded ----------------------------------------------
  void CreateCompileTask(int64_t local_device_id, std::shared_ptr<MultiMeshCompiler> compiler) override {
    tasks_->Compile(local_device_id, std::move(compiler));
  }

  void FenceCompilation() override { tasks_->FenceCompilation(); }

  zuku::Future<zuku::ArrayTile> CreateBuffer(int64_t local_device_id, int64_t global_device_id, int64_t size) override {
    return tasks_->CreateBuffer(local_device_id, global_device_id, size);
  }

  void CreateExecuteTask(int64_t run_id, int64_t local_device_id, int64_t global_device_id, zuku::DeviceList mesh,
                         std::shared_ptr<MultiMeshCompiler> compiler, const std::vector<ScalarArgument>& scalars,
                         const std::vector<StoreHandle>& inputs, const std::vector<StoreHandle>& outputs,
                         zuku::Future<zuku::ArrayTile>& temp_buffer, MultiMeshExecuteOptions options) override {
    Guard([&] {
      // the reshards queued so far leave (as one batch) before the task that reads their results
      ctx_->Flush();
      void* stream = nullptr;
      Check(mmr_context_stream(ctx_->raw(), &stream));
      const bool member = mesh.Contains(global_device_id);
      auto tiles = [&](const std::vector<StoreHandle>& stores, const char* kind) {
        std::vector<void*> out;
        out.reserve(stores.size());
        for (const StoreHandle& s : stores) {
          // a task's operands must hold a tile on the devices that run it (zuku_execute_context_impl.cc:271-290)
          if (member && !HasLocalShard(s)) {
            std::cerr << kind << " " << (s.impl ? s.impl->name : std::string("<null>")) << " has no tile on "
                      << global_device_id << " for task " << compiler->Name() << std::endl;
            std::abort();
          }
          // no host wait: the executable runs on the same stream as whatever produced the tile
          out.push_back(HasLocalShard(s) ? ctx_->TilePointer(s.impl->inner) : nullptr);
        }
        return out;
      };
      const std::vector<void*> in = tiles(inputs, "input"), out = tiles(outputs, "output");
      if (member)
        tasks_->Execute(stream, run_id, local_device_id, global_device_id, std::move(mesh), std::move(compiler), scalars,
                        in, out, temp_buffer, options);
    });
  }

 private:
  StoreHandle CreateStoreImpl(int64_t local_device_id, int64_t global_device_id, zuku::ShardedShape shape,
                              CreateStoreConfig config) override {
    StoreHandle handle;
    Guard([&] {
      mmr::StoreHandle inner = ctx_->CreateStore(
          local_device_id, global_device_id, FromZuku(shape),
          mmr::CreateStoreConfig{.name = config.name,
                                 .allocate_from_cache = config.allocate_from_cache,
                                 .min_cache_size = config.min_cache_size});
      handle = Wrap(std::move(inner), config.name.value_or("anonymous"));
    });
    return handle;
  }

  StoreHandle AssembleShardsImpl(int64_t local_device_id, int64_t global_device_id, zuku::ShardedShape shape,
                                 Shard shard, std::shared_ptr<MultiMeshStream> stream,
                                 std::optional<StoreHandle> existing_store) override {
    StoreHandle handle;
    Guard([&] {
      // The native shard's producer runs on the device's cached stream (GetCachedStream(backend, local id),
      // mm_utils.cc:53-70; the reference issues the copy on that stream, zuku_execute_context_impl.cc:410-414).
      // Here the copy runs on the context's stream behind an event recorded on the producer's: no host wait.
      std::shared_ptr<mmr::MultiMeshStream> producer;
      if (stream != nullptr) {
        auto se_stream = GetCachedStream(stream->mutable_backend(), shard.local_device_id);
        if (se_stream.ok())
          producer = std::make_shared<mmr::MultiMeshStream>(
              stream_executor::gpu::AsGpuStreamValue(*se_stream));  // the hipStream_t behind the se::Stream
      }
      std::optional<mmr::StoreHandle> existing;
      if (existing_store.has_value()) existing = Inner(*existing_store);
      mmr::StoreHandle inner =
          ctx_->AssembleShards(local_device_id, global_device_id, FromZuku(shape),
                               mmr::Shard{shard.data, shard.local_device_id, shard.size}, std::move(producer), existing);
      handle = existing_store.has_value() ? *existing_store : Wrap(std::move(inner), "anonymous");
    });
    return handle;
  }

  // zuku::ShardedShape{type, sharding{dims{size, sharding, permutation}, devices{start, num_devices}}} as
  // mm_sharding.cc:345-372, 427-431, 638-654 fills it  <->  mmr::ShardedShape (same fields; the type enumerators are
  // in the order of mm_sharding.cc:376-425).
  static mmr::ShardedShape FromZuku(const zuku::ShardedShape& s) {
    mmr::ShardedShape r;
    r.type = static_cast<mmr::SupportedType>(static_cast<int32_t>(s.type));
    for (const zuku::ShardingDim& d : s.sharding.dims)
      r.sharding.dims.push_back(mmr::ShardingDim{d.size, d.sharding, d.permutation});
    r.sharding.devices = mmr::DeviceList::Create(s.sharding.devices.start(), s.sharding.devices.size());
    return r;
  }

  static zuku::ShardedShape ToZuku(const mmr::ShardedShape& s) {
    zuku::ShardedShape r;
    r.type = static_cast<zuku::SupportedType>(static_cast<int32_t>(s.type));
    for (const mmr::ShardingDim& d : s.sharding.dims)
      r.sharding.dims.push_back(zuku::ShardingDim{.size = d.size, .sharding = d.sharding, .permutation = d.permutation});
    r.sharding.devices =
        zuku::DeviceList{{.start = s.sharding.devices.start(), .num_devices = s.sharding.devices.size()}};
    return r;
  }

  static StoreHandle Wrap(mmr::StoreHandle inner, std::string name) {
    const int64_t id = inner.unique_id;
    return StoreHandle{.impl = std::shared_ptr<StoreHandleImpl>(
                           new StoreHandleImpl{.name = std::move(name), .inner = std::move(inner)}),
                       .unique_id = id};
  }

  static const mmr::StoreHandle& Inner(const StoreHandle& h) {
    if (h.impl == nullptr) {
      std::cerr << "HipExecuteContextAdapter: empty store handle" << std::endl;
      std::abort();
    }
    return h.impl->inner;
  }

  static std::vector<mmr::StoreHandle> Inners(const std::vector<StoreHandle>& hs) {
    std::vector<mmr::StoreHandle> out;
    out.reserve(hs.size());
    for (const StoreHandle& h : hs) out.push_back(Inner(h));
    return out;
  }

  static void Check(int status) {
    if (status != MMR_OK) {
      std::cerr << "HipExecuteContextAdapter: " << mmr_last_error() << std::endl;
      std::abort();
    }
  }

  // The interface's methods return void or values and the reference aborts on invariant violations
  // (zuku_execute_context_impl.cc:271-290); the library reports them as exceptions.
  template <class Fn>
  static void Guard(Fn&& fn) {
    try {
      fn();
    } catch (const std::exception& e) {
      std::cerr << "HipExecuteContextAdapter: " << e.what() << std::endl;
      std::abort();
    }
  }

  std::shared_ptr<mmr::HipExecuteContext> ctx_;
  std::shared_ptr<HipTaskRunner> tasks_;
};

}  // namespace xla

#endif  // XLA_PJRT_MULTIMESH_HIP_EXECUTE_CONTEXT_ADAPTER_H_
