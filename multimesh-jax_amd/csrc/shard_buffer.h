// C++ mirror of the reference's caller-side buffer wrapper, MultiMeshPjRtBuffer
// (src/pjrt_client/mm_pjrt_buffer.h:28-179, mm_pjrt_buffer.cc), without XLA: what
// the plugin hands to JAX for one device's shard of an array.  A buffer holds
// EITHER a store handle (the array lives in the reshard runtime) OR a native
// buffer (device memory another runtime owns: a PjRtBuffer in the reference).
//
//   ToStore          native shard -> store tile (AssembleShards), or the store it
//                    already is                          mm_pjrt_buffer.cc:148-178
//   SliceStore       store -> zero-copy native view of this device's tile, kept
//                    alive by a reference that holds the store handle
//                                                        mm_pjrt_buffer.cc:27-36, 180-233
//   SliceLocalShard  either kind -> native view           mm_pjrt_buffer.cc:253-268
//   HasValidShard    false on devices outside the store's device list  :270-276
//   ToLiteral        blocking copy of the shard to host memory          :84-95
//   ~ShardBuffer     Destroy(store): drops this buffer's reference      :119-124
#ifndef MMR_CSRC_SHARD_BUFFER_H_
#define MMR_CSRC_SHARD_BUFFER_H_

#include <functional>
#include <memory>
#include <optional>
#include <string>
#include <variant>
#include <vector>

#include "hip_execute_context.h"

namespace mmr {

// Device memory owned elsewhere (the reference's native PjRtBuffer): a pointer, a size, and whatever keeps the
// memory alive for as long as this object exists.
class NativeBuffer {
 public:
  NativeBuffer(void* data, size_t size, std::shared_ptr<void> keep_alive = nullptr, std::function<void()> on_delete = {})
      : data_(data), size_(size), keep_alive_(std::move(keep_alive)), on_delete_(std::move(on_delete)) {}
  ~NativeBuffer() {
    if (on_delete_) on_delete_();
  }
  NativeBuffer(const NativeBuffer&) = delete;
  NativeBuffer& operator=(const NativeBuffer&) = delete;
  void* data() const { return data_; }
  size_t size() const { return size_; }

 private:
  void* data_;
  size_t size_;
  std::shared_ptr<void> keep_alive_;
  std::function<void()> on_delete_;
};

class ShardBuffer {
 public:
  using data_variant_t = std::variant<StoreHandle, std::shared_ptr<NativeBuffer>>;

  // global_shape / local_shape: extents of the whole array and of this device's shard (mm_pjrt_buffer.h:31-36).
  ShardBuffer(data_variant_t data, std::vector<int64_t> global_shape, std::vector<int64_t> local_shape, SupportedType type,
              std::shared_ptr<HipExecuteContext> context, int64_t local_device_id, int64_t global_device_id,
              std::optional<std::string> name = std::nullopt);
  ~ShardBuffer();
  ShardBuffer(const ShardBuffer&) = delete;
  ShardBuffer& operator=(const ShardBuffer&) = delete;

  bool has_store() const { return std::holds_alternative<StoreHandle>(data_); }
  bool has_native_buffer() const { return std::holds_alternative<std::shared_ptr<NativeBuffer>>(data_); }
  const StoreHandle& store() const;  // throws unless has_store()
  std::shared_ptr<NativeBuffer> shared_native_buffer() const;
  void set_store(const StoreHandle& store) { data_ = store; }
  std::string name() const { return name_.value_or("unnamed"); }
  const std::vector<int64_t>& on_device_shape() const { return local_shape_; }
  const std::vector<int64_t>& global_shape() const { return global_shape_; }
  int64_t local_device_id() const { return local_device_id_; }

  // The store this buffer is, or a store assembled from its native shard: every local device calls this with its own
  // shard and the same descriptor; member devices copy their shard into their tile, ordered behind `stream`'s work.
  StoreHandle ToStore(const ShardedShape& mm_shape, const std::shared_ptr<MultiMeshStream>& stream,
                      std::optional<StoreHandle> existing_store = std::nullopt) const;

  // This device's shard as a native buffer.  Of a store: a zero-copy view of the tile (blocks until the store's
  // pending work is done, like SliceLocalShard); the view holds the store handle, so the tile stays valid for as long
  // as the view lives, whatever happens to the other handles.
  std::unique_ptr<ShardBuffer> SliceLocalShard() const;

  // PjRtBuffer::ExternalReference of a store-backed buffer (StoreExternalReference, mm_pjrt_buffer.cc:27-36).
  struct ExternalReference {
    void* data{nullptr};
    std::optional<StoreHandle> store;  // pins the store
    std::shared_ptr<NativeBuffer> native;
  };
  ExternalReference AcquireExternalReference() const;

  bool HasValidShard() const;
  size_t GetOnDeviceSizeInBytes() const;  // ByteSizeOfElements(local_shape), mm_pjrt_buffer.cc:285-288
  // Blocking copy of the shard to host memory; `size` at most GetOnDeviceSizeInBytes().
  void ToLiteral(void* host_dst, size_t size) const;

  void Delete() { deleted_ = true; }
  bool IsDeleted() const { return deleted_; }

 private:
  std::unique_ptr<ShardBuffer> SliceStore() const;

  data_variant_t data_;
  std::vector<int64_t> global_shape_, local_shape_;
  SupportedType type_;
  std::shared_ptr<HipExecuteContext> context_;
  int64_t local_device_id_, global_device_id_;
  std::optional<std::string> name_;
  bool deleted_{false};
};

}  // namespace mmr

#endif  // MMR_CSRC_SHARD_BUFFER_H_
