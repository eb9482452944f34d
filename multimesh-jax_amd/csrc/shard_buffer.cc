// See shard_buffer.h.
#include "shard_buffer.h"

#include <hip/hip_runtime_api.h>

#include <stdexcept>

namespace mmr {

namespace {
[[noreturn]] void raise(const std::string& what) { throw std::runtime_error(what); }
}  // namespace

ShardBuffer::ShardBuffer(data_variant_t data, std::vector<int64_t> global_shape, std::vector<int64_t> local_shape,
                         SupportedType type, std::shared_ptr<HipExecuteContext> context, int64_t local_device_id,
                         int64_t global_device_id, std::optional<std::string> name)
    : data_(std::move(data)),
      global_shape_(std::move(global_shape)),
      local_shape_(std::move(local_shape)),
      type_(type),
      context_(std::move(context)),
      local_device_id_(local_device_id),
      global_device_id_(global_device_id),
      name_(std::move(name)) {
  if (!context_) raise("ShardBuffer: no execute context");
}

ShardBuffer::~ShardBuffer() {
  // mm_pjrt_buffer.cc:119-124: the buffer's own reference to the store goes; the store lives on through other handles
  if (has_store()) context_->Destroy(std::get<StoreHandle>(data_));
}

const StoreHandle& ShardBuffer::store() const {
  if (!has_store()) raise("ShardBuffer " + name() + " is not backed by a store");
  return std::get<StoreHandle>(data_);
}

std::shared_ptr<NativeBuffer> ShardBuffer::shared_native_buffer() const {
  if (!has_native_buffer()) raise("ShardBuffer " + name() + " holds no native buffer");
  return std::get<std::shared_ptr<NativeBuffer>>(data_);
}

StoreHandle ShardBuffer::ToStore(const ShardedShape& mm_shape, const std::shared_ptr<MultiMeshStream>& stream,
                                 std::optional<StoreHandle> existing_store) const {
  if (has_store()) return store();
  const std::shared_ptr<NativeBuffer> native = shared_native_buffer();
  Shard shard{native->data(), local_device_id_, native->size()};
  return context_->AssembleShards(local_device_id_, global_device_id_, mm_shape, shard, stream, std::move(existing_store));
}

size_t ShardBuffer::GetOnDeviceSizeInBytes() const {
  size_t n = static_cast<size_t>(mmr_itemsize(static_cast<int32_t>(type_)));
  for (int64_t e : local_shape_) n *= static_cast<size_t>(e);
  return n;
}

std::unique_ptr<ShardBuffer> ShardBuffer::SliceStore() const {
  // blocking, as in the reference: the pointer is handed to a runtime that knows nothing of this one's stream
  void* tile = context_->SliceLocalShard(local_device_id_, store());
  // the view's reference to the store: StoreExternalReference holds the handle by value
  auto keep = std::make_shared<StoreHandle>(store());
  auto native = std::make_shared<NativeBuffer>(tile, GetOnDeviceSizeInBytes(), std::move(keep));
  return std::make_unique<ShardBuffer>(std::move(native), local_shape_, local_shape_, type_, context_, local_device_id_,
                                       global_device_id_, name() + ".sliced");
}

std::unique_ptr<ShardBuffer> ShardBuffer::SliceLocalShard() const {
  if (has_native_buffer())
    return std::make_unique<ShardBuffer>(shared_native_buffer(), local_shape_, local_shape_, type_, context_,
                                         local_device_id_, global_device_id_, name() + ".sliced");
  return SliceStore();
}

ShardBuffer::ExternalReference ShardBuffer::AcquireExternalReference() const {
  ExternalReference ref;
  if (has_native_buffer()) {
    ref.native = shared_native_buffer();
    ref.data = ref.native->data();
    return ref;
  }
  ref.data = context_->SliceLocalShard(local_device_id_, store());
  ref.store = store();
  return ref;
}

bool ShardBuffer::HasValidShard() const {
  // this might be an empty dummy buffer for a sharded array (mm_pjrt_buffer.cc:270-276)
  if (has_store()) return context_->HasLocalShard(store());
  return true;
}

void ShardBuffer::ToLiteral(void* host_dst, size_t size) const {
  if (size > GetOnDeviceSizeInBytes()) raise("ToLiteral: more bytes than the shard holds");
  if (has_store()) {
    context_->CopyShardToHost(store(), host_dst, size);
    return;
  }
  // a native buffer: ordered behind the context's work (a view's tile may still be written by a queued reshard)
  const std::shared_ptr<NativeBuffer> native = shared_native_buffer();
  void* stream = nullptr;
  if (mmr_context_stream(context_->raw(), &stream) != MMR_OK) raise(std::string("ToLiteral: ") + mmr_last_error());
  hipError_t e = hipMemcpyAsync(host_dst, native->data(), size, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream));
  if (e == hipSuccess) e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
  if (e != hipSuccess) raise(std::string("ToLiteral: ") + hipGetErrorString(e));
}

}  // namespace mmr
