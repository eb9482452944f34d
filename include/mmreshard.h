/*
 * mmreshard - C ABI of the MI355X cross-submesh reshard path.
 *
 * This is the boundary the reference plugin's C++ host code binds instead of the
 * third-party runtime it forwards to today.  Every entry point names the
 * reference interface it stands in for (paths relative to the reference
 * checkout, src/pjrt_client/...).  Plain pointers and sizes only; all functions
 * return an mmr_status and leave a message for mmr_last_error() on failure.
 *
 * Model: every logical device of every submesh is a separate shard buffer in
 * the HBM of one GPU.  A store is one sharded array: one buffer per device of
 * its device list.  All device work is ordered on the context's HIP stream.
 */
#ifndef MMRESHARD_H_
#define MMRESHARD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MMR_MAX_DIMS 9 /* 8 tensor dims + the optional trailing replication entry */

typedef enum {
  MMR_OK = 0,
  MMR_INVALID_ARGUMENT = 1, /* absl::InvalidArgument in the reference */
  MMR_UNSUPPORTED = 2,      /* absl::Internal("Unsupported type") / Unimplemented */
  MMR_OUT_OF_MEMORY = 3,
  MMR_HIP_ERROR = 4,
  MMR_NOT_FOUND = 5, /* device outside a store's device list, unknown handle */
  MMR_INTERNAL = 6
} mmr_status;

/* Element types.  0..14 are zuku::SupportedType exactly as mm_sharding.cc:376-425
 * maps XLA primitive types; values >= 100 are extensions the reference rejects
 * with Internal("Unsupported type") and this library moves as opaque bytes. */
typedef enum {
  MMR_PRED = 0, MMR_F16 = 1, MMR_BF16 = 2, MMR_F32 = 3, MMR_F64 = 4,
  MMR_S8 = 5, MMR_S16 = 6, MMR_S32 = 7, MMR_S64 = 8,
  MMR_U8 = 9, MMR_U16 = 10, MMR_U32 = 11, MMR_U64 = 12,
  MMR_C64 = 13, MMR_C128 = 14,
  MMR_F8E4M3FN = 100, MMR_F8E5M2 = 101
} mmr_dtype;

/* zuku::ShardingDim as filled at mm_sharding.cc:366-367 and :643-649. */
typedef struct {
  int64_t size;        /* GLOBAL extent of the dim (1 for the replication entry) */
  int64_t sharding;    /* number of tiles along it (replication factor for that entry) */
  int64_t permutation; /* rank of the dim in device-id significance, 0 = most significant */
} mmr_sharding_dim;

/* zuku::ShardedShape {type, sharding{dims, devices{start, num_devices}}}
 * (mm_sharding.cc:427-431, :650-652), flattened to POD.  A trailing entry
 * {size 1, sharding R > 1} is the replication entry (mm_sharding.cc:356-358).
 * has_layout / minor_to_major are an extension: the reference's shards are
 * always dense row-major of the local shape. */
typedef struct {
  int32_t dtype; /* mmr_dtype */
  int32_t ndims; /* entries used in dims[], replication entry included */
  mmr_sharding_dim dims[MMR_MAX_DIMS];
  int64_t dev_start;
  int64_t dev_count;
  int32_t has_layout;                   /* 0: row-major shards */
  int32_t minor_to_major[MMR_MAX_DIMS]; /* XLA convention, tensor dims only */
} mmr_sharded_shape;

/* The subset of XLA's OpSharding proto that mm_sharding.cc reads. */
typedef enum { MMR_SHARDING_REPLICATED = 0, MMR_SHARDING_MAXIMAL = 1, MMR_SHARDING_OTHER = 3 } mmr_sharding_type;
typedef struct {
  int32_t type; /* mmr_sharding_type */
  int32_t n_tile_dims;
  int64_t tile_dims[MMR_MAX_DIMS];
  int32_t n_iota_dims; /* 0: explicit device list below */
  int64_t iota_reshape_dims[MMR_MAX_DIMS];
  int32_t iota_transpose_perm[MMR_MAX_DIMS];
  int32_t replicate_on_last_tile_dim;
  int64_t iota_offset;                    /* the plugin's extension field, mm_sharding.cc:270 */
  const int64_t* tile_assignment_devices; /* n_devices entries, or NULL */
  int64_t n_devices;
} mmr_op_sharding;

const char* mmr_last_error(void); /* thread-local, valid until the next failing call */
const char* mmr_version(void);
int mmr_itemsize(int32_t dtype); /* bytes per element, 0 if unknown */

/* ---------------------------------------------------------------------------
 * Descriptor front-end (host only, no GPU needed)
 * ------------------------------------------------------------------------- */

/* ComputeIndexSet, mm_sharding.h:63-77. out has n entries. */
int mmr_compute_index_set(int64_t global_index, const int64_t* dims, int32_t n, int64_t* out);
/* ComputeGlobalIndex, mm_sharding.h:79-91. */
int mmr_compute_global_index(const int64_t* indices, const int64_t* dims, int32_t n, int64_t* out);

/* LogicalToPhysicalSharding, mm_sharding.cc:183-273.  Logical dim i shards over
 * the device axes axes_flat[axes_begin[i] .. axes_begin[i+1]); axes_begin has
 * n_logical + 1 entries.  mesh_dims are the device-mesh axis sizes. */
int mmr_logical_to_physical_sharding(const int32_t* axes_flat, const int32_t* axes_begin, int32_t n_logical,
                                     int64_t dev_start, int64_t dev_count, const int64_t* mesh_dims,
                                     int32_t n_mesh, int32_t list_all_devices, mmr_op_sharding* out);

/* LogicalShardingToOpSharding, mpmd_logical_to_gspmd_sharding.cc:21-124: the
 * PartitionSpec-style logical axis names of one array, resolved through a
 * task's options (mesh dims and axis names, ordered logical -> device axis
 * pairs).  Tensor dim i carries the names spec_names[spec_begin[i] ..
 * spec_begin[i+1]).  list_all_devices is dev_count < total_devices (:87-88).
 * Shardings that do not divide the shape are rejected (:101-113). */
int mmr_logical_sharding_to_op_sharding(const int64_t* mesh_dims, const char* const* mesh_axis_names, int32_t n_mesh,
                                        const char* const* logical_names, const char* const* logical_device_axes,
                                        int32_t n_logical_axes, const char* const* spec_names, const int32_t* spec_begin,
                                        int32_t rank, const int64_t* shape, int64_t dev_start, int64_t dev_count,
                                        int64_t total_devices, mmr_op_sharding* out);

/* HloSharding::tile_assignment().array(): device id of every tile in row-major
 * tile order (what mm_sharding_test.cc:111-227 compares). Writes n entries. */
int mmr_tile_assignment_devices(const mmr_op_sharding* s, int64_t* out, int64_t capacity, int64_t* n);

/* CanonicalizeSharding, mm_sharding.cc:275-456. */
int mmr_canonicalize_sharding(const mmr_op_sharding* s, const int64_t* shape, int32_t rank, int32_t dtype,
                              int32_t shape_is_global, mmr_sharded_shape* out);

/* XlaShapeToZukuShape, mm_sharding.cc:583-671. */
int mmr_xla_shape_to_sharded_shape(const int64_t* shape, int32_t rank, int32_t dtype, int64_t dev_start,
                                   int64_t dev_count, const mmr_op_sharding* s, int32_t shape_is_global,
                                   mmr_sharded_shape* out);

/* MeshEquivalentSharding, mm_sharding.cc:40-51; NeedsReshard, mpmd_insert_reshard.cc:33-43. */
int mmr_mesh_equivalent_sharding(const mmr_op_sharding* lhs, const mmr_op_sharding* rhs, int32_t* out);
int mmr_needs_reshard(int64_t operand_dev_start, int64_t operand_dev_count, int64_t dev_start,
                      int64_t dev_count, const mmr_op_sharding* operand_sharding,
                      const mmr_op_sharding* sharding, int32_t* out);

/* CreateDeviceList(tile_assignment), mpmd_utils.cc:151-175: the contiguous device range a sharding covers; an explicit
 * list that is not consecutive ascending ids is MMR_UNSUPPORTED, as in the reference. */
int mmr_device_list_of_sharding(const mmr_op_sharding* s, int64_t* dev_start, int64_t* dev_count);

/* ToMpmdSharding, mpmd_partition.cc:128-166: a sharding written relative to a task's devices (ids 0..n-1, as it
 * stands inside the task's module) -> the sharding over global device ids.  rank = tensor rank.  An explicit
 * device list or a single device is written to devices_out (capacity entries) and out points at it. */
int mmr_to_mpmd_sharding(int32_t rank, const mmr_op_sharding* sharding, int64_t task_dev_start, int64_t task_dev_count,
                         int64_t global_dev_start, int64_t global_dev_count, mmr_op_sharding* out, int64_t* devices_out,
                         int64_t devices_capacity);

/* Shard geometry: what spmd::MakePartitionedShape + ByteSizeOfElements give the
 * plugin (mm_pjrt_executable.cc:537, mm_pjrt_buffer.cc:285-288) and what the
 * mock calls zuku::ShardSize (mm_mock_mm_xla.cc:75). */
/* ReplicateDims (mm_sharding.cc:458-582; used by sharding propagation, off the reshard path): the tiling of the
 * given tile-assignment dims moves into the trailing replication dim.  The result's iota is in XLA's canonical
 * form; the order of devices inside a replication group is not significant (HloSharding sorts each group). */
int mmr_replicate_dims(const mmr_op_sharding* sharding, const int64_t* replicated_dims, int32_t n_replicated,
                       mmr_op_sharding* out);
/* ResizeSharding (mm_sharding.cc:98-161): grows or shrinks the first tiled dim that can take it so that the tile
 * assignment has num_elements tiles.  *found = 0 where the reference returns nullopt.  dev_count = 0: no device
 * list given.  devices_out backs out->tile_assignment_devices when the input has an explicit device list. */
int mmr_resize_sharding(const int64_t* shape, int32_t rank, const mmr_op_sharding* sharding, int64_t num_elements,
                        int64_t dev_start, int64_t dev_count, mmr_op_sharding* out, int64_t* devices_out,
                        int64_t devices_capacity, int32_t* found);

int mmr_validate_sharded_shape(const mmr_sharded_shape* s);
int mmr_shard_extents(const mmr_sharded_shape* s, int64_t* extents, int32_t* rank);
int mmr_shard_bytes(const mmr_sharded_shape* s, int64_t* bytes);
int mmr_device_of_tile(const mmr_sharded_shape* s, const int64_t* tile_coord, int64_t* device);
int mmr_tile_of_device(const mmr_sharded_shape* s, int64_t device, int64_t* tile_coord);

/* ---------------------------------------------------------------------------
 * Copy plan (host side; this is what zuku::Reshard plans internally, call site
 * zuku_execute_context_impl.cc:450-451 "zuku will create and execute a
 * resharding plan").  Building and inspecting a plan needs no GPU.
 * ------------------------------------------------------------------------- */
typedef struct mmr_plan mmr_plan;

#define MMR_SLOT_FILL 0xFFFFFFFFu /* src_slot of a chunk that writes zeros (pad of short tiles) */

/* One workgroup's share of a strided copy: n2 x n1 rows of w contiguous bytes.
 * Slots index the launch's pointer table: for array a of a plan, source device
 * k is slot slot_base[a] + k and destination device k is
 * slot_base[a] + src.dev_count + k. */
typedef struct {
  uint32_t src_slot;
  uint32_t dst_slot;
  uint64_t src_off; /* bytes from the slot's base */
  uint64_t dst_off;
  uint32_t w;     /* contiguous bytes per row */
  uint32_t n1;    /* rows along the fast row dimension */
  uint32_t n2;    /* rows along the slow row dimension */
  uint32_t align; /* largest power of two <= 16 dividing every offset, stride and w */
  int64_t s1, d1; /* source / destination byte stride of the n1 dimension */
  int64_t s2, d2;
} mmr_copy_chunk;

/* One batch of tiles moved through LDS when source and destination disagree on
 * the minor-most dim.  x is contiguous in the source, y is contiguous in the
 * destination.  Tile edge: 64 elements (128 for 1-byte, 32 for 16-byte elements). */
typedef struct {
  uint32_t src_slot;
  uint32_t dst_slot;
  uint64_t src_off;
  uint64_t dst_off;
  uint32_t nx, ny;   /* tile extent in elements, each at most the tile edge */
  uint32_t nb;       /* tiles along the batch dimension */
  uint32_t itemsize; /* 1, 2, 4, 8 or 16 */
  int64_t src_ystride, dst_xstride; /* bytes */
  int64_t src_bstride, dst_bstride;
} mmr_transpose_chunk;

#define MMR_PLAN_ALL_GENERIC 1u /* treat every tile as ragged (aligned boxes go through the span kernel too; testing) */
#define MMR_PLAN_NO_AUTOTUNE 2u /* accepted and ignored: table orders are only timed on request (mmr_reshard_tune) */
#define MMR_PLAN_NO_SPAN 4u     /* ragged boxes become generic chunks instead of span groups (testing) */
#define MMR_PLAN_NO_INLINE 8u   /* group tables always live in device memory, never in the kernel's argument block */
#define MMR_PLAN_NO_SEGMENT_TABLES 16u /* no span group uses the per-span table of (row, piece) pairs (testing) */

typedef struct {
  uint32_t chunk_bytes; /* target bytes per copy chunk, 0 = default */
  uint32_t order;       /* 0 = default (2 for copy groups and tiles, 4 for span groups); 1 generation order,
                           2 by destination address, 3 by source address, 4 = by destination with the tiles of an
                           array interleaved in equal fractions (the same rows of all tiles together) */
  uint32_t xcd_mode;    /* workgroup -> chunk mapping. 0 = default; 1 = chunk i is workgroup i (the hardware deals
                           consecutive workgroups round-robin over the 8 XCDs); 2 = each XCD takes a contiguous
                           eighth of the table; G >= 16 = runs of G table neighbours share an XCD (and its L2) */
  uint32_t flags;       /* MMR_PLAN_* bits above (testing and probing switches);
                           bits 8-23: KiB per tile and round for order 4 (0 = default: 64 for copy groups, 4 for span groups) */
} mmr_plan_options;

typedef struct {
  int64_t n_arrays;
  int64_t n_boxes;             /* source-tile x destination-tile overlaps */
  int64_t n_copy16_chunks;     /* 16-byte aligned copy chunks (workgroups of the copy-group launch) */
  int64_t n_span_chunks;       /* destination spans (workgroups of the span launch, ragged rows) */
  int64_t n_groups;            /* records of the group tables ... */
  int64_t n_pieces;            /* ... and their pieces */
  int64_t n_copy_generic_chunks;
  int64_t n_transpose_chunks;
  int64_t n_fill_chunks;       /* included in the two copy counts */
  int64_t bytes_moved;         /* valid bytes written = valid bytes read */
  int64_t bytes_filled;        /* pad bytes zeroed */
  int64_t table_bytes;         /* device-resident plan size */
  int64_t n_slots;
  int64_t order_used;          /* table order in effect: 0 = the default mix, else a value of mmr_plan_options.order */
  int64_t interleave_kib;      /* order 4 only: KiB per tile and fraction */
  int64_t orders_timed;        /* how many launch orders mmr_reshard_tune timed for this plan (0 = never tuned) */
  int64_t n_copy16_launches;   /* launches the copy-group table leaves in (very long tables go in pieces) */
} mmr_plan_stats;

int mmr_plan_create(const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int32_t n_arrays,
                    const mmr_plan_options* options, mmr_plan** out);
void mmr_plan_destroy(mmr_plan* plan);
int mmr_plan_get_stats(const mmr_plan* plan, mmr_plan_stats* out);
/* kind: 0 = 16-byte aligned copy chunks, 1 = generic copy chunks. Returns how many were written. */
int64_t mmr_plan_get_copy_chunks(const mmr_plan* plan, int32_t kind, mmr_copy_chunk* out, int64_t capacity);
int64_t mmr_plan_get_transpose_chunks(const mmr_plan* plan, mmr_transpose_chunk* out, int64_t capacity);
int64_t mmr_plan_get_slot_bases(const mmr_plan* plan, int64_t* out, int64_t capacity);

/* ---------------------------------------------------------------------------
 * Execution: the store subset of xla::ZukuExecuteContext
 * (zuku_execute_context.h:38-133), one GPU, stream ordered.
 * ------------------------------------------------------------------------- */
typedef struct mmr_context mmr_context;
typedef struct mmr_store mmr_store;

/* ZukuExecuteContextImpl::Create, zuku_execute_context_impl.cc:559-577.
 * hip_stream may be NULL (the context then owns a stream) or a caller's
 * hipStream_t all work is ordered on. */
int mmr_context_create(int32_t hip_device, void* hip_stream, mmr_context** out);
void mmr_context_destroy(mmr_context* ctx);
int mmr_context_stream(mmr_context* ctx, void** hip_stream);
/* Default plan options of the context (chunk size, ordering); affects plans built afterwards. */
int mmr_context_set_plan_options(mmr_context* ctx, const mmr_plan_options* options);
/* Checking mode, kept from the reference's mock runtime: a rolling hash of the operation stream (kind, store ids,
 * descriptors; mm_mock_mm_xla.cc:259-262, compared between runs at mm_pjrt_executable_test.cc:760-766) and, on every
 * reshard, "every operand holds a tile on each of its devices" (mm_mock_mm_xla.cc:347-369).  Off by default. */
#define MMR_CHECK_INVARIANTS 1u
/* Every named timer that completes prints "<name> finished in <seconds>s" to stderr, the line the reference logs at
 * info level (zuku_execute_context_impl.cc:478-482). */
#define MMR_LOG_TIMERS 2u
int mmr_context_set_flags(mmr_context* ctx, uint32_t flags);

#define MMR_STORE_FROM_CACHE 1u    /* CreateStoreConfig::allocate_from_cache */
#define MMR_STORE_UNINITIALIZED 2u /* skip the zero fill: for stores whose every byte a reshard writes before it is read
                                      (a reshard writes the pad of short tiles too) */

/* CreateStore / CreateStoreImpl, zuku_execute_context.h:99-104,
 * zuku_execute_context_impl.cc:521-550: allocates the buffer of every device of
 * the descriptor's device list (zero-filled). */
int mmr_store_create(mmr_context* ctx, const mmr_sharded_shape* shape, const char* name, uint32_t flags,
                     mmr_store** out);
/* The same with CreateStoreConfig::min_cache_size (zuku_execute_context.h:29, passed to ArrayCache::Get at
 * zuku_execute_context_impl.cc:529-535; the mock prints value_or(1), mm_mock_mm_xla.cc:238).  ArrayCache itself is
 * third-party; read here as: with MMR_STORE_FROM_CACHE, the cache of this descriptor is made to hold at least
 * min_cache_size buffers in total (the one handed out included), so the next min_cache_size - 1 requests for the
 * descriptor are served without allocating.  Values < 1 count as 1. */
int mmr_store_create_ex(mmr_context* ctx, const mmr_sharded_shape* shape, const char* name, uint32_t flags,
                        int64_t min_cache_size, mmr_store** out);
/* Zero-copy import (what AssembleShards' "TODO: do the slicing" flat copy,
 * zuku_execute_context_impl.cc:405-415, would become when the native PjRt
 * shards may be used in place): a store whose buffer of device dev_start + k IS
 * device_ptrs[k] (caller-owned, 16-byte aligned, at least mmr_shard_bytes
 * long).  mmr_store_free on it waits for pending work and frees nothing. */
int mmr_store_adopt(mmr_context* ctx, const mmr_sharded_shape* shape, const char* name, void* const* device_ptrs,
                    mmr_store** out);

/* OffloadDtoH / OffloadHtoD, zuku_execute_context.h:61-68,
 * zuku_execute_context_impl.cc:162-211: the store's buffers move between the
 * device cache and a host cache of pinned buffers (both keyed by descriptor),
 * by an asynchronous copy on the context's stream; neither call waits for the
 * device.  The device memory an offload gives up goes to the device cache (the
 * next store of that descriptor created with MMR_STORE_FROM_CACHE takes it,
 * ordered on the stream behind the copy); the pinned buffer a reload gives up
 * goes to the host cache.  mmr_clear_store_cache releases both.
 * An offloaded store cannot be resharded, assembled or sliced (the mock's
 * invariant, mm_mock_mm_xla.cc:347-356); mmr_store_read_shard still works. */
int mmr_store_offload(mmr_context* ctx, mmr_store* store);
int mmr_store_reload(mmr_context* ctx, mmr_store* store);
int mmr_store_is_offloaded(const mmr_store* store, int32_t* out);

/* Free, zuku_execute_context_impl.cc:504-515 (keep_in_cache: buffers go back to
 * the per-shape cache); Destroy, :356-361. The handle is dead afterwards.  Without
 * keep_in_cache the memory returns to the context's allocator pool (the reference
 * allocates every store through its cache, :533-535): the next store of the same
 * byte size takes it, so freeing does not wait for the device. */
int mmr_store_free(mmr_context* ctx, mmr_store* store, int32_t keep_in_cache);
/* ClearStoreCache, zuku_execute_context_impl.cc:517-519: releases the per-shape cache, the allocator pool and the
 * pinned host cache. */
int mmr_clear_store_cache(mmr_context* ctx);

/* AssembleShards / Shard{data, local_device_id, size},
 * zuku_execute_context.h:20-24,89-97, zuku_execute_context_impl.cc:384-424: one
 * flat copy of `size` bytes into the buffer of `device`.  data_on_device == 1:
 * `data` is a device pointer (stream-ordered copy; large aligned shards go
 * through the library's own copy kernel); 0: host memory, consumed before the
 * call returns; 2: the HIP runtime tells which of the two; 3: a device pointer,
 * always copied by the runtime's hipMemcpyAsync (the reference's MemcpyDtoDAsync
 * as it is; also the independent kernel the traffic counters are calibrated on). */
int mmr_store_assemble(mmr_context* ctx, mmr_store* store, int64_t device, const void* data, size_t size,
                       int32_t data_on_device);

/* SliceLocalShard, zuku_execute_context.h:77-78, zuku_execute_context_impl.cc:
 * 367-377: blocks until the store's pending work is done and returns the base
 * pointer of the device's buffer (borrowed; valid until the store is freed). */
int mmr_store_shard_ptr(mmr_context* ctx, mmr_store* store, int64_t device, void** ptr);
/* Same, without waiting (for callers that stay on the context's stream). */
int mmr_store_shard_ptr_async(mmr_context* ctx, mmr_store* store, int64_t device, void** ptr);
/* What MultiMeshPjRtBuffer::ToLiteral does through SliceLocalShard
 * (mm_pjrt_buffer.cc:84-95): blocking copy of one shard to host memory. */
int mmr_store_read_shard(mmr_context* ctx, mmr_store* store, int64_t device, void* host_dst, size_t size);
/* HasLocalShard, zuku_execute_context_impl.cc:363-365. */
int mmr_store_has_shard(const mmr_store* store, int64_t device, int32_t* out);
/* GetStoreShardedShape, zuku_execute_context_impl.cc:379-382. */
int mmr_store_get_shape(const mmr_store* store, mmr_sharded_shape* out);
/* StoreHandle::unique_id, store_handle_fwd.h:15-19, zuku_execute_context_impl.cc:86-89. */
int64_t mmr_store_id(const mmr_store* store);

/* Reshard, zuku_execute_context.h:74-75, zuku_execute_context_impl.cc:437-452:
 * every destination buffer := its slice of the array the source buffers hold.
 * Asynchronous on the context's stream.  The plan is built on first use of a
 * (source descriptor, destination descriptor) pair and cached, keyed like
 * ReshardKey (mpmd_insert_reshard.cc:19-31). */
int mmr_reshard(mmr_context* ctx, mmr_store* src, mmr_store* dst);
/* All reshards of one schedule window in one plan and one launch per kernel
 * class (the reference issues one Reshard call per array,
 * mm_pjrt_executable.cc:616-658). */
int mmr_reshard_batch(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n);
/* Everything mmr_reshard_batch does for these stores except the launches: the plan
 * and the table of shard pointers are built, uploaded and cached, so that the next
 * mmr_reshard / mmr_reshard_batch of the same stores only launches kernels and can
 * be recorded into a HIP graph (stream capture forbids the allocations and copies
 * of a first use; a reshard that would need them while the stream is capturing
 * fails with MMR_INVALID_ARGUMENT and leaves the capture intact).  Schedule-build
 * time work like MpmdScheduler::AddReshardTask, mpmd_partition.cc:340-351. */
int mmr_reshard_bind(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n);
/* The argument checks of mmr_reshard without planning or launching anything (both stores of this context, distinct,
 * resident, same type and global extents): lets a caller that queues Reshard calls of one schedule window
 * (mm_pjrt_executable.cc:616-658) for a single mmr_reshard_batch report a bad call where it is made. */
int mmr_reshard_validate(mmr_context* ctx, mmr_store* src, mmr_store* dst);

/* No counterpart in the reference.  For callers that cannot allocate device memory where they reshard: code that
 * runs in tight serving loops or under harnesses that forbid allocation.  Does what mmr_reshard_batch does,
 * with the same kernels, but the chunk tables and the table of shard pointers of the launch live in a static device
 * array of MMR_STATIC_SCRATCH_BYTES per GPU instead of allocated memory: the call plans on the host, copies the tables
 * into that array on the context's stream (through a pinned staging buffer the context has held since its creation)
 * and launches; it calls no hipMalloc / hipFree.  A plan whose tables exceed the array is refused with MMR_INVALID_ARGUMENT (use mmr_reshard_batch).
 * It copies from host memory, so like every such entry point it is refused (MMR_INVALID_ARGUMENT, capture left
 * valid) while the context's stream is capturing a graph: a capturable reshard is mmr_reshard_bind + mmr_reshard.
 * Every call on a GPU shares that GPU's array.  Calls of one context follow each other on its stream; a call of
 * another context of this process on the same GPU makes its stream wait, on the device, for the kernels of the
 * previous user.  Streams of other processes and callers that bypass this entry point are not ordered: such calls
 * race.  No table order tuning. */
#define MMR_STATIC_SCRATCH_BYTES (1u << 20)
int mmr_reshard_batch_static(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n);

/* Times a few launch orders of the plan of these stores on the stores themselves (a reshard is idempotent) and keeps
 * the fastest for every later reshard of the same descriptors; *order_used receives its mmr_plan_options.order value
 * (0 = the default stayed).  Blocks the calling thread for a few dozen launches.  Nothing else ever times a plan: a
 * plain mmr_reshard plans, uploads and launches without waiting for the device, and its plan is the same on every
 * run.  Call it where the schedule is built (MpmdScheduler::AddReshardTask, mpmd_partition.cc:340-351), before any
 * graph capture of the reshard. */
int mmr_reshard_tune(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n, int64_t* order_used);
/* Drops every cached plan and binding (device tables) no launch in flight needs; pinned ones (mmr_reshard_bind) go
 * too, so graphs captured from them must not be replayed afterwards.  Waits for the stream. */
int mmr_context_clear_plans(mmr_context* ctx);

/* Build and upload the plan of n descriptor pairs (one batch) ahead of the first
 * reshard, i.e. when the schedule entry is created (MpmdScheduler::AddReshardTask,
 * mpmd_partition.cc:340-351) rather than when it first executes. */
int mmr_context_prepare(mmr_context* ctx, const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int32_t n);

/* Ordering against other streams without blocking the host, as the plugin ties
 * XLA's stream to the runtime's (RecordCuEvent, cuda_utils.cu.cc:78-83): the
 * context's stream waits for a caller's hipEvent_t / records one. */
int mmr_context_wait_event(mmr_context* ctx, void* hip_event);
int mmr_context_record_event(mmr_context* ctx, void* hip_event);

/* RunAfterAllTasks, zuku_execute_context.h:53-54, zuku_execute_context_impl.cc:347-354: fn(arg) runs once everything
 * queued on the context's stream so far is done; the call itself does not wait.  fn runs on a thread the context
 * owns (never on a thread of the HIP runtime), callbacks run one at a time in the order they were given, and fn may
 * call any entry point of this library except mmr_context_destroy - the reference's callback completes a future whose
 * continuations drop buffers (mm_pjrt_executable.cc:373-375).  mmr_context_destroy runs the callbacks still waiting
 * before it returns. */
int mmr_context_run_after(mmr_context* ctx, void (*fn)(void*), void* arg);

/* Blocks until everything queued on the context's stream is done and the callbacks of mmr_context_run_after given
 * before this call have returned (called from such a callback, it only waits for the stream). */
int mmr_sync(mmr_context* ctx);

/* StartTimer / StopTimer, zuku_execute_context.h:56-59, zuku_execute_context_impl.cc:462-486: named timers, any
 * number pending at once, and neither call waits for the device.  The reference defers a steady_clock reading
 * behind the last execute event on both sides and logs the difference from a deferred task; here both sides are
 * HIP events on the context's stream, so the interval is the device time between the two points.
 * mmr_timer_begin: a timer of that name that is already running is left as it is (pending_timers_.emplace, :466).
 * mmr_timer_end: MMR_NOT_FOUND if no such timer is running (the reference logs a warning and goes on, :471-474).
 * An interval is read once the device has passed its end, by whichever of these calls (or mmr_window_open) comes
 * next.  Marks that fall on the same point of the stream (nothing queued in between: the end of one execution's timer,
 * its window marker, the start of the next timer) share one event, while the context owns its stream and has not
 * handed it out through mmr_context_stream.  mmr_timer_poll never waits: *last_milliseconds is the most recent interval of `name` that has been read
 * (0 if none), *completed how many have been.  mmr_timer_wait is the blocking variant: it first waits until every
 * ended interval of `name` has been read (counted in host_blocking_syncs when it has to wait). */
int mmr_timer_begin(mmr_context* ctx, const char* name);
int mmr_timer_end(mmr_context* ctx, const char* name);
int mmr_timer_poll(mmr_context* ctx, const char* name, float* last_milliseconds, int64_t* completed);
int mmr_timer_wait(mmr_context* ctx, const char* name, float* last_milliseconds, int64_t* completed);

/* MarkProfile, zuku_execute_context.h:55, zuku_execute_context_impl.cc:458-460: a named mark in the profile.  Goes
 * out as a roctx marker (rocprofv3 --marker-trace shows it); the library also wraps plan building, table binding and
 * every launch of a reshard in roctx ranges ("mmreshard: build plan" / "bind tables" / "launch"), the counterpart of
 * the named region around every task of the reference (:292-308).  The roctx library is looked up at run time
 * (librocprofiler-sdk-roctx, then libroctx64); where neither is installed, or with MMR_ROCTX=0 in the environment,
 * the calls do nothing.  mmr_profile_available: 1 if marks reach a roctx library. */
int mmr_profile_mark(mmr_context* ctx, const char* name);
int mmr_profile_range_push(mmr_context* ctx, const char* name);
int mmr_profile_range_pop(mmr_context* ctx);
int mmr_profile_available(void);

/* OpenWindow / CloseWindow, zuku_execute_context.h:50-51, zuku_execute_context_impl.cc:128-143: one window per
 * execution of an executable (mm_pjrt_executable.cc:362, 705).  mmr_window_close marks the end of everything queued
 * so far; mmr_window_open returns at once while fewer than the limit (8, kMaxOpenWindows, :46) windows are still
 * running on the device and otherwise waits for the oldest one (counted in window_waits and host_blocking_syncs), so
 * a caller that never reads a result cannot run ahead of the device without bound.  (In the reference tree the line
 * that queues the marker, :140, is commented out, so its limit never triggers; the limit it declares is kept here.) */
int mmr_window_open(mmr_context* ctx);
int mmr_window_close(mmr_context* ctx);
int mmr_context_set_max_open_windows(mmr_context* ctx, int32_t n);

/* Unnamed HIP-event stopwatch on the context's stream for benchmarks: one interval at a time.  The events behind
 * every timer, mark and window marker of this library are made without the system-scope fence
 * (hipEventDisableSystemFence): they tell time and completion and cost the device no cache write-back in the middle
 * of a schedule; to read what the device wrote, wait with mmr_sync or read through mmr_store_read_shard. */
int mmr_timer_start(mmr_context* ctx);
int mmr_timer_stop_wait(mmr_context* ctx, float* milliseconds); /* blocks until the device reaches this point */
/* Per-launch timing of back-to-back work: mmr_timer_lap records a mark on the stream (between two launches, say);
 * mmr_timer_laps blocks until the last mark is reached, writes the device time between consecutive marks
 * (marks - 1 values, at most `capacity`; *count = how many) and forgets the marks. */
int mmr_timer_lap(mmr_context* ctx);
int mmr_timer_laps(mmr_context* ctx, float* milliseconds, int32_t capacity, int32_t* count);

typedef struct {
  int64_t plans_built;
  int64_t plan_cache_hits;
  int64_t bindings_built; /* pointer tables uploaded */
  int64_t binding_cache_hits;
  int64_t kernel_launches;
  int64_t reshard_calls;
  int64_t bytes_allocated; /* live device bytes in stores and caches */
  int64_t bytes_high_watermark;
  int64_t stores_live;
  int64_t cache_hits;      /* store buffers served from the per-shape cache */
  int64_t host_bytes_allocated; /* pinned host bytes of offloaded stores and of the host cache */
  int64_t host_bytes_high_watermark;
  int64_t host_blocking_syncs;  /* times an entry point made the calling thread wait for the device: every
                                   stream / event synchronisation and every hipFree the library issues */
  int64_t inline_launches;      /* launches whose table travelled in the kernel's argument block */
  int64_t device_allocations;   /* hipMalloc calls */
  int64_t host_cache_hits;      /* offloads served from the pinned host cache */
  int64_t pool_hits;            /* new stores whose memory came from the allocator's pool of freed stores */
  int64_t plans_cached;         /* plans held now */
  int64_t bindings_cached;      /* bound device tables held now */
  int64_t invariant_checks;     /* checks made in MMR_CHECK_INVARIANTS mode */
  int64_t operation_hash;       /* rolling hash of the operation stream in that mode */
  int64_t block_pool_hits;      /* table blocks (plans, bindings) served from the pool of recycled blocks */
  int64_t timers_resolved;      /* named timer intervals read so far */
  int64_t windows_opened;
  int64_t window_waits;         /* mmr_window_open calls that had to wait for an older window */
  int64_t profile_marks;
  int64_t events_recorded;      /* events the timers and windows put on the stream (points that coincide share one) */
} mmr_context_stats;
int mmr_context_get_stats(mmr_context* ctx, mmr_context_stats* out);
/* Stats of the cached plan of a store pair (builds it if needed). */
int mmr_reshard_plan_stats(mmr_context* ctx, mmr_store* src, mmr_store* dst, mmr_plan_stats* out);
/* The same for the plan of a batch (the arrays in the order mmr_reshard_batch was or will be given them). */
int mmr_reshard_batch_plan_stats(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n,
                                 mmr_plan_stats* out);

#ifdef __cplusplus
}
#endif
#endif /* MMRESHARD_H_ */
