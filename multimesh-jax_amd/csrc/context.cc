// Execution side of the C ABI: stores (one buffer per logical device, all in one
// GPU's HBM), the per-shape buffer cache, the plan cache, and the launches.
//
// Mirrors the store subset of xla::ZukuExecuteContext
// (zuku_execute_context.h:38-133) as ZukuExecuteContextImpl provides it
// (zuku_execute_context_impl.cc:356-452, 504-550), with the third-party
// zuku::Reshard behind it replaced by planner.cc + kernels.hip.
#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <initializer_list>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "common.h"
#include "chunk_ops.h"
#include "kernels.h"
#include "planner.h"

using mmr::fail;

namespace {

constexpr size_t kTileAlign = 4096;
constexpr size_t kMaxBindings = 64;  // unpinned device tables kept per context (least recently used go first)

std::atomic<int64_t> g_next_store_id{0};  // NextStoreId, zuku_execute_context_impl.cc:86-89

struct TransposeRun {
  uint32_t itemsize;
  bool vector_only;  // every chunk of the run satisfies transpose_is_vector
  int64_t begin, count;
};

// A plan plus what does not depend on the buffers it will run on.
struct DevicePlan {
  mmr_plan plan;
  std::vector<uint32_t> copy_hints, span_hints;
  std::vector<TransposeRun> transpose_runs;
  mmr_context* owner = nullptr;         // whose block pool the device tables came from
  mmr_copy_chunk* d_generic = nullptr;  // slot-relative tables, read through a launch's pointer table
  mmr_transpose_chunk* d_transposes = nullptr;
  size_t generic_capacity = 0, transposes_capacity = 0;
  bool inline_copy = false, inline_span = false;  // the group table fits the kernel's argument block
  uint64_t serial = 0;
  // Hashes of the buffer sets of the last launches that went without device tables.  As many as bindings are kept: a
  // schedule whose fresh output stores come round from the allocator's pool in a longer cycle than this list holds
  // would never see a set "again" and never get device tables (3 parameter sets x 4 output buffers in rotation
  // make 12 combinations).
  uint64_t recent[kMaxBindings] = {};
  uint32_t recent_at = 0;

  DevicePlan() = default;
  DevicePlan(const DevicePlan&) = delete;
  DevicePlan& operator=(const DevicePlan&) = delete;
  ~DevicePlan();  // the device tables go back to the owner's block pool (no device-wide wait)
  bool needs_ptrs() const { return !plan.generic.empty() || !plan.transposes.empty(); }
  // no launch of this plan can go without tables in device memory
  bool needs_binding() const {
    return needs_ptrs() || (plan.n_copy_chunks && !inline_copy) || (plan.n_span_chunks && !inline_span);
  }
};

// Where the tables of a launch lie inside one block of device memory (each 256-byte aligned).
struct BlockLayout {
  size_t ptrs = 0, cgroups = 0, cpieces = 0, chints = 0, sgroups = 0, smembers = 0, spieces = 0, shints = 0;
  size_t generic = 0, transposes = 0;  // only with chunk tables included
  size_t total = 0;
};

BlockLayout layout_block(const DevicePlan& dp, bool with_chunk_tables) {
  const mmr_plan& p = dp.plan;
  BlockLayout l;
  size_t at = 0;
  auto take = [&at](size_t bytes) {
    const size_t here = at;
    at += (bytes + 255) & ~static_cast<size_t>(255);
    return here;
  };
  l.ptrs = take((dp.needs_ptrs() || with_chunk_tables) ? static_cast<size_t>(p.n_slots) * sizeof(void*) : 0);
  l.cgroups = take(p.copy_groups.size() * sizeof(mmr::CopyGroup));
  l.cpieces = take(p.copy_pieces.size() * sizeof(mmr::CopyPiece));
  l.chints = take(dp.copy_hints.size() * sizeof(uint32_t));
  l.sgroups = take(p.span_groups.size() * sizeof(mmr::SpanGroup));
  l.smembers = take(p.span_members.size() * sizeof(mmr::SpanMember));
  l.spieces = take(p.span_pieces.size() * sizeof(mmr::SpanPiece));
  l.shints = take(dp.span_hints.size() * sizeof(uint32_t));
  if (with_chunk_tables) {
    l.generic = take(p.generic.size() * sizeof(mmr_copy_chunk));
    l.transposes = take(p.transposes.size() * sizeof(mmr_transpose_chunk));
  }
  l.total = at;
  return l;
}

// The device tables of a plan bound to one set of shard buffers: a pure function of (plan, buffer addresses), so
// stores that come and go at the same addresses (buffers recycled through the cache) find their tables again.
struct Binding {
  DevicePlan* plan = nullptr;
  std::vector<void*> ptrs;  // the key: every source and destination buffer, in slot order
  uint64_t key = 0;         // hash of (plan, ptrs): compared first, the vectors only on a match
  char* d_block = nullptr;  // from the context's block pool
  size_t capacity = 0;
  BlockLayout layout;
  bool pinned = false;  // made by mmr_reshard_bind or used under stream capture: never recycled
  uint64_t last_use = 0;
};

uint64_t hash_ptrs(const DevicePlan* dp, const std::vector<void*>& ptrs) {
  uint64_t h = 0xcbf29ce484222325ull ^ reinterpret_cast<uint64_t>(dp);
  for (void* q : ptrs) h = (h ^ reinterpret_cast<uint64_t>(q)) * 0x100000001b3ull;
  return h | 1;
}

// roctx markers and ranges (MarkProfile and the named region around every task of the reference,
// zuku_execute_context_impl.cc:292-308, 458-460), looked up at run time so that the library loads where no profiler
// library is installed; MMR_ROCTX=0 switches them off.
struct Roctx {
  void (*mark)(const char*) = nullptr;
  int (*push)(const char*) = nullptr;
  int (*pop)() = nullptr;
};

Roctx load_roctx() {
  Roctx r;
  const char* env = std::getenv("MMR_ROCTX");
  if (env && env[0] == '0') return r;
  for (const char* name : {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4", "libroctx64.so"}) {
    void* lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
    if (!lib) continue;
    r.mark = reinterpret_cast<void (*)(const char*)>(dlsym(lib, "roctxMarkA"));
    r.push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
    r.pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
    if (r.mark && r.push && r.pop) return r;
    r = Roctx{};
  }
  return r;
}

const Roctx& roctx() {
  static const Roctx r = load_roctx();
  return r;
}

struct ProfileRange {
  explicit ProfileRange(const char* name) : on(roctx().push != nullptr) {
    if (on) roctx().push(name);
  }
  ~ProfileRange() {
    if (on) roctx().pop();
  }
  ProfileRange(const ProfileRange&) = delete;
  ProfileRange& operator=(const ProfileRange&) = delete;
  bool on;
};

// A point on the stream's timeline: one timing event, shared by everything that marks the same point.  The end of
// one execution's timer, the marker of its window and the start of the next execution's timer fall on one point
// when no work was queued in between, and an event on the stream costs the device a few microseconds of idle time.
struct StreamPoint {
  hipEvent_t event = nullptr;
  int refs = 0;
  uint64_t epoch = 0;  // mmr_context::work_epoch when it was recorded
};

// A named interval whose two points are recorded and whose length nobody has read yet.
struct TimerInterval {
  std::string name;
  StreamPoint *start = nullptr, *stop = nullptr;
};
struct TimerResult {
  float last_ms = 0;
  int64_t completed = 0;
};

// One upload in flight out of the pinned staging arena: bytes [begin, end) are free again once `consumed` is reached.
struct StagedUpload {
  size_t begin = 0, end = 0;
  hipEvent_t consumed = nullptr;
};

struct CachedBuffer {
  char* base;
  size_t bytes;
};

}  // namespace

struct mmr_store {
  int64_t id = -1;
  int64_t ordinal = -1;  // per context: the hash of the operation stream must not depend on other contexts
  std::string name;
  mmr_sharded_shape shape{};
  mmr::Side side;
  std::string shape_key;
  char* base = nullptr;   // one allocation, the tile of device dev_start + k at base + slot(k) * pitch (null for adopted stores)
  size_t pitch = 0;
  size_t bytes = 0;
  std::vector<char*> adopted;  // caller-owned buffers, one per device (mmr_store_adopt)
  char* host = nullptr;        // pinned host copy while the store is offloaded (the device buffers are gone then)
  mmr_context* owner = nullptr;

  // Replicated stores keep the tiles of one replica together (replica after replica) whatever the order of the device
  // ids: a reshard reads the tiles of ONE replica, and with the replica digit in the middle of the device id those tiles
  // would lie a multiple of the pitch apart - with power-of-two shards a power of two, which lines the pieces that
  // neighbouring workgroups gather from them up on the same memory channels (a [4,32,2048,128] bf16 array, heads 4-way
  // x 2 replicas, gathered into sequence tiles: 25.4 us with tiles 32 MiB apart, 23.0 us with 16 MiB).
  int64_t replica_stride = 0, replication = 1;  // device-id stride of the replica digit; 1 replica: identity
  size_t slot(int64_t k) const {
    if (replication <= 1) return static_cast<size_t>(k);
    const int64_t r = (k / replica_stride) % replication;
    const int64_t data = (k / (replica_stride * replication)) * replica_stride + k % replica_stride;
    return static_cast<size_t>(r * (side.dev_count / replication) + data);
  }
  bool offloaded() const { return host != nullptr; }
  char* tile(int64_t k) const { return adopted.empty() ? base + slot(k) * pitch : adopted[static_cast<size_t>(k)]; }
};

// What a host function on the stream hands to the callback thread.
struct PendingCallback {
  void (*fn)(void*) = nullptr;
  void* arg = nullptr;
};

struct mmr_context {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  hipEvent_t t0 = nullptr, t1 = nullptr;
  std::vector<hipEvent_t> laps;  // mmr_timer_lap
  size_t laps_used = 0;
  mmr_plan_options options{};
  uint32_t flags = 0;
  std::mutex mu;
  std::unordered_map<std::string, std::unique_ptr<DevicePlan>> plans;  // by descriptor pair(s) and options
  std::list<std::string> plan_lru;                                     // most recently used first
  // last plan looked up, with the descriptors it was looked up by: a schedule that issues the same batch every
  // execution compares two arrays of descriptors instead of building and hashing a key string
  DevicePlan* last_plan = nullptr;
  std::vector<mmr_sharded_shape> last_srcs, last_dsts;
  mmr_plan_options last_options{};
  std::vector<std::unique_ptr<Binding>> bindings;
  std::unordered_multimap<uint64_t, Binding*> binding_index;  // Binding::key -> binding
  uint64_t clock = 0, next_plan_serial = 1;
  std::unordered_map<std::string, std::vector<CachedBuffer>> buffer_cache;  // ArrayCache: by descriptor
  std::unordered_map<std::string, std::vector<CachedBuffer>> host_cache;    // pinned buffers, by descriptor
  // "use the cache as a store allocator" (ArrayCache::Make, zuku_execute_context_impl.cc:533-535): allocations of stores
  // that were freed without keep_in_cache, by size; any new store of that size takes one (ordered on the stream behind
  // the work of its previous owner), so a loop that creates and drops its output stores every step neither allocates
  // nor frees.  mmr_clear_store_cache releases them.
  std::unordered_map<size_t, std::vector<char*>> free_pool;
  size_t free_pool_bytes = 0;
  std::unordered_map<int64_t, std::unique_ptr<mmr_store>> stores;
  int64_t next_ordinal = 0;
  mmr_context_stats stats{};
  // mmr_reshard_batch_static: this GPU's static scratch array, a pinned staging buffer of the same size and the event
  // that tells when the last copy out of the staging buffer is done
  char* static_scratch = nullptr;
  char* static_staging = nullptr;
  hipEvent_t static_copied = nullptr;
  hipEvent_t static_done = nullptr;  // recorded behind the kernels of this context's last static call
  bool static_copy_pending = false;
  // Device blocks of plan and binding tables, by capacity (powers of two): a block that a recycled binding or a
  // dropped plan gives up is reused by the next table of its size class, ordered on the stream behind the launches
  // that read it, so nothing on a step path frees device memory.
  std::map<size_t, std::vector<char*>> block_pool;
  // Pinned staging arena every table upload goes through (a byte ring): the copy engine reads pinned memory while
  // the host goes on; pageable sources would make the runtime stage or wait inside hipMemcpyAsync.
  char* staging = nullptr;
  size_t staging_head = 0;  // next free byte
  std::deque<StagedUpload> staged;
  std::vector<char> fill_scratch;  // tables are assembled here, then copied into the arena
  // events are created once and reused (creating one costs a runtime lock)
  std::vector<hipEvent_t> free_plain_events, free_timing_events;
  // Bumped by every entry point that may queue work on the stream; a StreamPoint is reused only while it is still
  // the last thing on the stream.  Once the caller has asked for the stream (mmr_context_stream) or brought its own,
  // work may arrive that the library does not see, and points are no longer shared.
  std::atomic<uint64_t> work_epoch{1};
  bool stream_exposed = false;
  StreamPoint* last_point = nullptr;
  // named deferred timers (StartTimer / StopTimer)
  std::unordered_map<std::string, StreamPoint*> pending_timers;
  std::deque<TimerInterval> resolving;
  std::unordered_map<std::string, TimerResult> timer_results;
  // execution windows (OpenWindow / CloseWindow)
  std::deque<StreamPoint*> window_markers;
  int32_t max_open_windows = 8;
  // callbacks of mmr_context_run_after: the stream's host function only queues them here; this thread runs them
  std::thread callback_thread;
  std::mutex callback_mu;
  std::condition_variable callback_cv;
  std::deque<PendingCallback> callbacks;
  int64_t callbacks_queued = 0, callbacks_done = 0;
  bool callback_stop = false;
};

namespace {

constexpr size_t kMaxPlans = 256;  // cached plans per context (least recently used go first)
constexpr size_t kFreePoolLimit = static_cast<size_t>(16) << 30;  // bytes the allocator keeps before it really frees

#ifndef MMR_TIMING_EVENT_FLAGS
#define MMR_TIMING_EVENT_FLAGS (hipEventDefault | hipEventDisableSystemFence)
#endif

#define MMR_HIP(expr)                                                                             \
  do {                                                                                            \
    hipError_t e_ = (expr);                                                                       \
    if (e_ != hipSuccess)                                                                         \
      return fail(e_ == hipErrorOutOfMemory ? MMR_OUT_OF_MEMORY : MMR_HIP_ERROR, "%s failed: %s", #expr, \
                  hipGetErrorString(e_));                                                         \
  } while (0)

void give_block(mmr_context* ctx, char* block, size_t capacity);

int use_device(mmr_context* ctx) {
  MMR_HIP(hipSetDevice(ctx->device));
  return MMR_OK;
}

bool capturing(mmr_context* ctx) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(ctx->stream, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
}

// Entry points that allocate, free, copy from pageable memory or wait may not run while the stream records a graph.
int refuse_capture(mmr_context* ctx, const char* what) {
  if (capturing(ctx))
    return fail(MMR_INVALID_ARGUMENT, "%s is not allowed while the context's stream is capturing a graph", what);
  return MMR_OK;
}

void account_alloc(mmr_context* ctx, int64_t bytes) {
  ctx->stats.bytes_allocated += bytes;
  ctx->stats.bytes_high_watermark = std::max(ctx->stats.bytes_high_watermark, ctx->stats.bytes_allocated);
}

int device_alloc(mmr_context* ctx, void** out, size_t bytes) {
  MMR_HIP(hipMalloc(out, bytes));
  ctx->stats.device_allocations += 1;
  return MMR_OK;
}

// Makes the calling thread wait for the stream; counted, because the reference's calls are asynchronous.
int blocking_sync(mmr_context* ctx) {
  ctx->stats.host_blocking_syncs += 1;
  MMR_HIP(hipStreamSynchronize(ctx->stream));
  return MMR_OK;
}

void hash_op(mmr_context* ctx, uint64_t kind, std::initializer_list<uint64_t> values, const std::string* text = nullptr) {
  if (!(ctx->flags & MMR_CHECK_INVARIANTS)) return;
  uint64_t h = static_cast<uint64_t>(ctx->stats.operation_hash);
  auto mix = [&h](uint64_t v) {  // FNV-1a over the 8 bytes of v
    for (int i = 0; i < 8; ++i) {
      h ^= (v >> (8 * i)) & 0xff;
      h *= 0x100000001b3ull;
    }
  };
  if (h == 0) h = 0xcbf29ce484222325ull;
  mix(kind);
  for (uint64_t v : values) mix(v);
  if (text)
    for (unsigned char c : *text) mix(c);
  ctx->stats.operation_hash = static_cast<int64_t>(h);
}

// Waits for one event; counted like every other host wait.
int blocking_wait(mmr_context* ctx, hipEvent_t e) {
  ctx->stats.host_blocking_syncs += 1;
  MMR_HIP(hipEventSynchronize(e));
  return MMR_OK;
}

// Events that only mark a point in time (timer marks, window markers, laps): nothing the host reads hangs on them, so
// they need no system-scope fence - which would write back and invalidate the caches in the middle of a schedule.
constexpr unsigned kTimingEventFlags = MMR_TIMING_EVENT_FLAGS;

int take_event(mmr_context* ctx, bool timing, hipEvent_t* out) {
  std::vector<hipEvent_t>& pool = timing ? ctx->free_timing_events : ctx->free_plain_events;
  if (!pool.empty()) {
    *out = pool.back();
    pool.pop_back();
    return MMR_OK;
  }
  MMR_HIP(hipEventCreateWithFlags(out, timing ? kTimingEventFlags : hipEventDisableTiming));
  return MMR_OK;
}

void give_event(mmr_context* ctx, bool timing, hipEvent_t e) {
  if (e) (timing ? ctx->free_timing_events : ctx->free_plain_events).push_back(e);
}

void release_point(mmr_context* ctx, StreamPoint* p) {
  if (!p || --p->refs > 0) return;
  give_event(ctx, true, p->event);
  delete p;
}

// The current end of the stream as a point the caller holds one reference to.
int mark_point(mmr_context* ctx, StreamPoint** out) {
  const uint64_t epoch = ctx->work_epoch.load();
  if (ctx->last_point && ctx->last_point->epoch == epoch && ctx->owns_stream && !ctx->stream_exposed) {
    ctx->last_point->refs += 1;
    *out = ctx->last_point;
    return MMR_OK;
  }
  auto p = std::make_unique<StreamPoint>();
  if (int rc = take_event(ctx, true, &p->event)) return rc;
  const hipError_t e = hipEventRecord(p->event, ctx->stream);
  if (e != hipSuccess) {
    give_event(ctx, true, p->event);
    return fail(MMR_HIP_ERROR, "hipEventRecord failed: %s", hipGetErrorString(e));
  }
  ctx->stats.events_recorded += 1;
  p->epoch = epoch;
  p->refs = 2;  // the caller's and last_point's
  release_point(ctx, ctx->last_point);
  ctx->last_point = p.get();
  *out = p.release();
  return MMR_OK;
}

void note_work(mmr_context* ctx) { ctx->work_epoch.fetch_add(1); }

constexpr size_t kStagingBytes = static_cast<size_t>(4) << 20;  // pinned arena of table uploads
constexpr size_t kStagingPiece = kStagingBytes / 4;            // longer uploads go in pieces of this size
constexpr size_t kMinBlockBytes = 16384;

size_t block_class(size_t bytes) {
  size_t c = kMinBlockBytes;
  while (c < bytes) c <<= 1;
  return c;
}

// A block of device memory for tables: from the pool of its size class, else new.
int take_block(mmr_context* ctx, size_t bytes, char** out, size_t* capacity) {
  const size_t cls = block_class(bytes);
  auto it = ctx->block_pool.find(cls);
  if (it != ctx->block_pool.end() && !it->second.empty()) {
    *out = it->second.back();
    it->second.pop_back();
    ctx->stats.block_pool_hits += 1;
  } else {
    if (int rc = device_alloc(ctx, reinterpret_cast<void**>(out), cls)) return rc;
  }
  *capacity = cls;
  return MMR_OK;
}

// Its next user writes it by a copy on the context's stream, behind every launch that still reads it.
void give_block(mmr_context* ctx, char* block, size_t capacity) {
  if (block) ctx->block_pool[capacity].push_back(block);
}

DevicePlan::~DevicePlan() {
  if (!owner) return;
  give_block(owner, reinterpret_cast<char*>(d_generic), generic_capacity);
  give_block(owner, reinterpret_cast<char*>(d_transposes), transposes_capacity);
}

// Frees the oldest staged uploads that the copy engine has consumed; with `wait`, waits for the oldest one.
int retire_staged(mmr_context* ctx, bool wait) {
  while (!ctx->staged.empty()) {
    StagedUpload& u = ctx->staged.front();
    if (hipEventQuery(u.consumed) != hipSuccess) {
      (void)hipGetLastError();
      if (!wait) break;
      if (int rc = blocking_wait(ctx, u.consumed)) return rc;
      wait = false;
    }
    give_event(ctx, false, u.consumed);
    ctx->staged.pop_front();
  }
  return MMR_OK;
}

// `bytes` (at most kStagingPiece) of the arena, free of any upload still in flight.
int staging_reserve(mmr_context* ctx, size_t bytes, char** out) {
  bytes = (bytes + 255) & ~static_cast<size_t>(255);
  for (;;) {
    if (int rc = retire_staged(ctx, false)) return rc;
    if (ctx->staged.empty()) ctx->staging_head = 0;
    size_t at = ctx->staging_head;
    if (at + bytes > kStagingBytes) at = 0;  // wrap: the tail of the arena stays unused this round
    bool free_range = true;
    for (const StagedUpload& u : ctx->staged) free_range &= u.end <= at || u.begin >= at + bytes;
    if (free_range) {
      ctx->staging_head = at + bytes;
      *out = ctx->staging + at;
      return MMR_OK;
    }
    if (int rc = retire_staged(ctx, true)) return rc;  // the ring is full: the host is that far ahead of the device
  }
}

// Copies host memory to the device through the pinned arena, on the context's stream; `host` may be reused as soon
// as the call returns.
int staged_upload(mmr_context* ctx, void* device, const void* host, size_t bytes) {
  const char* src = static_cast<const char*>(host);
  char* dst = static_cast<char*>(device);
  while (bytes) {
    const size_t piece = std::min(bytes, kStagingPiece);
    char* pinned = nullptr;
    if (int rc = staging_reserve(ctx, piece, &pinned)) return rc;
    std::memcpy(pinned, src, piece);
    StagedUpload u;
    u.begin = static_cast<size_t>(pinned - ctx->staging);
    u.end = u.begin + ((piece + 255) & ~static_cast<size_t>(255));
    if (int rc = take_event(ctx, false, &u.consumed)) return rc;
    hipError_t e = hipMemcpyAsync(dst, pinned, piece, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipEventRecord(u.consumed, ctx->stream);
    if (e != hipSuccess) {
      give_event(ctx, false, u.consumed);
      return fail(MMR_HIP_ERROR, "upload of %zu table bytes failed: %s", piece, hipGetErrorString(e));
    }
    ctx->staged.push_back(u);
    src += piece;
    dst += piece;
    bytes -= piece;
  }
  return MMR_OK;
}

template <class T>
int upload(mmr_context* ctx, const std::vector<T>& host, T** dev, size_t* capacity) {
  *dev = nullptr;
  *capacity = 0;
  if (host.empty()) return MMR_OK;
  char* block = nullptr;
  if (int rc = take_block(ctx, host.size() * sizeof(T), &block, capacity)) return rc;
  if (int rc = staged_upload(ctx, block, host.data(), host.size() * sizeof(T))) {
    give_block(ctx, block, *capacity);
    *capacity = 0;
    return rc;
  }
  *dev = reinterpret_cast<T*>(block);
  return MMR_OK;
}

// The transpose kernel's LDS tile and lane mapping assume bounds the planner keeps; checked before the first launch
// of a plan.  Also splits the table into runs of equal element width and kind, one launch each.
int check_transposes(const mmr_plan& plan, std::vector<TransposeRun>* runs) {
  const std::vector<mmr_transpose_chunk>& tr = plan.transposes;
  for (const mmr_transpose_chunk& c : tr) {
    uint32_t tile_x = 0, tile_y = 0;
    mmr::transpose_tile_extent(c.itemsize, &tile_x, &tile_y);
    const bool width_ok = c.itemsize == 1 || c.itemsize == 2 || c.itemsize == 4 || c.itemsize == 8 || c.itemsize == 16;
    if (!width_ok || c.nx == 0 || c.ny == 0)
      return fail(MMR_INTERNAL, "transpose chunk %u x %u of %u-byte elements", c.nx, c.ny, c.itemsize);
    if (mmr::transpose_is_thin(c)) {  // any shape, all batch entries in LDS at once
      if (static_cast<uint64_t>(c.nb) * c.nx * c.ny * c.itemsize > mmr::kTransposeLdsBytes)
        return fail(MMR_INTERNAL, "thin transpose chunk of %u x %u x %u elements exceeds the workgroup's LDS", c.nb, c.nx,
                    c.ny);
    } else if (c.nx > tile_x || c.ny > tile_y) {
      return fail(MMR_INTERNAL, "transpose chunk %u x %u of %u-byte elements does not fit the kernel's tile", c.nx, c.ny,
                  c.itemsize);
    }
  }
  for (int64_t i = 0; i < static_cast<int64_t>(tr.size()); ++i) {
    const bool vec = mmr::transpose_is_vector(tr[i]);
    if (i == 0 || tr[i].itemsize != tr[i - 1].itemsize || vec != runs->back().vector_only)
      runs->push_back({tr[i].itemsize, vec, i, 0});
    runs->back().count += 1;
  }
  return MMR_OK;
}

// What the span kernel's LDS staging assumes.
int check_spans(const mmr_plan& plan) {
  for (const mmr::SpanGroup& g : plan.span_groups)
    if (g.span == 0 || g.span > mmr::kSpanMaxBytes || g.head == 0 || g.head > g.span || g.W == 0 ||
        g.W > mmr::kSpanMaxRowBytes)
      return fail(MMR_INTERNAL, "span group with span %u, head %u, row %u", g.span, g.head, g.W);
  // a group that uses the segment table: one lane per (row, piece) pair that can touch a span
  for (const mmr::SpanGroup& g : plan.span_groups) {
    if (!g.table_mode) continue;
    for (uint32_t t = 0; t < g.il.members; ++t) {
      const mmr::SpanMember& m = plan.span_members[g.first_member + t];
      if (m.k == 0 || m.k > mmr::kSpanTablePieces || (static_cast<uint64_t>(g.span) / g.W + 2) * m.k > mmr::kSpanLanes)
        return fail(MMR_INTERNAL, "span group with %u pieces per row of %u bytes cannot use a segment table", m.k, g.W);
    }
  }
  return MMR_OK;
}

// Plans n descriptor pairs under `options`; the chunk tables that need no binding are uploaded.  With
// `device_tables` false nothing touches the device (the static entry point brings its own memory).
int make_device_plan(mmr_context* ctx, const std::vector<mmr_sharded_shape>& srcs, const std::vector<mmr_sharded_shape>& dsts,
                     const mmr_plan_options& options, bool device_tables, DevicePlan* dp) {
  const int n = static_cast<int>(srcs.size());
  if (int rc = mmr::build_plan(srcs.data(), dsts.data(), n, options, &dp->plan)) return rc;
  if (int rc = check_transposes(dp->plan, &dp->transpose_runs)) return rc;
  if (int rc = check_spans(dp->plan)) return rc;
  const mmr_plan& p = dp->plan;
  const bool may_inline = !(options.flags & MMR_PLAN_NO_INLINE);  // without it every launch builds device tables
  dp->inline_copy = may_inline && p.copy_groups.size() <= mmr::kInlineCopyGroups && p.copy_pieces.size() <= mmr::kInlineCopyPieces;
  dp->inline_span = may_inline && p.span_groups.size() <= mmr::kInlineSpanGroups &&
                    p.span_members.size() <= mmr::kInlineSpanMembers && p.span_pieces.size() <= mmr::kInlineSpanPieces;
  dp->copy_hints = mmr::group_hints(p.copy_groups, p.n_copy_chunks);
  dp->span_hints = mmr::group_hints(p.span_groups, p.n_span_chunks);
  dp->serial = ctx->next_plan_serial++;
  if (device_tables) {
    dp->owner = ctx;
    if (int rc = upload(ctx, dp->plan.generic, &dp->d_generic, &dp->generic_capacity)) return rc;
    if (int rc = upload(ctx, dp->plan.transposes, &dp->d_transposes, &dp->transposes_capacity)) return rc;
  }
  return MMR_OK;
}

void drop_bindings_of_plan(mmr_context* ctx, const DevicePlan* dp);

bool same_descriptors(const std::vector<mmr_sharded_shape>& a, const std::vector<mmr_sharded_shape>& b) {
  // descriptors are value-initialised PODs everywhere they are made, so their bytes compare
  return a.size() == b.size() && (a.empty() || std::memcmp(a.data(), b.data(), a.size() * sizeof(mmr_sharded_shape)) == 0);
}

void forget_last_plan(mmr_context* ctx) {
  ctx->last_plan = nullptr;
  ctx->last_srcs.clear();
  ctx->last_dsts.clear();
}

int get_plan(mmr_context* ctx, const std::vector<mmr_sharded_shape>& srcs, const std::vector<mmr_sharded_shape>& dsts,
             DevicePlan** out, std::string* key_out = nullptr) {
  const int n = static_cast<int>(srcs.size());
  // the batch of the previous call again (a schedule repeats its windows): no key is built
  if (!key_out && ctx->last_plan && std::memcmp(&ctx->last_options, &ctx->options, sizeof(ctx->options)) == 0 &&
      same_descriptors(ctx->last_srcs, srcs) && same_descriptors(ctx->last_dsts, dsts)) {
    ctx->stats.plan_cache_hits += 1;
    *out = ctx->last_plan;
    return MMR_OK;
  }
  std::string key = mmr::plan_key(srcs.data(), dsts.data(), n, ctx->options);
  if (key_out) *key_out = key;
  auto remember = [&](DevicePlan* dp) {
    ctx->last_plan = dp;
    ctx->last_srcs = srcs;
    ctx->last_dsts = dsts;
    ctx->last_options = ctx->options;
  };
  auto it = ctx->plans.find(key);
  if (it != ctx->plans.end()) {
    ctx->stats.plan_cache_hits += 1;
    *out = it->second.get();
    auto pos = std::find(ctx->plan_lru.begin(), ctx->plan_lru.end(), key);
    if (pos != ctx->plan_lru.begin() && pos != ctx->plan_lru.end()) ctx->plan_lru.splice(ctx->plan_lru.begin(), ctx->plan_lru, pos);
    remember(*out);
    return MMR_OK;
  }
  if (capturing(ctx))  // building a plan may allocate and copy
    return fail(MMR_INVALID_ARGUMENT,
                "the stream is capturing and this reshard has no cached plan yet: call mmr_reshard_bind (or run the "
                "reshard once) before the capture begins");
  ProfileRange range("mmreshard: build plan");
  auto dp = std::make_unique<DevicePlan>();
  if (int rc = make_device_plan(ctx, srcs, dsts, ctx->options, true, dp.get())) return rc;
  ctx->stats.plans_built += 1;
  *out = dp.get();
  ctx->plans.emplace(key, std::move(dp));
  ctx->plan_lru.push_front(std::move(key));
  // Least recently used plans go when the cache is full; the device tables of one that goes return to the block pool,
  // whose next user is ordered on the stream behind the launches that still read them.  Plans with bindings stay
  // until mmr_context_clear_plans (a captured graph may hold their tables).
  if (ctx->plans.size() > kMaxPlans) {
    for (auto pos = std::prev(ctx->plan_lru.end()); pos != ctx->plan_lru.begin();) {
      auto victim = ctx->plans.find(*pos);
      auto prev = std::prev(pos);
      bool bound = false;
      for (const auto& b : ctx->bindings) bound |= b->plan == victim->second.get();
      if (!bound) {
        if (ctx->last_plan == victim->second.get()) forget_last_plan(ctx);
        ctx->plans.erase(victim);
        ctx->plan_lru.erase(pos);
        if (ctx->plans.size() <= kMaxPlans) break;
      }
      pos = prev;
    }
  }
  ctx->stats.plans_cached = static_cast<int64_t>(ctx->plans.size());
  remember(*out);
  return MMR_OK;
}

// Slot -> buffer address for the stores of a batch.
void collect_ptrs(const mmr_plan& p, mmr_store* const* srcs, mmr_store* const* dsts, int n, std::vector<void*>* ptrs) {
  ptrs->assign(static_cast<size_t>(p.n_slots), nullptr);
  for (int a = 0; a < n; ++a) {
    size_t slot = static_cast<size_t>(p.slot_bases[a]);
    for (int64_t k = 0; k < srcs[a]->side.dev_count; ++k) (*ptrs)[slot++] = srcs[a]->tile(k);
    for (int64_t k = 0; k < dsts[a]->side.dev_count; ++k) (*ptrs)[slot++] = dsts[a]->tile(k);
  }
}

uint64_t address_of(const std::vector<void*>& ptrs, uint32_t slot, uint64_t off) {
  return slot == MMR_SLOT_FILL ? 0 : reinterpret_cast<uint64_t>(ptrs[slot]) + off;
}

void bind_copy_pieces(const mmr::CopyPiece* in, size_t n, const std::vector<void*>& ptrs, mmr::CopyPiece* out) {
  for (size_t i = 0; i < n; ++i) {
    out[i] = in[i];
    out[i].src = address_of(ptrs, in[i].src_slot, in[i].src);
    out[i].dst = address_of(ptrs, in[i].dst_slot, in[i].dst);
  }
}

void bind_span_tables(const mmr_plan& p, const std::vector<void*>& ptrs, mmr::SpanMember* members, mmr::SpanPiece* pieces) {
  for (size_t i = 0; i < p.span_members.size(); ++i) {
    members[i] = p.span_members[i];
    members[i].dst = address_of(ptrs, p.span_members[i].dst_slot, p.span_members[i].dst);
  }
  for (size_t i = 0; i < p.span_pieces.size(); ++i) {
    pieces[i] = p.span_pieces[i];
    pieces[i].src = address_of(ptrs, p.span_pieces[i].src_slot, p.span_pieces[i].src);
  }
}

// Fills `block` (layout l) with the tables of dp bound to ptrs.
void fill_block(const DevicePlan& dp, const BlockLayout& l, const std::vector<void*>& ptrs, bool with_chunk_tables, char* block) {
  const mmr_plan& p = dp.plan;
  if (dp.needs_ptrs() || with_chunk_tables) std::memcpy(block + l.ptrs, ptrs.data(), ptrs.size() * sizeof(void*));
  if (!p.copy_groups.empty()) {
    std::memcpy(block + l.cgroups, p.copy_groups.data(), p.copy_groups.size() * sizeof(mmr::CopyGroup));
    bind_copy_pieces(p.copy_pieces.data(), p.copy_pieces.size(), ptrs, reinterpret_cast<mmr::CopyPiece*>(block + l.cpieces));
    std::memcpy(block + l.chints, dp.copy_hints.data(), dp.copy_hints.size() * sizeof(uint32_t));
  }
  if (!p.span_groups.empty()) {
    std::memcpy(block + l.sgroups, p.span_groups.data(), p.span_groups.size() * sizeof(mmr::SpanGroup));
    bind_span_tables(p, ptrs, reinterpret_cast<mmr::SpanMember*>(block + l.smembers),
                     reinterpret_cast<mmr::SpanPiece*>(block + l.spieces));
    std::memcpy(block + l.shints, dp.span_hints.data(), dp.span_hints.size() * sizeof(uint32_t));
  }
  if (with_chunk_tables) {
    if (!p.generic.empty()) std::memcpy(block + l.generic, p.generic.data(), p.generic.size() * sizeof(mmr_copy_chunk));
    if (!p.transposes.empty())
      std::memcpy(block + l.transposes, p.transposes.data(), p.transposes.size() * sizeof(mmr_transpose_chunk));
  }
}

void unindex_binding(mmr_context* ctx, Binding* b) {
  auto range = ctx->binding_index.equal_range(b->key);
  for (auto it = range.first; it != range.second; ++it)
    if (it->second == b) {
      ctx->binding_index.erase(it);
      return;
    }
}

// The bindings of a plan that goes away: their blocks return to the pool (their next user is ordered on the stream
// behind the launches that still read them).
void drop_bindings_of_plan(mmr_context* ctx, const DevicePlan* dp) {
  for (auto it = ctx->bindings.begin(); it != ctx->bindings.end();) {
    if ((*it)->plan == dp) {
      unindex_binding(ctx, it->get());
      give_block(ctx, (*it)->d_block, (*it)->capacity);
      it = ctx->bindings.erase(it);
    } else {
      ++it;
    }
  }
  if (ctx->last_plan == dp) forget_last_plan(ctx);
  ctx->stats.bindings_cached = static_cast<int64_t>(ctx->bindings.size());
}

Binding* find_binding(mmr_context* ctx, const DevicePlan* dp, const std::vector<void*>& ptrs, uint64_t key) {
  auto range = ctx->binding_index.equal_range(key);
  for (auto it = range.first; it != range.second; ++it)
    if (it->second->plan == dp && it->second->ptrs == ptrs) return it->second;
  return nullptr;
}

// The binding of dp to ptrs: cached, else built in a recycled or new block and uploaded on the stream.
int get_binding(mmr_context* ctx, DevicePlan* dp, const std::vector<void*>& ptrs, bool pin, bool count_hit, Binding** out) {
  const uint64_t key = hash_ptrs(dp, ptrs);
  if (Binding* b = find_binding(ctx, dp, ptrs, key)) {
    b->last_use = ++ctx->clock;
    b->pinned |= pin || capturing(ctx);
    if (count_hit) ctx->stats.binding_cache_hits += 1;
    *out = b;
    return MMR_OK;
  }
  if (capturing(ctx))
    return fail(MMR_INVALID_ARGUMENT,
                "the stream is capturing and this reshard has no bound device tables yet: call mmr_reshard_bind (or "
                "run the reshard once) before the capture begins");
  ProfileRange range("mmreshard: bind tables");
  const BlockLayout l = layout_block(*dp, false);
  // a block to put it in: the least recently used unpinned binding's once the cache is full, else one from the pool
  std::unique_ptr<Binding> b;
  size_t unpinned = 0;
  for (auto& x : ctx->bindings) unpinned += x->pinned ? 0 : 1;
  if (unpinned >= kMaxBindings) {
    size_t victim = ctx->bindings.size();
    for (size_t i = 0; i < ctx->bindings.size(); ++i)
      if (!ctx->bindings[i]->pinned && (victim == ctx->bindings.size() || ctx->bindings[i]->last_use < ctx->bindings[victim]->last_use))
        victim = i;
    b = std::move(ctx->bindings[victim]);
    ctx->bindings.erase(ctx->bindings.begin() + static_cast<std::ptrdiff_t>(victim));
    unindex_binding(ctx, b.get());
    if (b->capacity < l.total) {  // too small: swapped for one of the right size class
      give_block(ctx, b->d_block, b->capacity);
      b->d_block = nullptr;
      b->capacity = 0;
    }
  } else {
    b = std::make_unique<Binding>();
  }
  if (!b->d_block)
    if (int rc = take_block(ctx, l.total, &b->d_block, &b->capacity)) return rc;
  b->plan = dp;
  b->ptrs = ptrs;
  b->key = key;
  b->layout = l;
  b->pinned = pin;
  b->last_use = ++ctx->clock;
  ctx->fill_scratch.assign(l.total, 0);
  fill_block(*dp, l, ptrs, false, ctx->fill_scratch.data());
  // stream-ordered: launches queued earlier that still read a recycled block finish before the copy overwrites it
  if (int rc = staged_upload(ctx, b->d_block, ctx->fill_scratch.data(), l.total)) {
    give_block(ctx, b->d_block, b->capacity);
    ctx->stats.bindings_cached = static_cast<int64_t>(ctx->bindings.size());
    return rc;
  }
  ctx->stats.bindings_built += 1;
  *out = b.get();
  ctx->binding_index.emplace(key, b.get());
  ctx->bindings.push_back(std::move(b));
  ctx->stats.bindings_cached = static_cast<int64_t>(ctx->bindings.size());
  return MMR_OK;
}

// Launches over tables in device memory: `block` laid out by l; the generic and transpose chunk tables at the
// given addresses.
int launch_block(mmr_context* ctx, const DevicePlan& dp, const char* block, const BlockLayout& l,
                 const mmr_copy_chunk* d_generic, const mmr_transpose_chunk* d_transposes, bool copies, bool spans) {
  const mmr_plan& p = dp.plan;
  const uint32_t xm = p.options.xcd_mode == 0 ? 64 : p.options.xcd_mode;  // runs of 64 table neighbours per XCD (measured)
  if (copies && p.n_copy_chunks) {
    uint32_t starts[mmr::kMaxDirectGroups];
    const bool direct = p.copy_groups.size() <= mmr::kMaxDirectGroups;
    for (size_t i = 0; direct && i < p.copy_groups.size(); ++i) starts[i] = p.copy_groups[i].first_chunk;
    MMR_HIP(mmr::launch_copy_groups(reinterpret_cast<const mmr::CopyGroup*>(block + l.cgroups),
                                    static_cast<uint32_t>(p.copy_groups.size()),
                                    reinterpret_cast<const mmr::CopyPiece*>(block + l.cpieces),
                                    reinterpret_cast<const uint32_t*>(block + l.chints), direct ? starts : nullptr,
                                    p.n_copy_chunks, xm, ctx->stream));
  }
  if (spans && p.n_span_chunks)
    MMR_HIP(mmr::launch_spans(reinterpret_cast<const mmr::SpanGroup*>(block + l.sgroups),
                              static_cast<uint32_t>(p.span_groups.size()),
                              reinterpret_cast<const mmr::SpanMember*>(block + l.smembers),
                              reinterpret_cast<const mmr::SpanPiece*>(block + l.spieces),
                              reinterpret_cast<const uint32_t*>(block + l.shints), p.n_span_chunks, xm, ctx->stream));
  void* const* d_ptrs = reinterpret_cast<void* const*>(block + l.ptrs);
  MMR_HIP(mmr::launch_copy_generic(d_generic, static_cast<int64_t>(p.generic.size()), d_ptrs, xm, ctx->stream));
  for (const TransposeRun& run : dp.transpose_runs)
    // tiles are ordered in 8 x 8 blocks; runs of 64 table neighbours per XCD keep a block in one L2 (measured best)
    MMR_HIP(mmr::launch_transpose(d_transposes + run.begin, run.count, d_ptrs, xm, run.itemsize, run.vector_only, ctx->stream));
  return MMR_OK;
}

int64_t launches_of(const DevicePlan* dp) {
  const uint32_t xm = dp->plan.options.xcd_mode == 0 ? 64 : dp->plan.options.xcd_mode;
  return mmr::copy_group_launches(dp->plan.n_copy_chunks, xm) + (dp->plan.n_span_chunks ? 1 : 0) +
         (dp->plan.generic.empty() ? 0 : 1) + static_cast<int64_t>(dp->transpose_runs.size());
}

// One launch per kernel class.  Tables in device memory, bound to these buffers, are the fast way (a workgroup's
// table reads stay in the caches); they cost an allocation and an upload the first time.  Group tables small enough
// can instead travel in the kernel's argument block, bound right here: nothing to allocate, upload or keep alive
// (about a microsecond slower per launch).  So: the first launch of a plan on a set of buffers goes through the
// argument block where it can, the second one on the same buffers builds the device tables, and every later one
// finds them (as does any launch after mmr_reshard_bind).  `tables`: 0 = that policy, 1 = device tables now.
int launch_plan(mmr_context* ctx, DevicePlan* dp, const std::vector<void*>& ptrs, int tables, bool count_hit) {
  const mmr_plan& p = dp->plan;
  const uint32_t xm = p.options.xcd_mode == 0 ? 64 : p.options.xcd_mode;
  ProfileRange range("mmreshard: launch");
  const uint64_t key = hash_ptrs(dp, ptrs);
  Binding* binding = find_binding(ctx, dp, ptrs, key);
  if (binding) {
    binding->last_use = ++ctx->clock;
    binding->pinned |= capturing(ctx);
    if (count_hit) ctx->stats.binding_cache_hits += 1;
  } else {
    bool want = dp->needs_binding() || tables == 1;
    if (!want && !capturing(ctx)) {  // seen these buffers before?
      for (uint64_t r : dp->recent) want |= r == key;
      if (!want) dp->recent[dp->recent_at++ % kMaxBindings] = key;
    }
    if (want)
      if (int rc = get_binding(ctx, dp, ptrs, /*pin=*/false, /*count_hit=*/false, &binding)) return rc;
  }
  const bool inline_copy = !binding && dp->inline_copy, inline_span = !binding && dp->inline_span;
  if (p.n_copy_chunks && inline_copy) {
    mmr::InlineCopyTable t{};
    t.n_groups = static_cast<uint32_t>(p.copy_groups.size());
    t.n_chunks = p.n_copy_chunks;
    std::copy(p.copy_groups.begin(), p.copy_groups.end(), t.groups);
    bind_copy_pieces(p.copy_pieces.data(), p.copy_pieces.size(), ptrs, t.pieces);
    MMR_HIP(mmr::launch_copy_groups_inline(t, xm, ctx->stream));
    ctx->stats.inline_launches += 1;
  }
  if (p.n_span_chunks && inline_span) {
    mmr::InlineSpanTable t{};
    t.n_groups = static_cast<uint32_t>(p.span_groups.size());
    t.n_chunks = p.n_span_chunks;
    std::copy(p.span_groups.begin(), p.span_groups.end(), t.groups);
    bind_span_tables(p, ptrs, t.members, t.pieces);
    MMR_HIP(mmr::launch_spans_inline(t, xm, ctx->stream));
    ctx->stats.inline_launches += 1;
  }
  if (binding)
    if (int rc = launch_block(ctx, *dp, binding->d_block, binding->layout, dp->d_generic, dp->d_transposes, true, true))
      return rc;
  ctx->stats.kernel_launches += launches_of(dp);
  return MMR_OK;
}

int check_store(mmr_context* ctx, const mmr_store* s, const char* what) {
  if (!s) return fail(MMR_INVALID_ARGUMENT, "%s store is null", what);
  if (s->owner != ctx) return fail(MMR_INVALID_ARGUMENT, "%s store belongs to another context", what);
  return MMR_OK;
}

// Argument checks shared by every reshard entry point.
int check_batch(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int n) {
  for (int a = 0; a < n; ++a) {
    if (int rc = check_store(ctx, srcs[a], "source")) return rc;
    if (int rc = check_store(ctx, dsts[a], "destination")) return rc;
    if (srcs[a] == dsts[a]) return fail(MMR_INVALID_ARGUMENT, "array %d: source and destination are the same store", a);
    // the mock's invariant (mm_mock_mm_xla.cc:164-173, 347-356): an offloaded store cannot take part in device work
    if (srcs[a]->offloaded() || dsts[a]->offloaded())
      return fail(MMR_INVALID_ARGUMENT, "array %d: store %lld is still offloaded to host memory", a,
                  (long long)(srcs[a]->offloaded() ? srcs[a]->id : dsts[a]->id));
  }
  for (int a = 0; a < n; ++a)
    for (int b = 0; b < n; ++b)
      if (dsts[a] == srcs[b] || (a != b && dsts[a] == dsts[b]))
        return fail(MMR_INVALID_ARGUMENT, "store %lld is written by array %d and used again by array %d of the same batch",
                    (long long)dsts[a]->id, a, b);
  if (ctx->flags & MMR_CHECK_INVARIANTS) {
    // mm_mock_mm_xla.cc:347-369: every operand holds a tile on each device of its list
    for (int a = 0; a < n; ++a)
      for (mmr_store* s : {srcs[a], dsts[a]}) {
        ctx->stats.invariant_checks += 1;
        for (int64_t k = 0; k < s->side.dev_count; ++k)
          if (s->side.shard_bytes > 0 && !s->tile(k))
            return fail(MMR_INTERNAL, "invariant violated: store %lld has no tile on device %lld", (long long)s->id,
                        (long long)(s->side.dev_start + k));
        hash_op(ctx, 2 /* Reshard */, {static_cast<uint64_t>(s->ordinal)}, &s->shape_key);
      }
  }
  return MMR_OK;
}

void shapes_of(mmr_store* const* srcs, mmr_store* const* dsts, int n, std::vector<mmr_sharded_shape>* s,
               std::vector<mmr_sharded_shape>* d) {
  s->resize(static_cast<size_t>(n));
  d->resize(static_cast<size_t>(n));
  for (int a = 0; a < n; ++a) {
    (*s)[a] = srcs[a]->shape;
    (*d)[a] = dsts[a]->shape;
  }
}

int reshard_locked(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int n, bool launch = true) {
  if (n == 0) return MMR_OK;
  if (int rc = use_device(ctx)) return rc;
  if (int rc = check_batch(ctx, srcs, dsts, n)) return rc;
  std::vector<mmr_sharded_shape> sshapes, dshapes;
  shapes_of(srcs, dsts, n, &sshapes, &dshapes);
  DevicePlan* dp = nullptr;
  if (int rc = get_plan(ctx, sshapes, dshapes, &dp)) return rc;
  std::vector<void*> ptrs;
  collect_ptrs(dp->plan, srcs, dsts, n, &ptrs);
  if (!launch) {  // mmr_reshard_bind: everything but the launches; the tables stay until the plans are cleared
    Binding* binding = nullptr;
    return get_binding(ctx, dp, ptrs, /*pin=*/true, /*count_hit=*/false, &binding);
  }
  ctx->stats.reshard_calls += 1;
  return launch_plan(ctx, dp, ptrs, /*tables=*/0, /*count_hit=*/true);
}

// mmr_reshard_tune: times the default order and a few interleaved ones on the caller's buffers.
int tune_locked(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int n, int64_t* order_used) {
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_reshard_tune")) return rc;
  if (int rc = check_batch(ctx, srcs, dsts, n)) return rc;
  std::vector<mmr_sharded_shape> sshapes, dshapes;
  shapes_of(srcs, dsts, n, &sshapes, &dshapes);
  DevicePlan* dp = nullptr;
  std::string key;
  if (int rc = get_plan(ctx, sshapes, dshapes, &dp, &key)) return rc;
  const mmr_plan_options base = dp->plan.options;
  if (order_used) *order_used = dp->plan.stats.order_used;
  const size_t chunks = static_cast<size_t>(dp->plan.n_copy_chunks) + dp->plan.n_span_chunks + dp->plan.generic.size();
  if (base.order != 0 || chunks < 1024) return MMR_OK;  // a fixed order, or too small to matter
  std::vector<void*> ptrs;
  collect_ptrs(dp->plan, srcs, dsts, n, &ptrs);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  MMR_HIP(hipEventCreate(&e0));
  if (hipEventCreate(&e1) != hipSuccess) {
    (void)hipEventDestroy(e0);
    return fail(MMR_HIP_ERROR, "hipEventCreate failed");
  }
  int reps = 3;  // launches per measurement; raised after the first one so that a measurement spans ~0.5 ms
  auto time_plan = [&](DevicePlan* plan, float* ms) -> int {
    if (int rc = launch_plan(ctx, plan, ptrs, 1, false)) return rc;  // warm-up (and upload of its tables)
    MMR_HIP(hipEventRecord(e0, ctx->stream));
    for (int i = 0; i < reps; ++i)
      if (int rc = launch_plan(ctx, plan, ptrs, 1, false)) return rc;
    MMR_HIP(hipEventRecord(e1, ctx->stream));
    ctx->stats.host_blocking_syncs += 1;
    MMR_HIP(hipEventSynchronize(e1));
    MMR_HIP(hipEventElapsedTime(ms, e0, e1));
    *ms /= static_cast<float>(reps);
    return MMR_OK;
  };
  float best_ms = 0;
  int64_t timed = 0;
  int rc = time_plan(dp, &best_ms);
  if (rc == MMR_OK && best_ms > 0 && best_ms * 3 < 0.5f) {  // short kernels: average over more launches
    reps = std::min(24, static_cast<int>(0.5f / best_ms) + 1);
    rc = time_plan(dp, &best_ms);
  }
  if (rc != MMR_OK) {  // the default plan itself does not run: report it
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return rc;
  }
  timed = 1;
  struct Candidate {
    uint32_t order, kib;
  };
  const Candidate candidates[] = {{4, 64}, {4, 512}, {4, 2048}, {4, 4096}, {2, 0}};
  std::unique_ptr<DevicePlan> best;
  for (const Candidate& cand : candidates) {
    if (cand.order == 2 && dp->plan.n_span_chunks == 0) continue;  // what a plan without span groups does by default
    mmr_plan_options o = base;
    o.order = cand.order;
    o.flags = (o.flags & 0xffu) | (cand.kib << 8);
    auto alt = std::make_unique<DevicePlan>();
    float ms = 0;
    // a candidate that fails to build or to run (out of memory, say) is skipped: the default stays valid
    int crc = make_device_plan(ctx, dp->plan.srcs, dp->plan.dsts, o, true, alt.get());
    if (crc == MMR_OK) crc = time_plan(alt.get(), &ms);
    if (crc == MMR_OK) {
      timed += 1;
      if (ms < 0.98f * best_ms) {  // only a clear win replaces the default
        if (best) drop_bindings_of_plan(ctx, best.get());
        best_ms = ms;
        best = std::move(alt);
        continue;
      }
    } else {
      (void)hipGetLastError();
    }
    drop_bindings_of_plan(ctx, alt.get());
  }
  if (best) {
    // Two more paired measurements must confirm the win (three wins in all), the challenger measured first in one
    // pair and second in the other so that a drift of the clocks favours neither side.
    for (int round = 0; round < 2 && best; ++round) {
      float again_default = 0, again_best = 0;
      DevicePlan* first = round == 0 ? dp : best.get();
      DevicePlan* second = round == 0 ? best.get() : dp;
      float first_ms = 0, second_ms = 0;
      const bool ran = time_plan(first, &first_ms) == MMR_OK && time_plan(second, &second_ms) == MMR_OK;
      again_default = round == 0 ? first_ms : second_ms;
      again_best = round == 0 ? second_ms : first_ms;
      if (!ran || !(again_best < 0.98f * again_default)) {
        (void)hipGetLastError();
        drop_bindings_of_plan(ctx, best.get());
        best.reset();
      }
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (best) {  // the winner takes the default's place in the cache
    drop_bindings_of_plan(ctx, dp);
    drop_bindings_of_plan(ctx, best.get());
    best->plan.stats.order_used = best->plan.options.order;
    best->plan.options = base;  // still the plan of the context's options
    ctx->plans[key] = std::move(best);
    dp = ctx->plans[key].get();
  }
  dp->plan.stats.orders_timed = timed;
  if (order_used) *order_used = dp->plan.stats.order_used;
  return MMR_OK;
}

// Who used a GPU's static scratch array last, in this process, and the event its kernels are done at.
struct StaticArrayUser {
  std::mutex mu;
  mmr_context* last = nullptr;
  hipEvent_t done = nullptr;
};

StaticArrayUser& static_array_user(int device) {
  static StaticArrayUser users[64];
  return users[device & 63];
}

// mmr_reshard_batch_static: the same argument checks, plan and kernels as reshard_locked, but every table of the
// launch goes into this GPU's static scratch array (pinned staging -> one stream-ordered copy) and nothing is
// allocated on the device.
int reshard_static_locked(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int n) {
  if (n == 0) return MMR_OK;
  if (int rc = use_device(ctx)) return rc;
  // Captured, the copy into the array would be replayed from a staging buffer and into an array that later calls
  // rewrite, with kernel arguments frozen for the tables of this call: refused like every entry point that copies
  // from host memory.
  if (int rc = refuse_capture(ctx, "mmr_reshard_batch_static")) return rc;
  if (int rc = check_batch(ctx, srcs, dsts, n)) return rc;
  std::vector<mmr_sharded_shape> sshapes, dshapes;
  shapes_of(srcs, dsts, n, &sshapes, &dshapes);
  // host-side plans of their own (a cached DevicePlan may hold device tables; this path may not create any)
  std::string key = "static:" + mmr::plan_key(sshapes.data(), dshapes.data(), n, ctx->options);
  auto it = ctx->plans.find(key);
  if (it == ctx->plans.end()) {
    auto dp = std::make_unique<DevicePlan>();
    if (int rc = make_device_plan(ctx, sshapes, dshapes, ctx->options, /*device_tables=*/false, dp.get())) return rc;
    it = ctx->plans.emplace(key, std::move(dp)).first;
    ctx->plan_lru.push_back(key);
    ctx->stats.plans_cached = static_cast<int64_t>(ctx->plans.size());
  }
  const DevicePlan& dp = *it->second;
  const BlockLayout l = layout_block(dp, /*with_chunk_tables=*/true);
  if (l.total > MMR_STATIC_SCRATCH_BYTES)
    return fail(MMR_INVALID_ARGUMENT,
                "the tables of this reshard take %zu bytes, the static scratch array holds %u: use mmr_reshard_batch", l.total,
                static_cast<unsigned>(MMR_STATIC_SCRATCH_BYTES));
  if (ctx->static_copy_pending) {  // the staging buffer is free again once the previous call's copy has read it
    if (hipEventQuery(ctx->static_copied) != hipSuccess) {
      ctx->stats.host_blocking_syncs += 1;
      MMR_HIP(hipEventSynchronize(ctx->static_copied));
    }
    ctx->static_copy_pending = false;
  }
  std::vector<void*> ptrs;
  collect_ptrs(dp.plan, srcs, dsts, n, &ptrs);
  fill_block(dp, l, ptrs, true, ctx->static_staging);
  // The array is one per GPU and process: if another context's kernels were the last to read it, this stream waits
  // for them on the device (no host wait).  Calls of one context are ordered by its stream anyway.
  StaticArrayUser& user = static_array_user(ctx->device);
  std::lock_guard<std::mutex> array_lock(user.mu);
  if (user.last && user.last != ctx) MMR_HIP(hipStreamWaitEvent(ctx->stream, user.done, 0));
  // stream-ordered: the copy waits for the kernels of the previous call on this stream, which still read the array
  MMR_HIP(hipMemcpyAsync(ctx->static_scratch, ctx->static_staging, l.total, hipMemcpyHostToDevice, ctx->stream));
  MMR_HIP(hipEventRecord(ctx->static_copied, ctx->stream));
  ctx->static_copy_pending = true;
  ctx->stats.reshard_calls += 1;
  const char* base = ctx->static_scratch;
  int rc = launch_block(ctx, dp, base, l, reinterpret_cast<const mmr_copy_chunk*>(base + l.generic),
                        reinterpret_cast<const mmr_transpose_chunk*>(base + l.transposes), true, true);
  // recorded even after a failed launch: what did get queued still reads the array
  const hipError_t e = hipEventRecord(ctx->static_done, ctx->stream);
  user.last = ctx;
  user.done = ctx->static_done;
  if (rc != MMR_OK) return rc;
  if (e != hipSuccess) return fail(MMR_HIP_ERROR, "hipEventRecord failed: %s", hipGetErrorString(e));
  ctx->stats.kernel_launches += launches_of(&dp);
  return MMR_OK;
}

struct CallbackTicket {
  mmr_context* ctx;
  PendingCallback cb;
};

// Host function on the stream: the work before it is done; hands the callback to the context's own thread.
void callback_ready(void* p) {
  std::unique_ptr<CallbackTicket> t(static_cast<CallbackTicket*>(p));
  {
    std::lock_guard<std::mutex> lock(t->ctx->callback_mu);
    t->ctx->callbacks.push_back(t->cb);
  }
  t->ctx->callback_cv.notify_all();
}

// The context's callback thread: runs callbacks in the order the stream released them.  They may call into the
// library (free stores, issue work); mmr_context_destroy is the one call they may not make.
void callback_loop(mmr_context* ctx) {
  std::unique_lock<std::mutex> lock(ctx->callback_mu);
  for (;;) {
    ctx->callback_cv.wait(lock, [&] { return ctx->callback_stop || !ctx->callbacks.empty(); });
    if (ctx->callbacks.empty()) return;  // stopping, nothing left
    PendingCallback cb = ctx->callbacks.front();
    ctx->callbacks.pop_front();
    lock.unlock();
    cb.fn(cb.arg);
    lock.lock();
    ctx->callbacks_done += 1;
    ctx->callback_cv.notify_all();
  }
}

// Reads the intervals whose stop event the device has reached (in stream order) into timer_results.  With
// `wait_for`, first waits until no interval of that name is left unread.
int resolve_timers(mmr_context* ctx, const char* wait_for) {
  if (wait_for) {
    hipEvent_t last = nullptr;
    for (const TimerInterval& t : ctx->resolving)
      if (t.name == wait_for) last = t.stop->event;
    if (last && hipEventQuery(last) != hipSuccess) {
      (void)hipGetLastError();
      if (int rc = blocking_wait(ctx, last)) return rc;
    }
  }
  while (!ctx->resolving.empty()) {
    TimerInterval& t = ctx->resolving.front();
    if (hipEventQuery(t.stop->event) != hipSuccess) {
      (void)hipGetLastError();
      break;
    }
    float ms = 0;
    if (t.start != t.stop) MMR_HIP(hipEventElapsedTime(&ms, t.start->event, t.stop->event));
    TimerResult& r = ctx->timer_results[t.name];
    r.last_ms = ms;
    r.completed += 1;
    ctx->stats.timers_resolved += 1;
    if (ctx->flags & MMR_LOG_TIMERS)  // "<name> finished in <s>s" (zuku_execute_context_impl.cc:478-482)
      std::fprintf(stderr, "%s finished in %gs\n", t.name.c_str(), static_cast<double>(ms) * 1e-3);
    release_point(ctx, t.start);
    release_point(ctx, t.stop);
    ctx->resolving.pop_front();
  }
  return MMR_OK;
}

int tile_index(const mmr_store* s, int64_t device, int64_t* k) {
  const int64_t rel = device - s->side.dev_start;
  if (rel < 0 || rel >= s->side.dev_count)
    return fail(MMR_NOT_FOUND, "device %lld holds no shard of store %lld (devices [%lld, +%lld))", (long long)device,
                (long long)s->id, (long long)s->side.dev_start, (long long)s->side.dev_count);
  *k = rel;
  return MMR_OK;
}

}  // namespace

extern "C" {

int mmr_context_create(int32_t hip_device, void* hip_stream, mmr_context** out) {
  if (!out) return fail(MMR_INVALID_ARGUMENT, "null output");
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0)
    return fail(MMR_HIP_ERROR, "no HIP device is available (%s); this library has no CPU fallback",
                e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
  if (hip_device < 0 || hip_device >= count) return fail(MMR_INVALID_ARGUMENT, "HIP device %d of %d", hip_device, count);
  // a failure part-way releases what was made so far
  struct Guard {
    mmr_context* ctx;
    ~Guard() {
      if (ctx) mmr_context_destroy(ctx);
    }
  } guard{new mmr_context()};
  mmr_context* ctx = guard.ctx;
  ctx->device = hip_device;
  MMR_HIP(hipSetDevice(hip_device));
  if (hip_stream) {
    ctx->stream = static_cast<hipStream_t>(hip_stream);
  } else {
    MMR_HIP(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking));  // default priority
    ctx->owns_stream = true;
  }
  MMR_HIP(hipEventCreateWithFlags(&ctx->t0, kTimingEventFlags));
  MMR_HIP(hipEventCreateWithFlags(&ctx->t1, kTimingEventFlags));
  MMR_HIP(hipHostMalloc(reinterpret_cast<void**>(&ctx->staging), kStagingBytes, hipHostMallocDefault));
  // set-up of the entry point that may not allocate: everything it needs exists from here on
  MMR_HIP(mmr::static_scratch_address(hip_device, reinterpret_cast<void**>(&ctx->static_scratch)));
  MMR_HIP(hipHostMalloc(reinterpret_cast<void**>(&ctx->static_staging), MMR_STATIC_SCRATCH_BYTES, hipHostMallocDefault));
  MMR_HIP(hipEventCreateWithFlags(&ctx->static_copied, hipEventDisableTiming));
  MMR_HIP(hipEventCreateWithFlags(&ctx->static_done, hipEventDisableTiming));
  (void)roctx();  // looked up once, outside any timed path
  guard.ctx = nullptr;
  *out = ctx;
  return MMR_OK;
}

void mmr_context_destroy(mmr_context* ctx) {
  if (!ctx) return;
  (void)hipSetDevice(ctx->device);
  if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
  // Every host function of the stream has run by now, so every callback is queued.  The thread ends once it has run
  // them all, including those that a callback queued in turn (run_after counts them before it returns).
  if (ctx->callback_thread.joinable()) {
    {
      std::unique_lock<std::mutex> lock(ctx->callback_mu);
      ctx->callback_cv.wait(lock, [&] { return ctx->callbacks_done >= ctx->callbacks_queued; });
      ctx->callback_stop = true;
    }
    ctx->callback_cv.notify_all();
    ctx->callback_thread.join();
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);  // work the last callbacks queued
  }
  for (auto& b : ctx->bindings) give_block(ctx, b->d_block, b->capacity);
  ctx->bindings.clear();
  ctx->binding_index.clear();
  ctx->plans.clear();  // their device tables go to the block pool ...
  for (auto& c : ctx->block_pool)
    for (char* b : c.second) (void)hipFree(b);  // ... which is released here
  for (auto& s : ctx->stores) {
    (void)hipFree(s.second->base);
    if (s.second->host) (void)hipHostFree(s.second->host);
  }
  for (auto& c : ctx->buffer_cache)
    for (auto& b : c.second) (void)hipFree(b.base);
  for (auto& c : ctx->free_pool)
    for (char* b : c.second) (void)hipFree(b);
  for (auto& c : ctx->host_cache)
    for (auto& b : c.second) (void)hipHostFree(b.base);
  if (ctx->t0) (void)hipEventDestroy(ctx->t0);
  if (ctx->t1) (void)hipEventDestroy(ctx->t1);
  for (hipEvent_t e : ctx->laps) (void)hipEventDestroy(e);
  for (auto& u : ctx->staged) (void)hipEventDestroy(u.consumed);
  for (auto& t : ctx->pending_timers) release_point(ctx, t.second);
  for (auto& t : ctx->resolving) {
    release_point(ctx, t.start);
    release_point(ctx, t.stop);
  }
  for (StreamPoint* p : ctx->window_markers) release_point(ctx, p);
  release_point(ctx, ctx->last_point);  // every point's event is back in the pool now
  for (hipEvent_t e : ctx->free_plain_events) (void)hipEventDestroy(e);
  for (hipEvent_t e : ctx->free_timing_events) (void)hipEventDestroy(e);
  {  // the stream is idle: whoever uses the static array next has nothing of this context to wait for
    StaticArrayUser& user = static_array_user(ctx->device);
    std::lock_guard<std::mutex> array_lock(user.mu);
    if (user.last == ctx) {
      user.last = nullptr;
      user.done = nullptr;
    }
  }
  if (ctx->static_copied) (void)hipEventDestroy(ctx->static_copied);
  if (ctx->static_done) (void)hipEventDestroy(ctx->static_done);
  if (ctx->static_staging) (void)hipHostFree(ctx->static_staging);
  if (ctx->staging) (void)hipHostFree(ctx->staging);
  if (ctx->owns_stream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

int mmr_context_stream(mmr_context* ctx, void** hip_stream) {
  if (!ctx || !hip_stream) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  ctx->stream_exposed = true;  // the caller may queue work the library does not see
  *hip_stream = ctx->stream;
  return MMR_OK;
}

int mmr_context_set_plan_options(mmr_context* ctx, const mmr_plan_options* options) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  ctx->options = options ? *options : mmr_plan_options{};  // part of every plan's cache key
  return MMR_OK;
}

int mmr_context_set_flags(mmr_context* ctx, uint32_t flags) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  ctx->flags = flags;
  return MMR_OK;
}

int mmr_context_clear_plans(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_context_clear_plans")) return rc;
  if (int rc = blocking_sync(ctx)) return rc;
  for (auto& b : ctx->bindings) give_block(ctx, b->d_block, b->capacity);
  ctx->bindings.clear();
  ctx->binding_index.clear();
  forget_last_plan(ctx);
  ctx->plans.clear();
  ctx->plan_lru.clear();
  for (auto& c : ctx->block_pool)  // the stream is idle: nothing reads the tables any more
    for (char* b : c.second) MMR_HIP(hipFree(b));
  ctx->block_pool.clear();
  ctx->stats.plans_cached = 0;
  ctx->stats.bindings_cached = 0;
  return MMR_OK;
}

int mmr_store_create_ex(mmr_context* ctx, const mmr_sharded_shape* shape, const char* name, uint32_t flags,
                        int64_t min_cache_size, mmr_store** out) {
  if (!ctx || !shape || !out) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  if (int rc = use_device(ctx)) return rc;
  auto s = std::make_unique<mmr_store>();
  if (int rc = mmr::make_side(*shape, &s->side)) return rc;
  s->shape = *shape;
  s->shape_key = mmr::descriptor_key(*shape);
  s->name = name ? name : "anonymous";  // zuku_execute_context_impl.cc:538-543
  s->owner = ctx;
  s->pitch = (static_cast<size_t>(std::max<int64_t>(s->side.shard_bytes, 1)) + kTileAlign - 1) / kTileAlign * kTileAlign;

  s->bytes = s->pitch * static_cast<size_t>(s->side.dev_count);
  s->replication = s->side.replication;
  s->replica_stride = s->side.replication > 1 ? s->side.dev_stride[s->side.ndims - 1] : 0;
  // Where the buffer comes from is decided first; anything that can fail (a capture in progress, an allocation, the
  // zero fill) either happens before a buffer is taken or gives it back.
  std::vector<CachedBuffer>* parked = (flags & MMR_STORE_FROM_CACHE) ? &ctx->buffer_cache[s->shape_key] : nullptr;
  const bool from_cache = parked && !parked->empty();
  auto pooled = ctx->free_pool.find(s->bytes);
  const bool from_pool = !from_cache && pooled != ctx->free_pool.end() && !pooled->second.empty();
  const bool fill = !from_cache && !(flags & MMR_STORE_UNINITIALIZED);
  const int64_t extra = (!from_cache && parked) ? std::max<int64_t>(min_cache_size, 1) - 1 : 0;
  if (!from_cache && !from_pool)
    if (int rc = refuse_capture(ctx, "creating a store that needs new device memory")) return rc;
  if (fill)
    if (int rc = refuse_capture(ctx, "zero-filling a new store")) return rc;
  if (extra > 0)
    if (int rc = refuse_capture(ctx, "filling a store cache")) return rc;
  if (from_cache) {
    s->base = parked->back().base;
    parked->pop_back();
    ctx->stats.cache_hits += 1;
  } else if (from_pool) {
    s->base = pooled->second.back();
    pooled->second.pop_back();
    ctx->free_pool_bytes -= s->bytes;
    ctx->stats.pool_hits += 1;
  } else {
    if (int rc = device_alloc(ctx, reinterpret_cast<void**>(&s->base), s->bytes)) return rc;
    account_alloc(ctx, static_cast<int64_t>(s->bytes));
  }
  // the buffer returns to the allocator's pool (it is accounted for either way) if the call fails from here on
  auto give_back = [&](int rc) {
    ctx->free_pool[s->bytes].push_back(s->base);
    ctx->free_pool_bytes += s->bytes;
    s->base = nullptr;
    return rc;
  };
  if (fill) {
    const hipError_t e = hipMemsetAsync(s->base, 0, s->bytes, ctx->stream);
    if (e != hipSuccess) return give_back(fail(MMR_HIP_ERROR, "hipMemsetAsync failed: %s", hipGetErrorString(e)));
  }
  // ArrayCache::Get(shape, min_cache_size): the cache of this descriptor holds at least that many buffers
  for (int64_t i = 0; i < extra; ++i) {
    char* more = nullptr;
    if (int rc = device_alloc(ctx, reinterpret_cast<void**>(&more), s->bytes)) return give_back(rc);
    account_alloc(ctx, static_cast<int64_t>(s->bytes));
    parked->push_back(CachedBuffer{more, s->bytes});  // owned by the cache from here on, whatever happens next
    if (!(flags & MMR_STORE_UNINITIALIZED)) {
      const hipError_t e = hipMemsetAsync(more, 0, s->bytes, ctx->stream);
      if (e != hipSuccess) return give_back(fail(MMR_HIP_ERROR, "hipMemsetAsync failed: %s", hipGetErrorString(e)));
    }
  }
  s->id = g_next_store_id.fetch_add(1);
  s->ordinal = ctx->next_ordinal++;
  hash_op(ctx, 1 /* CreateStore */, {static_cast<uint64_t>(s->ordinal)}, &s->shape_key);
  ctx->stats.stores_live += 1;
  *out = s.get();
  ctx->stores.emplace(s->id, std::move(s));
  return MMR_OK;
}

int mmr_store_create(mmr_context* ctx, const mmr_sharded_shape* shape, const char* name, uint32_t flags,
                     mmr_store** out) {
  return mmr_store_create_ex(ctx, shape, name, flags, 1, out);
}

int mmr_store_free(mmr_context* ctx, mmr_store* store, int32_t keep_in_cache) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = check_store(ctx, store, "freed")) return rc;
  if (int rc = use_device(ctx)) return rc;
  hash_op(ctx, 3 /* Free */, {static_cast<uint64_t>(store->ordinal), static_cast<uint64_t>(keep_in_cache != 0)});
  if (store->host) {
    // the pinned buffer goes back to the host cache (a copy still in flight on the stream is ordered before its next use)
    ctx->host_cache[store->shape_key].push_back(CachedBuffer{store->host, store->bytes});
  } else if (!store->adopted.empty()) {
    // caller-owned buffers: in-flight work on them must finish before the caller may reuse them
    if (int rc = refuse_capture(ctx, "freeing a store of adopted buffers")) return rc;
    if (int rc = blocking_sync(ctx)) return rc;
  } else if (keep_in_cache) {
    ctx->buffer_cache[store->shape_key].push_back(CachedBuffer{store->base, store->bytes});
  } else if (ctx->free_pool_bytes + store->bytes <= kFreePoolLimit) {
    ctx->free_pool[store->bytes].push_back(store->base);  // back to the allocator's pool: no device-wide wait
    ctx->free_pool_bytes += store->bytes;
  } else {
    if (int rc = refuse_capture(ctx, "freeing device memory")) return rc;
    MMR_HIP(hipFree(store->base));  // waits for the device
    ctx->stats.host_blocking_syncs += 1;
    ctx->stats.bytes_allocated -= static_cast<int64_t>(store->bytes);
  }
  ctx->stats.stores_live -= 1;
  ctx->stores.erase(store->id);
  return MMR_OK;
}

int mmr_clear_store_cache(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_clear_store_cache")) return rc;
  // a buffer leaves its list before it is freed, so a failure part-way leaves the lists true
  bool freed = false;
  for (auto& c : ctx->buffer_cache)
    while (!c.second.empty()) {
      const CachedBuffer b = c.second.back();
      c.second.pop_back();
      MMR_HIP(hipFree(b.base));  // waits for the device
      ctx->stats.bytes_allocated -= static_cast<int64_t>(b.bytes);
      freed = true;
    }
  ctx->buffer_cache.clear();
  for (auto& c : ctx->free_pool)
    while (!c.second.empty()) {
      char* b = c.second.back();
      c.second.pop_back();
      ctx->free_pool_bytes -= c.first;
      MMR_HIP(hipFree(b));
      ctx->stats.bytes_allocated -= static_cast<int64_t>(c.first);
      freed = true;
    }
  ctx->free_pool.clear();
  if (freed) ctx->stats.host_blocking_syncs += 1;
  bool any_host = false;
  for (auto& c : ctx->host_cache) any_host |= !c.second.empty();
  if (any_host)
    if (int rc = blocking_sync(ctx)) return rc;  // a reload may still be reading one of them
  for (auto& c : ctx->host_cache) {
    for (auto& b : c.second) {
      MMR_HIP(hipHostFree(b.base));
      ctx->stats.host_bytes_allocated -= static_cast<int64_t>(b.bytes);
    }
  }
  ctx->host_cache.clear();
  return MMR_OK;
}

int mmr_store_assemble(mmr_context* ctx, mmr_store* store, int64_t device, const void* data, size_t size,
                       int32_t data_on_device) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  if (int rc = check_store(ctx, store, "assembled")) return rc;
  int64_t k = 0;
  if (int rc = tile_index(store, device, &k)) return rc;
  if (size > static_cast<size_t>(store->side.shard_bytes))
    return fail(MMR_INVALID_ARGUMENT, "shard of %zu bytes does not fit the %lld-byte buffer of store %lld", size,
                (long long)store->side.shard_bytes, (long long)store->id);
  hash_op(ctx, 4 /* AssembleShards */, {static_cast<uint64_t>(store->ordinal), static_cast<uint64_t>(device), size});
  if (size == 0) return MMR_OK;
  if (!data) return fail(MMR_INVALID_ARGUMENT, "null shard data");
  if (int rc = use_device(ctx)) return rc;
  // one flat copy of the shard's bytes, as AssembleShardsImpl does
  // (zuku_execute_context_impl.cc:405-415)
  const bool runtime_copy = data_on_device == 3;  // a device pointer, copied by the runtime's own kernel
  if (runtime_copy) data_on_device = 1;
  const hipMemcpyKind kind = data_on_device == 1   ? hipMemcpyDeviceToDevice
                             : data_on_device == 0 ? hipMemcpyHostToDevice
                                                   : hipMemcpyDefault;  // the runtime looks the pointer up
  if (store->offloaded()) return fail(MMR_INVALID_ARGUMENT, "store %lld is offloaded to host memory", (long long)store->id);
  if (data_on_device == 2) {  // ask the runtime where the pointer lives: a device-resident shard needs no host wait
    hipPointerAttribute_t attr{};
    if (hipPointerGetAttributes(&attr, data) == hipSuccess) {
      if (attr.type == hipMemoryTypeDevice && attr.device == ctx->device) data_on_device = 1;
    } else {
      (void)hipGetLastError();  // plain host memory is unknown to the runtime: not an error here
    }
  }
  // a large device-resident shard goes through the library's own copy kernel (6.4 TB/s against 5.3 TB/s for the
  // runtime's device-to-device copy on MI355X); anything else through the runtime
  const uintptr_t bits = reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(store->tile(k));
  if (data_on_device == 1 && !runtime_copy && size >= (1u << 20) && (bits & 15u) == 0) {
    const size_t body = size & ~static_cast<size_t>(15);
    MMR_HIP(mmr::launch_flat_copy(data, store->tile(k), body, ctx->stream));
    ctx->stats.kernel_launches += 1;
    if (size > body)
      MMR_HIP(hipMemcpyAsync(static_cast<char*>(store->tile(k)) + body, static_cast<const char*>(data) + body, size - body,
                             hipMemcpyDeviceToDevice, ctx->stream));
    return MMR_OK;
  }
  if (data_on_device != 1)
    if (int rc = refuse_capture(ctx, "assembling a shard from host memory")) return rc;
  MMR_HIP(hipMemcpyAsync(store->tile(k), data, size, kind, ctx->stream));
  if (data_on_device != 1)
    if (int rc = blocking_sync(ctx)) return rc;  // host data is consumed before returning
  return MMR_OK;
}

int mmr_store_shard_ptr_async(mmr_context* ctx, mmr_store* store, int64_t device, void** ptr) {
  if (!ctx || !ptr) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = check_store(ctx, store, "sliced")) return rc;
  int64_t k = 0;
  if (int rc = tile_index(store, device, &k)) return rc;
  if (store->offloaded()) return fail(MMR_INVALID_ARGUMENT, "store %lld is offloaded to host memory", (long long)store->id);
  *ptr = store->tile(k);
  return MMR_OK;
}

int mmr_store_shard_ptr(mmr_context* ctx, mmr_store* store, int64_t device, void** ptr) {
  if (int rc = mmr_store_shard_ptr_async(ctx, store, device, ptr)) return rc;
  return mmr_sync(ctx);
}

int mmr_store_read_shard(mmr_context* ctx, mmr_store* store, int64_t device, void* host_dst, size_t size) {
  if (!ctx || !host_dst) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  if (int rc = check_store(ctx, store, "read")) return rc;
  int64_t k = 0;
  if (int rc = tile_index(store, device, &k)) return rc;
  if (size > static_cast<size_t>(store->side.shard_bytes))
    return fail(MMR_INVALID_ARGUMENT, "read of %zu bytes exceeds the %lld-byte shard", size,
                (long long)store->side.shard_bytes);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "reading a shard back")) return rc;
  if (store->offloaded()) {
    if (int rc = blocking_sync(ctx)) return rc;  // the copy to the pinned buffer is done after this
    std::memcpy(host_dst, store->host + store->slot(k) * store->pitch, size);
    return MMR_OK;
  }
  if (size) MMR_HIP(hipMemcpyAsync(host_dst, store->tile(k), size, hipMemcpyDeviceToHost, ctx->stream));
  return blocking_sync(ctx);
}

int mmr_store_has_shard(const mmr_store* store, int64_t device, int32_t* out) {
  if (!store || !out) return fail(MMR_INVALID_ARGUMENT, "null argument");
  const int64_t rel = device - store->side.dev_start;
  *out = rel >= 0 && rel < store->side.dev_count;
  return MMR_OK;
}

int mmr_store_get_shape(const mmr_store* store, mmr_sharded_shape* out) {
  if (!store || !out) return fail(MMR_INVALID_ARGUMENT, "null argument");
  *out = store->shape;
  return MMR_OK;
}

int64_t mmr_store_id(const mmr_store* store) { return store ? store->id : -1; }

int mmr_store_adopt(mmr_context* ctx, const mmr_sharded_shape* shape, const char* name, void* const* device_ptrs,
                    mmr_store** out) {
  if (!ctx || !shape || !out || !device_ptrs) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  auto s = std::make_unique<mmr_store>();
  if (int rc = mmr::make_side(*shape, &s->side)) return rc;
  for (int64_t k = 0; k < s->side.dev_count; ++k) {
    if (!device_ptrs[k] && s->side.shard_bytes > 0) return fail(MMR_INVALID_ARGUMENT, "buffer of device %lld is null", (long long)(s->side.dev_start + k));
    if (reinterpret_cast<uintptr_t>(device_ptrs[k]) % 16)
      return fail(MMR_INVALID_ARGUMENT, "buffer of device %lld is not 16-byte aligned", (long long)(s->side.dev_start + k));
    s->adopted.push_back(static_cast<char*>(device_ptrs[k]));
  }
  s->shape = *shape;
  s->shape_key = mmr::descriptor_key(*shape);
  s->name = name ? name : "anonymous";
  s->owner = ctx;
  s->pitch = static_cast<size_t>(s->side.shard_bytes);
  s->bytes = 0;
  s->id = g_next_store_id.fetch_add(1);
  s->ordinal = ctx->next_ordinal++;
  hash_op(ctx, 5 /* adopt */, {static_cast<uint64_t>(s->ordinal)}, &s->shape_key);
  ctx->stats.stores_live += 1;
  *out = s.get();
  ctx->stores.emplace(s->id, std::move(s));
  return MMR_OK;
}

int mmr_store_offload(mmr_context* ctx, mmr_store* store) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  if (int rc = check_store(ctx, store, "offloaded")) return rc;
  if (store->offloaded()) return MMR_OK;
  if (!store->adopted.empty()) return fail(MMR_INVALID_ARGUMENT, "store %lld lives in caller-owned buffers", (long long)store->id);
  if (int rc = use_device(ctx)) return rc;
  hash_op(ctx, 6 /* OffloadDtoH */, {static_cast<uint64_t>(store->ordinal)});
  // a pinned buffer from the host cache of this descriptor, else a new one (allocated pinned, never registered
  // after the fact)
  std::vector<CachedBuffer>& pool = ctx->host_cache[store->shape_key];
  char* host = nullptr;
  if (!pool.empty()) {
    host = pool.back().base;
    pool.pop_back();
    ctx->stats.host_cache_hits += 1;
  } else {
    if (int rc = refuse_capture(ctx, "offloading a store that needs a new pinned buffer")) return rc;
    MMR_HIP(hipHostMalloc(reinterpret_cast<void**>(&host), store->bytes, hipHostMallocDefault));
    ctx->stats.host_bytes_allocated += static_cast<int64_t>(store->bytes);
    ctx->stats.host_bytes_high_watermark = std::max(ctx->stats.host_bytes_high_watermark, ctx->stats.host_bytes_allocated);
  }
  // ordered on the stream behind whatever produced the store (the `pipelined` stores of OffloadDtoH included); the
  // device buffer goes to the device cache at once: its next user is ordered on the same stream behind this copy
  const hipError_t e = hipMemcpyAsync(host, store->base, store->bytes, hipMemcpyDeviceToHost, ctx->stream);
  if (e != hipSuccess) {  // the store stays on the device; the pinned buffer is kept for the next offload
    pool.push_back(CachedBuffer{host, store->bytes});
    return fail(MMR_HIP_ERROR, "copy of store %lld to host memory failed: %s", (long long)store->id, hipGetErrorString(e));
  }
  store->host = host;
  ctx->buffer_cache[store->shape_key].push_back(CachedBuffer{store->base, store->bytes});
  store->base = nullptr;
  return MMR_OK;
}

int mmr_store_reload(mmr_context* ctx, mmr_store* store) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  if (int rc = check_store(ctx, store, "reloaded")) return rc;
  if (!store->offloaded()) return MMR_OK;
  if (int rc = use_device(ctx)) return rc;
  hash_op(ctx, 7 /* OffloadHtoD */, {static_cast<uint64_t>(store->ordinal)});
  std::vector<CachedBuffer>& parked = ctx->buffer_cache[store->shape_key];
  char* base = nullptr;
  if (!parked.empty()) {
    base = parked.back().base;
    parked.pop_back();
    ctx->stats.cache_hits += 1;
  } else {
    if (int rc = refuse_capture(ctx, "reloading a store that needs new device memory")) return rc;
    if (int rc = device_alloc(ctx, reinterpret_cast<void**>(&base), store->bytes)) return rc;
    account_alloc(ctx, static_cast<int64_t>(store->bytes));
  }
  const hipError_t e = hipMemcpyAsync(base, store->host, store->bytes, hipMemcpyHostToDevice, ctx->stream);
  if (e != hipSuccess) {  // the store stays offloaded; the device buffer is kept for the next reload
    parked.push_back(CachedBuffer{base, store->bytes});
    return fail(MMR_HIP_ERROR, "copy of store %lld back to the device failed: %s", (long long)store->id, hipGetErrorString(e));
  }
  store->base = base;
  // the pinned buffer goes to the host cache at once: the next offload into it is ordered behind this copy
  ctx->host_cache[store->shape_key].push_back(CachedBuffer{store->host, store->bytes});
  store->host = nullptr;
  return MMR_OK;
}

int mmr_store_is_offloaded(const mmr_store* store, int32_t* out) {
  if (!store || !out) return fail(MMR_INVALID_ARGUMENT, "null argument");
  *out = store->offloaded();
  return MMR_OK;
}

int mmr_context_prepare(mmr_context* ctx, const mmr_sharded_shape* srcs, const mmr_sharded_shape* dsts, int32_t n) {
  if (!ctx || n < 0 || (n > 0 && (!srcs || !dsts))) return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  if (n == 0) return MMR_OK;
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  if (int rc = use_device(ctx)) return rc;
  std::vector<mmr_sharded_shape> s(srcs, srcs + n), d(dsts, dsts + n);
  DevicePlan* dp = nullptr;
  return get_plan(ctx, s, d, &dp);
}

int mmr_context_wait_event(mmr_context* ctx, void* hip_event) {
  if (!ctx || !hip_event) return fail(MMR_INVALID_ARGUMENT, "null argument");
  note_work(ctx);
  MMR_HIP(hipStreamWaitEvent(ctx->stream, static_cast<hipEvent_t>(hip_event), 0));
  return MMR_OK;
}

int mmr_context_record_event(mmr_context* ctx, void* hip_event) {
  if (!ctx || !hip_event) return fail(MMR_INVALID_ARGUMENT, "null argument");
  MMR_HIP(hipEventRecord(static_cast<hipEvent_t>(hip_event), ctx->stream));
  return MMR_OK;
}

int mmr_reshard(mmr_context* ctx, mmr_store* src, mmr_store* dst) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  return reshard_locked(ctx, &src, &dst, 1);
}

int mmr_reshard_batch(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n) {
  if (!ctx || n < 0 || (n > 0 && (!srcs || !dsts))) return fail(MMR_INVALID_ARGUMENT, "bad batch arguments");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  return reshard_locked(ctx, srcs, dsts, n);
}

int mmr_reshard_batch_static(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n) {
  if (!ctx || n < 0 || (n > 0 && (!srcs || !dsts))) return fail(MMR_INVALID_ARGUMENT, "bad batch arguments");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  return reshard_static_locked(ctx, srcs, dsts, n);
}

int mmr_reshard_tune(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n, int64_t* order_used) {
  if (!ctx || n <= 0 || !srcs || !dsts) return fail(MMR_INVALID_ARGUMENT, "bad batch arguments");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  return tune_locked(ctx, srcs, dsts, n, order_used);
}

int mmr_reshard_validate(mmr_context* ctx, mmr_store* src, mmr_store* dst) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = check_store(ctx, src, "source")) return rc;
  if (int rc = check_store(ctx, dst, "destination")) return rc;
  if (src == dst) return fail(MMR_INVALID_ARGUMENT, "source and destination are the same store");
  if (src->offloaded() || dst->offloaded())
    return fail(MMR_INVALID_ARGUMENT, "store %lld is still offloaded to host memory",
                (long long)(src->offloaded() ? src->id : dst->id));
  const mmr::Side& S = src->side;
  const mmr::Side& D = dst->side;
  if (S.dtype != D.dtype)
    return fail(MMR_INVALID_ARGUMENT, "source type %d differs from destination type %d", S.dtype, D.dtype);
  if (S.rank != D.rank) return fail(MMR_INVALID_ARGUMENT, "source rank %d differs from destination rank %d", S.rank, D.rank);
  for (int i = 0; i < S.rank; ++i)
    if (S.size[i] != D.size[i])
      return fail(MMR_INVALID_ARGUMENT, "dim %d is %lld in the source and %lld in the destination", i,
                  (long long)S.size[i], (long long)D.size[i]);
  return MMR_OK;
}

int mmr_reshard_bind(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n) {
  if (!ctx || n < 0 || (n > 0 && (!srcs || !dsts))) return fail(MMR_INVALID_ARGUMENT, "bad batch arguments");
  std::lock_guard<std::mutex> lock(ctx->mu);
  note_work(ctx);
  return reshard_locked(ctx, srcs, dsts, n, /*launch=*/false);
}

int mmr_context_run_after(mmr_context* ctx, void (*fn)(void*), void* arg) {
  if (!ctx || !fn) return fail(MMR_INVALID_ARGUMENT, "null argument");
  MMR_HIP(hipSetDevice(ctx->device));
  note_work(ctx);
  {
    std::lock_guard<std::mutex> lock(ctx->callback_mu);
    if (!ctx->callback_thread.joinable()) ctx->callback_thread = std::thread(callback_loop, ctx);
    ctx->callbacks_queued += 1;
  }
  // The stream's host function runs on a thread of the HIP runtime, where no HIP call is allowed and where a lock
  // of this library could be held by a thread that waits for this very stream: it only passes fn on.
  auto* boxed = new CallbackTicket{ctx, {fn, arg}};
  const hipError_t e = hipLaunchHostFunc(ctx->stream, callback_ready, boxed);
  if (e != hipSuccess) {
    delete boxed;
    std::lock_guard<std::mutex> lock(ctx->callback_mu);
    ctx->callbacks_queued -= 1;
    return fail(MMR_HIP_ERROR, "hipLaunchHostFunc failed: %s", hipGetErrorString(e));
  }
  return MMR_OK;
}

int mmr_sync(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  MMR_HIP(hipSetDevice(ctx->device));
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    ctx->stats.host_blocking_syncs += 1;
  }
  MMR_HIP(hipStreamSynchronize(ctx->stream));
  // ... and until the callbacks whose turn has come have run (not when called from one of them)
  std::unique_lock<std::mutex> lock(ctx->callback_mu);
  if (ctx->callback_thread.joinable() && std::this_thread::get_id() != ctx->callback_thread.get_id()) {
    const int64_t target = ctx->callbacks_queued;
    ctx->callback_cv.wait(lock, [&] { return ctx->callbacks_done >= target; });
  }
  return MMR_OK;
}

int mmr_timer_start(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  MMR_HIP(hipEventRecord(ctx->t0, ctx->stream));
  return MMR_OK;
}

int mmr_timer_stop_wait(mmr_context* ctx, float* milliseconds) {
  if (!ctx || !milliseconds) return fail(MMR_INVALID_ARGUMENT, "null argument");
  MMR_HIP(hipEventRecord(ctx->t1, ctx->stream));
  {
    std::lock_guard<std::mutex> lock(ctx->mu);
    ctx->stats.host_blocking_syncs += 1;
  }
  MMR_HIP(hipEventSynchronize(ctx->t1));
  MMR_HIP(hipEventElapsedTime(milliseconds, ctx->t0, ctx->t1));
  return MMR_OK;
}

int mmr_timer_lap(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (ctx->laps_used == ctx->laps.size()) {
    hipEvent_t e = nullptr;
    MMR_HIP(hipEventCreateWithFlags(&e, kTimingEventFlags));
    ctx->laps.push_back(e);
  }
  MMR_HIP(hipEventRecord(ctx->laps[ctx->laps_used], ctx->stream));
  ctx->laps_used += 1;
  return MMR_OK;
}

int mmr_timer_laps(mmr_context* ctx, float* milliseconds, int32_t capacity, int32_t* count) {
  if (!ctx || !count || (capacity > 0 && !milliseconds)) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  const size_t n = ctx->laps_used > 0 ? ctx->laps_used - 1 : 0;
  if (ctx->laps_used > 0)
    if (int rc = blocking_wait(ctx, ctx->laps[ctx->laps_used - 1])) return rc;
  *count = static_cast<int32_t>(std::min<size_t>(n, static_cast<size_t>(std::max(capacity, 0))));
  for (int32_t i = 0; i < *count; ++i) MMR_HIP(hipEventElapsedTime(&milliseconds[i], ctx->laps[i], ctx->laps[i + 1]));
  ctx->laps_used = 0;
  return MMR_OK;
}

int mmr_timer_begin(mmr_context* ctx, const char* name) {
  if (!ctx || !name) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_timer_begin")) return rc;
  if (int rc = resolve_timers(ctx, nullptr)) return rc;
  // pending_timers_.emplace(name, ...) (zuku_execute_context_impl.cc:466): a timer of that name already running stays
  if (ctx->pending_timers.count(name)) return MMR_OK;
  StreamPoint* start = nullptr;
  if (int rc = mark_point(ctx, &start)) return rc;
  ctx->pending_timers.emplace(name, start);
  return MMR_OK;
}

int mmr_timer_end(mmr_context* ctx, const char* name) {
  if (!ctx || !name) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_timer_end")) return rc;
  auto it = ctx->pending_timers.find(name);
  if (it == ctx->pending_timers.end())  // "cannot stop timer ..., does not exist": a warning in the reference (:471-474)
    return fail(MMR_NOT_FOUND, "cannot stop timer %s, does not exist", name);
  TimerInterval t;
  t.name = it->first;
  t.start = it->second;
  if (int rc = mark_point(ctx, &t.stop)) return rc;
  ctx->pending_timers.erase(it);
  ctx->resolving.push_back(std::move(t));
  return resolve_timers(ctx, nullptr);
}

int mmr_timer_poll(mmr_context* ctx, const char* name, float* last_milliseconds, int64_t* completed) {
  if (!ctx || !name) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = resolve_timers(ctx, nullptr)) return rc;
  auto it = ctx->timer_results.find(name);
  if (last_milliseconds) *last_milliseconds = it == ctx->timer_results.end() ? 0.0f : it->second.last_ms;
  if (completed) *completed = it == ctx->timer_results.end() ? 0 : it->second.completed;
  return MMR_OK;
}

int mmr_timer_wait(mmr_context* ctx, const char* name, float* last_milliseconds, int64_t* completed) {
  if (!ctx || !name) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_timer_wait")) return rc;
  if (int rc = resolve_timers(ctx, name)) return rc;
  auto it = ctx->timer_results.find(name);
  if (last_milliseconds) *last_milliseconds = it == ctx->timer_results.end() ? 0.0f : it->second.last_ms;
  if (completed) *completed = it == ctx->timer_results.end() ? 0 : it->second.completed;
  return MMR_OK;
}

int mmr_profile_mark(mmr_context* ctx, const char* name) {
  if (!ctx || !name) return fail(MMR_INVALID_ARGUMENT, "null argument");
  if (roctx().mark) roctx().mark(name);
  std::lock_guard<std::mutex> lock(ctx->mu);
  ctx->stats.profile_marks += 1;
  return MMR_OK;
}

int mmr_profile_range_push(mmr_context* ctx, const char* name) {
  if (!ctx || !name) return fail(MMR_INVALID_ARGUMENT, "null argument");
  if (roctx().push) roctx().push(name);
  return MMR_OK;
}

int mmr_profile_range_pop(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  if (roctx().pop) roctx().pop();
  return MMR_OK;
}

int mmr_profile_available(void) { return roctx().mark != nullptr; }

int mmr_window_open(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_window_open")) return rc;
  // windows the device has finished are no longer in flight
  while (!ctx->window_markers.empty() && hipEventQuery(ctx->window_markers.front()->event) == hipSuccess) {
    release_point(ctx, ctx->window_markers.front());
    ctx->window_markers.pop_front();
  }
  (void)hipGetLastError();  // hipErrorNotReady of the query that ended the loop
  // "we have to limit the maximum number of open windows" (zuku_execute_context_impl.cc:128-136): the caller waits
  // for the oldest window while max_open_windows are still running
  while (static_cast<int64_t>(ctx->window_markers.size()) >= ctx->max_open_windows) {
    StreamPoint* oldest = ctx->window_markers.front();
    ctx->window_markers.pop_front();
    ctx->stats.window_waits += 1;
    const int rc = blocking_wait(ctx, oldest->event);
    release_point(ctx, oldest);
    if (rc != MMR_OK) return rc;
  }
  ctx->stats.windows_opened += 1;
  return resolve_timers(ctx, nullptr);
}

int mmr_window_close(mmr_context* ctx) {
  if (!ctx) return fail(MMR_INVALID_ARGUMENT, "null context");
  std::lock_guard<std::mutex> lock(ctx->mu);
  if (int rc = use_device(ctx)) return rc;
  if (int rc = refuse_capture(ctx, "mmr_window_close")) return rc;
  StreamPoint* marker = nullptr;  // merge_events(last_execute_events_) (:139): everything queued so far
  if (int rc = mark_point(ctx, &marker)) return rc;
  ctx->window_markers.push_back(marker);
  return MMR_OK;
}

int mmr_context_set_max_open_windows(mmr_context* ctx, int32_t n) {
  if (!ctx || n < 1) return fail(MMR_INVALID_ARGUMENT, "at least one window must be allowed");
  std::lock_guard<std::mutex> lock(ctx->mu);
  ctx->max_open_windows = n;
  return MMR_OK;
}

int mmr_context_get_stats(mmr_context* ctx, mmr_context_stats* out) {
  if (!ctx || !out) return fail(MMR_INVALID_ARGUMENT, "null argument");
  std::lock_guard<std::mutex> lock(ctx->mu);
  *out = ctx->stats;
  return MMR_OK;
}

int mmr_reshard_batch_plan_stats(mmr_context* ctx, mmr_store* const* srcs, mmr_store* const* dsts, int32_t n,
                                 mmr_plan_stats* out) {
  if (!ctx || !out || n <= 0 || !srcs || !dsts) return fail(MMR_INVALID_ARGUMENT, "bad arguments");
  std::lock_guard<std::mutex> lock(ctx->mu);
  for (int a = 0; a < n; ++a) {
    if (int rc = check_store(ctx, srcs[a], "source")) return rc;
    if (int rc = check_store(ctx, dsts[a], "destination")) return rc;
  }
  std::vector<mmr_sharded_shape> s, d;
  shapes_of(srcs, dsts, n, &s, &d);
  if (int rc = use_device(ctx)) return rc;
  note_work(ctx);  // a plan built here uploads its tables
  DevicePlan* dp = nullptr;
  if (int rc = get_plan(ctx, s, d, &dp)) return rc;
  *out = dp->plan.stats;
  return MMR_OK;
}

int mmr_reshard_plan_stats(mmr_context* ctx, mmr_store* src, mmr_store* dst, mmr_plan_stats* out) {
  return mmr_reshard_batch_plan_stats(ctx, &src, &dst, 1, out);
}

}  // extern "C"
