/*
 * CPU restatement of the reference's reshard, in plain C.
 *
 * TEST INFRASTRUCTURE ONLY: the checker the GPU path is compared with and the
 * "cpu_baseline" leg of the benchmark.  The shipped library never links it.
 *
 * The reference hands two sharded arrays to a third-party runtime
 * (src/pjrt_client/zuku_execute_context_impl.cc:437-452 -> zuku::Reshard; zuku
 * 24.9.0 and its Realm copy engine are fetched at build time and are not in
 * the reference tree).  On CPU that runtime moves one contiguous run per
 * memcpy on a pool of DMA threads; this file restates exactly that: every
 * (source tile x destination tile) overlap becomes a box, a box becomes runs,
 * runs are spread over pthreads.
 *
 * Descriptor semantics follow how the reference fills zuku::ShardedShape
 * (src/pjrt_client/mm_sharding.cc:345-372, 427-431, 638-654):
 *   dims[i] = {size (global extent), sharding (#tiles), permutation (rank of
 *   the dim in device-id significance, 0 = most significant)}; an optional
 *   trailing {1, R} entry replicates; devices = [start, start + count).
 *   Tile extent = ceil(size / sharding) (spmd::MakePartitionedShape, call
 *   sites mm_sharding.cc:69, mm_pjrt_executable.cc:537).
 * Pinned against the NumPy oracle and single-element brute force in
 * tests/test_oracle.py.  Pad content (zero) and the per-shard layout
 * (minor_to_major) are not reference behaviour: parity unpinned for those.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_DIMS 9

typedef struct {
  int32_t itemsize;
  int32_t ndims; /* entries of size/sharding/permutation, replication dim included */
  int64_t size[ORC_MAX_DIMS];
  int64_t sharding[ORC_MAX_DIMS];
  int64_t permutation[ORC_MAX_DIMS];
  int64_t dev_start;
  int64_t dev_count;
  int32_t has_layout;
  int32_t minor_to_major[ORC_MAX_DIMS];
} orc_desc;

typedef struct {
  int rank;
  int64_t ext[ORC_MAX_DIMS];  /* box extent per logical dim (elements) */
  int64_t sstr[ORC_MAX_DIMS]; /* source stride per logical dim (elements) */
  int64_t dstr[ORC_MAX_DIMS];
  const char* src;
  char* dst;
  int run_dim;   /* dim contiguous on both sides, or -1 */
  int64_t rows;  /* number of memcpy calls this box needs */
} orc_box;

typedef struct {
  const orc_box* boxes;
  const int64_t* row_prefix;
  int nboxes;
  int64_t row_lo, row_hi;
  int itemsize;
} orc_job;

static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static int64_t min64(int64_t a, int64_t b) { return a < b ? a : b; }
static int64_t max64(int64_t a, int64_t b) { return a > b ? a : b; }

static int tensor_rank(const orc_desc* d) {
  int n = d->ndims;
  if (n > 0 && d->size[n - 1] == 1 && d->sharding[n - 1] > 1) return n - 1;
  return n;
}

/* stride of every descriptor dim inside the device id */
static int device_strides(const orc_desc* d, int64_t* st) {
  int64_t acc = 1;
  for (int rank = d->ndims - 1; rank >= 0; --rank) {
    int found = -1;
    for (int i = 0; i < d->ndims; ++i)
      if (d->permutation[i] == rank) found = i;
    if (found < 0) return -1;
    st[found] = acc;
    acc *= d->sharding[found];
  }
  return acc == d->dev_count ? 0 : -1;
}

/* element strides of a shard buffer per logical dim */
static void shard_strides(const orc_desc* d, int rank, const int64_t* tile_ext, int64_t* str) {
  int64_t acc = 1;
  for (int k = 0; k < rank; ++k) {
    int dim = d->has_layout ? d->minor_to_major[k] : rank - 1 - k;
    str[dim] = acc;
    acc *= tile_ext[dim];
  }
}

static void* worker(void* arg) {
  orc_job* job = (orc_job*)arg;
  int b = 0;
  for (int64_t row = job->row_lo; row < job->row_hi;) {
    while (b + 1 < job->nboxes && job->row_prefix[b + 1] <= row) ++b;
    const orc_box* bx = &job->boxes[b];
    int64_t local = row - job->row_prefix[b];
    int64_t local_end = min64(job->row_hi, job->row_prefix[b] + bx->rows) - job->row_prefix[b];
    for (; local < local_end; ++local, ++row) {
      /* row-major decomposition of `local` over the non-run dims */
      int64_t rem = local, so = 0, dof = 0;
      for (int i = bx->rank - 1; i >= 0; --i) {
        if (i == bx->run_dim) continue;
        int64_t idx = rem % bx->ext[i];
        rem /= bx->ext[i];
        so += idx * bx->sstr[i];
        dof += idx * bx->dstr[i];
      }
      if (bx->run_dim >= 0) {
        memcpy(bx->dst + dof * job->itemsize, bx->src + so * job->itemsize,
               (size_t)(bx->ext[bx->run_dim] * job->itemsize));
      } else {
        memcpy(bx->dst + dof * job->itemsize, bx->src + so * job->itemsize, (size_t)job->itemsize);
      }
    }
  }
  return NULL;
}

/*
 * src_bufs[k] / dst_bufs[k]: shard buffer of device dev_start + k.
 * Returns 0, or a negative code for an invalid descriptor pair.
 */
int orc_reshard(const orc_desc* src, const void* const* src_bufs, const orc_desc* dst,
                void* const* dst_bufs, int nthreads) {
  int rank = tensor_rank(src);
  if (rank != tensor_rank(dst) || src->itemsize != dst->itemsize) return -1;
  for (int i = 0; i < rank; ++i)
    if (src->size[i] != dst->size[i]) return -2;
  int64_t sdev[ORC_MAX_DIMS], ddev[ORC_MAX_DIMS];
  if (device_strides(src, sdev) || device_strides(dst, ddev)) return -3;

  int64_t sext[ORC_MAX_DIMS], dext[ORC_MAX_DIMS], sstr[ORC_MAX_DIMS], dstr[ORC_MAX_DIMS];
  int64_t dshard_elems = 1;
  for (int i = 0; i < rank; ++i) {
    sext[i] = ceil_div(src->size[i], src->sharding[i]);
    dext[i] = ceil_div(dst->size[i], dst->sharding[i]);
    dshard_elems *= dext[i];
  }
  shard_strides(src, rank, sext, sstr);
  shard_strides(dst, rank, dext, dstr);

  int cap = 64, nboxes = 0;
  orc_box* boxes = (orc_box*)malloc(sizeof(orc_box) * cap);

  for (int64_t dd = 0; dd < dst->dev_count; ++dd) {
    int64_t dcoord[ORC_MAX_DIMS], lo[ORC_MAX_DIMS], hi[ORC_MAX_DIMS];
    int padded = 0, empty = 0;
    for (int i = 0; i < dst->ndims; ++i) dcoord[i] = (dd / ddev[i]) % dst->sharding[i];
    for (int i = 0; i < rank; ++i) {
      lo[i] = min64(dcoord[i] * dext[i], dst->size[i]);
      hi[i] = min64(lo[i] + dext[i], dst->size[i]);
      if (hi[i] - lo[i] < dext[i]) padded = 1;
      if (hi[i] == lo[i]) empty = 1;
    }
    char* dbuf = (char*)dst_bufs[dd];
    if (padded) memset(dbuf, 0, (size_t)(dshard_elems * dst->itemsize));
    if (empty) continue;

    /* range of source tiles that overlap, per dim */
    int64_t t_lo[ORC_MAX_DIMS], t_n[ORC_MAX_DIMS], combos = 1;
    for (int i = 0; i < rank; ++i) {
      t_lo[i] = lo[i] / sext[i];
      t_n[i] = (hi[i] - 1) / sext[i] - t_lo[i] + 1;
      combos *= t_n[i];
    }
    for (int64_t c = 0; c < combos; ++c) {
      int64_t rem = c, sdevice = 0;
      orc_box bx;
      bx.rank = rank;
      int64_t soff = 0, doff = 0;
      for (int i = rank - 1; i >= 0; --i) {
        int64_t t = t_lo[i] + rem % t_n[i];
        rem /= t_n[i];
        int64_t s_lo = t * sext[i];
        int64_t b_lo = max64(lo[i], s_lo);
        int64_t b_hi = min64(hi[i], min64(s_lo + sext[i], src->size[i]));
        bx.ext[i] = b_hi - b_lo;
        bx.sstr[i] = sstr[i];
        bx.dstr[i] = dstr[i];
        soff += (b_lo - s_lo) * sstr[i];
        doff += (b_lo - lo[i]) * dstr[i];
        sdevice += t * sdev[i]; /* replica 0: the replication coordinate stays 0 */
      }
      bx.src = (const char*)src_bufs[sdevice] + soff * src->itemsize;
      bx.dst = dbuf + doff * dst->itemsize;
      bx.run_dim = -1;
      bx.rows = 1;
      for (int i = 0; i < rank; ++i)
        if (sstr[i] == 1 && dstr[i] == 1) bx.run_dim = i;
      for (int i = 0; i < rank; ++i)
        if (i != bx.run_dim) bx.rows *= bx.ext[i];
      if (nboxes == cap) {
        cap *= 2;
        boxes = (orc_box*)realloc(boxes, sizeof(orc_box) * cap);
      }
      boxes[nboxes++] = bx;
    }
  }

  int64_t* prefix = (int64_t*)malloc(sizeof(int64_t) * (nboxes + 1));
  prefix[0] = 0;
  for (int b = 0; b < nboxes; ++b) prefix[b + 1] = prefix[b] + boxes[b].rows;
  int64_t total = prefix[nboxes];

  if (nthreads < 1) nthreads = 1;
  if (nthreads > 256) nthreads = 256;
  orc_job jobs[256];
  pthread_t tids[256];
  for (int t = 0; t < nthreads; ++t) {
    jobs[t].boxes = boxes;
    jobs[t].row_prefix = prefix;
    jobs[t].nboxes = nboxes;
    jobs[t].row_lo = total * t / nthreads;
    jobs[t].row_hi = total * (t + 1) / nthreads;
    jobs[t].itemsize = src->itemsize;
  }
  if (nthreads == 1) {
    worker(&jobs[0]);
  } else {
    for (int t = 0; t < nthreads; ++t) pthread_create(&tids[t], NULL, worker, &jobs[t]);
    for (int t = 0; t < nthreads; ++t) pthread_join(tids[t], NULL);
  }
  free(prefix);
  free(boxes);
  return 0;
}
