// Context, caching allocator, upload/download, and the metadata-only view
// operations of the backend.  The view operations mirror what ox-arrays does
// with strides for the `Concrete` instance of horde-ad
// (src/HordeAd/Core/OpsConcrete.hs:243-246,641-652): no element is touched.
#include "common.hpp"

#include <hip/hiprtc.h>

#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <cerrno>
#include <cstdlib>
#include <fstream>

namespace hg {

int fail(hgpu_ctx* ctx, int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  if (ctx) {
    std::lock_guard<std::mutex> g(ctx->mu);
    ctx->err = buf;
  }
  return code;
}

int check_hip(hgpu_ctx* ctx, hipError_t e, const char* what) {
  if (e == hipSuccess) return HGPU_OK;
  return fail(ctx, e == hipErrorOutOfMemory ? HGPU_ERR_OOM : HGPU_ERR_DEVICE, "%s: %s", what,
              hipGetErrorString(e));
}

static size_t round_block(size_t bytes) {
  if (bytes < 256) return 256;
  if (bytes <= (1u << 20)) {  // powers of two up to 1 MiB
    size_t p = 256;
    while (p < bytes) p <<= 1;
    return p;
  }
  const size_t mib = 1u << 20;  // then multiples of 1 MiB
  return (bytes + mib - 1) / mib * mib;
}

static void drop_cache_locked(hgpu_ctx* ctx) {
  for (auto& kv : ctx->cache) {
    (void)hipFree(kv.second);
    ctx->reserved -= kv.first;
  }
  ctx->cache.clear();
}

// Every block has at least kSlack bytes behind the bytes asked for: kernels that
// move whole 16-byte vectors may read (never write) up to one vector past the
// last element of an array without leaving the block.
constexpr size_t kSlack = 16;

int buffer_alloc(hgpu_ctx* ctx, size_t bytes, hgpu_buffer** out) {
  size_t blk = round_block(bytes + kSlack);
  void* p = nullptr;
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    std::multimap<size_t, void*>& cache = ctx->cap ? ctx->cap->cache : ctx->cache;
    auto it = cache.find(blk);
    if (it != cache.end()) {
      p = it->second;
      cache.erase(it);
    } else {
      if (ctx->fail_after >= 0 && (int64_t)ctx->n_device_allocs >= ctx->fail_after) {
        ctx->err = "device allocation failed (injected)";
        return HGPU_ERR_OOM;
      }
      (void)hipSetDevice(ctx->device);
      hipError_t e = hipMalloc(&p, blk);
      if (e != hipSuccess && !ctx->cap) {
        (void)hipGetLastError();
        // Cached blocks may still be read by enqueued kernels: drain first.
        (void)hipStreamSynchronize(ctx->stream);
        drop_cache_locked(ctx);
        e = hipMalloc(&p, blk);
      }
      if (e != hipSuccess) {
        (void)hipGetLastError();
        char msg[160];
        snprintf(msg, sizeof msg, "device allocation of %zu bytes failed: %s", blk, hipGetErrorString(e));
        ctx->err = msg;
        return HGPU_ERR_OOM;
      }
      ctx->reserved += blk;
      ctx->n_device_allocs++;
    }
    ctx->in_use += blk;
  }
  hgpu_buffer* b = new hgpu_buffer;
  b->ctx = ctx;
  b->ptr = p;
  b->bytes = blk;
  b->refs.store(1);
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    b->pool = ctx->cap;
    if (b->pool) b->pool->refs++;
  }
  *out = b;
  return HGPU_OK;
}

void buffer_retain(hgpu_buffer* b) {
  if (b) b->refs.fetch_add(1);
}

void buffer_release(hgpu_buffer* b) {
  if (!b) return;
  if (b->refs.fetch_sub(1) == 1) {
    hgpu_ctx* ctx = b->ctx;
    {
      // The block goes back to the cache at once: all work that reads it is
      // already enqueued on the in-order stream, and whatever reuses it is
      // enqueued behind that work.
      std::lock_guard<std::mutex> g(ctx->mu);
      hgpu_cap_pool* pool = b->pool;
      if (pool && pool->alive) pool->cache.emplace(b->bytes, b->ptr);
      else ctx->cache.emplace(b->bytes, b->ptr);
      if (pool && --pool->refs == 0) delete pool;
      ctx->in_use -= b->bytes;
    }
    delete b;
  }
}

}  // namespace hg

namespace {
struct ArrayBlocks {
  struct Node { Node* next; };
  Node* head = nullptr;
  size_t n = 0;
  ~ArrayBlocks() {
    while (head) { Node* x = head; head = head->next; ::operator delete(x); }
  }
};
thread_local ArrayBlocks array_blocks;
constexpr size_t kArrayBlocksKept = 16384;
}  // namespace

void* hgpu_array::operator new(size_t n) {
  ArrayBlocks& ab = array_blocks;
  if (n == sizeof(hgpu_array) && ab.head) {
    ArrayBlocks::Node* x = ab.head;
    ab.head = x->next;
    --ab.n;
    return x;
  }
  return ::operator new(n < sizeof(hgpu_array) ? sizeof(hgpu_array) : n);
}
void hgpu_array::operator delete(void* p) {
  if (!p) return;
  ArrayBlocks& ab = array_blocks;
  if (ab.n >= kArrayBlocksKept) { ::operator delete(p); return; }
  auto* x = static_cast<ArrayBlocks::Node*>(p);
  x->next = ab.head;
  ab.head = x;
  ++ab.n;
}

namespace hg {
hgpu_array* new_view(hgpu_ctx* ctx, hgpu_buffer* buf, int dtype, int rank, const int64_t* shape,
                     const int64_t* strides, int64_t offset) {
  hgpu_array* a = new hgpu_array;
  a->ctx = ctx;
  a->refs.store(1);
  a->buf = buf;
  buffer_retain(buf);
  a->dtype = dtype;
  a->rank = rank;
  for (int i = 0; i < rank; ++i) {
    a->shape[i] = shape[i];
    a->strides[i] = strides[i];
  }
  a->offset = offset;
  return a;
}

int new_dense(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape, hgpu_array** out) {
  if (rank < 0 || rank > HGPU_MAX_RANK) return fail(ctx, HGPU_ERR_INVALID, "rank %d out of range", rank);
  int64_t n = 1;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] < 0) return fail(ctx, HGPU_ERR_INVALID, "negative extent");
    n *= shape[i];
  }
  int64_t st[HGPU_MAX_RANK];
  dense_strides(rank, shape, st);
  hgpu_buffer* buf = nullptr;
  if (n > 0) {
    int rc = buffer_alloc(ctx, (size_t)n * dtype_size(dtype), &buf);
    if (rc) return rc;
  }
  *out = new_view(ctx, buf, dtype, rank, shape, st, 0);
  buffer_release(buf);  // the view holds the only reference
  return HGPU_OK;
}

int new_zeros(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape, hgpu_array** out) {
  int rc = new_dense(ctx, dtype, rank, shape, out);
  if (rc) return rc;
  int64_t n = nelem(*out);
  if (n > 0) {
    // A fill kernel, not hipMemsetAsync: callers may capture the stream.
    rc = zero_fill(ctx, data_ptr(*out), (size_t)n * dtype_size(dtype));
    if (rc) {
      hgpu_release(*out);
      *out = nullptr;
      return rc;
    }
  }
  return HGPU_OK;
}

bool is_dense(const hgpu_array* a) {
  int64_t s = 1;
  for (int i = a->rank - 1; i >= 0; --i) {
    if (a->shape[i] != 1 && a->strides[i] != s) return false;
    s *= a->shape[i];
  }
  return true;
}

bool same_shape(const hgpu_array* a, const hgpu_array* b) {
  if (a->rank != b->rank) return false;
  for (int i = 0; i < a->rank; ++i)
    if (a->shape[i] != b->shape[i]) return false;
  return true;
}

bool collapse(int rank, const int64_t* shape, int nops, const int64_t* const* strides, Dims* out) {
  Dims d;
  d.nd = 0;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] == 1) continue;
    bool merged = false;
    if (d.nd > 0) {
      int p = d.nd - 1;
      bool ok = true;
      for (int k = 0; k < nops; ++k)
        if (d.st[k][p] != strides[k][i] * shape[i]) { ok = false; break; }
      if (ok) {
        d.shape[p] *= shape[i];
        for (int k = 0; k < nops; ++k) d.st[k][p] = strides[k][i];
        merged = true;
      }
    }
    if (!merged) {
      if (d.nd == HG_KDIMS) return false;
      d.shape[d.nd] = shape[i];
      for (int k = 0; k < nops; ++k) d.st[k][d.nd] = strides[k][i];
      d.nd++;
    }
  }
  if (d.nd == 0) {
    d.nd = 1;
    d.shape[0] = 1;
    for (int k = 0; k < nops; ++k) d.st[k][0] = 0;
  }
  for (int i = d.nd; i < HG_KDIMS; ++i) {
    d.shape[i] = 1;
    for (int k = 0; k < 4; ++k) d.st[k][i] = 0;
  }
  for (int k = nops; k < 4; ++k)
    for (int i = 0; i < HG_KDIMS; ++i) d.st[k][i] = 0;
  *out = d;
  return true;
}

static int ensure_staging(hgpu_ctx* ctx, size_t bytes) {
  if (ctx->staging_bytes >= bytes) return HGPU_OK;
  if (ctx->staging) (void)hipHostFree(ctx->staging);
  ctx->staging = nullptr;
  ctx->staging_bytes = 0;
  hipError_t e = hipHostMalloc(&ctx->staging, bytes, hipHostMallocDefault);
  if (e != hipSuccess) return check_hip(ctx, e, "hipHostMalloc");
  ctx->staging_bytes = bytes;
  return HGPU_OK;
}

}  // namespace hg

using namespace hg;

namespace hg {
int no_capture(hgpu_ctx* ctx, const char* what) {
  if (ctx->cap) return fail(ctx, HGPU_ERR_UNSUPPORTED, "%s: not while a graph is being captured (it needs the host)", what);
  return HGPU_OK;
}

int zero_block(hgpu_ctx* ctx, const void** out) {
  if (!ctx->zero_block) {
    hgpu_buffer* b = nullptr;
    int rc = buffer_alloc(ctx, 256, &b);
    if (rc) return rc;
    rc = zero_fill(ctx, b->ptr, 256);
    if (rc) { buffer_release(b); return rc; }
    ctx->zero_block = b;
  }
  *out = ctx->zero_block->ptr;
  return HGPU_OK;
}

int ticket_block(hgpu_ctx* ctx, void** out) {
  if (!ctx->ticket_block) {
    if (int rc0 = no_capture(ctx, "the first reduction that draws tickets")) return rc0;
    hgpu_buffer* b = nullptr;
    int rc = buffer_alloc(ctx, 4096, &b);
    if (rc) return rc;
    rc = zero_fill(ctx, b->ptr, 4096);
    if (rc) { buffer_release(b); return rc; }
    ctx->ticket_block = b;
  }
  *out = ctx->ticket_block->ptr;
  return HGPU_OK;
}
}  // namespace hg

extern "C" {

int hgpu_init(int device, hgpu_ctx** out) {
  if (!out) return HGPU_ERR_INVALID;
  *out = nullptr;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n) {
    (void)hipGetLastError();
    return HGPU_ERR_DEVICE;
  }
  if (hipSetDevice(device) != hipSuccess) return HGPU_ERR_DEVICE;
  hgpu_ctx* ctx = new hgpu_ctx;
  ctx->device = device;
  if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
    delete ctx;
    return HGPU_ERR_DEVICE;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) == hipSuccess) ctx->num_cu = prop.multiProcessorCount;
  const void* z = nullptr;
  (void)zero_block(ctx, &z);     // made now, so that no capture ever owns it
  void* tk = nullptr;
  (void)ticket_block(ctx, &tk);
  *out = ctx;
  return HGPU_OK;
}

// ---- graphs: one captured sequence of launches, replayed as a unit ---------

int hgpu_capture_begin(hgpu_ctx* ctx) {
  if (!ctx) return HGPU_ERR_INVALID;
  if (ctx->cap) return fail(ctx, HGPU_ERR_INVALID, "capture_begin: a capture is already open");
  (void)hipSetDevice(ctx->device);
  flush_deferred(ctx);
  hipError_t e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) return check_hip(ctx, e, "capture_begin");
  hgpu_cap_pool* pool = new hgpu_cap_pool;
  {
    // The warm blocks of the context move into the capture's pool: a capture
    // after a warm-up run allocates nothing.
    std::lock_guard<std::mutex> g(ctx->mu);
    pool->cache.swap(ctx->cache);
  }
  e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) {
    std::lock_guard<std::mutex> g(ctx->mu);
    ctx->cache.swap(pool->cache);
    delete pool;
    return check_hip(ctx, e, "hipStreamBeginCapture");
  }
  std::lock_guard<std::mutex> g(ctx->mu);
  ctx->cap = pool;
  return HGPU_OK;
}

static void retire_pool(hgpu_ctx* ctx, hgpu_cap_pool* pool) {
  std::lock_guard<std::mutex> g(ctx->mu);
  pool->alive = false;
  for (auto& kv : pool->cache) ctx->cache.emplace(kv.first, kv.second);
  pool->cache.clear();
  if (--pool->refs == 0) delete pool;
}

int hgpu_capture_end(hgpu_ctx* ctx, hgpu_graph** out) {
  if (!ctx || !out) return HGPU_ERR_INVALID;
  if (!ctx->cap) return fail(ctx, HGPU_ERR_INVALID, "capture_end: no capture is open");
  (void)hipSetDevice(ctx->device);
  flush_deferred(ctx);          // launches still held back belong to the graph
  int held_rc;
  {
    std::lock_guard<std::mutex> lk(ctx->launch_mu);
    held_rc = take_deferred_rc(ctx);
  }
  hgpu_cap_pool* pool;
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    pool = ctx->cap;
    ctx->cap = nullptr;
  }
  hgpu_graph* gr = new hgpu_graph;
  gr->ctx = ctx;
  gr->pool = pool;
  hipError_t e = hipStreamEndCapture(ctx->stream, &gr->graph);
  if (e == hipSuccess && !held_rc) e = hipGraphInstantiate(&gr->exec, gr->graph, nullptr, nullptr, 0);
  if (e != hipSuccess || held_rc) {
    (void)hipGetLastError();
    if (gr->graph) (void)hipGraphDestroy(gr->graph);
    retire_pool(ctx, pool);
    delete gr;
    return held_rc ? held_rc : check_hip(ctx, e, "capture_end");   // a recording that lacks a launch is no recording
  }
  *out = gr;
  return HGPU_OK;
}

int hgpu_graph_launch(hgpu_graph* gr) {
  if (!gr) return HGPU_ERR_INVALID;
  hgpu_ctx* ctx = gr->ctx;
  if (ctx->cap) return fail(ctx, HGPU_ERR_INVALID, "graph_launch: not inside a capture");
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  (void)hipSetDevice(ctx->device);
  if (ctx->dq_pending) flush_deferred_locked(ctx);
  if (int rc = take_deferred_rc(ctx)) return rc;
  return check_hip(ctx, hipGraphLaunch(gr->exec, ctx->stream), "hipGraphLaunch");
}

int hgpu_graph_destroy(hgpu_graph* gr) {
  if (!gr) return HGPU_ERR_INVALID;
  hgpu_ctx* ctx = gr->ctx;
  (void)hipSetDevice(ctx->device);
  flush_deferred(ctx);
  (void)hipStreamSynchronize(ctx->stream);     // a replay may still be running on the blocks
  if (gr->exec) (void)hipGraphExecDestroy(gr->exec);
  if (gr->graph) (void)hipGraphDestroy(gr->graph);
  retire_pool(ctx, gr->pool);
  delete gr;
  return HGPU_OK;
}

int hgpu_shutdown(hgpu_ctx* ctx) {
  if (!ctx) return HGPU_ERR_INVALID;
  (void)hipSetDevice(ctx->device);
  drop_deferred(ctx);
  (void)hipStreamSynchronize(ctx->stream);
  forget_remembered_sums(ctx);
  if (ctx->zero_block) { buffer_release(ctx->zero_block); ctx->zero_block = nullptr; }
  if (ctx->ticket_block) { buffer_release(ctx->ticket_block); ctx->ticket_block = nullptr; }
  {
    std::lock_guard<std::mutex> g(ctx->mu);
    drop_cache_locked(ctx);
  }
  if (ctx->staging) (void)hipHostFree(ctx->staging);
  ctx->staging = nullptr;
  ctx->staging_bytes = 0;
  // The context itself stays allocated: arrays released later (finalizers)
  // still find their allocator.
  return HGPU_OK;
}

int hgpu_sync(hgpu_ctx* ctx) {
  if (!ctx) return HGPU_ERR_INVALID;
  if (int rc = no_capture(ctx, "sync")) return rc;
  (void)hipSetDevice(ctx->device);
  flush_deferred(ctx);
  int rc = check_hip(ctx, hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  if (int held_rc = take_deferred_rc(ctx)) rc = held_rc;      // a launch that was held back failed after its call had returned
  return rc;
}

const char* hgpu_last_error(hgpu_ctx* ctx) {
  static thread_local std::string copy;
  if (!ctx) return "no context";
  std::lock_guard<std::mutex> g(ctx->mu);
  copy = ctx->err;
  return copy.c_str();
}

int hgpu_mem_stats(hgpu_ctx* ctx, uint64_t* in_use, uint64_t* reserved, uint64_t* n_allocs) {
  if (!ctx) return HGPU_ERR_INVALID;
  flush_deferred(ctx);      // launches that are held back hold their buffers
  std::lock_guard<std::mutex> g(ctx->mu);
  if (in_use) *in_use = ctx->in_use;
  if (reserved) *reserved = ctx->reserved;
  if (n_allocs) *n_allocs = ctx->n_device_allocs;
  return HGPU_OK;
}

void* hgpu_stream(hgpu_ctx* ctx) {
  if (!ctx) return nullptr;
  flush_deferred(ctx);      // whoever enqueues on the stream next comes after everything issued so far
  return (void*)ctx->stream;
}

int hgpu_inject_alloc_failure(hgpu_ctx* ctx, int64_t limit) {
  if (!ctx) return HGPU_ERR_INVALID;
  flush_deferred(ctx);
  std::lock_guard<std::mutex> g(ctx->mu);
  if (limit < 0) {
    ctx->fail_after = -1;
  } else {
    ctx->fail_after = (int64_t)ctx->n_device_allocs + limit;
    // Cached blocks would satisfy requests without a device allocation.
    (void)hipStreamSynchronize(ctx->stream);
    drop_cache_locked(ctx);
  }
  return HGPU_OK;
}

int hgpu_profile_enable(hgpu_ctx* ctx, int on) {
  if (!ctx) return HGPU_ERR_INVALID;
  std::lock_guard<std::mutex> g(ctx->launch_mu);
  if (ctx->dq_pending) flush_deferred_locked(ctx);
  (void)hipStreamSynchronize(ctx->stream);
  for (auto& r : ctx->prof) { (void)hipEventDestroy(r.a); (void)hipEventDestroy(r.b); }
  ctx->prof.clear();
  ctx->profiling = on != 0;
  ctx->profile_shapes = on == 2;
  return HGPU_OK;
}

int hgpu_profile_report(hgpu_ctx* ctx, char* buf, size_t n) {
  if (!ctx || !buf || n == 0) return HGPU_ERR_INVALID;
  std::lock_guard<std::mutex> g(ctx->launch_mu);
  if (ctx->dq_pending) flush_deferred_locked(ctx);
  (void)hipStreamSynchronize(ctx->stream);
  struct Agg { long count = 0; double ms = 0, bytes = 0, flops = 0; };
  std::map<std::string, Agg> agg;
  for (auto& r : ctx->prof) {
    float ms = 0;
    if (hipEventElapsedTime(&ms, r.a, r.b) != hipSuccess) continue;
    Agg& a = agg[r.name];
    a.count++;
    a.ms += ms;
    a.bytes += r.bytes;
    a.flops += r.flops;
  }
  std::string out;
  char line[256];
  for (auto& kv : agg) {
    snprintf(line, sizeof line, "%s %ld %.6f %.0f %.0f\n", kv.first.c_str(), kv.second.count, kv.second.ms, kv.second.bytes, kv.second.flops);
    out += line;
  }
  snprintf(buf, n, "%s", out.c_str());
  return HGPU_OK;
}

int hgpu_upload(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape, const void* host, hgpu_array** out) {
  if (!ctx || !out) return HGPU_ERR_INVALID;
  *out = nullptr;
  if (dtype_size(dtype) == 0) return fail(ctx, HGPU_ERR_INVALID, "unknown dtype %d", dtype);
  if (int rc0 = no_capture(ctx, "upload")) return rc0;
  hgpu_array* a = nullptr;
  int rc = new_dense(ctx, dtype, rank, shape, &a);
  if (rc) return rc;
  size_t bytes = (size_t)nelem(a) * dtype_size(dtype);
  if (bytes > 0) {
    if (!host) {
      hgpu_release(a);
      return fail(ctx, HGPU_ERR_INVALID, "null host pointer");
    }
    LaunchGuard lg(ctx);
    // Pageable source: hipMemcpyAsync stages it and the host block may be
    // reused by the caller as soon as we return, so wait for the copy.
    hipError_t e = hipMemcpyAsync(data_ptr(a), host, bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
      hgpu_release(a);
      return check_hip(ctx, e, "upload");
    }
    if (nelem(a) == 1 && a->buf && a->offset == 0) {      // a constant of a program: remember when it is zero
      bool zero = true;
      for (size_t i = 0; i < bytes; ++i) zero = zero && ((const unsigned char*)host)[i] == 0;
      if (zero) a->buf->known = hgpu_buffer::kZeroScalar;
    }
  }
  *out = a;
  return HGPU_OK;
}

int hgpu_overwrite(hgpu_ctx* ctx, hgpu_array* a, const void* host) {
  if (!ctx || !a) return HGPU_ERR_INVALID;
  if (int rc = no_capture(ctx, "overwrite")) return rc;
  if (!is_dense(a)) return fail(ctx, HGPU_ERR_INVALID, "overwrite: the array is a strided view");
  size_t bytes = (size_t)nelem(a) * dtype_size(a->dtype);
  if (bytes == 0) return HGPU_OK;
  if (!host) return fail(ctx, HGPU_ERR_INVALID, "null host pointer");
  if (a->buf->known_relied_on) return fail(ctx, HGPU_ERR_INVALID, "overwrite: a kernel has been chosen for this array's contents (an index vector or a zero constant)");
  a->buf->known = hgpu_buffer::kUnknown;
  LaunchGuard lg(ctx);
  ctx->write_epoch++;
  hipError_t e = hipMemcpyAsync(data_ptr(a), host, bytes, hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  return check_hip(ctx, e, "overwrite");
}

int hgpu_assign(hgpu_ctx* ctx, hgpu_array* dst, const hgpu_array* src) {
  if (!ctx || !dst || !src) return HGPU_ERR_INVALID;
  if (dst->dtype != src->dtype || !same_shape(dst, src)) return fail(ctx, HGPU_ERR_INVALID, "assign: shapes or dtypes differ");
  if (!is_dense(dst)) return fail(ctx, HGPU_ERR_INVALID, "assign: the destination is a strided view");
  if (nelem(dst) == 0) return HGPU_OK;
  if (dst->buf == src->buf) return fail(ctx, HGPU_ERR_INVALID, "assign: source and destination share memory");
  if (dst->buf->known_relied_on) return fail(ctx, HGPU_ERR_INVALID, "assign: a kernel has been chosen for the destination's contents (an index vector or a zero constant)");
  dst->buf->known = hgpu_buffer::kUnknown;
  {
    std::lock_guard<std::mutex> lk(ctx->launch_mu);
    ctx->write_epoch++;
  }
  return copy_view(ctx, dst->dtype, dst->rank, dst->shape, data_ptr(src), src->strides, data_ptr(dst), dst->strides);
}

int hgpu_download(hgpu_ctx* ctx, const hgpu_array* a, void* host) {
  if (!ctx || !a) return HGPU_ERR_INVALID;
  if (int rc = no_capture(ctx, "download")) return rc;
  int64_t n = nelem(a);
  if (n == 0) return HGPU_OK;
  if (!host) return fail(ctx, HGPU_ERR_INVALID, "null host pointer");
  size_t bytes = (size_t)n * dtype_size(a->dtype);
  hgpu_array* dense = nullptr;
  const hgpu_array* src = a;
  if (!is_dense(a)) {
    int rc = hgpu_materialize(ctx, a, &dense);
    if (rc) return rc;
    src = dense;
  }
  hipError_t e;
  int held_rc;
  {
    LaunchGuard lg(ctx);
    held_rc = take_deferred_rc(ctx);
    e = hipMemcpyAsync(host, data_ptr(src), bytes, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  }
  if (dense) hgpu_release(dense);
  if (held_rc) return held_rc;
  return check_hip(ctx, e, "download");
}

int hgpu_read_scalar(hgpu_ctx* ctx, const hgpu_array* a, void* host) {
  if (!ctx || !a || !host) return HGPU_ERR_INVALID;
  if (nelem(a) != 1) return fail(ctx, HGPU_ERR_INVALID, "read_scalar of an array with %lld elements", (long long)nelem(a));
  if (int rc = no_capture(ctx, "read_scalar")) return rc;
  LaunchGuard lg(ctx);
  const int held_rc = take_deferred_rc(ctx);
  hipError_t e = hipMemcpyAsync(host, data_ptr(a), dtype_size(a->dtype), hipMemcpyDeviceToHost, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (held_rc) return held_rc;
  return check_hip(ctx, e, "read_scalar");
}

int hgpu_retain(hgpu_array* a) {
  if (!a) return HGPU_ERR_INVALID;
  a->refs.fetch_add(1);
  return HGPU_OK;
}

int hgpu_release(hgpu_array* a) {
  if (!a) return HGPU_OK;
  if (a->refs.fetch_sub(1) == 1) {
    buffer_release(a->buf);
    delete a;
  }
  return HGPU_OK;
}

int hgpu_rank(const hgpu_array* a) { return a ? a->rank : -1; }
int hgpu_dtype_of(const hgpu_array* a) { return a ? a->dtype : -1; }
int64_t hgpu_size(const hgpu_array* a) { return a ? nelem(a) : -1; }
int hgpu_shape(const hgpu_array* a, int64_t* s) {
  if (!a || !s) return HGPU_ERR_INVALID;
  for (int i = 0; i < a->rank; ++i) s[i] = a->shape[i];
  return HGPU_OK;
}
int hgpu_strides(const hgpu_array* a, int64_t* s) {
  if (!a || !s) return HGPU_ERR_INVALID;
  for (int i = 0; i < a->rank; ++i) s[i] = a->strides[i];
  return HGPU_OK;
}
int hgpu_is_dense(const hgpu_array* a) { return a && is_dense(a) ? 1 : 0; }

/* -------------------------------------------------------------------- views */

int hgpu_transpose(hgpu_ctx* ctx, const hgpu_array* a, int nperm, const int* perm, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (nperm < 0 || nperm > a->rank) return fail(ctx, HGPU_ERR_INVALID, "transpose: permutation longer than rank");
  int64_t sh[HGPU_MAX_RANK], st[HGPU_MAX_RANK];
  bool seen[HGPU_MAX_RANK] = {false};
  for (int i = 0; i < a->rank; ++i) {
    int s = i;
    if (i < nperm) {
      s = perm[i];
      if (s < 0 || s >= nperm || seen[s]) return fail(ctx, HGPU_ERR_INVALID, "transpose: not a permutation");
      seen[s] = true;
    }
    sh[i] = a->shape[s];
    st[i] = a->strides[s];
  }
  *out = new_view(ctx, a->buf, a->dtype, a->rank, sh, st, a->offset);
  return HGPU_OK;
}

// Tries to express `shape` as a view of a; fills strides on success.
static bool reshape_view(const hgpu_array* a, int rank, const int64_t* shape, int64_t* st) {
  // Merge a's dims into maximal contiguous runs, then split them.
  int64_t rsh[HGPU_MAX_RANK], rst[HGPU_MAX_RANK];
  int nr = 0;
  for (int i = 0; i < a->rank; ++i) {
    if (a->shape[i] == 1) continue;
    if (nr > 0 && rst[nr - 1] == a->strides[i] * a->shape[i]) {
      rsh[nr - 1] *= a->shape[i];
      rst[nr - 1] = a->strides[i];
    } else {
      rsh[nr] = a->shape[i];
      rst[nr] = a->strides[i];
      nr++;
    }
  }
  int r = 0;
  int64_t rem = nr > 0 ? rsh[0] : 1;  // elements of the current run not yet consumed (outer part)
  for (int i = 0; i < rank; ++i) {
    int64_t s = shape[i];
    if (s == 1) { st[i] = 0; continue; }
    if (r >= nr) return false;
    if (rem % s != 0) return false;
    rem /= s;
    st[i] = rst[r] * rem;
    if (rem == 1) {
      r++;
      rem = r < nr ? rsh[r] : 1;
    }
  }
  return r == nr;
}

int hgpu_reshape(hgpu_ctx* ctx, const hgpu_array* a, int rank, const int64_t* shape, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (rank < 0 || rank > HGPU_MAX_RANK) return fail(ctx, HGPU_ERR_INVALID, "reshape: bad rank");
  int64_t n = 1;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  if (n != nelem(a)) return fail(ctx, HGPU_ERR_INVALID, "reshape: %lld elements into %lld", (long long)nelem(a), (long long)n);
  int64_t st[HGPU_MAX_RANK];
  if (n == 0) {
    dense_strides(rank, shape, st);
    *out = new_view(ctx, nullptr, a->dtype, rank, shape, st, 0);
    return HGPU_OK;
  }
  if (reshape_view(a, rank, shape, st)) {
    *out = new_view(ctx, a->buf, a->dtype, rank, shape, st, a->offset);
    return HGPU_OK;
  }
  hgpu_array* d = nullptr;
  int rc = hgpu_materialize(ctx, a, &d);
  if (rc) return rc;
  dense_strides(rank, shape, st);
  *out = new_view(ctx, d->buf, d->dtype, rank, shape, st, d->offset);
  hgpu_release(d);
  return HGPU_OK;
}

int hgpu_slice(hgpu_ctx* ctx, const hgpu_array* a, int dim, int64_t start, int64_t len, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (dim < 0 || dim >= a->rank) return fail(ctx, HGPU_ERR_INVALID, "slice: dim %d of rank %d", dim, a->rank);
  if (start < 0 || len < 0 || start + len > a->shape[dim])
    return fail(ctx, HGPU_ERR_INVALID, "slice: [%lld,+%lld) outside extent %lld", (long long)start, (long long)len, (long long)a->shape[dim]);
  int64_t sh[HGPU_MAX_RANK];
  for (int i = 0; i < a->rank; ++i) sh[i] = a->shape[i];
  sh[dim] = len;
  *out = new_view(ctx, len == 0 ? nullptr : a->buf, a->dtype, a->rank, sh, a->strides, a->offset + start * a->strides[dim]);
  return HGPU_OK;
}

int hgpu_reverse(hgpu_ctx* ctx, const hgpu_array* a, int dim, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (dim < 0 || dim >= a->rank) return fail(ctx, HGPU_ERR_INVALID, "reverse: dim %d of rank %d", dim, a->rank);
  int64_t st[HGPU_MAX_RANK];
  for (int i = 0; i < a->rank; ++i) st[i] = a->strides[i];
  int64_t off = a->offset;
  if (a->shape[dim] > 0) off += (a->shape[dim] - 1) * a->strides[dim];
  st[dim] = -st[dim];
  *out = new_view(ctx, a->buf, a->dtype, a->rank, a->shape, st, off);
  return HGPU_OK;
}

int hgpu_replicate(hgpu_ctx* ctx, const hgpu_array* a, int np, const int64_t* pre, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (np < 0 || np + a->rank > HGPU_MAX_RANK) return fail(ctx, HGPU_ERR_INVALID, "replicate: rank too large");
  int64_t sh[HGPU_MAX_RANK], st[HGPU_MAX_RANK];
  bool empty = false;
  for (int i = 0; i < np; ++i) {
    if (pre[i] < 0) return fail(ctx, HGPU_ERR_INVALID, "replicate: negative extent");
    sh[i] = pre[i];
    st[i] = 0;
    if (pre[i] == 0) empty = true;
  }
  for (int i = 0; i < a->rank; ++i) {
    sh[np + i] = a->shape[i];
    st[np + i] = a->strides[i];
  }
  *out = new_view(ctx, empty ? nullptr : a->buf, a->dtype, np + a->rank, sh, st, a->offset);
  return HGPU_OK;
}

int hgpu_index_prefix(hgpu_ctx* ctx, const hgpu_array* a, int n, const int64_t* ix, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (n < 0 || n > a->rank) return fail(ctx, HGPU_ERR_INVALID, "index: %d indices into rank %d", n, a->rank);
  int64_t off = a->offset;
  bool oob = false;
  for (int i = 0; i < n; ++i) {
    if (ix[i] < 0 || ix[i] >= a->shape[i]) oob = true;
    off += ix[i] * a->strides[i];
  }
  if (oob) return new_zeros(ctx, a->dtype, a->rank - n, a->shape + n, out);
  *out = new_view(ctx, a->buf, a->dtype, a->rank - n, a->shape + n, a->strides + n, off);
  return HGPU_OK;
}

int hgpu_as_strided(hgpu_ctx* ctx, const hgpu_array* a, int rank, const int64_t* shape, const int64_t* strides,
                    int64_t offset, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (rank < 0 || rank > HGPU_MAX_RANK) return fail(ctx, HGPU_ERR_INVALID, "as_strided: bad rank");
  int64_t lo = a->offset + offset, hi = lo;
  bool empty = false;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] < 0) return fail(ctx, HGPU_ERR_INVALID, "as_strided: negative extent");
    if (shape[i] == 0) { empty = true; continue; }
    int64_t span = (shape[i] - 1) * strides[i];
    if (span > 0) hi += span; else lo += span;
  }
  if (!empty) {
    if (!a->buf) return fail(ctx, HGPU_ERR_INVALID, "as_strided: view of an empty array");
    // The addressed range must stay inside the elements a itself addresses.
    int64_t alo = a->offset, ahi = a->offset;
    for (int i = 0; i < a->rank; ++i) {
      int64_t span = (a->shape[i] - 1) * a->strides[i];
      if (span > 0) ahi += span; else alo += span;
    }
    if (lo < alo || hi > ahi)
      return fail(ctx, HGPU_ERR_INVALID, "as_strided: elements [%lld,%lld] outside the source view [%lld,%lld]",
                  (long long)lo, (long long)hi, (long long)alo, (long long)ahi);
  }
  *out = new_view(ctx, empty ? nullptr : a->buf, a->dtype, rank, shape, strides, a->offset + offset);
  return HGPU_OK;
}

}  // extern "C"

// ---- run-time compilation with a cache on disk -----------------------------

namespace hg {
namespace {

uint64_t fnv1a(const std::string& s, uint64_t h) {
  for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
  return h;
}

// "" when there is to be no cache
std::string rtc_cache_dir() {
  std::string dir;
  if (const char* e = getenv("HORDEAD_GPU_CACHE")) {
    dir = e;
    if (dir.empty() || dir == "off" || dir == "0") return "";
  } else if (const char* x = getenv("XDG_CACHE_HOME")) {
    if (*x) dir = std::string(x) + "/hordead_gpu";
  }
  if (dir.empty()) {
    const char* home = getenv("HOME");
    if (!home || !*home) return "";
    dir = std::string(home) + "/.cache";
    mkdir(dir.c_str(), 0700);
    dir += "/hordead_gpu";
  }
  if (mkdir(dir.c_str(), 0700) != 0 && errno != EEXIST) return "";
  return dir;
}

const char* kRtcOpts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};

}  // namespace

int rtc_compile(hgpu_ctx* ctx, const std::string& src, const char* what, std::vector<char>* code) {
  // the key: everything the code object depends on
  int major = 0, minor = 0;
  hiprtcVersion(&major, &minor);
  std::string stamp = "hiprtc " + std::to_string(major) + "." + std::to_string(minor);
  for (const char* o : kRtcOpts) { stamp += " "; stamp += o; }
  const uint64_t h1 = fnv1a(src, fnv1a(stamp, 14695981039346656037ull)), h2 = fnv1a(stamp, fnv1a(src, 1469598103934665603ull));
  char name[64];
  snprintf(name, sizeof name, "%016llx%016llx.co", (unsigned long long)h1, (unsigned long long)h2);
  const std::string dir = rtc_cache_dir();
  const std::string path = dir.empty() ? "" : dir + "/" + name;
  const std::string header = stamp + "\n" + std::to_string(src.size()) + "\n";
  // HORDEAD_GPU_KEEP_SOURCES=<dir>: the generated sources are written there,
  // under the names of their code objects, for reading or compiling by hand
  if (const char* keep = getenv("HORDEAD_GPU_KEEP_SOURCES")) {
    if (*keep) {
      std::string sp = std::string(keep) + "/" + name;
      sp.replace(sp.size() - 3, 3, ".hip");
      std::ofstream f(sp, std::ios::trunc);
      if (f) f << "// " << what << "\n" << src;
    }
  }
  if (!path.empty()) {
    std::ifstream f(path, std::ios::binary);
    if (f) {
      std::string all((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
      if (all.size() > header.size() && all.compare(0, header.size(), header) == 0) {
        code->assign(all.begin() + (long)header.size(), all.end());
        return HGPU_OK;
      }
    }
  }
  hiprtcProgram prog;
  if (hiprtcCreateProgram(&prog, src.c_str(), "hordead_gpu_rtc.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
    return fail(ctx, HGPU_ERR_DEVICE, "hiprtcCreateProgram failed");
  // packed FP32 instructions stay off, as in the ahead-of-time build.  There is
  // no retry without the switch: a compiler that rejects it fails here, with its
  // log, rather than handing back code built under other options than the key says.
  hiprtcResult r = hiprtcCompileProgram(prog, (int)(sizeof kRtcOpts / sizeof kRtcOpts[0]), kRtcOpts);
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    return fail(ctx, HGPU_ERR_DEVICE, "hiprtc (%s): %s: %.600s", what, hiprtcGetErrorString(r), log.c_str());
  }
  size_t n = 0;
  hiprtcGetCodeSize(prog, &n);
  code->resize(n);
  hiprtcGetCode(prog, code->data());
  hiprtcDestroyProgram(&prog);
  if (!path.empty()) {   // written under another name first: a reader never sees half a file
    const std::string tmp = path + "." + std::to_string((long)getpid()) + ".tmp";
    std::ofstream f(tmp, std::ios::binary | std::ios::trunc);
    if (f) {
      f.write(header.data(), (std::streamsize)header.size());
      f.write(code->data(), (std::streamsize)code->size());
      f.close();
      if (!f || rename(tmp.c_str(), path.c_str()) != 0) unlink(tmp.c_str());
    }
  }
  return HGPU_OK;
}

}  // namespace hg
