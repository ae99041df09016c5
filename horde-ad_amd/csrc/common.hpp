// Shared host-side definitions of the gfx950 backend: context, buffer, array
// view, dimension collapsing and launch helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "hordead_gpu.h"

// Largest number of dimensions a kernel sees after adjacent dimensions that
// are contiguous in every operand have been merged.
#define HG_KDIMS 10

// Blocks handed out while a graph is being captured belong to the capture's
// pool: replays of the graph write them again, so they may be reused by the
// capture itself but never by other work while the graph lives.
struct hgpu_cap_pool {
  std::multimap<size_t, void*> cache;   // guarded by the context's allocator mutex
  bool alive = true;                    // false once the graph is destroyed: blocks return to the context's cache
  int refs = 1;                         // the graph (or the open capture) + every live buffer
};

struct hgpu_buffer {
  hgpu_ctx* ctx;
  void* ptr;
  size_t bytes;      // size of the block handed out by the allocator
  std::atomic<int> refs;
  hgpu_cap_pool* pool = nullptr;
  // What the library knows about the block's contents without reading them (arrays are written
  // once): element i is the I64 value i (hgpu_iota), or the block holds a single element of all
  // zero bits.  A kernel chosen because of that knowledge marks the block, and the two entry points
  // that write into existing arrays (hgpu_overwrite, hgpu_assign) refuse a marked block.
  enum { kUnknown = 0, kIotaI64 = 1, kZeroScalar = 2 };
  int known = kUnknown;
  bool known_relied_on = false;
};

struct hgpu_array {
  hgpu_ctx* ctx;
  std::atomic<int> refs;
  hgpu_buffer* buf;  // nullptr for zero-size arrays
  int dtype;
  int rank;
  int64_t shape[HGPU_MAX_RANK];
  int64_t strides[HGPU_MAX_RANK];  // in elements
  int64_t offset;                  // in elements, from buf->ptr
  // Arrays (views included) come and go by the thousand in a training step, most of them freed together
  // when the step's tape goes: their blocks are kept on a list per thread instead of going back to the
  // allocator, whose per-thread cache holds only a few blocks of one size.
  static void* operator new(size_t n);
  static void operator delete(void* p);
};

namespace hg {
struct DeferredQueue;                         // launches held back to be grouped (smallk.hip)
void flush_deferred_locked(hgpu_ctx* ctx);    // the caller holds launch_mu
void flush_deferred(hgpu_ctx* ctx);
void drop_deferred(hgpu_ctx* ctx);            // flush, then free the queue
void forget_remembered_sums(hgpu_ctx* ctx);   // results kept for a later call, and the arrays held for them (footprint.hip)
}  // namespace hg

struct hgpu_ctx {
  int device;
  hipStream_t stream;
  std::mutex mu;                 // guards allocator state and `err`
  std::multimap<size_t, void*> cache;
  uint64_t in_use = 0, reserved = 0, n_device_allocs = 0;
  int64_t fail_after = -1;
  std::string err;
  void* staging = nullptr;       // pinned host staging block
  size_t staging_bytes = 0;
  std::mutex launch_mu;          // serialises enqueue order across host threads
  uint64_t write_epoch = 0;      // counts the writes into existing arrays (hgpu_overwrite, hgpu_assign): results remembered for given inputs end with it
  int num_cu = 256;
  // JIT cache of fused elementwise kernels, keyed by generated source.
  std::map<std::string, void*> jit_cache;
  // Optional per-launch timing (hgpu_profile_enable): one event pair per launch.
  struct ProfRec { const char* name; hipEvent_t a, b; double bytes, flops; };
  bool profiling = false;
  bool profile_shapes = false;           // hgpu_profile_enable(ctx, 2): labels carry the problem shape
  std::set<std::string> label_pool;
  std::mutex label_mu;                    // guards label_pool: labels are made on any calling thread
  std::vector<ProfRec> prof;
  hgpu_buffer* zero_block = nullptr;     // 256 zero bytes, for kernels that want a dummy table
  hgpu_buffer* ticket_block = nullptr;   // counters (zero between launches) for kernels whose last block finishes a reduction
  hgpu_cap_pool* cap = nullptr;          // non-null while the stream is capturing into a graph
  // Small products whose launch is held back until something else needs the
  // stream: those that do not depend on one another then go out as one kernel.
  hg::DeferredQueue* dq = nullptr;
  bool dq_pending = false;
  int deferred_rc = 0;                   // first error of a held-back launch, reported by the next call that hands results to the host
};

struct hgpu_graph {
  hgpu_ctx* ctx;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  hgpu_cap_pool* pool = nullptr;
};

namespace hg {

inline size_t dtype_size(int dt) {
  switch (dt) {
    case HGPU_F64: case HGPU_I64: return 8;
    case HGPU_F32: case HGPU_I32: return 4;
    case HGPU_I16: return 2;
    case HGPU_I8: case HGPU_BOOL: return 1;
  }
  return 0;
}
inline bool dtype_is_float(int dt) { return dt == HGPU_F64 || dt == HGPU_F32; }
inline bool dtype_is_int(int dt) { return dt >= HGPU_I64 && dt <= HGPU_I8; }

int fail(hgpu_ctx* ctx, int code, const char* fmt, ...);
int check_hip(hgpu_ctx* ctx, hipError_t e, const char* what);

// Allocator (runtime.hip).
int buffer_alloc(hgpu_ctx* ctx, size_t bytes, hgpu_buffer** out);
int zero_block(hgpu_ctx* ctx, const void** out);   // a context-lifetime block of 256 zero bytes
// Context-lifetime counters (1024 of 32 bits, zero between launches) for kernels whose blocks draw tickets: the
// last one finishes the reduction and sets its counter back to zero.  Launches on the context's stream follow one
// another, so the same counters serve them all.
int ticket_block(hgpu_ctx* ctx, void** out);
// Fails (HGPU_ERR_UNSUPPORTED) when the stream is capturing: for entry points that must talk to the host.
int no_capture(hgpu_ctx* ctx, const char* what);
void buffer_retain(hgpu_buffer* b);
void buffer_release(hgpu_buffer* b);

// Array construction helpers (runtime.hip).
hgpu_array* new_view(hgpu_ctx* ctx, hgpu_buffer* buf, int dtype, int rank, const int64_t* shape,
                     const int64_t* strides, int64_t offset);
int new_dense(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape, hgpu_array** out);
int new_zeros(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape, hgpu_array** out);
inline int64_t nelem(const hgpu_array* a) {
  int64_t n = 1;
  for (int i = 0; i < a->rank; ++i) n *= a->shape[i];
  return n;
}
inline void* data_ptr(const hgpu_array* a) {
  if (!a->buf) return nullptr;
  return (char*)a->buf->ptr + a->offset * (int64_t)dtype_size(a->dtype);
}
bool is_dense(const hgpu_array* a);
bool same_shape(const hgpu_array* a, const hgpu_array* b);

// Up to four operands viewed over one iteration space.  `nd` dimensions of
// extent `shape`, operand k advancing by `st[k][d]` elements along dim d.
struct Dims {
  int nd;
  int64_t shape[HG_KDIMS];
  int64_t st[4][HG_KDIMS];
};

// One single-launch reduction of hgpu_contract (contract.hip) with every argument of its kernel: such a launch
// can be held back like a small product, and reductions that do not read one another's results then go out as
// one kernel (the bias and readout gradients at the end of a reverse pass).
struct RedJob {
  int dtype = 0;              // element type of operands and result
  int variant = 0;            // 0: a block per output, 1: a wavefront per output, 2: a lane per output
  int hasb = 0;
  Dims keep, red;
  int64_t n_out = 0, R = 0, Q = 0, Lin = 0, sa = 0, sb = 0, chunk = 0;
  unsigned grid = 0;
  const void* a = nullptr;
  const void* b = nullptr;
  void* out = nullptr;
  const char* label = nullptr;
  double bytes = 0, flops = 0;
};
// contract.hip: launches up to four such reductions of one element type as one kernel (the caller holds launch_mu)
hipError_t launch_reduction_group(hgpu_ctx* ctx, const RedJob* const* jobs, int n);
// smallk.hip: holds the launch back (retaining the buffers it reads and writes); false: the caller launches it now
bool hold_reduction(hgpu_ctx* ctx, const RedJob& job, hgpu_buffer* const* reads, int n_reads, hgpu_buffer* write);

// Builds the merged iteration space of `nops` operands that share `shape`.
// Size-1 dims vanish; adjacent dims merge when every operand's strides allow.
// Returns false when more than HG_KDIMS dims remain.
bool collapse(int rank, const int64_t* shape, int nops, const int64_t* const* strides, Dims* out);

inline void dense_strides(int rank, const int64_t* shape, int64_t* st) {
  int64_t s = 1;
  for (int i = rank - 1; i >= 0; --i) { st[i] = s; s *= shape[i]; }
}

inline unsigned grid_for(int64_t n, int block, int max_blocks) {
  int64_t g = (n + block - 1) / block;
  if (g < 1) g = 1;
  if (g > max_blocks) g = max_blocks;
  return (unsigned)g;
}

// Compiles `src` for gfx950 at run time (runtime.hip) and hands back the code
// object.  Code objects are kept on disk between processes, keyed by the
// source, the options and the compiler's version: a kernel that was compiled
// once (a second or so for the larger ones) is read back in under a
// millisecond.  The directory is $HORDEAD_GPU_CACHE, else
// $XDG_CACHE_HOME/hordead_gpu, else $HOME/.cache/hordead_gpu; HORDEAD_GPU_CACHE=off
// (or an unwritable directory) means no files.  `what` names the caller in errors.
int rtc_compile(hgpu_ctx* ctx, const std::string& src, const char* what, std::vector<char>* code);

// Zeroes `bytes` bytes (rounded up to 16) with a fill kernel (ewise.hip).
int zero_fill(hgpu_ctx* ctx, void* p, size_t bytes);
// Strided copy between two views of equal shape (ewise.hip).
int copy_view(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape, const void* src,
              const int64_t* sst, void* dst, const int64_t* dst_st);

// Serialises enqueueing and, when profiling is on, brackets the launches made
// while it lives with an event pair labelled `name`; `bytes` / `flops` are the
// ALGORITHMIC traffic and work of those launches.
struct LaunchGuard {
  hgpu_ctx* ctx;
  bool timed = false;
  explicit LaunchGuard(hgpu_ctx* c, const char* name = nullptr, double bytes = 0, double flops = 0) : ctx(c) {
    c->launch_mu.lock();
    (void)hipSetDevice(c->device);
    if (c->dq_pending) flush_deferred_locked(c);   // what was held back goes first: stream order is program order
    static const bool trace = getenv("HORDEAD_GPU_TRACE_LAUNCHES") != nullptr;   // one line per launch, in program order
    if (trace && name) fprintf(stderr, "hordead_gpu: launch %s\n", name);
    if (c->profiling && name && !c->cap) {
      hgpu_ctx::ProfRec r{name, nullptr, nullptr, bytes, flops};
      if (hipEventCreate(&r.a) == hipSuccess && hipEventCreate(&r.b) == hipSuccess) {
        (void)hipEventRecord(r.a, c->stream);
        c->prof.push_back(r);
        timed = true;
      }
    }
  }
  ~LaunchGuard() {
    if (timed && !stop_carried) (void)hipEventRecord(ctx->prof.back().b, ctx->stream);
    ctx->launch_mu.unlock();
  }
  // The guard's events for a launch that carries them itself (hipExtModuleLaunchKernel, hipExtLaunchKernel): they
  // then hold the kernel's own begin and end, which is what a profiler's kernel trace reports.  Events recorded
  // around a launch also time its dispatch and the cache write-back after it, 3-4 us more on this device.  The
  // first launch under the guard takes start_event(), the last one stop_event(); both are null while nothing is timed.
  bool stop_carried = false;
  hipEvent_t start_event() { return timed ? ctx->prof.back().a : nullptr; }
  hipEvent_t stop_event() {
    if (!timed) return nullptr;
    stop_carried = true;
    return ctx->prof.back().b;
  }
};

// Launch of a run-time compiled kernel under a guard: `first` / `last` say whether this is the first / last
// launch the guard's record is to cover.
inline hipError_t launch_module(LaunchGuard& lg, hipFunction_t fn, unsigned grid, unsigned block, void** args, bool first = true, bool last = true) {
  if (!lg.timed || (uint64_t)grid * block > 0xffffffffull) return hipModuleLaunchKernel(fn, grid, 1, 1, block, 1, 1, 0, lg.ctx->stream, args, nullptr);
  return hipExtModuleLaunchKernel(fn, grid * block, 1, 1, block, 1, 1, 0, lg.ctx->stream, args, nullptr, first ? lg.start_event() : nullptr,
                                  last ? lg.stop_event() : nullptr, 0);
}

// A label with the lifetime of the context (profiling records keep the pointer).
inline const char* intern_label(hgpu_ctx* c, const std::string& s) {
  std::lock_guard<std::mutex> g(c->label_mu);
  return c->label_pool.insert(s).first->c_str();
}

// The first error of a launch that had been held back and failed after its own
// call returned; cleared once handed out.  Every entry point that hands data or
// a finished recording to the host reports it, since the caller would otherwise
// read a result that was never written.  Call with launch_mu held.
inline int take_deferred_rc(hgpu_ctx* c) {
  const int rc = c->deferred_rc;
  c->deferred_rc = 0;
  return rc;
}

}  // namespace hg

#define HG_DISPATCH_DTYPE(dt, T, ...)                                   \
  switch (dt) {                                                         \
    case HGPU_F64: { using T = double; __VA_ARGS__; break; }            \
    case HGPU_F32: { using T = float; __VA_ARGS__; break; }             \
    case HGPU_I64: { using T = int64_t; __VA_ARGS__; break; }           \
    case HGPU_I32: { using T = int32_t; __VA_ARGS__; break; }           \
    case HGPU_I16: { using T = int16_t; __VA_ARGS__; break; }           \
    case HGPU_I8: { using T = int8_t; __VA_ARGS__; break; }             \
    case HGPU_BOOL: { using T = uint8_t; __VA_ARGS__; break; }          \
    default: break;                                                     \
  }

#define HG_CHECK_LAUNCH(ctx, what)                                      \
  do {                                                                  \
    hipError_t e__ = hipGetLastError();                                 \
    if (e__ != hipSuccess) return hg::check_hip(ctx, e__, what);        \
  } while (0)

// Device-side decomposition of a linear index over a merged iteration space.
#ifdef __HIPCC__
namespace hg {
template <int NOPS>
__device__ __forceinline__ void decompose(const Dims& d, int64_t lin, int64_t* off) {
#pragma unroll
  for (int k = 0; k < NOPS; ++k) off[k] = 0;
  if (lin < (int64_t)0x7fffffff) {
    uint32_t r = (uint32_t)lin;
    for (int i = d.nd - 1; i > 0; --i) {
      uint32_t s = (uint32_t)d.shape[i];
      uint32_t q = r / s;
      uint32_t c = r - q * s;
      r = q;
#pragma unroll
      for (int k = 0; k < NOPS; ++k) off[k] += (int64_t)c * d.st[k][i];
    }
#pragma unroll
    for (int k = 0; k < NOPS; ++k) off[k] += (int64_t)r * d.st[k][0];
  } else {
    int64_t r = lin;
    for (int i = d.nd - 1; i > 0; --i) {
      int64_t s = d.shape[i];
      int64_t q = r / s;
      int64_t c = r - q * s;
      r = q;
#pragma unroll
      for (int k = 0; k < NOPS; ++k) off[k] += c * d.st[k][i];
    }
#pragma unroll
    for (int k = 0; k < NOPS; ++k) off[k] += r * d.st[k][0];
  }
}
}  // namespace hg
#endif
