// Whole-array comparison giving one Bool: the EqH / OrdH instances of
// `Concrete` on arrays (src/HordeAd/Core/CarriersConcrete.hs:310-331) compare
// the row-major element sequences lexicographically.  The device finds the
// first differing position with an atomic minimum and decides there.
#include "common.hpp"

using namespace hg;

namespace {

constexpr int kBlock = 256;

template <typename T>
__global__ void __launch_bounds__(kBlock) k_first_diff(Dims d, int64_t n, const T* __restrict__ a, const T* __restrict__ b, unsigned long long* first) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  unsigned long long mine = ~0ull;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off[2];
    decompose<2>(d, i, off);
    if (!(a[off[0]] == b[off[1]])) { mine = (unsigned long long)i; break; }
  }
  if (mine != ~0ull) atomicMin(first, mine);
}

template <typename T>
__global__ void k_decide(Dims d, int64_t n, int cmp, const T* __restrict__ a, const T* __restrict__ b, const unsigned long long* first, int* result) {
  unsigned long long f = *first;
  if (f >= (unsigned long long)n) {
    *result = (cmp == HGPU_LT) ? 0 : 1;
    return;
  }
  int64_t off[2];
  decompose<2>(d, (int64_t)f, off);
  T x = a[off[0]], y = b[off[1]];
  *result = cmp == HGPU_EQ ? 0 : (cmp == HGPU_LEQ ? (x <= y) : (x < y));
}

__global__ void k_set_u64(unsigned long long* p, unsigned long long v) { *p = v; }

}  // namespace

extern "C" int hgpu_compare_all(hgpu_ctx* ctx, int cmp, const hgpu_array* a, const hgpu_array* b, int* result) {
  if (!ctx || !a || !b || !result) return HGPU_ERR_INVALID;
  if (cmp < HGPU_LEQ || cmp > HGPU_LT) return fail(ctx, HGPU_ERR_INVALID, "compare_all: unknown opcode %d", cmp);
  if (a->dtype != b->dtype) return fail(ctx, HGPU_ERR_INVALID, "compare_all: dtypes differ");
  if (!same_shape(a, b)) return fail(ctx, HGPU_ERR_INVALID, "compare_all: shapes differ");
  if (int rc = no_capture(ctx, "compare_all")) return rc;
  int64_t n = nelem(a);
  if (n == 0) {
    *result = cmp == HGPU_LT ? 0 : 1;
    return HGPU_OK;
  }
  const int64_t* sts[2] = {a->strides, b->strides};
  Dims d;
  if (!collapse(a->rank, a->shape, 2, sts, &d)) return fail(ctx, HGPU_ERR_UNSUPPORTED, "compare_all: too many dims");
  hgpu_buffer* scratch = nullptr;
  int rc = buffer_alloc(ctx, 256, &scratch);
  if (rc) return rc;
  unsigned long long* first = (unsigned long long*)scratch->ptr;
  int* flag = (int*)((char*)scratch->ptr + 64);
  int host = 0, held_rc;
  hipError_t e;
  {
    LaunchGuard lg(ctx, "compare_all", 2.0 * n * dtype_size(a->dtype), (double)n);
    held_rc = take_deferred_rc(ctx);
    hipLaunchKernelGGL(k_set_u64, dim3(1), dim3(1), 0, ctx->stream, first, ~0ull);
    unsigned g = grid_for(n, kBlock, ctx->num_cu * 8);
    HG_DISPATCH_DTYPE(a->dtype, T, {
      hipLaunchKernelGGL(k_first_diff<T>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const T*)data_ptr(a), (const T*)data_ptr(b), first);
      hipLaunchKernelGGL(k_decide<T>, dim3(1), dim3(1), 0, ctx->stream, d, n, cmp, (const T*)data_ptr(a), (const T*)data_ptr(b), first, flag);
    });
    e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(&host, flag, sizeof(int), hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  }
  buffer_release(scratch);
  if (held_rc) return held_rc;
  if (e != hipSuccess) return check_hip(ctx, e, "compare_all");
  *result = host;
  return HGPU_OK;
}
