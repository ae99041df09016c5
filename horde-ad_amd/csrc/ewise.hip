// Elementwise kernels over strided views: the Num / Fractional / Floating /
// IntegralH instances of arrays that horde-ad's `Concrete` backend takes from
// ox-arrays (src/HordeAd/Core/CarriersConcrete.hs:40-56,333-343), comparisons,
// conversions, and the copying structural operations (append, pad, oneHot).
//
// Every kernel walks the OUTPUT in linear order, one element per lane per
// grid-stride step, so stores are always coalesced; loads are coalesced
// whenever the operand's innermost merged dimension has unit stride.  When all
// operands are dense (or one-element broadcasts) the index decomposition is
// skipped and each lane moves 16-byte vectors.
#include "common.hpp"

using namespace hg;

namespace {

constexpr int kBlock = 256;

template <typename T> struct is_fp { static constexpr bool value = false; };
template <> struct is_fp<double> { static constexpr bool value = true; };
template <> struct is_fp<float> { static constexpr bool value = true; };

template <typename T>
__device__ __forceinline__ T apply1(int op, T x) {
  if constexpr (is_fp<T>::value) {
    switch (op) {
      case HGPU_NEG: return -x;
      case HGPU_ABS: return fabs(x);
      case HGPU_SIGNUM: return x > T(0) ? T(1) : (x < T(0) ? T(-1) : x);
      case HGPU_RECIP: return T(1) / x;
      case HGPU_EXP: return exp(x);
      case HGPU_LOG: return log(x);
      case HGPU_SQRT: return sqrt(x);
      case HGPU_SIN: return sin(x);
      case HGPU_COS: return cos(x);
      case HGPU_TAN: return tan(x);
      case HGPU_ASIN: return asin(x);
      case HGPU_ACOS: return acos(x);
      case HGPU_ATAN: return atan(x);
      case HGPU_SINH: return sinh(x);
      case HGPU_COSH: return cosh(x);
      case HGPU_TANH: return tanh(x);
      case HGPU_ASINH: return asinh(x);
      case HGPU_ACOSH: return acosh(x);
      case HGPU_ATANH: return atanh(x);
    }
    return x;
  } else {
    switch (op) {
      case HGPU_NEG: return (T)(-x);
      case HGPU_ABS: return x < 0 ? (T)(-x) : x;
      case HGPU_SIGNUM: return x > 0 ? T(1) : (x < 0 ? T(-1) : T(0));
      case HGPU_NOT: return (T)(x == 0 ? 1 : 0);
    }
    return x;
  }
}

template <typename T>
__device__ __forceinline__ T apply2(int op, T x, T y) {
  if constexpr (is_fp<T>::value) {
    switch (op) {
      case HGPU_ADD: return x + y;
      case HGPU_MUL: return x * y;
      case HGPU_SUB: return x - y;
      case HGPU_DIV: return x / y;
      case HGPU_POW: return pow(x, y);
      case HGPU_LOGBASE: return log(y) / log(x);  // logBase x y = log y / log x
      case HGPU_ATAN2: return atan2(x, y);
      case HGPU_MIN: return x <= y ? x : y;
      case HGPU_MAX: return x >= y ? x : y;
    }
    return x;
  } else {
    switch (op) {
      case HGPU_ADD: return (T)(x + y);
      case HGPU_MUL: return (T)(x * y);
      case HGPU_SUB: return (T)(x - y);
      case HGPU_QUOT: return y == 0 ? x : (T)(x / y);  // quot a 1 = a
      case HGPU_REM: return y == 0 ? T(0) : (T)(x % y);  // array rule: rem a 1 = 0
      case HGPU_REM_SCALAR: return y == 0 ? x : (T)(x % y);
      case HGPU_MIN: return x <= y ? x : y;
      case HGPU_MAX: return x >= y ? x : y;
      case HGPU_AND: return (T)((x != 0 && y != 0) ? 1 : 0);
    }
    return x;
  }
}

template <typename T>
__device__ __forceinline__ uint8_t applycmp(int op, T x, T y) {
  switch (op) {
    case HGPU_LEQ: return x <= y;
    case HGPU_EQ: return x == y;
    case HGPU_LT: return x < y;
  }
  return 0;
}

// ---- generic strided kernels (operand 0 is the dense output) --------------

template <typename T>
__global__ void __launch_bounds__(kBlock) k_ewise1(int op, Dims d, int64_t n, const T* __restrict__ a, T* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off[1];
    decompose<1>(d, i, off);
    o[i] = apply1<T>(op, a[off[0]]);
  }
}

template <typename T>
__global__ void __launch_bounds__(kBlock) k_ewise2(int op, Dims d, int64_t n, const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off[2];
    decompose<2>(d, i, off);
    o[i] = apply2<T>(op, a[off[0]], b[off[1]]);
  }
}

template <typename T>
__global__ void __launch_bounds__(kBlock) k_cmp(int op, Dims d, int64_t n, const T* __restrict__ a, const T* __restrict__ b, uint8_t* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off[2];
    decompose<2>(d, i, off);
    o[i] = applycmp<T>(op, a[off[0]], b[off[1]]);
  }
}

template <typename T>
__global__ void __launch_bounds__(kBlock) k_select(Dims d, int64_t n, const uint8_t* __restrict__ c, const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off[3];
    decompose<3>(d, i, off);
    o[i] = c[off[0]] ? a[off[1]] : b[off[2]];
  }
}

template <typename S, typename D>
__device__ __forceinline__ D conv1(S x, int mode) {
  if constexpr (is_fp<S>::value && !is_fp<D>::value) {
    if (mode == HGPU_CONV_FLOOR) return (D)(int64_t)floor((double)x);
    return (D)(int64_t)x;
  } else {
    return (D)x;
  }
}

template <typename S, typename D>
__global__ void __launch_bounds__(kBlock) k_convert(int mode, Dims d, int64_t n, const S* __restrict__ a, D* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off[1];
    decompose<1>(d, i, off);
    o[i] = conv1<S, D>(a[off[0]], mode);
  }
}

// Copy between two strided views of one shape (operand 0 = source, 1 = dest).
template <typename T>
__global__ void __launch_bounds__(kBlock) k_copy(Dims d, int64_t n, const T* __restrict__ a, T* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off[2];
    decompose<2>(d, i, off);
    o[off[1]] = a[off[0]];
  }
}

// Zero padding in one pass over the result: the dims of the (dense) result in
// memory order, for each the padding in front, the source's extent and stride.
struct PadDims {
  int nd;
  int64_t shape[HG_KDIMS], lo[HG_KDIMS], ext[HG_KDIMS], sst[HG_KDIMS];
};

struct alignas(16) Bytes16 { uint64_t lo, hi; };

template <typename T>
__global__ void __launch_bounds__(kBlock) k_pad(PadDims d, int64_t n, const T* __restrict__ a, T* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) {
    int64_t off = 0;
    bool inside = true;
    if (n <= (int64_t)0x7fffffff) {
      uint32_t r = (uint32_t)i;
      for (int k = d.nd - 1; k >= 0; --k) {
        uint32_t s = (uint32_t)d.shape[k];
        uint32_t q = k > 0 ? r / s : 0;
        int64_t c = (int64_t)(r - q * s) - d.lo[k];
        r = q;
        inside = inside && (uint64_t)c < (uint64_t)d.ext[k];
        off += c * d.sst[k];
      }
    } else {
      int64_t r = i;
      for (int k = d.nd - 1; k >= 0; --k) {
        int64_t s = d.shape[k];
        int64_t q = k > 0 ? r / s : 0;
        int64_t c = r - q * s - d.lo[k];
        r = q;
        inside = inside && (uint64_t)c < (uint64_t)d.ext[k];
        off += c * d.sst[k];
      }
    }
    o[i] = inside ? a[off] : T{};
  }
}

// ---- dense fast paths: 16-byte vectors, flags say which operands broadcast --

template <typename T> struct Vec16 { static constexpr int N = 16 / sizeof(T); T v[N]; };

template <typename T, bool BA, bool BB>
__global__ void __launch_bounds__(kBlock) k_ewise2_dense(int op, int64_t n, const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ o) {
  constexpr int N = Vec16<T>::N;
  int64_t nv = n / N;
  int64_t step = (int64_t)gridDim.x * kBlock;
  T sa = BA ? a[0] : T(0), sb = BB ? b[0] : T(0);
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < nv; i += step) {
    Vec16<T> va, vb, vo;
    if (!BA) va = reinterpret_cast<const Vec16<T>*>(a)[i];
    if (!BB) vb = reinterpret_cast<const Vec16<T>*>(b)[i];
#pragma unroll
    for (int k = 0; k < N; ++k) vo.v[k] = apply2<T>(op, BA ? sa : va.v[k], BB ? sb : vb.v[k]);
    reinterpret_cast<Vec16<T>*>(o)[i] = vo;
  }
  int64_t t = nv * N + (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t < n) o[t] = apply2<T>(op, BA ? sa : a[t], BB ? sb : b[t]);
}

template <typename T>
__global__ void __launch_bounds__(kBlock) k_ewise1_dense(int op, int64_t n, const T* __restrict__ a, T* __restrict__ o) {
  constexpr int N = Vec16<T>::N;
  int64_t nv = n / N;
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < nv; i += step) {
    Vec16<T> va = reinterpret_cast<const Vec16<T>*>(a)[i], vo;
#pragma unroll
    for (int k = 0; k < N; ++k) vo.v[k] = apply1<T>(op, va.v[k]);
    reinterpret_cast<Vec16<T>*>(o)[i] = vo;
  }
  int64_t t = nv * N + (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t < n) o[t] = apply1<T>(op, a[t]);
}

__global__ void __launch_bounds__(kBlock) k_zero16(int64_t n16, uint4* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n16; i += step) o[i] = make_uint4(0, 0, 0, 0);
}

template <typename T>
__global__ void __launch_bounds__(kBlock) k_iota(int64_t n, T* __restrict__ o) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += step) o[i] = (T)i;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// 0 = general view, 1 = dense, 2 = every stride zero (one element broadcast).
inline int layout_class(const hgpu_array* a) {
  bool all0 = true;
  for (int i = 0; i < a->rank; ++i)
    if (a->shape[i] != 1 && a->strides[i] != 0) all0 = false;
  if (all0) return 2;
  return is_dense(a) ? 1 : 0;
}

inline int max_blocks(hgpu_ctx* ctx) { return ctx->num_cu * 8; }

}  // namespace

namespace hg {

int zero_fill(hgpu_ctx* ctx, void* p, size_t bytes) {
  // Blocks come from the allocator in multiples of 256 bytes, so rounding the
  // length up to 16 stays inside the block.
  int64_t n16 = (int64_t)((bytes + 15) / 16);
  if (n16 == 0) return HGPU_OK;
  LaunchGuard lg(ctx, "zero_fill", (double)bytes, 0);
  hipLaunchKernelGGL(k_zero16, dim3(grid_for(n16, kBlock, max_blocks(ctx))), dim3(kBlock), 0, ctx->stream, n16, (uint4*)p);
  HG_CHECK_LAUNCH(ctx, "zero_fill");
  return HGPU_OK;
}

int copy_view(hgpu_ctx* ctx, int dtype, int rank, const int64_t* shape, const void* src, const int64_t* sst,
              void* dst, const int64_t* dst_st) {
  int64_t n = 1;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  if (n == 0) return HGPU_OK;
  // A copy may visit the elements in any order: walk the dims in the
  // destination's memory order (largest stride first) so that stores coalesce.
  int order[HGPU_MAX_RANK];
  for (int i = 0; i < rank; ++i) order[i] = i;
  auto mag = [&](int dim) { return dst_st[dim] < 0 ? -dst_st[dim] : dst_st[dim]; };
  for (int i = 1; i < rank; ++i)
    for (int j = i; j > 0 && mag(order[j]) > mag(order[j - 1]); --j) { int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
  int64_t psh[HGPU_MAX_RANK], pss[HGPU_MAX_RANK], pds[HGPU_MAX_RANK];
  for (int i = 0; i < rank; ++i) { psh[i] = shape[order[i]]; pss[i] = sst[order[i]]; pds[i] = dst_st[order[i]]; }
  const int64_t* sts[2] = {pss, pds};
  Dims d;
  if (!collapse(rank, psh, 2, sts, &d)) return fail(ctx, HGPU_ERR_UNSUPPORTED, "copy: more than %d merged dims", HG_KDIMS);
  const char* label = "copy_view";
  if (ctx->profiling && ctx->profile_shapes) {
    char buf[200];
    int w = snprintf(buf, sizeof buf, "copy_view[es%d", (int)dtype_size(dtype));
    for (int i = 0; i < d.nd && w < (int)sizeof buf - 60; ++i)
      w += snprintf(buf + w, sizeof buf - w, ",%lld:%lld>%lld", (long long)d.shape[i], (long long)d.st[0][i], (long long)d.st[1][i]);
    snprintf(buf + w, sizeof buf - w, "]");
    label = intern_label(ctx, buf);
  }
  LaunchGuard lg(ctx, label, 2.0 * n * dtype_size(dtype), 0);
  unsigned g = grid_for(n, kBlock, max_blocks(ctx));
  switch (dtype_size(dtype)) {
    case 8: hipLaunchKernelGGL(k_copy<uint64_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint64_t*)src, (uint64_t*)dst); break;
    case 4: hipLaunchKernelGGL(k_copy<uint32_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint32_t*)src, (uint32_t*)dst); break;
    case 2: hipLaunchKernelGGL(k_copy<uint16_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint16_t*)src, (uint16_t*)dst); break;
    default: hipLaunchKernelGGL(k_copy<uint8_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint8_t*)src, (uint8_t*)dst); break;
  }
  HG_CHECK_LAUNCH(ctx, "copy_view");
  return HGPU_OK;
}

}  // namespace hg

extern "C" {

int hgpu_materialize(hgpu_ctx* ctx, const hgpu_array* a, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  hgpu_array* o = nullptr;
  int rc = new_dense(ctx, a->dtype, a->rank, a->shape, &o);
  if (rc) return rc;
  rc = copy_view(ctx, a->dtype, a->rank, a->shape, data_ptr(a), a->strides, data_ptr(o), o->strides);
  if (rc) { hgpu_release(o); return rc; }
  *out = o;
  return HGPU_OK;
}

int hgpu_pad(hgpu_ctx* ctx, const hgpu_array* a, const int64_t* lo, const int64_t* hi, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  int64_t sh[HGPU_MAX_RANK];
  for (int i = 0; i < a->rank; ++i) {
    if (lo[i] < 0 || hi[i] < 0) return fail(ctx, HGPU_ERR_INVALID, "pad: negative padding");
    sh[i] = a->shape[i] + lo[i] + hi[i];
  }
  // The result keeps the operand's order of dims IN MEMORY (a transposed view is
  // padded into a transposed array): the copy is coalesced on both sides and
  // whatever was contiguous stays contiguous for the consumer.
  int order[HGPU_MAX_RANK];
  for (int i = 0; i < a->rank; ++i) order[i] = i;
  auto key = [&](int d) -> int64_t {
    int64_t s = a->strides[d] < 0 ? -a->strides[d] : a->strides[d];
    return (s == 0 || a->shape[d] == 1) ? INT64_MAX : s;   // replicated dims go outermost
  };
  for (int i = 1; i < a->rank; ++i)   // stable insertion sort, largest stride first
    for (int j = i; j > 0 && key(order[j]) > key(order[j - 1]); --j) { int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
  int64_t psh[HGPU_MAX_RANK];
  for (int i = 0; i < a->rank; ++i) psh[i] = sh[order[i]];
  // dims of the result in memory order; neighbours without padding whose source
  // strides nest become one dim, dims of extent 1 vanish
  PadDims d;
  d.nd = 0;
  int64_t n = 1;
  for (int i = 0; i < a->rank; ++i) {
    const int dim = order[i];
    n *= psh[i];
    if (psh[i] == 1 && a->shape[dim] == 1) continue;
    const bool plain = lo[dim] == 0 && hi[dim] == 0;
    if (d.nd > 0 && plain && d.lo[d.nd - 1] == 0 && d.ext[d.nd - 1] == d.shape[d.nd - 1] && d.sst[d.nd - 1] == a->strides[dim] * a->shape[dim]) {
      d.shape[d.nd - 1] *= psh[i];
      d.ext[d.nd - 1] *= psh[i];
      d.sst[d.nd - 1] = a->strides[dim];
      continue;
    }
    if (d.nd == HG_KDIMS) return fail(ctx, HGPU_ERR_UNSUPPORTED, "pad: more than %d merged dims", HG_KDIMS);
    d.shape[d.nd] = psh[i];
    d.lo[d.nd] = lo[dim];
    d.ext[d.nd] = a->shape[dim];
    d.sst[d.nd] = a->strides[dim];
    ++d.nd;
  }
  if (d.nd == 0) { d.nd = 1; d.shape[0] = 1; d.lo[0] = 0; d.ext[0] = 1; d.sst[0] = 0; }
  hgpu_array* phys = nullptr;
  int rc = new_dense(ctx, a->dtype, a->rank, psh, &phys);
  if (rc) return rc;
  int64_t st[HGPU_MAX_RANK];
  for (int i = 0; i < a->rank; ++i) st[order[i]] = phys->strides[i];
  hgpu_array* o = new_view(ctx, phys->buf, a->dtype, a->rank, sh, st, 0);
  hgpu_release(phys);
  if (n > 0) {
    const char* label = "pad";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[200];
      int w = snprintf(buf, sizeof buf, "pad[es%d", (int)dtype_size(a->dtype));
      for (int i = 0; i < d.nd && w < (int)sizeof buf - 80; ++i)
        w += snprintf(buf + w, sizeof buf - w, ",%lld+%lld/%lld:%lld", (long long)d.lo[i], (long long)d.ext[i], (long long)d.shape[i], (long long)d.sst[i]);
      snprintf(buf + w, sizeof buf - w, "]");
      label = intern_label(ctx, buf);
    }
    LaunchGuard lg(ctx, label, (double)(n + nelem(a)) * dtype_size(a->dtype), 0);
    const void* src = data_ptr(a);
    void* dst = data_ptr(o);
    // rows whose extents, paddings and addresses are all multiples of 16 bytes move as 16-byte elements
    size_t es = dtype_size(a->dtype);
    const int64_t f = 16 / (int64_t)es;
    const int in = d.nd - 1;
    bool wide = es < 16 && d.sst[in] == 1 && d.shape[in] % f == 0 && d.lo[in] % f == 0 && d.ext[in] % f == 0 && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0;
    for (int i = 0; i < in && wide; ++i) wide = d.sst[i] % f == 0;
    if (wide) {
      d.shape[in] /= f;
      d.lo[in] /= f;
      d.ext[in] /= f;
      for (int i = 0; i < in; ++i) d.sst[i] /= f;
      n /= f;
      es = 16;
    }
    unsigned g = grid_for(n, kBlock, max_blocks(ctx));
    switch (es) {
      case 16: hipLaunchKernelGGL(k_pad<Bytes16>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const Bytes16*)src, (Bytes16*)dst); break;
      case 8: hipLaunchKernelGGL(k_pad<uint64_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint64_t*)src, (uint64_t*)dst); break;
      case 4: hipLaunchKernelGGL(k_pad<uint32_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint32_t*)src, (uint32_t*)dst); break;
      case 2: hipLaunchKernelGGL(k_pad<uint16_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint16_t*)src, (uint16_t*)dst); break;
      default: hipLaunchKernelGGL(k_pad<uint8_t>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint8_t*)src, (uint8_t*)dst); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "pad"); }
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_scatter_affine(hgpu_ctx* ctx, const hgpu_array* src, int rank_m, int n_ix, const int64_t* c0, const int64_t* coef,
                        const int64_t* shp, hgpu_array** out) {
  if (!ctx || !src || !out || (n_ix > 0 && (!c0 || !shp)) || (n_ix > 0 && rank_m > 0 && !coef)) return HGPU_ERR_INVALID;
  if (rank_m < 0 || rank_m > src->rank || n_ix < 0) return fail(ctx, HGPU_ERR_INVALID, "scatter_affine: bad ranks");
  const int rank_n = src->rank - rank_m, rank_o = n_ix + rank_n;
  if (rank_o > HGPU_MAX_RANK) return fail(ctx, HGPU_ERR_INVALID, "scatter_affine: result rank too large");
  int64_t osh[HGPU_MAX_RANK];
  for (int j = 0; j < n_ix; ++j) osh[j] = shp[j];
  for (int i = 0; i < rank_n; ++i) osh[n_ix + i] = src->shape[rank_m + i];
  const int64_t n_src = nelem(src);
  int64_t n_out = 1;
  for (int i = 0; i < rank_o; ++i) n_out *= osh[i];
  if (n_src > 0) {
    for (int j = 0; j < n_ix; ++j) {   // range of every component over the box of positions
      int64_t lo = c0[j], hi = c0[j];
      for (int d = 0; d < rank_m; ++d) {
        int64_t span = coef[d * n_ix + j] * (src->shape[d] - 1);
        if (span > 0) hi += span; else lo += span;
      }
      if (lo < 0 || hi > shp[j] - 1) return fail(ctx, HGPU_ERR_INVALID, "scatter_affine: a position leaves the bounds");
    }
  }
  // The result keeps src's order of dims in memory: an output dim is as
  // contiguous as the most contiguous source dim that moves it.
  int64_t key[HGPU_MAX_RANK];
  auto mag = [](int64_t v) { return v < 0 ? -v : v; };
  for (int j = 0; j < n_ix; ++j) {
    key[j] = INT64_MAX;
    for (int d = 0; d < rank_m; ++d)
      if (coef[d * n_ix + j] != 0 && src->shape[d] > 1 && src->strides[d] != 0 && mag(src->strides[d]) < key[j]) key[j] = mag(src->strides[d]);
  }
  for (int i = 0; i < rank_n; ++i) {
    int d = rank_m + i;
    key[n_ix + i] = (src->shape[d] > 1 && src->strides[d] != 0) ? mag(src->strides[d]) : INT64_MAX;
  }
  int order[HGPU_MAX_RANK];
  for (int i = 0; i < rank_o; ++i) order[i] = i;
  for (int i = 1; i < rank_o; ++i)   // stable insertion sort, largest key first
    for (int j = i; j > 0 && key[order[j]] > key[order[j - 1]]; --j) { int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
  int64_t psh[HGPU_MAX_RANK];
  for (int i = 0; i < rank_o; ++i) psh[i] = osh[order[i]];
  hgpu_array* phys = nullptr;
  // distinct positions fill distinct places: with as many positions as places nothing stays zero
  int rc = (n_src == n_out) ? new_dense(ctx, src->dtype, rank_o, psh, &phys) : new_zeros(ctx, src->dtype, rank_o, psh, &phys);
  if (rc) return rc;
  int64_t st[HGPU_MAX_RANK];
  for (int i = 0; i < rank_o; ++i) st[order[i]] = phys->strides[i];
  hgpu_array* o = new_view(ctx, phys->buf, src->dtype, rank_o, osh, st, 0);
  hgpu_release(phys);
  if (n_src > 0) {
    int64_t off = 0, ds[HGPU_MAX_RANK];
    for (int j = 0; j < n_ix; ++j) off += c0[j] * st[j];
    for (int d = 0; d < rank_m; ++d) {
      ds[d] = 0;
      for (int j = 0; j < n_ix; ++j) ds[d] += coef[d * n_ix + j] * st[j];
    }
    for (int i = 0; i < rank_n; ++i) ds[rank_m + i] = st[n_ix + i];
    rc = copy_view(ctx, src->dtype, src->rank, src->shape, data_ptr(src), src->strides,
                   (char*)data_ptr(o) + off * (int64_t)dtype_size(src->dtype), ds);
    if (rc) { hgpu_release(o); return rc; }
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_ewise1(hgpu_ctx* ctx, int op, const hgpu_array* a, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (op < 0 || op >= HGPU_OP1_COUNT) return fail(ctx, HGPU_ERR_INVALID, "ewise1: unknown opcode %d", op);
  bool fp = dtype_is_float(a->dtype);
  if (op >= HGPU_RECIP && op <= HGPU_ATANH && !fp) return fail(ctx, HGPU_ERR_INVALID, "ewise1: floating opcode %d on a non-floating array", op);
  if (op == HGPU_NOT && a->dtype != HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "ewise1: NOT on a non-Bool array");
  if (a->dtype == HGPU_BOOL && op != HGPU_NOT) return fail(ctx, HGPU_ERR_INVALID, "ewise1: arithmetic on a Bool array");
  hgpu_array* o = nullptr;
  int rc = new_dense(ctx, a->dtype, a->rank, a->shape, &o);
  if (rc) return rc;
  int64_t n = nelem(o);
  if (n > 0) {
    LaunchGuard lg(ctx, "ewise1", 2.0 * n * dtype_size(a->dtype), (double)n);
    if (layout_class(a) == 1 && aligned16(data_ptr(a))) {
      unsigned g = grid_for(n, kBlock * 4, max_blocks(ctx));
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_ewise1_dense<T>, dim3(g), dim3(kBlock), 0, ctx->stream, op, n, (const T*)data_ptr(a), (T*)data_ptr(o)));
    } else {
      const int64_t* sts[1] = {a->strides};
      Dims d;
      if (!collapse(a->rank, a->shape, 1, sts, &d)) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "ewise1: too many dims"); }
      unsigned g = grid_for(n, kBlock, max_blocks(ctx));
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_ewise1<T>, dim3(g), dim3(kBlock), 0, ctx->stream, op, d, n, (const T*)data_ptr(a), (T*)data_ptr(o)));
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "ewise1"); }
  }
  *out = o;
  return HGPU_OK;
}

static int check_binary(hgpu_ctx* ctx, const char* who, const hgpu_array* a, const hgpu_array* b) {
  if (a->dtype != b->dtype) return fail(ctx, HGPU_ERR_INVALID, "%s: dtypes %d and %d differ", who, a->dtype, b->dtype);
  if (!same_shape(a, b)) return fail(ctx, HGPU_ERR_INVALID, "%s: shapes differ", who);
  return HGPU_OK;
}

int hgpu_ewise2(hgpu_ctx* ctx, int op, const hgpu_array* a, const hgpu_array* b, hgpu_array** out) {
  if (!ctx || !a || !b || !out) return HGPU_ERR_INVALID;
  if (op < 0 || op >= HGPU_OP2_COUNT) return fail(ctx, HGPU_ERR_INVALID, "ewise2: unknown opcode %d", op);
  int rc = check_binary(ctx, "ewise2", a, b);
  if (rc) return rc;
  bool fp = dtype_is_float(a->dtype);
  if (op >= HGPU_DIV && op <= HGPU_ATAN2 && !fp) return fail(ctx, HGPU_ERR_INVALID, "ewise2: floating opcode %d on a non-floating array", op);
  if (op >= HGPU_QUOT && op <= HGPU_REM_SCALAR && !dtype_is_int(a->dtype)) return fail(ctx, HGPU_ERR_INVALID, "ewise2: integral opcode %d on a non-integral array", op);
  if (op == HGPU_AND && a->dtype != HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "ewise2: AND on a non-Bool array");
  if (a->dtype == HGPU_BOOL && op != HGPU_AND) return fail(ctx, HGPU_ERR_INVALID, "ewise2: arithmetic on a Bool array");
  hgpu_array* o = nullptr;
  rc = new_dense(ctx, a->dtype, a->rank, a->shape, &o);
  if (rc) return rc;
  int64_t n = nelem(o);
  if (n > 0) {
    LaunchGuard lg(ctx, "ewise2", 3.0 * n * dtype_size(a->dtype), (double)n);
    int la = layout_class(a), lb = layout_class(b);
    bool fast = la != 0 && lb != 0 && !(la == 2 && lb == 2) && (la == 2 || aligned16(data_ptr(a))) && (lb == 2 || aligned16(data_ptr(b)));
    if (fast) {
      unsigned g = grid_for(n, kBlock * 4, max_blocks(ctx));
      HG_DISPATCH_DTYPE(a->dtype, T, {
        const T* pa = (const T*)data_ptr(a);
        const T* pb = (const T*)data_ptr(b);
        T* po = (T*)data_ptr(o);
        if (la == 2) hipLaunchKernelGGL((k_ewise2_dense<T, true, false>), dim3(g), dim3(kBlock), 0, ctx->stream, op, n, pa, pb, po);
        else if (lb == 2) hipLaunchKernelGGL((k_ewise2_dense<T, false, true>), dim3(g), dim3(kBlock), 0, ctx->stream, op, n, pa, pb, po);
        else hipLaunchKernelGGL((k_ewise2_dense<T, false, false>), dim3(g), dim3(kBlock), 0, ctx->stream, op, n, pa, pb, po);
      });
    } else {
      const int64_t* sts[2] = {a->strides, b->strides};
      Dims d;
      if (!collapse(a->rank, a->shape, 2, sts, &d)) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "ewise2: too many dims"); }
      unsigned g = grid_for(n, kBlock, max_blocks(ctx));
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_ewise2<T>, dim3(g), dim3(kBlock), 0, ctx->stream, op, d, n, (const T*)data_ptr(a), (const T*)data_ptr(b), (T*)data_ptr(o)));
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "ewise2"); }
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_compare(hgpu_ctx* ctx, int cmp, const hgpu_array* a, const hgpu_array* b, hgpu_array** out) {
  if (!ctx || !a || !b || !out) return HGPU_ERR_INVALID;
  if (cmp < HGPU_LEQ || cmp > HGPU_LT) return fail(ctx, HGPU_ERR_INVALID, "compare: unknown opcode %d", cmp);
  int rc = check_binary(ctx, "compare", a, b);
  if (rc) return rc;
  hgpu_array* o = nullptr;
  rc = new_dense(ctx, HGPU_BOOL, a->rank, a->shape, &o);
  if (rc) return rc;
  int64_t n = nelem(o);
  if (n > 0) {
    const int64_t* sts[2] = {a->strides, b->strides};
    Dims d;
    if (!collapse(a->rank, a->shape, 2, sts, &d)) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "compare: too many dims"); }
    LaunchGuard lg(ctx, "compare", n * (2.0 * dtype_size(a->dtype) + 1), (double)n);
    unsigned g = grid_for(n, kBlock, max_blocks(ctx));
    HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_cmp<T>, dim3(g), dim3(kBlock), 0, ctx->stream, cmp, d, n, (const T*)data_ptr(a), (const T*)data_ptr(b), (uint8_t*)data_ptr(o)));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "compare"); }
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_select(hgpu_ctx* ctx, const hgpu_array* c, const hgpu_array* a, const hgpu_array* b, hgpu_array** out) {
  if (!ctx || !c || !a || !b || !out) return HGPU_ERR_INVALID;
  if (c->dtype != HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "select: condition is not Bool");
  int rc = check_binary(ctx, "select", a, b);
  if (rc) return rc;
  if (!same_shape(c, a)) return fail(ctx, HGPU_ERR_INVALID, "select: condition shape differs");
  hgpu_array* o = nullptr;
  rc = new_dense(ctx, a->dtype, a->rank, a->shape, &o);
  if (rc) return rc;
  int64_t n = nelem(o);
  if (n > 0) {
    const int64_t* sts[3] = {c->strides, a->strides, b->strides};
    Dims d;
    if (!collapse(a->rank, a->shape, 3, sts, &d)) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "select: too many dims"); }
    LaunchGuard lg(ctx, "select", n * (3.0 * dtype_size(a->dtype) + 1), (double)n);
    unsigned g = grid_for(n, kBlock, max_blocks(ctx));
    HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_select<T>, dim3(g), dim3(kBlock), 0, ctx->stream, d, n, (const uint8_t*)data_ptr(c), (const T*)data_ptr(a), (const T*)data_ptr(b), (T*)data_ptr(o)));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "select"); }
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_convert(hgpu_ctx* ctx, const hgpu_array* a, int dtype, int mode, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (dtype_size(dtype) == 0) return fail(ctx, HGPU_ERR_INVALID, "convert: unknown dtype %d", dtype);
  if (mode == HGPU_CONV_FLOOR && !(dtype_is_float(a->dtype) && dtype_is_int(dtype)))
    return fail(ctx, HGPU_ERR_INVALID, "convert: floor needs a floating source and an integral target");
  hgpu_array* o = nullptr;
  int rc = new_dense(ctx, dtype, a->rank, a->shape, &o);
  if (rc) return rc;
  int64_t n = nelem(o);
  if (n > 0) {
    const int64_t* sts[1] = {a->strides};
    Dims d;
    if (!collapse(a->rank, a->shape, 1, sts, &d)) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "convert: too many dims"); }
    LaunchGuard lg(ctx, "convert", (double)n * (dtype_size(a->dtype) + dtype_size(dtype)), (double)n);
    unsigned g = grid_for(n, kBlock, max_blocks(ctx));
    HG_DISPATCH_DTYPE(a->dtype, S, {
      HG_DISPATCH_DTYPE(dtype, D, hipLaunchKernelGGL((k_convert<S, D>), dim3(g), dim3(kBlock), 0, ctx->stream, mode, d, n, (const S*)data_ptr(a), (D*)data_ptr(o)));
    });
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "convert"); }
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_iota(hgpu_ctx* ctx, int64_t n, int dtype, hgpu_array** out) {
  if (!ctx || !out) return HGPU_ERR_INVALID;
  if (n < 0 || dtype_size(dtype) == 0 || dtype == HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "iota: bad arguments");
  hgpu_array* o = nullptr;
  int rc = new_dense(ctx, dtype, 1, &n, &o);
  if (rc) return rc;
  if (n > 0) {
    LaunchGuard lg(ctx, "iota", (double)n * dtype_size(dtype), 0);
    unsigned g = grid_for(n, kBlock, max_blocks(ctx));
    HG_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL(k_iota<T>, dim3(g), dim3(kBlock), 0, ctx->stream, n, (T*)data_ptr(o)));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "iota"); }
    if (dtype == HGPU_I64 && o->buf && o->offset == 0) o->buf->known = hgpu_buffer::kIotaI64;
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_concat(hgpu_ctx* ctx, int n, const hgpu_array* const* parts, hgpu_array** out) {
  if (!ctx || !parts || !out || n < 1) return HGPU_ERR_INVALID;
  const hgpu_array* p0 = parts[0];
  if (p0->rank < 1) return fail(ctx, HGPU_ERR_INVALID, "concat: rank 0");
  int64_t sh[HGPU_MAX_RANK];
  for (int i = 0; i < p0->rank; ++i) sh[i] = p0->shape[i];
  sh[0] = 0;
  for (int k = 0; k < n; ++k) {
    const hgpu_array* p = parts[k];
    if (!p || p->rank != p0->rank || p->dtype != p0->dtype) return fail(ctx, HGPU_ERR_INVALID, "concat: part %d has another rank or dtype", k);
    for (int i = 1; i < p0->rank; ++i)
      if (p->shape[i] != p0->shape[i]) return fail(ctx, HGPU_ERR_INVALID, "concat: part %d differs in dim %d", k, i);
    sh[0] += p->shape[0];
  }
  hgpu_array* o = nullptr;
  int rc = new_dense(ctx, p0->dtype, p0->rank, sh, &o);
  if (rc) return rc;
  int64_t row = 0;
  for (int k = 0; k < n && !rc; ++k) {
    const hgpu_array* p = parts[k];
    if (nelem(p) > 0)
      rc = copy_view(ctx, p->dtype, p->rank, p->shape, data_ptr(p), p->strides,
                     (char*)data_ptr(o) + row * o->strides[0] * (int64_t)dtype_size(p->dtype), o->strides);
    row += p->shape[0];
  }
  if (rc) { hgpu_release(o); return rc; }
  *out = o;
  return HGPU_OK;
}

int hgpu_onehot(hgpu_ctx* ctx, const hgpu_array* v, int n, const int64_t* ix, const int64_t* shp, hgpu_array** out) {
  if (!ctx || !v || !out || n < 0 || n + v->rank > HGPU_MAX_RANK) return HGPU_ERR_INVALID;
  int64_t sh[HGPU_MAX_RANK];
  bool oob = false;
  for (int i = 0; i < n; ++i) {
    sh[i] = shp[i];
    if (ix[i] < 0 || ix[i] >= shp[i]) oob = true;
  }
  for (int i = 0; i < v->rank; ++i) sh[n + i] = v->shape[i];
  hgpu_array* o = nullptr;
  int rc = new_zeros(ctx, v->dtype, n + v->rank, sh, &o);
  if (rc) return rc;
  if (!oob && nelem(v) > 0) {
    int64_t off = 0;
    for (int i = 0; i < n; ++i) off += ix[i] * o->strides[i];
    rc = copy_view(ctx, v->dtype, v->rank, v->shape, data_ptr(v), v->strides,
                   (char*)data_ptr(o) + off * (int64_t)dtype_size(v->dtype), o->strides + n);
  }
  if (rc) { hgpu_release(o); return rc; }
  *out = o;
  return HGPU_OK;
}

}  // extern "C"
