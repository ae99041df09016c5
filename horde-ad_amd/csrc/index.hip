// Indexing kernels: gather and scatter-add driven by index ARRAYS.
//
// horde-ad's gather/scatter take an index FUNCTION and the `Concrete` backend
// evaluates it once per position on the host (tgatherZSScalar / tscatterZSScalar,
// src/HordeAd/Core/OpsConcrete.hs:1581-1665).  Here the host layer evaluates
// the function once over all positions at a time and hands over one I64 array
// per indexed dimension; each array is a view over the position space shm, so
// an index that ignores some position variables costs no memory (stride 0).
//
// Out-of-bounds rule (OpsConcrete.hs:923-950): a position with any index
// outside [0, extent) reads zeros in gather and is skipped in scatter.
#include "common.hpp"

using namespace hg;

namespace {

constexpr int kBlock = 256;
constexpr int kMaxIx = 8;

struct IxSpace {
  int nd;                          // merged position dims
  int n_ix;
  int64_t shape[HG_KDIMS];
  int64_t st[kMaxIx][HG_KDIMS];    // strides of each index array over the position dims
  int64_t data_st[HG_KDIMS];       // strides of the data operand over the position dims (scatter)
  const int64_t* ix[kMaxIx];
  int64_t extent[kMaxIx];          // indexed extents of the table
  int64_t table_st[kMaxIx];        // strides of the table over the indexed dims
};

__device__ __forceinline__ bool resolve(const IxSpace& sp, int64_t m, int64_t* table_off, int64_t* data_off) {
  int64_t off[kMaxIx];
#pragma unroll
  for (int k = 0; k < kMaxIx; ++k) off[k] = 0;
  int64_t doff = 0;
  int64_t r = m;
  for (int i = sp.nd - 1; i >= 0; --i) {
    int64_t c;
    if (i > 0) {
      int64_t q = r / sp.shape[i];
      c = r - q * sp.shape[i];
      r = q;
    } else {
      c = r;
    }
    doff += c * sp.data_st[i];
#pragma unroll
    for (int k = 0; k < kMaxIx; ++k)
      if (k < sp.n_ix) off[k] += c * sp.st[k][i];
  }
  bool ok = true;
  int64_t t = 0;
#pragma unroll
  for (int k = 0; k < kMaxIx; ++k) {
    if (k < sp.n_ix) {
      int64_t v = sp.ix[k][off[k]];
      ok = ok && v >= 0 && v < sp.extent[k];
      t += v * sp.table_st[k];
    }
  }
  *table_off = t;
  *data_off = doff;
  return ok;
}

// out dense [M, N]; src inner part described by `inner` (operand 0 = src strides over shn).
template <typename T>
__global__ void __launch_bounds__(kBlock) k_gather(IxSpace sp, Dims inner, int64_t M, int64_t N, const T* __restrict__ src, T* __restrict__ out) {
  int64_t total = M * N;
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += step) {
    int64_t m = N == 1 ? i : i / N;
    int64_t n = N == 1 ? 0 : i - m * N;
    int64_t toff, doff;
    bool ok = resolve(sp, m, &toff, &doff);
    T v = T(0);
    if (ok) {
      int64_t io[1];
      decompose<1>(inner, n, io);
      v = src[toff + io[0]];
    }
    out[i] = v;
  }
}

template <typename T> struct atomic_ok { static constexpr bool value = false; };
template <> struct atomic_ok<double> { static constexpr bool value = true; };
template <> struct atomic_ok<float> { static constexpr bool value = true; };
template <> struct atomic_ok<int32_t> { static constexpr bool value = true; };
template <> struct atomic_ok<int64_t> { static constexpr bool value = true; };

template <typename T>
__device__ __forceinline__ void atomic_add(T* p, T v) {
  if constexpr (sizeof(T) == 8 && !std::is_floating_point<T>::value) {
    atomicAdd(reinterpret_cast<unsigned long long*>(p), (unsigned long long)v);
  } else if constexpr (std::is_floating_point<T>::value) {
    unsafeAtomicAdd(p, v);
  } else {
    atomicAdd(p, v);
  }
}

// src is a view [M (position dims), N (inner dims)]; out dense [P, N], zeroed.
template <typename T, bool INJECTIVE>
__global__ void __launch_bounds__(kBlock) k_scatter(IxSpace sp, Dims inner, int64_t M, int64_t N, const T* __restrict__ src, T* __restrict__ out) {
  int64_t total = M * N;
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += step) {
    int64_t m = N == 1 ? i : i / N;
    int64_t n = N == 1 ? 0 : i - m * N;
    int64_t toff, doff;
    bool ok = resolve(sp, m, &toff, &doff);
    if (ok) {
      int64_t io[1];
      decompose<1>(inner, n, io);
      T v = src[doff + io[0]];
      if constexpr (INJECTIVE) out[toff + n] = v;
      else atomic_add<T>(&out[toff + n], v);
    }
  }
}

int build_space(hgpu_ctx* ctx, const char* who, int n_ix, const hgpu_array* const* ix, int rank_m, const int64_t* shm,
                const int64_t* data_st, IxSpace* sp) {
  if (n_ix < 0 || n_ix > kMaxIx) return fail(ctx, HGPU_ERR_UNSUPPORTED, "%s: %d index arrays (at most %d)", who, n_ix, kMaxIx);
  int64_t zero[HGPU_MAX_RANK] = {0};
  // merge position dims jointly over all index arrays and the data operand
  const int64_t* sts[kMaxIx + 1];
  for (int k = 0; k < n_ix; ++k) {
    const hgpu_array* a = ix[k];
    if (!a || a->dtype != HGPU_I64) return fail(ctx, HGPU_ERR_INVALID, "%s: index array %d is not I64", who, k);
    if (a->rank != rank_m) return fail(ctx, HGPU_ERR_INVALID, "%s: index array %d has rank %d, positions have rank %d", who, k, a->rank, rank_m);
    for (int i = 0; i < rank_m; ++i)
      if (a->shape[i] != shm[i]) return fail(ctx, HGPU_ERR_INVALID, "%s: index array %d differs from shm in dim %d", who, k, i);
    sts[k] = a->strides;
  }
  sts[n_ix] = data_st ? data_st : zero;
  // collapse() handles 4 operands; do the merge here for up to kMaxIx + 1.
  int nops = n_ix + 1;
  sp->nd = 0;
  sp->n_ix = n_ix;
  for (int i = 0; i < rank_m; ++i) {
    if (shm[i] == 1) continue;
    bool merged = false;
    if (sp->nd > 0) {
      int p = sp->nd - 1;
      bool ok = true;
      for (int k = 0; k < nops; ++k) {
        int64_t prev = k < n_ix ? sp->st[k][p] : sp->data_st[p];
        if (prev != sts[k][i] * shm[i]) { ok = false; break; }
      }
      if (ok) {
        sp->shape[p] *= shm[i];
        for (int k = 0; k < n_ix; ++k) sp->st[k][p] = sts[k][i];
        sp->data_st[p] = sts[n_ix][i];
        merged = true;
      }
    }
    if (!merged) {
      if (sp->nd == HG_KDIMS) return fail(ctx, HGPU_ERR_UNSUPPORTED, "%s: more than %d merged position dims", who, HG_KDIMS);
      sp->shape[sp->nd] = shm[i];
      for (int k = 0; k < n_ix; ++k) sp->st[k][sp->nd] = sts[k][i];
      sp->data_st[sp->nd] = sts[n_ix][i];
      sp->nd++;
    }
  }
  if (sp->nd == 0) {
    sp->nd = 1;
    sp->shape[0] = 1;
    for (int k = 0; k < n_ix; ++k) sp->st[k][0] = 0;
    sp->data_st[0] = 0;
  }
  for (int k = 0; k < kMaxIx; ++k) {
    sp->ix[k] = k < n_ix ? (const int64_t*)data_ptr(ix[k]) : nullptr;
    sp->extent[k] = 0;
    sp->table_st[k] = 0;
  }
  return HGPU_OK;
}

}  // namespace

extern "C" {

int hgpu_gather(hgpu_ctx* ctx, const hgpu_array* src, int n_ix, const hgpu_array* const* ix, int rank_m, const int64_t* shm, hgpu_array** out) {
  if (!ctx || !src || !out || rank_m < 0) return HGPU_ERR_INVALID;
  if (n_ix > src->rank) return fail(ctx, HGPU_ERR_INVALID, "gather: %d indices into rank %d", n_ix, src->rank);
  int rank_n = src->rank - n_ix;
  if (rank_m + rank_n > HGPU_MAX_RANK) return fail(ctx, HGPU_ERR_INVALID, "gather: result rank too large");
  int64_t osh[HGPU_MAX_RANK];
  int64_t M = 1, N = 1;
  for (int i = 0; i < rank_m; ++i) { osh[i] = shm[i]; M *= shm[i]; }
  for (int i = 0; i < rank_n; ++i) { osh[rank_m + i] = src->shape[n_ix + i]; N *= src->shape[n_ix + i]; }
  IxSpace sp;
  int rc = build_space(ctx, "gather", n_ix, ix, rank_m, shm, nullptr, &sp);
  if (rc) return rc;
  bool empty_table = false;
  for (int k = 0; k < n_ix; ++k) {
    sp.extent[k] = src->shape[k];
    sp.table_st[k] = src->strides[k];
    if (src->shape[k] == 0) empty_table = true;
  }
  hgpu_array* o = nullptr;
  if (M * N == 0 || empty_table) {
    rc = new_zeros(ctx, src->dtype, rank_m + rank_n, osh, &o);
    if (rc) return rc;
    *out = o;
    return HGPU_OK;
  }
  rc = new_dense(ctx, src->dtype, rank_m + rank_n, osh, &o);
  if (rc) return rc;
  const int64_t* is[1] = {src->strides + n_ix};
  Dims inner;
  if (!collapse(rank_n, src->shape + n_ix, 1, is, &inner)) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "gather: too many inner dims"); }
  {
    const char* label = "gather";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[120];
      snprintf(buf, sizeof buf, "gather[es%d,M%lld,N%lld,ix%d]", (int)dtype_size(src->dtype), (long long)M, (long long)N, n_ix);
      label = ctx->label_pool.insert(buf).first->c_str();
    }
    LaunchGuard lg(ctx, label, 2.0 * M * N * dtype_size(src->dtype) + 8.0 * M * n_ix, 0);
    unsigned g = grid_for(M * N, kBlock, ctx->num_cu * 8);
    switch (dtype_size(src->dtype)) {
      case 8: hipLaunchKernelGGL(k_gather<uint64_t>, dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const uint64_t*)data_ptr(src), (uint64_t*)data_ptr(o)); break;
      case 4: hipLaunchKernelGGL(k_gather<uint32_t>, dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const uint32_t*)data_ptr(src), (uint32_t*)data_ptr(o)); break;
      case 2: hipLaunchKernelGGL(k_gather<uint16_t>, dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const uint16_t*)data_ptr(src), (uint16_t*)data_ptr(o)); break;
      default: hipLaunchKernelGGL(k_gather<uint8_t>, dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const uint8_t*)data_ptr(src), (uint8_t*)data_ptr(o)); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "gather"); }
  }
  *out = o;
  return HGPU_OK;
}

int hgpu_scatter_add(hgpu_ctx* ctx, const hgpu_array* src, int n_ix, const hgpu_array* const* ix, int rank_m, const int64_t* shp, int flags, hgpu_array** out) {
  if (!ctx || !src || !out || rank_m < 0 || n_ix < 0) return HGPU_ERR_INVALID;
  if (rank_m > src->rank) return fail(ctx, HGPU_ERR_INVALID, "scatter: %d position dims in rank %d", rank_m, src->rank);
  int rank_n = src->rank - rank_m;
  if (n_ix + rank_n > HGPU_MAX_RANK) return fail(ctx, HGPU_ERR_INVALID, "scatter: result rank too large");
  if (src->dtype == HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "scatter: Bool arrays have no sum");
  int64_t osh[HGPU_MAX_RANK];
  int64_t M = 1, N = 1;
  for (int i = 0; i < n_ix; ++i) osh[i] = shp[i];
  for (int i = 0; i < rank_m; ++i) M *= src->shape[i];
  for (int i = 0; i < rank_n; ++i) { osh[n_ix + i] = src->shape[rank_m + i]; N *= src->shape[rank_m + i]; }
  hgpu_array* o = nullptr;
  int rc = new_zeros(ctx, src->dtype, n_ix + rank_n, osh, &o);
  if (rc) return rc;
  if (M * N == 0 || nelem(o) == 0) { *out = o; return HGPU_OK; }
  IxSpace sp;
  rc = build_space(ctx, "scatter", n_ix, ix, rank_m, src->shape, src->strides, &sp);
  if (rc) { hgpu_release(o); return rc; }
  for (int k = 0; k < n_ix; ++k) {
    sp.extent[k] = shp[k];
    sp.table_st[k] = o->strides[k];
  }
  const int64_t* is[1] = {src->strides + rank_m};
  Dims inner;
  if (!collapse(rank_n, src->shape + rank_m, 1, is, &inner)) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "scatter: too many inner dims"); }
  bool inj = (flags & 1) != 0;
  bool launched = false;
  {
    LaunchGuard lg(ctx, inj ? "scatter_store" : "scatter_atomic", 2.0 * M * N * dtype_size(src->dtype) + 8.0 * M * n_ix, (double)M * N);
    unsigned g = grid_for(M * N, kBlock, ctx->num_cu * 8);
    HG_DISPATCH_DTYPE(src->dtype, T, {
      if constexpr (atomic_ok<T>::value) {
        if (inj) hipLaunchKernelGGL((k_scatter<T, true>), dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const T*)data_ptr(src), (T*)data_ptr(o));
        else hipLaunchKernelGGL((k_scatter<T, false>), dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const T*)data_ptr(src), (T*)data_ptr(o));
        launched = true;
      } else {
        if (inj) { hipLaunchKernelGGL((k_scatter<T, true>), dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const T*)data_ptr(src), (T*)data_ptr(o)); launched = true; }
      }
    });
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "scatter"); }
  }
  if (!launched) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "scatter: no accumulating kernel for dtype %d", src->dtype); }
  *out = o;
  return HGPU_OK;
}

}  // extern "C"
