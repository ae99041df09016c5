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
//
// Scatter-add adds colliding positions in ascending row-major order of the
// positions, the reference's own order (tscatterZSScalar walks `shsEnum shm`,
// OpsConcrete.hs:1581-1619), and without atomics: the positions are sorted by
// destination with a stable radix sort, and every destination's run is summed
// front to back by one lane per element.  Results do not depend on the run and,
// for floating point, carry the rounding of that very order as long as no
// destination is hit more than 256 times; a longer run is summed in segments
// of 256 entries (each front to back) whose sums are added in ascending order,
// so that the serial part of a scatter into a handful of cells stays bounded.
#include "common.hpp"

#include <rocprim/rocprim.hpp>

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

// Slices that are contiguous in the table and a whole number of V-sized units
// (16 bytes when sizes and strides allow): a lane moves one unit, so the lanes
// of a slice read consecutive units of one place in the table, and the position
// of a slice is resolved by each of its lanes from the same few index entries
// (one cache line).  `units` = units per slice; tbl_unit = table element size /
// sizeof(V) as a fraction num/den folded into the offsets by the caller:
// table offsets arrive in elements and are scaled by es_over_v (elements per unit
// inverted: unit offset = element offset / elems_per_unit, exact by the caller's checks).
template <typename V>
__global__ void __launch_bounds__(kBlock) k_gather_units(IxSpace sp, int64_t M, int64_t units, int64_t elems_per_unit, const V* __restrict__ src, V* __restrict__ out) {
  const int64_t total = M * units;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  const bool small = total < (int64_t)0x7fffffff;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += step) {
    int64_t m, u;
    if (small) {
      const uint32_t q = (uint32_t)i / (uint32_t)units;
      m = q;
      u = (uint32_t)i - q * (uint32_t)units;
    } else {
      m = i / units;
      u = i - m * units;
    }
    int64_t toff, doff;
    const bool ok = resolve(sp, m, &toff, &doff);
    V v{};
    if (ok) v = src[toff / elems_per_unit + u];
    out[i] = v;
  }
}

// src is a view [M (position dims), N (inner dims)]; out dense [P, N], zeroed.
// Distinct positions go to distinct places (the caller's promise): plain stores.
template <typename T>
__global__ void __launch_bounds__(kBlock) k_scatter_store(IxSpace sp, Dims inner, int64_t M, int64_t N, const T* __restrict__ src, T* __restrict__ out) {
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
      out[toff + n] = src[doff + io[0]];
    }
  }
}

// Entries of one run that a lane adds front to back.  A destination hit by at most
// kSeg positions is summed in exactly the reference's order; a longer run is cut,
// from its first entry, into segments of kSeg entries that separate lanes add up,
// and the segment sums are then added in ascending order (k_scatter_combine).
constexpr int kSeg = 256;

// key[m] = where position m's slice starts in out (the same for colliding
// positions), or `skip` when an index is out of bounds; val[m] = m.  Also clears
// long_head, one entry per kSeg sorted entries (see k_scatter_runs).
template <typename K>
__global__ void __launch_bounds__(kBlock) k_scatter_keys(IxSpace sp, int64_t M, K skip, K* __restrict__ key, uint32_t* __restrict__ val,
                                                         uint32_t* __restrict__ long_head, int64_t n_buckets) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t m = (int64_t)blockIdx.x * kBlock + threadIdx.x; m < M; m += step) {
    int64_t toff, doff;
    bool ok = resolve(sp, m, &toff, &doff);
    key[m] = ok ? (K)toff : skip;
    val[m] = (uint32_t)m;
    if (m < n_buckets) long_head[m] = 0;
  }
}

// the data operand's offset of position m (resolve() without the index arrays)
__device__ __forceinline__ int64_t data_offset(const IxSpace& sp, int64_t m) {
  int64_t doff = 0, r = m;
  for (int i = sp.nd - 1; i >= 0; --i) {
    int64_t c = r;
    if (i > 0) { int64_t q = r / sp.shape[i]; c = r - q * sp.shape[i]; r = q; }
    doff += c * sp.data_st[i];
  }
  return doff;
}

// key / val sorted by key, equal keys in ascending position order.  One lane per
// (sorted entry, inner element); a lane works when its entry starts a SEGMENT:
// the first entry of a run, or an entry a multiple of kSeg entries after it.
// It adds the segment's slices front to back, starting from zero.  A run of one
// segment is written to `out` at once.  The segment sums of a longer run go to
// `part`, two places per bucket of kSeg sorted entries -- a bucket holds at most
// one first segment of a long run (place 1) and one later segment (place 0),
// because segments of one run start kSeg entries apart and a long run is
// longer than a bucket -- and long_head[bucket] remembers where the run starts.
// Is sorted entry `at` (key k, not the first entry of its run) the start of a later segment of a long run?
template <typename K>
__device__ __forceinline__ bool later_segment_start(const K* __restrict__ key, int64_t at, K k) {
  if (at < kSeg || key[at - kSeg] != k) return false;   // fewer than kSeg entries of this run before this one
  int64_t lo = 0, hi = at - kSeg;                       // the run's first entry: the first key that is not smaller
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (key[mid] < k) lo = mid + 1; else hi = mid;
  }
  return (at - lo) % kSeg == 0;
}

// Adds entries j .. end - 1 of the run with key k to acc, front to back; stops at the first other key.
// Keys, positions and values of four entries are in flight together.  Returns the first entry not added.
template <typename T, typename K>
__device__ __forceinline__ int64_t add_run(const IxSpace& sp, const K* __restrict__ key, const uint32_t* __restrict__ val, const T* __restrict__ src, int64_t io,
                                           K k, int64_t j, int64_t end, int64_t M, T* acc) {
  while (j < end) {
    const int64_t j1 = j + 1 < M ? j + 1 : M - 1, j2 = j + 2 < M ? j + 2 : M - 1, j3 = j + 3 < M ? j + 3 : M - 1;
    const K k0 = key[j], k1 = key[j1], k2 = key[j2], k3 = key[j3];
    const uint32_t p0 = val[j], p1 = val[j1], p2 = val[j2], p3 = val[j3];
    if (k0 != k) return j;
    const bool m1 = j + 1 < end && k1 == k, m2 = m1 && j + 2 < end && k2 == k, m3 = m2 && j + 3 < end && k3 == k;
    const T v0 = src[data_offset(sp, (int64_t)p0) + io];
    const T v1 = src[data_offset(sp, (int64_t)(m1 ? p1 : p0)) + io];
    const T v2 = src[data_offset(sp, (int64_t)(m2 ? p2 : p0)) + io];
    const T v3 = src[data_offset(sp, (int64_t)(m3 ? p3 : p0)) + io];
    *acc = (T)(*acc + v0);
    if (!m1) return j + 1;
    *acc = (T)(*acc + v1);
    if (!m2) return j + 2;
    *acc = (T)(*acc + v2);
    if (!m3) return j + 3;
    *acc = (T)(*acc + v3);
    j += 4;
  }
  return j;
}

// key / val sorted by key, equal keys in ascending position order.  One lane per
// (sorted entry, inner element); a lane works when its entry starts a SEGMENT:
// the first entry of a run, or an entry a multiple of kSeg entries after it.
// It adds the segment's slices front to back, starting from zero.  A run of one
// segment is written to `out` at once.  The segment sums of a longer run go to
// `part`, two places per bucket of kSeg sorted entries -- a bucket holds at most
// one first segment of a long run (place 1) and one later segment (place 0),
// because segments of one run start kSeg entries apart and a long run is
// longer than a bucket -- and long_head[bucket] remembers where the run starts.
template <typename T, typename K>
__global__ void __launch_bounds__(kBlock) k_scatter_runs(IxSpace sp, Dims inner, int64_t M, int64_t N, K skip, const K* __restrict__ key,
                                                         const uint32_t* __restrict__ val, const T* __restrict__ src, T* __restrict__ out,
                                                         T* __restrict__ part, uint32_t* __restrict__ long_head) {
  int64_t total = M * N;
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += step) {
    int64_t at = i / N;
    int64_t n = i - at * N;
    const K k = key[at];
    if (k == skip) continue;
    const bool head = at == 0 || key[at - 1] != k;
    if (!head && !later_segment_start(key, at, k)) continue;
    int64_t io[1];
    decompose<1>(inner, n, io);
    const int64_t end = at + kSeg < M ? at + kSeg : M;
    T acc = T(0);
    const int64_t j = add_run(sp, key, val, src, io[0], k, at, end, M, &acc);
    const bool more = j < M && key[j] == k;
    if (head && !more) {
      out[(int64_t)k + n] = acc;
    } else {
      const int64_t q = at / kSeg;
      part[(q * 2 + (head ? 1 : 0)) * N + n] = acc;
      if (head && n == 0) long_head[q] = (uint32_t)(at - q * kSeg) + 1;
    }
  }
}

// The same for single elements (N = 1), a wavefront per 64 sorted entries: EVERY
// lane fetches its entry's value (coalesced keys and positions, one gather), and
// the lane at a segment's start then collects the values of the lanes behind it
// through the wavefront, nearest first -- the same order, without a chain of
// dependent loads.  What lies beyond the wavefront's 64 entries it adds itself.
template <typename T, typename K>
__global__ void __launch_bounds__(kBlock) k_scatter_runs1(IxSpace sp, int64_t M, K skip, const K* __restrict__ key, const uint32_t* __restrict__ val,
                                                          const T* __restrict__ src, T* __restrict__ out, T* __restrict__ part, uint32_t* __restrict__ long_head) {
  const int lane = threadIdx.x & 63;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t base = (int64_t)blockIdx.x * kBlock + (threadIdx.x & ~63); base < M; base += step) {   // the same trips for all lanes of a wavefront
    const int64_t at = base + lane;
    const bool valid = at < M;
    const K k = valid ? key[at] : skip;
    const bool live = valid && k != skip;
    const T v = live ? src[data_offset(sp, (int64_t)val[at])] : T(0);
    K before = (K)__shfl_up((unsigned long long)k, 1);
    if (lane == 0) before = at > 0 && valid ? key[at - 1] : (K)~k;
    const bool head = live && (at == 0 || before != k);
    const bool start = head || (live && later_segment_start(key, at, k));
    T acc = (T)(T(0) + v);
    bool open = start;                      // still inside the run
    int reach = 1;                          // entries of the segment this lane has added
    for (int d = 1; d < 64; ++d) {
      const K kd = (K)__shfl_down((unsigned long long)k, d);
      const T vd = __shfl_down(v, d);
      const bool take = open && lane + d < 64 && kd == k;      // (a segment is longer than a wavefront's share, so its end is not met here)
      if (open && lane + d < 64 && !take) open = false;
      if (take) { acc = (T)(acc + vd); reach = d + 1; }
      if (!__any(take)) break;
    }
    if (!start) continue;
    int64_t j = at + reach;
    if (open && lane + reach >= 64) {       // the run goes on behind the wavefront's entries
      const int64_t end = at + kSeg < M ? at + kSeg : M;
      j = add_run(sp, key, val, src, (int64_t)0, k, j, end, M, &acc);
    }
    const bool more = j < M && key[j] == k && j - at >= kSeg;
    if (head && !more) {
      out[(int64_t)k] = acc;
    } else {
      const int64_t q = at / kSeg;
      part[q * 2 + (head ? 1 : 0)] = acc;
      if (head) long_head[q] = (uint32_t)(at - q * kSeg) + 1;
    }
  }
}

// One lane per (bucket, inner element): where a long run starts in the bucket,
// its segment sums are added in ascending order and written to `out`.
template <typename T, typename K>
__global__ void __launch_bounds__(kBlock) k_scatter_combine(int64_t M, int64_t N, int64_t n_buckets, const K* __restrict__ key, const T* __restrict__ part,
                                                            const uint32_t* __restrict__ long_head, T* __restrict__ out) {
  int64_t total = n_buckets * N;
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += step) {
    int64_t q = N == 1 ? i : i / N;
    int64_t n = N == 1 ? 0 : i - q * N;
    const uint32_t h = long_head[q];
    if (!h) continue;
    const int64_t at = q * kSeg + (int64_t)h - 1;
    const K k = key[at];
    T acc = part[(q * 2 + 1) * N + n];
    for (int64_t a = at + kSeg; a < M && key[a] == k; a += kSeg) acc = (T)(acc + part[(a / kSeg) * 2 * N + n]);
    out[(int64_t)k + n] = acc;
  }
}

// k_scatter_keys -> stable radix sort by key -> k_scatter_runs -> k_scatter_combine.
// bufs: keys (in, out), positions (in, out), sort workspace, segment sums, long_head.
template <typename K>
hipError_t scatter_sorted(hgpu_ctx* ctx, const IxSpace& sp, const Dims& inner, int64_t M, int64_t N, const hgpu_array* src, hgpu_array* o, int* rc_out) {
  const K skip = (K)nelem(o);   // larger than every slice start
  int end_bit = 1;
  while (end_bit < (int)(8 * sizeof(K)) && ((uint64_t)skip >> end_bit) != 0) ++end_bit;
  const int64_t n_buckets = (M + kSeg - 1) / kSeg;
  const size_t es = dtype_size(src->dtype);
  hgpu_buffer *kb = nullptr, *vb = nullptr, *tb = nullptr, *pb = nullptr, *hb = nullptr;
  auto drop = [&] { for (hgpu_buffer* b : {kb, vb, tb, pb, hb}) if (b) buffer_release(b); };
  int rc = buffer_alloc(ctx, (size_t)M * 2 * sizeof(K), &kb);
  if (!rc) rc = buffer_alloc(ctx, (size_t)M * 8, &vb);
  if (!rc) rc = buffer_alloc(ctx, (size_t)n_buckets * 2 * (size_t)N * es, &pb);
  if (!rc) rc = buffer_alloc(ctx, (size_t)n_buckets * 4, &hb);
  if (rc) { drop(); *rc_out = rc; return hipSuccess; }
  K* key_in = (K*)kb->ptr;
  K* key_out = key_in + M;
  uint32_t* val_in = (uint32_t*)vb->ptr;
  uint32_t* val_out = val_in + M;
  uint32_t* long_head = (uint32_t*)hb->ptr;
  size_t temp_bytes = 0;
  hipError_t e = rocprim::radix_sort_pairs(nullptr, temp_bytes, key_in, key_out, val_in, val_out, (size_t)M, 0, (unsigned)end_bit, ctx->stream);
  if (e == hipSuccess) {
    rc = buffer_alloc(ctx, temp_bytes > 0 ? temp_bytes : 1, &tb);
    if (rc) { drop(); *rc_out = rc; return hipSuccess; }
    hipLaunchKernelGGL(k_scatter_keys<K>, dim3(grid_for(M, kBlock, ctx->num_cu * 8)), dim3(kBlock), 0, ctx->stream, sp, M, skip, key_in, val_in, long_head, n_buckets);
    e = rocprim::radix_sort_pairs(tb->ptr, temp_bytes, key_in, key_out, val_in, val_out, (size_t)M, 0, (unsigned)end_bit, ctx->stream);
    if (e == hipSuccess) {
      unsigned g = grid_for(M * N, kBlock, ctx->num_cu * 8);
      if (N == 1) {
        HG_DISPATCH_DTYPE(src->dtype, T, hipLaunchKernelGGL((k_scatter_runs1<T, K>), dim3(g), dim3(kBlock), 0, ctx->stream, sp, M, skip, (const K*)key_out, (const uint32_t*)val_out,
                                                            (const T*)data_ptr(src), (T*)data_ptr(o), (T*)pb->ptr, long_head));
      } else {
        HG_DISPATCH_DTYPE(src->dtype, T, hipLaunchKernelGGL((k_scatter_runs<T, K>), dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, skip, (const K*)key_out, (const uint32_t*)val_out,
                                                            (const T*)data_ptr(src), (T*)data_ptr(o), (T*)pb->ptr, long_head));
      }
      e = hipGetLastError();
    }
    if (e == hipSuccess) {
      unsigned g = grid_for(n_buckets * N, kBlock, ctx->num_cu * 8);
      HG_DISPATCH_DTYPE(src->dtype, T, hipLaunchKernelGGL((k_scatter_combine<T, K>), dim3(g), dim3(kBlock), 0, ctx->stream, M, N, n_buckets, (const K*)key_out, (const T*)pb->ptr,
                                                          (const uint32_t*)long_head, (T*)data_ptr(o)));
      e = hipGetLastError();
    }
  }
  drop();
  *rc_out = HGPU_OK;
  return e;
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
      label = intern_label(ctx, buf);
    }
    LaunchGuard lg(ctx, label, 2.0 * M * N * dtype_size(src->dtype) + 8.0 * M * n_ix, 0);
    // contiguous slices of whole 16-byte (or 8-byte) units: one unit per lane
    const int64_t es = (int64_t)dtype_size(src->dtype);
    int unit = 0;
    if (N > 1 && inner.nd == 1 && inner.st[0][0] == 1) {
      for (int cand : {16, 8}) {
        if (cand <= es || (N * es) % cand != 0 || ((uintptr_t)data_ptr(src)) % (uintptr_t)cand != 0) continue;
        bool ok = true;
        for (int k = 0; k < n_ix && ok; ++k) ok = (src->strides[k] * es) % cand == 0;
        if (ok) { unit = cand; break; }
      }
    }
    if (unit) {
      const int64_t units = N * es / unit, epu = unit / es;
      unsigned g = grid_for(M * units, kBlock, ctx->num_cu * 16);
      if (unit == 16) hipLaunchKernelGGL(k_gather_units<uint4>, dim3(g), dim3(kBlock), 0, ctx->stream, sp, M, units, epu, (const uint4*)data_ptr(src), (uint4*)data_ptr(o));
      else hipLaunchKernelGGL(k_gather_units<uint64_t>, dim3(g), dim3(kBlock), 0, ctx->stream, sp, M, units, epu, (const uint64_t*)data_ptr(src), (uint64_t*)data_ptr(o));
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "gather"); }
      *out = o;
      return HGPU_OK;
    }
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
  if (inj) {
    LaunchGuard lg(ctx, "scatter_store", 2.0 * M * N * dtype_size(src->dtype) + 8.0 * M * n_ix, 0);
    unsigned g = grid_for(M * N, kBlock, ctx->num_cu * 8);
    HG_DISPATCH_DTYPE(src->dtype, T, hipLaunchKernelGGL((k_scatter_store<T>), dim3(g), dim3(kBlock), 0, ctx->stream, sp, inner, M, N, (const T*)data_ptr(src), (T*)data_ptr(o)));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "scatter"); }
    *out = o;
    return HGPU_OK;
  }
  // sort the positions by destination (stable: colliding positions stay in ascending order), then sum every run in that order
  if (M >= (int64_t)1 << 32) { hgpu_release(o); return fail(ctx, HGPU_ERR_UNSUPPORTED, "scatter: %lld positions", (long long)M); }
  hipError_t e;
  {
    LaunchGuard lg(ctx, "scatter_sorted", 2.0 * M * N * dtype_size(src->dtype) + 8.0 * M * n_ix, (double)M * N);
    // destinations that fit 32 bits sort as 32-bit keys: half the bytes per sorting pass
    e = nelem(o) < (int64_t)0xffffffff ? scatter_sorted<uint32_t>(ctx, sp, inner, M, N, src, o, &rc) : scatter_sorted<uint64_t>(ctx, sp, inner, M, N, src, o, &rc);
  }
  if (rc) { hgpu_release(o); return rc; }
  if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "scatter"); }
  *out = o;
  return HGPU_OK;
}

}  // extern "C"
