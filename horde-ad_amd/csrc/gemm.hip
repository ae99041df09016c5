// Matrix-core (MFMA) path of hgpu_contract.
//
// horde-ad's `Concrete` backend computes matmul2 as "dot over the innermost
// dim of two broadcast views" (src/HordeAd/Core/OpsConcrete.hs:237-242) and
// convolutions as the same contraction over gathered windows
// (test/simplified/TestMnistPP.hs:735).  Seen through strides these are all ONE
// pattern:  every kept dim advances only A (an "M" dim), only B (an "N" dim) or
// both (a batch dim), and every reduced dim advances both (a "K" dim).  Then
//     A[m, k] sits at  offAm(m) + offAk(k),   B[n, k] at  offBn(n) + offBk(k),
//     C[m, n] at  offCm(m) + offCn(n),
// with m, n, k multi-indices -- a matrix product whose operands are addressed
// through separable offset maps.  No operand is copied or re-laid-out: the
// im2col "patch matrix" of a convolution exists only as such a map.
//
// Kernel: 256 threads = 4 wavefronts, K-step 16; the block tile ranges from
// 128x128 (wavefronts 2x2, each 4x4 MFMA tiles of 16x16) down to 256x16 / 16x256
// and 32x32 for skinny or tiny outputs (a convolution with 16 output channels
// has N = 16).  v_mfma_f64_16x16x4_f64 / v_mfma_f32_16x16x4_f32, accumulators
// in registers.
// Operand tiles are staged through LDS in [k][m] order (one element of padding
// per row keeps both the transposing stores and the MFMA-fragment loads free
// of bank conflicts); the global loads of tile t+1 are issued before the MFMAs
// of tile t.  Lanes run along whichever of m or k is contiguous in memory, so
// loads coalesce for both plain and transposed operands.  Tiles are numbered
// so that each XCD (blockIdx mod 8) works on a contiguous run of tiles and its
// L2 sees neighbouring rows of A.  Small outputs with long K are split along K
// into partial products summed by a second launch (fixed order: reproducible).
#include <algorithm>
#include <cmath>

#include "gemm_kernel.hpp"

using namespace hg;
using namespace hg::gemm;

namespace {

// K offset tables of both operands, Kp >= K entries: entries past K repeat the
// last four valid k (so that a 4-element vector load at a padded entry stays
// inside the operand).
__global__ void k_koff(Group k, int64_t K, int64_t Kp, int64_t* __restrict__ ka, int64_t* __restrict__ kb) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < Kp) {
    int64_t idx = i;
    if (i >= K) {
      idx = K >= 4 ? K - 4 + (i & 3) : K - 1;
      if (idx > K - 1) idx = K - 1;
    }
    int64_t a, b, c;
    group_off(k, idx, &a, &b, &c);
    ka[i] = a;
    kb[i] = b;
  }
}

// Sums the split-K partials: out[i] = sum_s part[s * stride + i].  A block owns
// OPB consecutive outputs; its 256 / OPB groups of lanes each take every
// (256 / OPB)-th partial (coalesced rows of OPB elements), several loads in
// flight at a time, and combine through LDS in a fixed order.  Few outputs get
// the narrow blocks: more of them, and fewer partials for a lane to walk through.
template <typename T, int OPB>
__global__ void __launch_bounds__(256) k_sum_partials(int64_t n, int S, int64_t stride, const T* __restrict__ part, T* __restrict__ out, int64_t n1, T* __restrict__ out2) {
  constexpr int G = 256 / OPB;
  __shared__ T red[G][OPB + 1];
  const int ol = threadIdx.x % OPB, g = threadIdx.x / OPB;
  for (int64_t base = (int64_t)blockIdx.x * OPB; base < n; base += (int64_t)gridDim.x * OPB) {
    int64_t i = base + ol;
    T acc = T(0);
    if (i < n) {
#pragma unroll 8
      for (int s = g; s < S; s += G) acc += part[(int64_t)s * stride + i];
    }
    red[g][ol] = acc;
    __syncthreads();
    if (g == 0 && i < n) {
      T t = red[0][ol];
#pragma unroll
      for (int k = 1; k < G; ++k) t += red[k][ol];
      if (i < n1) out[i] = t;
      else out2[i - n1] = t;
    }
    __syncthreads();
  }
}

// The same sum for a handful of partials (S <= 8), where the blocks above would
// leave most of their lane groups without a partial: one output per lane, the
// partials added in the same order (0 + p0 + p1 + ...), four loads in flight.
template <typename T>
__global__ void __launch_bounds__(256) k_sum_partials_few(int64_t n, int S, int64_t stride, const T* __restrict__ part, T* __restrict__ out, int64_t n1, T* __restrict__ out2) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const T* p = part + i;
    T acc = T(0);
    int s = 0;
    for (; s + 3 < S; s += 4) {
      const T a = p[(int64_t)s * stride], b = p[(int64_t)(s + 1) * stride], c = p[(int64_t)(s + 2) * stride], d = p[(int64_t)(s + 3) * stride];
      acc += a;
      acc += b;
      acc += c;
      acc += d;
    }
    if (s + 1 < S) {
      const T a = p[(int64_t)s * stride], b = p[(int64_t)(s + 1) * stride];
      acc += a;
      acc += b;
      s += 2;
    }
    if (s < S) acc += p[(int64_t)s * stride];
    if (i < n1) out[i] = acc;
    else out2[i - n1] = acc;
  }
}

// Outputs [0, n1) go to `out`, the rest to `out2` (two results whose partial sums one kernel wrote side by side).
template <typename T>
void launch_sum_partials(hgpu_ctx* ctx, int64_t n, int S, const T* part, T* out, int64_t n1 = -1, T* out2 = nullptr) {
  if (n1 < 0) n1 = n;
  if (S <= 8)
    hipLaunchKernelGGL((k_sum_partials_few<T>), dim3(grid_for(n, 256, ctx->num_cu * 8)), dim3(256), 0, ctx->stream, n, S, n, part, out, n1, out2);
  else if (sizeof(T) == 4)   // rows of 32 floats are whole 128-byte lines (16384 outputs x 270 partials: 12.9 us with rows of 8, 7.1 us with rows of 32)
    hipLaunchKernelGGL((k_sum_partials<T, 32>), dim3(grid_for(n, 32, ctx->num_cu * 8)), dim3(256), 0, ctx->stream, n, S, n, part, out, n1, out2);
  else if (n <= 32768 && S >= 32)
    hipLaunchKernelGGL((k_sum_partials<T, 8>), dim3(grid_for(n, 8, ctx->num_cu * 8)), dim3(256), 0, ctx->stream, n, S, n, part, out, n1, out2);
  else
    hipLaunchKernelGGL((k_sum_partials<T, 32>), dim3(grid_for(n, 32, ctx->num_cu * 8)), dim3(256), 0, ctx->stream, n, S, n, part, out, n1, out2);
}

// Appends dim (extent e, strides a, b, c) to a group, merging with the previous dim when all strides allow.
bool push_dim(Group& g, int64_t e, int64_t a, int64_t b, int64_t c) {
  if (e == 1) return true;
  if (g.nd > 0) {
    int p = g.nd - 1;
    if (g.sa[p] == a * e && g.sb[p] == b * e && g.sc[p] == c * e) {
      g.shape[p] *= e;
      g.sa[p] = a;
      g.sb[p] = b;
      g.sc[p] = c;
      return true;
    }
  }
  if (g.nd == GD) return false;
  g.shape[g.nd] = e;
  g.sa[g.nd] = a;
  g.sb[g.nd] = b;
  g.sc[g.nd] = c;
  g.nd++;
  return true;
}

void finish(Group& g) {
  if (g.nd == 0) {
    g.nd = 1;
    g.shape[0] = 1;
    g.sa[0] = g.sb[0] = g.sc[0] = 0;
  }
  for (int i = g.nd; i < GD; ++i) {
    g.shape[i] = 1;
    g.sa[i] = g.sb[i] = g.sc[i] = 0;
  }
}

int64_t total(const Group& g) {
  int64_t n = 1;
  for (int i = 0; i < g.nd; ++i) n *= g.shape[i];
  return n;
}

// True when 16-byte loads along the direction the staging lanes run are safe
// for one operand: unit stride there and an extent that is a multiple of the
// vector, so that the elements of a vector are neighbours in memory.  The
// vectors need element alignment only.
bool vector_ok(size_t es, const Group& run, int run_dim, const int64_t* run_st) {
  const int64_t v = (int64_t)(16 / es);
  return run_st[run_dim] == 1 && run.shape[run_dim] % v == 0;
}
// Products with at most 32 rows or columns: the LDS-free kernel, the small side as N.
int gemm_direct(hgpu_ctx* ctx, GemmParams p, int dtype, const void* pa, const void* pb, hgpu_array* out, bool* handled, int n_terms) {
  if (p.N > 32) {   // swap the roles of the operands: C^T = B A^T
    std::swap(p.m, p.n);
    std::swap(p.M, p.N);
    std::swap(pa, pb);
    for (int t = 0; t < n_terms; ++t) std::swap(p.a_term[t], p.b_term[t]);
    for (Group* g : {&p.m, &p.n, &p.k, &p.bt})
      for (int i = 0; i < GD; ++i) std::swap(g->sa[i], g->sb[i]);
  }
  const int tn = p.N <= 16 ? 1 : 2, tm = p.M <= 16 ? 1 : (p.M <= 32 ? 2 : 4);
  const int64_t tiles = ((p.M + 16 * tm - 1) / (16 * tm)) * ((p.N + 16 * tn - 1) / (16 * tn));
  if (tiles > 0x3fffffff) return HGPU_OK;
  // one wavefront per (tile, K chunk): aim at one per SIMD (more, shorter chunks
  // measured slower: set-up and partial sums per wavefront), chunks of at least 64
  const int64_t want = (int64_t)ctx->num_cu * 4;
  const int64_t out_elems = p.M * p.N * p.BT;
  const int64_t nt = n_terms > 0 ? n_terms : 1;      // products summed by this launch
  int64_t split = 1;
  if (tiles * p.BT * nt * 2 <= want && p.K >= 128) {
    split = (want + tiles * p.BT * nt - 1) / (tiles * p.BT * nt);
    int64_t cap = (int64_t)((double)(p.M + p.N) * p.K * p.BT / (2.0 * out_elems));   // partials stay small next to the operands
    if (cap > 4096) cap = 4096;
    if (split > cap) split = cap;
    if (split > p.K / 64) split = p.K / 64;
    if (split < 1) split = 1;
  }
  p.kchunk = ((p.K + split - 1) / split + 15) / 16 * 16;
  p.term_split = (int)((p.K + p.kchunk - 1) / p.kchunk);
  p.n_terms = n_terms;
  p.split = (int)(p.term_split * nt);                // K chunks of all terms
  split = p.split;
  p.a_kc = p.b_kc = 0;
  p.c_rows_contig = 0;

  const size_t es = dtype_size(dtype);
  const int64_t out_n = nelem(out);
  const void* zero_tab = nullptr;
  int rc = zero_block(ctx, &zero_tab);
  if (rc) return rc;
  hgpu_buffer* koff = nullptr;
  const int64_t Kp = (p.K + 15) / 16 * 16 + 32;   // padded tables (see k_gemm_direct)
  rc = buffer_alloc(ctx, (size_t)Kp * 16, &koff);
  if (rc) return rc;
  hgpu_buffer* part = nullptr;
  if (split > 1) {
    rc = buffer_alloc(ctx, (size_t)out_n * split * es, &part);
    if (rc) { buffer_release(koff); return rc; }
  }
  p.c_split_stride = split > 1 ? out_n : 0;
  int64_t* ka = (int64_t*)koff->ptr;
  int64_t* kb = ka + Kp;
  dim3 grid((unsigned)((tiles * split + 3) / 4), 1, (unsigned)p.BT);
  {
    double flops = 2.0 * p.M * p.N * p.K * p.BT * nt;
    double bytes = (((double)p.M * p.K + (double)p.N * p.K) * nt + (double)p.M * p.N) * p.BT * es;
    const char* label = dtype == HGPU_F64 ? "gemm_f64" : "gemm_f32";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[128];
      snprintf(buf, sizeof buf, "%s[M%lldxN%lldxK%lldxB%lld,s%d,direct,t%dx%d,k%lld:%lld/%lld]", label, (long long)p.M, (long long)p.N, (long long)p.K, (long long)p.BT, (int)split, 16 * tm, 16 * tn, (long long)p.k.shape[p.k.nd - 1], (long long)p.k.sa[p.k.nd - 1], (long long)p.k.sb[p.k.nd - 1]);
      label = intern_label(ctx, buf);
    }
    // the helper launches are timed under their own names, the label times the MFMA kernel alone
    if (p.k.nd > 1) {
      LaunchGuard lk(ctx, "gemm_k_offsets", (double)Kp * 16, 0);
      hipLaunchKernelGGL(k_koff, dim3((unsigned)((Kp + 255) / 256)), dim3(256), 0, ctx->stream, p.k, p.K, Kp, ka, kb);
      p.kmask = -1;
      p.ksa = p.ksb = 0;
    } else {   // single K dim: offsets are k * stride, the table a block of zeros
      ka = kb = (int64_t*)zero_tab;
      p.kmask = 0;
      p.ksa = p.k.sa[0];
      p.ksb = p.k.sb[0];
    }
    void* cdst = split > 1 ? part->ptr : data_ptr(out);
    // an operand contiguous along K is read four elements at a time
    auto k_vector = [&](const void* base, const int64_t* ks, const int64_t* rs, const Group& rows, const int64_t* bs) {
      const int64_t v = (int64_t)(16 / es);
      const int kd = p.k.nd - 1;
      if (((uintptr_t)base & 15) != 0 || p.K < 16 || ks[kd] != 1 || p.k.shape[kd] % 4 != 0) return false;
      for (int i = 0; i < kd; ++i) if (ks[i] % v != 0) return false;
      for (int i = 0; i < rows.nd; ++i) if (rs[i] % v != 0) return false;
      for (int i = 0; i < p.bt.nd; ++i) if (bs[i] % v != 0) return false;
      return true;
    };
    const bool va = k_vector(pa, p.k.sa, p.m.sa, p.m, p.bt.sa), vb = k_vector(pb, p.k.sb, p.n.sb, p.n, p.bt.sb);
    LaunchArgs la{ctx->stream, -1, tm, tn, va, vb, grid, pa, pb, cdst, ka, kb};
    {
      LaunchGuard lg(ctx, label, bytes, flops);
      la.ev_start = lg.start_event();
      la.ev_stop = lg.stop_event();
      if (dtype == HGPU_F64) launch_f64(p, la);
      else launch_f32(p, la);
    }
    if (split > 1) {
      LaunchGuard ls(ctx, "gemm_sum_partials", (double)out_n * (split + 1) * es, (double)out_n * split);
      if (dtype == HGPU_F64) launch_sum_partials<double>(ctx, out_n, (int)split, (const double*)part->ptr, (double*)data_ptr(out));
      else launch_sum_partials<float>(ctx, out_n, (int)split, (const float*)part->ptr, (float*)data_ptr(out));
    }
  }
  hipError_t e = hipGetLastError();
  buffer_release(koff);
  if (part) buffer_release(part);
  if (e != hipSuccess) return check_hip(ctx, e, "gemm");
  *handled = true;
  return HGPU_OK;
}

}  // namespace

namespace hg {

int try_footprint(hgpu_ctx* ctx, const GemmParams& p, int dtype, const void* pa, const void* pb, hgpu_array* out, bool* handled);
int try_smallk(hgpu_ctx* ctx, int n_terms, const hgpu_array* const* as, const hgpu_array* const* bs, int n_keep, int n_in, const hgpu_array* const* in, int c_slot,
               int n_instr, const hgpu_fused_instr* prog, const std::vector<int>& dt, int n_out, const int* out_slots, hgpu_array* const* outs, bool* handled);

// The dims of a contraction out[kept] = sum a[kept, red] * b[kept, red] sorted
// into row (M), column (N), reduced (K) and batch groups by which operand moves
// along them; false when the strides do not make it a matrix product.
bool classify_contraction(int rank, const int64_t* shape, const int64_t* st_a, const int64_t* st_b, const int64_t* st_c, int n_keep, GemmParams* p) {
  p->m.nd = p->n.nd = p->k.nd = p->bt.nd = 0;
  // Classify the dims.  The dims of a group are an index SET: any order works
  // as long as A, B and C agree, so each group is sorted with the dim that is
  // most contiguous in memory last (innermost) -- that is the dim the lanes of
  // a load run along -- and only then merged.
  struct DimRec { int64_t e, sa, sb, sc; };
  std::vector<DimRec> gm, gn, gk, gb;
  for (int i = 0; i < n_keep; ++i) {
    int64_t e = shape[i], sa = st_a[i], sb = st_b[i], sc = st_c[i];
    if (e == 1) continue;
    if (sa != 0 && sb == 0) gm.push_back({e, sa, 0, sc});
    else if (sa == 0 && sb != 0) gn.push_back({e, 0, sb, sc});
    else if (sa != 0 && sb != 0) gb.push_back({e, sa, sb, sc});
    else return false;  // an output dim neither operand depends on
  }
  for (int i = n_keep; i < rank; ++i) {
    int64_t e = shape[i], sa = st_a[i], sb = st_b[i];
    if (e == 1) continue;
    if (sa == 0 || sb == 0) return false;  // a plain sum hidden in the contraction
    gk.push_back({e, sa, sb, 0});
  }
  auto mag = [](int64_t v) { return v < 0 ? -v : v; };
  std::stable_sort(gm.begin(), gm.end(), [&](const DimRec& x, const DimRec& y) { return mag(x.sa) > mag(y.sa); });
  std::stable_sort(gn.begin(), gn.end(), [&](const DimRec& x, const DimRec& y) { return mag(x.sb) > mag(y.sb); });
  {
    // K: follow the operand that has a unit-stride K dim; when both or neither
    // do, the one that is larger (more rows to stream)
    int64_t rows_a = 1, rows_b = 1;
    for (auto& d : gm) rows_a *= d.e;
    for (auto& d : gn) rows_b *= d.e;
    bool a_unit = false, b_unit = false;
    for (auto& d : gk) { a_unit = a_unit || mag(d.sa) == 1; b_unit = b_unit || mag(d.sb) == 1; }
    bool by_a = (a_unit != b_unit) ? a_unit : rows_a >= rows_b;
    std::stable_sort(gk.begin(), gk.end(), [&](const DimRec& x, const DimRec& y) { return by_a ? mag(x.sa) > mag(y.sa) : mag(x.sb) > mag(y.sb); });
  }
  for (auto& d : gm) if (!push_dim(p->m, d.e, d.sa, d.sb, d.sc)) return false;
  for (auto& d : gn) if (!push_dim(p->n, d.e, d.sa, d.sb, d.sc)) return false;
  for (auto& d : gk) if (!push_dim(p->k, d.e, d.sa, d.sb, d.sc)) return false;
  for (auto& d : gb) if (!push_dim(p->bt, d.e, d.sa, d.sb, d.sc)) return false;
  finish(p->m);
  finish(p->n);
  finish(p->k);
  finish(p->bt);
  p->M = total(p->m);
  p->N = total(p->n);
  p->K = total(p->k);
  p->BT = total(p->bt);
  return true;
}

int sum_partials(hgpu_ctx* ctx, int dtype, int64_t n, int parts, const void* part, void* out) {
  size_t es = dtype_size(dtype);
  LaunchGuard ls(ctx, "gemm_sum_partials", (double)n * (parts + 1) * es, (double)n * parts);
  if (dtype == HGPU_F64) launch_sum_partials<double>(ctx, n, parts, (const double*)part, (double*)out);
  else launch_sum_partials<float>(ctx, n, parts, (const float*)part, (float*)out);
  HG_CHECK_LAUNCH(ctx, "gemm_sum_partials");
  return HGPU_OK;
}

// `parts` partial results of n1 + n2 elements each: the first n1 summed into out1, the other n2 into out2.
int sum_partials_split(hgpu_ctx* ctx, int dtype, int64_t n1, int64_t n2, int parts, const void* part, void* out1, void* out2) {
  const size_t es = dtype_size(dtype);
  const int64_t n = n1 + n2;
  LaunchGuard ls(ctx, "gemm_sum_partials", (double)n * (parts + 1) * es, (double)n * parts);
  if (dtype == HGPU_F64) launch_sum_partials<double>(ctx, n, parts, (const double*)part, (double*)out1, n1, (double*)out2);
  else launch_sum_partials<float>(ctx, n, parts, (const float*)part, (float*)out1, n1, (float*)out2);
  HG_CHECK_LAUNCH(ctx, "gemm_sum_partials");
  return HGPU_OK;
}

int try_gemm(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array* out, bool* handled,
             int n_terms, const hgpu_array* const* as, const hgpu_array* const* bs, hgpu_array** partials_out) {
  // n_terms > 0: out = sum_t contract(as[t], bs[t]); all terms have the shapes,
  // strides and dtype of a = as[0], b = bs[0] (the caller has checked).
  // partials_out: a caller that runs an elementwise pass over the result anyway
  // takes the two or three partial results of a product split along K instead
  // (an array of shape [parts, kept dims...]; `out` is then left unwritten) and
  // adds them in that pass.
  *handled = false;
  if (partials_out) *partials_out = nullptr;
  if (!b) return HGPU_OK;
  if (a->dtype != HGPU_F64 && a->dtype != HGPU_F32) return HGPU_OK;
  GemmParams p;
  if (!classify_contraction(a->rank, a->shape, a->strides, b->strides, out->strides, n_keep, &p)) return HGPU_OK;
  // Worth the matrix cores only when there is reuse on both sides.
  if (p.K < 4 || p.M * p.N < 256) return HGPU_OK;
  if (p.BT > 65535) return HGPU_OK;
  if ((double)p.M * p.N * p.K * p.BT < 2.0e6) return HGPU_OK;
  // a thousand outputs under a long K (the last layer's weight gradient: 100 x 10
  // over 5000): the split-K kernels have a handful of wavefronts to work with,
  // a wavefront per output in the reduction kernels has a thousand
  if ((p.M <= 16 || p.N <= 16) && p.K > 1024 && (double)p.M * p.N * p.K * p.BT < 2.0e7) return HGPU_OK;

  const void* pa = data_ptr(a);
  const void* pb = data_ptr(b);
  // A small output under a long K (weight gradients, the last layer of a
  // classifier) is better served by independent wavefronts than by staged tiles.
  static_assert(kMaxTerms == 32, "hgpu_contract_sum groups 32 terms to a launch");
  if (n_terms > kMaxTerms) return HGPU_OK;
  p.n_terms = n_terms;
  p.term_loop = 0;
  for (int t = 0; t < n_terms; ++t) { p.a_term[t] = data_ptr(as[t]); p.b_term[t] = data_ptr(bs[t]); }
  if (n_terms == 0) {   // windows into small footprints: operands from LDS
    int rc = try_footprint(ctx, p, a->dtype, pa, pb, out, handled);
    if (rc || *handled) return rc;
  }
  if ((p.K <= 512 || (p.K <= 1024 && p.M * p.N <= 160000)) && p.BT == 1) {   // the whole contracted dim in LDS: no K loop, no K table
    const hgpu_array* const* ta = n_terms > 0 ? as : &a;
    const hgpu_array* const* tb = n_terms > 0 ? bs : &b;
    const hgpu_array* none = nullptr;
    const int slot = 0;
    int rc = try_smallk(ctx, n_terms > 0 ? n_terms : 1, ta, tb, n_keep, 1, &none, 0, 0, nullptr, std::vector<int>{a->dtype}, 1, &slot, &out, handled);
    if (rc || *handled) return rc;
  }
  // (under a long K the staged kernel's coalesced tile loads win even with most of a 32-wide tile empty: the recurrent network's
  // input weight gradient, 128 x 28 over 28 x 5000, 52 -> 45 us)
  if ((p.M <= 32 || p.N <= 32) && p.M <= 1024 && p.N <= 1024 && p.K < 4096) return gemm_direct(ctx, p, a->dtype, pa, pb, out, handled, n_terms);

  const int64_t nt = n_terms > 0 ? n_terms : 1;      // products summed by this launch
  const int64_t out_elems = p.M * p.N * p.BT;
  // K chunks for a tile shape, and how well the blocks then fill the device
  // (blocks / places of the rounds they take)
  auto plan_split = [&](int c, double* fill_out) {
    const int64_t bm = kTiles[c].wgm * kTiles[c].tm * 16, bn = kTiles[c].wgn * kTiles[c].tn * 16;
    const int64_t tl = ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn);
    // small tiles do little work per K step and hide the latency of a step only
    // behind other blocks on the CU: ask for more of them
    const int64_t per_cu = bm * bn >= 128 * 64 ? 2 : (bm * bn >= 64 * 64 ? 4 : 8);
    const double slots = (double)ctx->num_cu * per_cu;
    auto fill = [&](int cand) {
      const double blocks = (double)tl * p.BT * nt * cand;
      return blocks / (std::ceil(blocks / slots) * slots);
    };
    int split = 1;
    const int64_t want = (int64_t)ctx->num_cu * per_cu;
    if (tl * p.BT * nt < want && p.K >= 8 * BK) {
      split = (int)((want + tl * p.BT * nt - 1) / (tl * p.BT * nt));
      int64_t max_split = p.K / (4 * BK);
      if (split > max_split) split = (int)max_split;
      // the partial products must stay small next to the operands, or small outright
      int64_t cap = out_elems > 0 ? (int64_t)((double)(p.M + p.N) * p.K * p.BT / (2.0 * out_elems)) : 1;
      if (out_elems * (int64_t)dtype_size(a->dtype) <= (1 << 20) && cap < 16) cap = 16;
      if (cap > 512) cap = 512;
      if (cap < 1) cap = 1;
      if (split > cap) split = (int)cap;
      if (split < 1) split = 1;
      // fewer tiles than CUs: two K halves per tile keep every CU busy, and the
      // second pass over the output costs less than the idle quarter of the device
      if (split == 1 && tl * p.BT * nt < ctx->num_cu && p.K >= 16 * BK) split = 2;
      // A few more chunks when they fill the last round of blocks: with `per_cu`
      // blocks resident on a CU, blocks run in rounds of num_cu * per_cu, and a
      // round that is three quarters empty costs as much as a full one.  (300 x 784
      // over K 5000 in 64 x 128 tiles: 11 chunks = 385 blocks take 82 us, 14 chunks
      // = 490 blocks 70 us, 15 chunks = 525 blocks 94 us.)
      if (split > 1) {
        int best_s = split;
        double best_fill = fill(split);
        const int hi = (int)std::min<int64_t>(max_split, split + (split * 3 + 9) / 10);
        for (int cand = split + 1; cand <= hi; ++cand)
          if (fill(cand) > best_fill + 0.1) { best_fill = fill(cand); best_s = cand; }
        // ... or a few less, when that makes whole rounds (28 products of 128 x 128 over
        // K 5000 in 64 x 64 tiles: 12 chunks each = 1344 blocks on 1024 places, 9 = 1008)
        const int lo = std::max(2, split - (split * 3 + 9) / 10);
        for (int cand = split - 1; cand >= lo; --cand)
          if (fill(cand) > best_fill + 0.1) { best_fill = fill(cand); best_s = cand; }
        split = best_s;
      }
    }
    if (fill_out) *fill_out = fill(split);
    return split;
  };
  // tile shape: least padded work per unit of efficiency and of device filled
  const bool f64 = a->dtype == HGPU_F64;
  int cfg = 0;
  double best = 1e300;
  double costs[kNumTiles];
  for (int c = 0; c < (a->dtype == HGPU_F32 ? kNumTiles : kFirstF32OnlyTile); ++c) {
    int64_t bm = kTiles[c].wgm * kTiles[c].tm * 16, bn = kTiles[c].wgn * kTiles[c].tn * 16;
    double padded = (double)((p.M + bm - 1) / bm * bm) * (double)((p.N + bn - 1) / bn * bn);
    // fp64: the instruction is slow next to LDS, so the operand reuse of a larger
    // tile buys little and three 64 x 64 blocks on a CU run it as well as two of
    // 64 x 128 (300 x 784 over K 5000: 64 against 74 us)
    const double eff = (f64 && bm == 64 && bn == 64) ? 0.85 : kTiles[c].eff;
    double cost = padded / eff;
    // a tile shape that cannot occupy the device even with K split pays for the idle CUs
    double blocks = (double)((p.M + bm - 1) / bm) * (double)((p.N + bn - 1) / bn) * (double)p.BT;
    double can_split = (double)(p.K / (4 * BK));
    double cap0 = (double)(p.M + p.N) * p.K / (2.0 * p.M * p.N);
    if (can_split > cap0) can_split = cap0;
    if (can_split > 512) can_split = 512;
    if (can_split < 1) can_split = 1;
    if (blocks * can_split < ctx->num_cu) cost *= ctx->num_cu / (blocks * can_split);
    costs[c] = cost;
    if (cost < best * 0.999) { best = cost; cfg = c; }
  }
  if (f64) {
    // among shapes within 15 % of the least, the one whose blocks fill their rounds
    // best (the fp32 choices were tuned without this step)
    double best2 = 1e300;
    for (int c = 0; c < kFirstF32OnlyTile; ++c) {
      if (costs[c] > best * 1.15) continue;
      double fl = 1;
      (void)plan_split(c, &fl);
      const double c2 = costs[c] / std::max(fl, 0.25);
      if (c2 < best2 * 0.999) { best2 = c2; cfg = c; }
    }
  }
  const int64_t BM = kTiles[cfg].wgm * kTiles[cfg].tm * 16, BN = kTiles[cfg].wgn * kTiles[cfg].tn * 16;
  int64_t tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  if (tiles > 0x7fffffff) return HGPU_OK;
  int split = plan_split(cfg, nullptr);
  if (const char* e = getenv("HORDEAD_GEMM_SPLIT")) {   // for measurements
    int v = atoi(e);
    if (v >= 1 && v <= p.K / BK) split = v;
  }
  p.kchunk = ((p.K + split - 1) / split + BK - 1) / BK * BK;
  p.term_split = (int)((p.K + p.kchunk - 1) / p.kchunk);
  p.split = (int)(p.term_split * nt);                // K chunks of all terms
  // terms that are one chunk each, under tiles that fill the device by
  // themselves: every block adds the terms up in its registers, no partials
  p.term_loop = (nt > 1 && p.term_split == 1 && tiles * p.BT >= ctx->num_cu / 2 &&
                 term_loop_tile(kTiles[cfg].wgm, kTiles[cfg].wgn, kTiles[cfg].tm, kTiles[cfg].tn)) ? 1 : 0;
  if (p.term_loop) p.split = 1;
  split = p.split;
  if (split > 65535) return HGPU_OK;

  size_t es = dtype_size(a->dtype);
  int64_t out_n = nelem(out);
  const void* zero_tab = nullptr;
  int rc = zero_block(ctx, &zero_tab);
  if (rc) return rc;
  hgpu_buffer* koff = nullptr;
  const int64_t Kp = p.K;
  rc = buffer_alloc(ctx, (size_t)Kp * 16, &koff);
  if (rc) return rc;
  hgpu_buffer* part = nullptr;
  if (split > 1) {
    rc = buffer_alloc(ctx, (size_t)out_n * split * es, &part);
    if (rc) { buffer_release(koff); return rc; }
  }
  p.c_split_stride = split > 1 ? out_n : 0;
  int64_t* ka = (int64_t*)koff->ptr;
  int64_t* kb = ka + p.K;
  // lanes run along k when the innermost K dim is contiguous and long enough to
  // fill a 16-lane group, or when running along m / n would be no better
  auto along_k = [](int64_t sk, int64_t ek, int64_t srow) {
    if (sk < 0) sk = -sk;
    if (srow < 0) srow = -srow;
    if (sk == 1 && (ek >= 16 || srow != 1)) return true;
    return srow != 1 && sk < srow;
  };
  bool akc = along_k(p.k.sa[p.k.nd - 1], p.k.shape[p.k.nd - 1], p.m.sa[p.m.nd - 1]);
  bool bkc = along_k(p.k.sb[p.k.nd - 1], p.k.shape[p.k.nd - 1], p.n.sb[p.n.nd - 1]);
  p.a_kc = akc ? 1 : 0;
  p.b_kc = bkc ? 1 : 0;
  p.c_rows_contig = (p.m.sc[p.m.nd - 1] == 1 && p.n.sc[p.n.nd - 1] != 1 && p.M >= 64) ? 1 : 0;
  bool va, vb;
  {
    va = vector_ok(es, akc ? p.k : p.m, (akc ? p.k.nd : p.m.nd) - 1, akc ? p.k.sa : p.m.sa);
    vb = vector_ok(es, bkc ? p.k : p.n, (bkc ? p.k.nd : p.n.nd) - 1, bkc ? p.k.sb : p.n.sb);
  }
  dim3 grid((unsigned)tiles, (unsigned)split, (unsigned)p.BT);
  {
    double flops = 2.0 * p.M * p.N * p.K * p.BT * nt;
    double bytes = (((double)p.M * p.K + (double)p.N * p.K) * nt + (double)p.M * p.N) * p.BT * es;
    const char* label = a->dtype == HGPU_F64 ? "gemm_f64" : "gemm_f32";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[128];
      char terms[24] = "";
      if (nt > 1) snprintf(terms, sizeof terms, ",terms%lld%s", (long long)nt, p.term_loop ? "loop" : "");
      snprintf(buf, sizeof buf, "%s[M%lldxN%lldxK%lldxB%lld,s%d,%s%s,t%lldx%lld%s]", label, (long long)p.M, (long long)p.N, (long long)p.K, (long long)p.BT, split, akc ? (va ? "K" : "k") : (va ? "M" : "m"), bkc ? (vb ? "K" : "k") : (vb ? "N" : "n"), (long long)BM, (long long)BN, terms);
      label = intern_label(ctx, buf);
    }
    // the helper launches are timed under their own names, the label times the MFMA kernel alone
    if (p.k.nd > 1) {
      LaunchGuard lk(ctx, "gemm_k_offsets", (double)Kp * 16, 0);
      hipLaunchKernelGGL(k_koff, dim3((unsigned)((Kp + 255) / 256)), dim3(256), 0, ctx->stream, p.k, p.K, Kp, ka, kb);
      p.kmask = -1;
      p.ksa = p.ksb = 0;
    } else {   // single K dim: offsets are k * stride, the table a block of zeros
      ka = kb = (int64_t*)zero_tab;
      p.kmask = 0;
      p.ksa = p.k.sa[0];
      p.ksb = p.k.sb[0];
    }
    void* cdst = split > 1 ? part->ptr : data_ptr(out);
    LaunchArgs la{ctx->stream, cfg, 0, 0, va, vb, grid, data_ptr(a), data_ptr(b), cdst, ka, kb};
    {
      LaunchGuard lg(ctx, label, bytes, flops);
      la.ev_start = lg.start_event();
      la.ev_stop = lg.stop_event();
      if (a->dtype == HGPU_F64) launch_f64(p, la);
      else launch_f32(p, la);
    }
    if (split > 1 && partials_out && split <= 3 && is_dense(out)) {
      int64_t sh[HGPU_MAX_RANK + 1], st[HGPU_MAX_RANK + 1];
      sh[0] = split;
      for (int d = 0; d < out->rank; ++d) sh[d + 1] = out->shape[d];
      dense_strides(out->rank + 1, sh, st);
      *partials_out = new_view(ctx, part, a->dtype, out->rank + 1, sh, st, 0);
    } else if (split > 1) {
      LaunchGuard ls(ctx, "gemm_sum_partials", (double)out_n * (split + 1) * es, (double)out_n * split);
      if (a->dtype == HGPU_F64) launch_sum_partials<double>(ctx, out_n, (int)split, (const double*)part->ptr, (double*)data_ptr(out));
      else launch_sum_partials<float>(ctx, out_n, (int)split, (const float*)part->ptr, (float*)data_ptr(out));
    }
  }
  hipError_t e = hipGetLastError();
  buffer_release(koff);
  if (part) buffer_release(part);
  if (e != hipSuccess) {
    if (partials_out && *partials_out) { hgpu_release(*partials_out); *partials_out = nullptr; }
    return check_hip(ctx, e, "gemm");
  }
  *handled = true;
  return HGPU_OK;
}

}  // namespace hg

// ---- the matrix cores' ceiling, measured -----------------------------------
// Loops of nothing but one MFMA instruction on independent accumulators: what
// a product kernel built on that instruction cannot exceed on this part.
namespace {
typedef __attribute__((ext_vector_type(4))) double probe_d4;
typedef __attribute__((ext_vector_type(4))) float probe_f4;
typedef __attribute__((ext_vector_type(16))) float probe_f16;

__global__ void __launch_bounds__(256) mfma_probe_f64_16x16x4(double* out, int iters) {
  probe_d4 acc[4];
  for (int i = 0; i < 4; ++i) acc[i] = probe_d4{0, 0, 0, 0};
  const double a = threadIdx.x * 0.001, b = threadIdx.x * 0.002;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[i], 0, 0, 0);
  }
  double s = 0;
  for (int i = 0; i < 4; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
__global__ void __launch_bounds__(256) mfma_probe_f64_4x4x4(double* out, int iters) {
  double acc[8];
  for (int i = 0; i < 8; ++i) acc[i] = 0;
  const double a = threadIdx.x * 0.001, b = threadIdx.x * 0.002;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f64_4x4x4f64(a, b, acc[i], 0, 0, 0);
  }
  double s = 0;
  for (int i = 0; i < 8; ++i) s += acc[i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
__global__ void __launch_bounds__(256) mfma_probe_f32_16x16x4(float* out, int iters) {
  probe_f4 acc[4];
  for (int i = 0; i < 4; ++i) acc[i] = probe_f4{0, 0, 0, 0};
  const float a = threadIdx.x * 0.001f, b = threadIdx.x * 0.002f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
  }
  float s = 0;
  for (int i = 0; i < 4; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
__global__ void __launch_bounds__(256) mfma_probe_f32_32x32x2(float* out, int iters) {
  probe_f16 acc[2];
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 16; ++j) acc[i][j] = 0;
  const float a = threadIdx.x * 0.001f, b = threadIdx.x * 0.002f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 2; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
  }
  float s = 0;
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 16; ++j) s += acc[i][j];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
// The same instruction fed the way a product kernel feeds it: four wavefronts
// hold a 64 x 64 tile (2 x 2 blocks each), every K step of 16 reads its
// fragments from LDS and ends with a barrier; nothing is loaded from memory.
__global__ void __launch_bounds__(256) mfma_probe_f64_16x16x4_lds(double* out, int iters) {
  __shared__ double As[16][65], Bs[16][65];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave >> 1, wn = wave & 1;
  for (int i = t; i < 16 * 65; i += 256) { (&As[0][0])[i] = i * 1e-3; (&Bs[0][0])[i] = i * 2e-3; }
  __syncthreads();
  probe_d4 acc[2][2];
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 2; ++j) acc[i][j] = probe_d4{0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int kk = 0; kk < 16; kk += 4) {
      double fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = As[kk + (lane >> 4)][wm * 32 + i * 16 + (lane & 15)];
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = Bs[kk + (lane >> 4)][wn * 32 + j * 16 + (lane & 15)];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  double s = 0;
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 2; ++j) s += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  out[blockIdx.x * 256 + t] = s;
}
}  // namespace

extern "C" int hgpu_mfma_probe(hgpu_ctx* ctx, int variant, int iters, double* tflops) {
  if (!ctx || !tflops || iters < 1) return HGPU_ERR_INVALID;
  if (int rc = no_capture(ctx, "mfma_probe")) return rc;
  // 16 wavefronts per CU: every SIMD has four to pick from; the LDS-fed variants 4, 5, 6 run one, two, four per SIMD
  const int blocks = ctx->num_cu * (variant == 4 ? 1 : variant == 5 ? 2 : 4);
  hgpu_buffer* buf = nullptr;
  int rc = buffer_alloc(ctx, (size_t)blocks * 256 * 8, &buf);
  if (rc) return rc;
  double flops_per_wave_iter = 0;
  auto launch = [&]() {
    switch (variant) {
      case 0: hipLaunchKernelGGL(mfma_probe_f64_16x16x4, dim3(blocks), dim3(256), 0, ctx->stream, (double*)buf->ptr, iters); flops_per_wave_iter = 4 * 2.0 * 16 * 16 * 4; break;
      case 1: hipLaunchKernelGGL(mfma_probe_f64_4x4x4, dim3(blocks), dim3(256), 0, ctx->stream, (double*)buf->ptr, iters); flops_per_wave_iter = 8 * 2.0 * 4 * 4 * 4 * 4; break;
      case 2: hipLaunchKernelGGL(mfma_probe_f32_16x16x4, dim3(blocks), dim3(256), 0, ctx->stream, (float*)buf->ptr, iters); flops_per_wave_iter = 4 * 2.0 * 16 * 16 * 4; break;
      case 3: hipLaunchKernelGGL(mfma_probe_f32_32x32x2, dim3(blocks), dim3(256), 0, ctx->stream, (float*)buf->ptr, iters); flops_per_wave_iter = 2 * 2.0 * 32 * 32 * 2; break;
      case 4: case 5: case 6:
        hipLaunchKernelGGL(mfma_probe_f64_16x16x4_lds, dim3(blocks), dim3(256), 0, ctx->stream, (double*)buf->ptr, iters);
        flops_per_wave_iter = 16 * 2.0 * 16 * 16 * 4;
        break;
      default: break;
    }
  };
  if (variant < 0 || variant > 6) { buffer_release(buf); return fail(ctx, HGPU_ERR_INVALID, "mfma_probe: variant %d", variant); }
  hipEvent_t e0, e1;
  LaunchGuard lg(ctx);
  launch();   // warm-up
  hipError_t e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  if (e == hipSuccess) {
    (void)hipEventRecord(e0, ctx->stream);
    launch();
    (void)hipEventRecord(e1, ctx->stream);
    e = hipEventSynchronize(e1);
  }
  float ms = 0;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  buffer_release(buf);
  if (e != hipSuccess || ms <= 0) return check_hip(ctx, e == hipSuccess ? hipErrorUnknown : e, "mfma_probe");
  *tflops = flops_per_wave_iter * (double)iters * (double)blocks * 4.0 / ((double)ms * 1e-3) / 1e12;
  return HGPU_OK;
}
