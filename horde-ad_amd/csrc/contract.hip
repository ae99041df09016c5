// Reductions and contractions over strided views:
//   out[o] = sum_r a[o,r] * b[o,r]
// which, with free views, is horde-ad's tssum / tssumN / tssum0 / tsdot0 /
// tsdot1In / tsmatvecmul / tsmatmul2 (src/HordeAd/Core/OpsConcrete.hs:215-242).
//
// This file holds the general path, bound by HBM bandwidth:
//   * lane-per-output: adjacent lanes own adjacent outputs and walk the
//     reduced index space with an odometer (coalesced when the kept innermost
//     dimension has unit stride: sums over outer dimensions);
//   * wave-per-output: the 64 lanes of a wavefront stride over the innermost
//     reduced dimension and combine with a shuffle tree (coalesced when the
//     reduced innermost dimension has unit stride: dot1In, sum0, dot0).
// Long reductions with few outputs are split into S chunks whose partial sums
// (double / int64 accumulators) are combined by a second launch, so the
// summation order is fixed by the shape alone: results are reproducible from
// run to run.  GEMM-shaped contractions are routed to the MFMA kernels first.
#include "common.hpp"

using namespace hg;

namespace hg {
// gemm.hip: returns HGPU_OK and sets *handled when the contraction was
// recognised as a matrix product and executed on the matrix cores.
int try_gemm(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array* out, bool* handled,
             int n_terms = 0, const hgpu_array* const* as = nullptr, const hgpu_array* const* bs = nullptr, hgpu_array** partials_out = nullptr);
constexpr int kGemmMaxTerms = 32;   // products one launch of try_gemm sums (kMaxTerms of the kernels)
}

namespace {

constexpr int kBlock = 256;

template <typename T> struct acc_of { using type = int64_t; };
template <> struct acc_of<double> { using type = double; };
template <> struct acc_of<float> { using type = double; };

// Several products of one layout reduced by one launch (hgpu_contract_sum):
// the chunk index s of a work item also selects the term, s = term * s_per +
// chunk within the term, and the term's operands replace the kernel's pointer
// arguments.  n == 0: one product.
struct TermPtrs {
  int n, s_per;
  const void* a[hg::kGemmMaxTerms];
  const void* b[hg::kGemmMaxTerms];
};

template <typename A>
__device__ __forceinline__ A wave_sum(A v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    if constexpr (sizeof(A) == 8) {
      unsigned long long u = *reinterpret_cast<unsigned long long*>(&v);
      unsigned lo = __shfl_down((unsigned)(u & 0xffffffffu), off, 64);
      unsigned hi = __shfl_down((unsigned)(u >> 32), off, 64);
      unsigned long long w = ((unsigned long long)hi << 32) | lo;
      v += *reinterpret_cast<A*>(&w);
    } else {
      v += __shfl_down(v, off, 64);
    }
  }
  return v;
}

// Work item = (output o, chunk s); s-th chunk covers reduced linear indices
// [s*chunk, min(R, (s+1)*chunk)).  out is dense [n_out, S].
// (`bid` of `nb` blocks: the kernels below pass their own block index; the grouped kernel at the end of this
// file passes a block's place among the blocks of its problem.  tp == nullptr: one product.)
template <typename TI, typename TO, bool HASB>
__device__ __forceinline__ void lane_body(const Dims& keep, const Dims& red, int64_t n_out, int64_t R, int S, int64_t chunk,
                                          const TI* __restrict__ a0, const TI* __restrict__ b0, TO* __restrict__ out, const TermPtrs* tp, unsigned bid, unsigned nb) {
  using A = typename acc_of<TI>::type;
  int64_t items = n_out * S;
  int64_t step = (int64_t)nb * kBlock;
  for (int64_t item = (int64_t)bid * kBlock + threadIdx.x; item < items; item += step) {
    int64_t o = item % n_out, s = item / n_out;
    const int64_t s_all = s;
    const TI* a = a0;
    const TI* b = b0;
    if (tp && tp->n) {
      int term = (int)(s / tp->s_per);
      s -= (int64_t)term * tp->s_per;
      a = (const TI*)tp->a[term];
      b = (const TI*)tp->b[term];
    }
    int64_t ko[2];
    decompose<2>(keep, o, ko);
    int64_t r0 = s * chunk, r1 = r0 + chunk;
    if (r1 > R) r1 = R;
    // odometer over the reduced dims, started at r0
    int64_t idx[HG_KDIMS];
    int64_t oa = ko[0], ob = ko[1];
    {
      int64_t r = r0;
      for (int i = red.nd - 1; i >= 0; --i) {
        int64_t q = i > 0 ? r / red.shape[i] : 0;
        int64_t c = i > 0 ? r - q * red.shape[i] : r;
        idx[i] = c;
        oa += c * red.st[0][i];
        ob += c * red.st[1][i];
        r = q;
      }
    }
    A acc = 0;
    const int last = red.nd - 1;
    for (int64_t r = r0; r < r1; ++r) {
      A x = (A)a[oa];
      if (HASB) x *= (A)b[ob];
      acc += x;
      // advance
      int i = last;
      idx[i]++;
      oa += red.st[0][i];
      ob += red.st[1][i];
      while (i > 0 && idx[i] == red.shape[i]) {
        oa -= idx[i] * red.st[0][i];
        ob -= idx[i] * red.st[1][i];
        idx[i] = 0;
        --i;
        idx[i]++;
        oa += red.st[0][i];
        ob += red.st[1][i];
      }
    }
    out[o * S + s_all] = (TO)acc;
  }
}
template <typename TI, typename TO, bool HASB>
__global__ void __launch_bounds__(kBlock) k_contract_lane(Dims keep, Dims red, int64_t n_out, int64_t R, int S, int64_t chunk,
                                                           const TI* __restrict__ a0, const TI* __restrict__ b0, TO* __restrict__ out, TermPtrs tp) {
  lane_body<TI, TO, HASB>(keep, red, n_out, R, S, chunk, a0, b0, out, &tp, blockIdx.x, gridDim.x);
}

// Sum over j = j_first, j_first + 64, ... < j_end of a[j * sa] (* b[j * sb]): four
// independent accumulators keep four loads per operand in flight.
template <typename TI, typename A, bool HASB>
__device__ __forceinline__ A lane_strided_sum(const TI* __restrict__ pa, const TI* __restrict__ pb, int64_t sa, int64_t sb, int64_t j_first, int64_t j_end) {
  A acc0 = 0, acc1 = 0, acc2 = 0, acc3 = 0;
  int64_t j = j_first;
  for (; j + 192 < j_end; j += 256) {
    A x0 = (A)pa[j * sa], x1 = (A)pa[(j + 64) * sa], x2 = (A)pa[(j + 128) * sa], x3 = (A)pa[(j + 192) * sa];
    if (HASB) {
      x0 *= (A)pb[j * sb];
      x1 *= (A)pb[(j + 64) * sb];
      x2 *= (A)pb[(j + 128) * sb];
      x3 *= (A)pb[(j + 192) * sb];
    }
    acc0 += x0;
    acc1 += x1;
    acc2 += x2;
    acc3 += x3;
  }
  for (; j < j_end; j += 64) {
    A x = (A)pa[j * sa];
    if (HASB) x *= (A)pb[j * sb];
    acc0 += x;
  }
  return (acc0 + acc1) + (acc2 + acc3);
}

// One wavefront per work item.  `red` has its innermost dim split off:
// Lin = extent, (sa_in, sb_in) = strides; `red` keeps the outer reduced dims
// with Q = their product.  Chunks split Q when Q > 1, else Lin.
template <typename TI, typename TO, bool HASB>
__device__ __forceinline__ void wave_body(const Dims& keep, const Dims& red, int64_t n_out, int64_t Q, int64_t Lin, int64_t sa_in, int64_t sb_in,
                                          int S, int64_t chunk, const TI* __restrict__ a0, const TI* __restrict__ b0, TO* __restrict__ out, const TermPtrs* tp, unsigned bid, unsigned nb) {
  using A = typename acc_of<TI>::type;
  const int lane = threadIdx.x & 63;
  int64_t wave = ((int64_t)bid * kBlock + threadIdx.x) >> 6;
  int64_t nwaves = ((int64_t)nb * kBlock) >> 6;
  int64_t items = n_out * S;
  for (int64_t item = wave; item < items; item += nwaves) {
    int64_t o = item / S;
    int s = (int)(item - o * S);
    const TI* a = a0;
    const TI* b = b0;
    if (tp && tp->n) {
      int term = s / tp->s_per;
      s -= term * tp->s_per;
      a = (const TI*)tp->a[term];
      b = (const TI*)tp->b[term];
    }
    int64_t ko[2];
    decompose<2>(keep, o, ko);
    int64_t q0 = 0, q1 = Q, j0 = 0, j1 = Lin;
    if (Q > 1) { q0 = s * chunk; q1 = q0 + chunk; if (q1 > Q) q1 = Q; }
    else { j0 = s * chunk; j1 = j0 + chunk; if (j1 > Lin) j1 = Lin; }
    A acc = 0;
    int64_t q = q0;
    if (Lin <= 1024) {
      // short inner rows: four outer indices at a time, so that a lane has four
      // loads per operand in flight although a row gives it only a few elements
      for (; q + 3 < q1; q += 4) {
        const TI* pa[4];
        const TI* pb[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          int64_t ro[2];
          decompose<2>(red, q + u, ro);
          pa[u] = a + ko[0] + ro[0];
          pb[u] = HASB ? b + ko[1] + ro[1] : nullptr;
        }
        A c[4] = {0, 0, 0, 0};
        for (int64_t j = j0 + lane; j < j1; j += 64) {
          A x[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) x[u] = (A)pa[u][j * sa_in];
          if (HASB) {
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] *= (A)pb[u][j * sb_in];
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) c[u] += x[u];
        }
        acc += (c[0] + c[1]) + (c[2] + c[3]);
      }
    }
    for (; q < q1; ++q) {
      int64_t ro[2];
      decompose<2>(red, q, ro);
      const TI* pa = a + ko[0] + ro[0];
      const TI* pb = HASB ? b + ko[1] + ro[1] : nullptr;
      acc += lane_strided_sum<TI, A, HASB>(pa, pb, sa_in, sb_in, j0 + lane, j1);
    }
    acc = wave_sum<A>(acc);
    if (lane == 0) out[item] = (TO)acc;
  }
}
template <typename TI, typename TO, bool HASB>
__global__ void __launch_bounds__(kBlock) k_contract_wave(Dims keep, Dims red, int64_t n_out, int64_t Q, int64_t Lin, int64_t sa_in, int64_t sb_in,
                                                           int S, int64_t chunk, const TI* __restrict__ a0, const TI* __restrict__ b0, TO* __restrict__ out, TermPtrs tp) {
  wave_body<TI, TO, HASB>(keep, red, n_out, Q, Lin, sa_in, sb_in, S, chunk, a0, b0, out, &tp, blockIdx.x, gridDim.x);
}

// One block of four wavefronts per output: for a few hundred outputs with a few
// thousand reduced elements each, where one wavefront per output leaves most of
// the device idle and splitting into chunks would cost a second launch.  The
// wavefronts take every fourth outer reduced index (or a quarter of the inner
// dim when there is no outer one) and combine through LDS in a fixed order.
template <typename TI, typename TO, bool HASB>
__device__ __forceinline__ void block_body(const Dims& keep, const Dims& red, int64_t n_out, int64_t Q, int64_t Lin, int64_t sa_in, int64_t sb_in,
                                           const TI* __restrict__ a, const TI* __restrict__ b, TO* __restrict__ out, unsigned bid, unsigned nb) {
  using A = typename acc_of<TI>::type;
  __shared__ A part[kBlock / 64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  constexpr int NW = kBlock / 64;
  for (int64_t o = bid; o < n_out; o += nb) {
    int64_t ko[2];
    decompose<2>(keep, o, ko);
    A acc = 0;
    if (Q > 1) {
      for (int64_t q = w; q < Q; q += NW) {
        int64_t ro[2];
        decompose<2>(red, q, ro);
        acc += lane_strided_sum<TI, A, HASB>(a + ko[0] + ro[0], HASB ? b + ko[1] + ro[1] : nullptr, sa_in, sb_in, lane, Lin);
      }
    } else {
      const int64_t quarter = (Lin + NW - 1) / NW;
      const int64_t j0 = w * quarter, j1 = j0 + quarter < Lin ? j0 + quarter : Lin;
      acc = lane_strided_sum<TI, A, HASB>(a + ko[0], HASB ? b + ko[1] : nullptr, sa_in, sb_in, j0 + lane, j1);
    }
    acc = wave_sum<A>(acc);
    if (lane == 0) part[w] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
      A t = part[0];
#pragma unroll
      for (int k = 1; k < NW; ++k) t += part[k];
      out[o] = (TO)t;
    }
    __syncthreads();
  }
}
template <typename TI, typename TO, bool HASB>
__global__ void __launch_bounds__(kBlock) k_contract_block(Dims keep, Dims red, int64_t n_out, int64_t Q, int64_t Lin, int64_t sa_in, int64_t sb_in,
                                                            const TI* __restrict__ a, const TI* __restrict__ b, TO* __restrict__ out) {
  block_body<TI, TO, HASB>(keep, red, n_out, Q, Lin, sa_in, sb_in, a, b, out, blockIdx.x, gridDim.x);
}

// Up to four single-launch reductions of one element type as one kernel: the first blocks are problem 0's, the
// next ones problem 1's, ...; every block runs the code of the kernel its problem would have been launched with.
struct RedArgs {
  Dims keep, red;
  int64_t n_out, R, Q, Lin, sa, sb, chunk;
  int variant, hasb;
  unsigned grid, pad_;
  const void* a;
  const void* b;
  void* out;
};
struct RedGroup {
  int n, pad_;
  RedArgs j[4];
};
static_assert(sizeof(RedGroup) <= 4000, "the grouped reduction's arguments must fit the kernel argument block");

template <typename T>
__global__ void __launch_bounds__(kBlock) k_contract_group(RedGroup g) {
  unsigned bid = blockIdx.x;
  int k = 0;
  while (k < g.n - 1 && bid >= g.j[k].grid) { bid -= g.j[k].grid; ++k; }
  const RedArgs& r = g.j[k];
  const T* a = (const T*)r.a;
  const T* b = (const T*)r.b;
  T* out = (T*)r.out;
  if (r.variant == 0) {
    if (r.hasb) block_body<T, T, true>(r.keep, r.red, r.n_out, r.Q, r.Lin, r.sa, r.sb, a, b, out, bid, r.grid);
    else block_body<T, T, false>(r.keep, r.red, r.n_out, r.Q, r.Lin, r.sa, r.sb, a, b, out, bid, r.grid);
  } else if (r.variant == 1) {
    if (r.hasb) wave_body<T, T, true>(r.keep, r.red, r.n_out, r.Q, r.Lin, r.sa, r.sb, 1, r.chunk, a, b, out, nullptr, bid, r.grid);
    else wave_body<T, T, false>(r.keep, r.red, r.n_out, r.Q, r.Lin, r.sa, r.sb, 1, r.chunk, a, b, out, nullptr, bid, r.grid);
  } else {
    if (r.hasb) lane_body<T, T, true>(r.keep, r.red, r.n_out, r.R, 1, r.chunk, a, b, out, nullptr, bid, r.grid);
    else lane_body<T, T, false>(r.keep, r.red, r.n_out, r.R, 1, r.chunk, a, b, out, nullptr, bid, r.grid);
  }
}

// First (want_max = 0: minimal, 1: maximal) element along the last dim.
template <typename T>
__global__ void __launch_bounds__(kBlock) k_argminmax(Dims keep, int64_t n_out, int64_t L, int64_t sl, int want_max, const T* __restrict__ a, int64_t* __restrict__ out, T* __restrict__ vals) {
  int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t o = (int64_t)blockIdx.x * kBlock + threadIdx.x; o < n_out; o += step) {
    int64_t ko[1];
    decompose<1>(keep, o, ko);
    const T* p = a + ko[0];
    T best = p[0];
    int64_t bi = 0;
    for (int64_t j = 1; j < L; ++j) {
      T x = p[j * sl];
      bool better = want_max ? (x > best) : (x < best);
      if (better) { best = x; bi = j; }
    }
    out[o] = bi;
    if (vals) vals[o] = best;
  }
}

// The same with one wavefront per row, for long rows: every lane scans a
// strided subsequence keeping its first extremum, then lanes combine; on equal
// values the smaller index wins, which keeps "first occurrence".
template <typename T>
__global__ void __launch_bounds__(kBlock) k_argminmax_wave(Dims keep, int64_t n_out, int64_t L, int64_t sl, int want_max, const T* __restrict__ a, int64_t* __restrict__ out, T* __restrict__ vals) {
  const int lane = threadIdx.x & 63;
  int64_t wave = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
  int64_t nwaves = ((int64_t)gridDim.x * kBlock) >> 6;
  for (int64_t o = wave; o < n_out; o += nwaves) {
    int64_t ko[1];
    decompose<1>(keep, o, ko);
    const T* p = a + ko[0];
    bool have = lane < L;
    T best = have ? p[(int64_t)lane * sl] : T(0);
    int64_t bi = lane;
    for (int64_t j = lane + 64; j < L; j += 64) {
      T x = p[j * sl];
      bool better = want_max ? (x > best) : (x < best);
      if (better) { best = x; bi = j; }
    }
    for (int off = 32; off > 0; off >>= 1) {
      int o_have = __shfl_down((int)have, off, 64);
      long long o_bi = __shfl_down((long long)bi, off, 64);
      T o_best;
      if constexpr (sizeof(T) == 8) {
        unsigned long long u = *reinterpret_cast<unsigned long long*>(&best);
        unsigned lo = __shfl_down((unsigned)(u & 0xffffffffu), off, 64);
        unsigned hi = __shfl_down((unsigned)(u >> 32), off, 64);
        unsigned long long w = ((unsigned long long)hi << 32) | lo;
        o_best = *reinterpret_cast<T*>(&w);
      } else if constexpr (sizeof(T) == 4) {
        unsigned u = *reinterpret_cast<unsigned*>(&best);
        unsigned w = __shfl_down(u, off, 64);
        o_best = *reinterpret_cast<T*>(&w);
      } else {
        int w = __shfl_down((int)best, off, 64);
        o_best = (T)w;
      }
      if (o_have) {
        bool better = !have || (want_max ? (o_best > best) : (o_best < best)) || (o_best == best && o_bi < bi);
        if (better) { best = o_best; bi = o_bi; have = true; }
      }
    }
    if (lane == 0) {
      out[o] = bi;
      if (vals) vals[o] = best;
    }
  }
}

// One block of 1024 lanes per row, for a few very long rows (the minimum of a
// whole tensor): lanes scan strided subsequences, then combine through LDS with
// the same "smaller index wins ties" rule.
template <typename T>
__global__ void __launch_bounds__(1024) k_argminmax_block(Dims keep, int64_t L, int64_t sl, int want_max, const T* __restrict__ a, int64_t* __restrict__ out, T* __restrict__ vals) {
  __shared__ T sbest[1024];
  __shared__ int64_t sidx[1024];
  int64_t ko[1];
  decompose<1>(keep, blockIdx.x, ko);
  const T* p = a + ko[0];
  const int t = threadIdx.x;
  bool have = t < L;
  T best = have ? p[(int64_t)t * sl] : T(0);
  int64_t bi = t;
  // eight loads in flight; the comparisons keep the order of the positions
  int64_t j = (int64_t)t + 1024;
  for (; j + 7 * 1024 < L; j += 8 * 1024) {
    T x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) x[u] = p[(j + u * 1024) * sl];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      bool better = want_max ? (x[u] > best) : (x[u] < best);
      if (better) { best = x[u]; bi = j + u * 1024; }
    }
  }
  for (; j < L; j += 1024) {
    T x = p[j * sl];
    bool better = want_max ? (x > best) : (x < best);
    if (better) { best = x; bi = j; }
  }
  sbest[t] = best;
  sidx[t] = have ? bi : INT64_MAX;
  __syncthreads();
  for (int off = 512; off > 0; off >>= 1) {
    if (t < off) {
      T ob = sbest[t + off];
      int64_t oi = sidx[t + off];
      if (oi != INT64_MAX) {
        bool mine = sidx[t] != INT64_MAX;
        bool better = !mine || (want_max ? (ob > sbest[t]) : (ob < sbest[t])) || (ob == sbest[t] && oi < sidx[t]);
        if (better) { sbest[t] = ob; sidx[t] = oi; }
      }
    }
    __syncthreads();
  }
  if (t == 0) {
    out[blockIdx.x] = sidx[0];
    if (vals) vals[blockIdx.x] = sbest[0];
  }
}

// A few very long rows whose data one CU cannot fetch fast enough (a block
// draws some tens of GB/s): G blocks per row scan consecutive pieces, then one
// wavefront per row picks among the G candidates, the earlier piece winning ties.
template <typename T>
__global__ void __launch_bounds__(kBlock) k_argminmax_pieces(Dims keep, int64_t L, int64_t sl, int want_max, int G, int64_t piece, const T* __restrict__ a,
                                                              T* __restrict__ pbest, int64_t* __restrict__ pidx) {
  __shared__ T sbest[kBlock];
  __shared__ int64_t sidx[kBlock];
  const int row = blockIdx.x / G, g = blockIdx.x % G;
  int64_t ko[1];
  decompose<1>(keep, row, ko);
  const T* p = a + ko[0];
  const int t = threadIdx.x;
  const int64_t j0 = (int64_t)g * piece, j1 = j0 + piece < L ? j0 + piece : L;
  T best = T(0);
  int64_t bi = INT64_MAX;
  int64_t j = j0 + t;
  for (; j + 3 * kBlock < j1; j += 4 * kBlock) {
    T x[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) x[u] = p[(j + u * kBlock) * sl];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      bool better = bi == INT64_MAX || (want_max ? (x[u] > best) : (x[u] < best));
      if (better) { best = x[u]; bi = j + u * kBlock; }
    }
  }
  for (; j < j1; j += kBlock) {
    T x = p[j * sl];
    bool better = bi == INT64_MAX || (want_max ? (x > best) : (x < best));
    if (better) { best = x; bi = j; }
  }
  sbest[t] = best;
  sidx[t] = bi;
  __syncthreads();
  for (int off = kBlock / 2; off > 0; off >>= 1) {
    if (t < off) {
      T ob = sbest[t + off];
      int64_t oi = sidx[t + off];
      if (oi != INT64_MAX) {
        bool mine = sidx[t] != INT64_MAX;
        bool better = !mine || (want_max ? (ob > sbest[t]) : (ob < sbest[t])) || (ob == sbest[t] && oi < sidx[t]);
        if (better) { sbest[t] = ob; sidx[t] = oi; }
      }
    }
    __syncthreads();
  }
  if (t == 0) { pbest[blockIdx.x] = sbest[0]; pidx[blockIdx.x] = sidx[0]; }
}
template <typename T>
__global__ void __launch_bounds__(64) k_argminmax_pick(int G, int want_max, const T* __restrict__ pbest, const int64_t* __restrict__ pidx, int64_t* __restrict__ out,
                                                        T* __restrict__ vals) {
  const int row = blockIdx.x, lane = threadIdx.x;
  T best = T(0);
  int64_t bi = INT64_MAX;
  for (int g = lane; g < G; g += 64) {
    T x = pbest[row * G + g];
    int64_t xi = pidx[row * G + g];
    if (xi == INT64_MAX) continue;
    bool better = bi == INT64_MAX || (want_max ? (x > best) : (x < best));    // pieces of a lane come in ascending order
    if (better) { best = x; bi = xi; }
  }
  for (int off = 32; off > 0; off >>= 1) {
    T ob = __shfl_down(best, off);
    int64_t oi = __shfl_down(bi, off);
    if (oi != INT64_MAX) {
      bool better = bi == INT64_MAX || (want_max ? (ob > best) : (ob < best)) || (ob == best && oi < bi);
      if (better) { best = ob; bi = oi; }
    }
  }
  if (lane == 0) {
    out[row] = bi;
    if (vals) vals[row] = best;
  }
}

// The buffers of a reduction whose launch may be held back (see RedJob): what it reads and what it writes.
struct HoldBufs { hgpu_buffer* a; hgpu_buffer* b; hgpu_buffer* out; };

template <typename TI, typename TO>
int launch_stage(hgpu_ctx* ctx, bool use_wave, const Dims& keep, const Dims& red_full, int64_t n_out, int64_t R, int S, const void* a, const void* b, void* out,
                 const TermPtrs* terms = nullptr, const HoldBufs* hold = nullptr, int dtype = -1) {
  // with terms, S counts the chunks of all of them; each term is cut into s_per
  TermPtrs tp;
  tp.n = 0;
  tp.s_per = S;
  if (terms) tp = *terms;
  const int S_per = tp.n ? tp.s_per : S;
  const char* label = b ? (use_wave ? "contract_dot_wave" : "contract_dot_lane") : (use_wave ? "contract_sum_wave" : "contract_sum_lane");
  if (ctx->profiling && ctx->profile_shapes) {
    char buf[160];
    int n = snprintf(buf, sizeof buf, "%s[out%lld,R%lld,S%d,red", label, (long long)n_out, (long long)R, S);
    for (int i = 0; i < red_full.nd && n < (int)sizeof buf - 40; ++i)
      n += snprintf(buf + n, sizeof buf - n, "_%lld:%lld/%lld", (long long)red_full.shape[i], (long long)red_full.st[0][i], (long long)red_full.st[1][i]);
    n += snprintf(buf + n, sizeof buf - n, ",keep");
    for (int i = 0; i < keep.nd && n < (int)sizeof buf - 40; ++i)
      n += snprintf(buf + n, sizeof buf - n, "_%lld:%lld/%lld", (long long)keep.shape[i], (long long)keep.st[0][i], (long long)keep.st[1][i]);
    snprintf(buf + n, sizeof buf - n, "]");
    label = intern_label(ctx, buf);
  }
  const double nterms = tp.n ? tp.n : 1;
  // algorithmic bytes: every operand's distinct elements once (an operand that stands still along a dim is not read again along it)
  auto distinct = [&](int k) {
    double n = 1;
    for (int i = 0; i < keep.nd; ++i) if (keep.st[k][i] != 0) n *= (double)keep.shape[i];
    for (int i = 0; i < red_full.nd; ++i) if (red_full.st[k][i] != 0) n *= (double)red_full.shape[i];
    return n;
  };
  const double bytes = (distinct(0) + (b ? distinct(1) : 0.0)) * sizeof(TI) * nterms + (double)n_out * (S > 0 ? S : 1) * sizeof(TO),
               flops = (double)n_out * R * (b ? 2 : 1) * nterms;
  int maxb = ctx->num_cu * 8;
  // A single-launch reduction of at most eight million terms is held back: the next ones that do not read its result share its launch.
  if (hold && !terms && S <= 1 && std::is_same<TI, TO>::value && (double)n_out * (double)R <= 8.0e6) {
    RedJob j;
    j.dtype = dtype;
    j.hasb = b ? 1 : 0;
    j.keep = keep;
    j.red = red_full;
    j.n_out = n_out;
    j.R = R;
    j.a = a;
    j.b = b;
    j.out = out;
    j.label = label;
    j.bytes = bytes;
    j.flops = flops;
    if (use_wave) {
      int last = j.red.nd - 1;
      j.Lin = j.red.shape[last];
      j.sa = j.red.st[0][last];
      j.sb = j.red.st[1][last];
      j.Q = R / j.Lin;
      if (j.red.nd > 1) { j.red.nd -= 1; } else { j.red.shape[0] = 1; j.red.st[0][0] = j.red.st[1][0] = 0; }
      if (S == 0) {
        j.variant = 0;
        j.grid = (unsigned)(n_out < (int64_t)maxb ? n_out : maxb);
      } else {
        j.variant = 1;
        j.chunk = j.Q > 1 ? j.Q : j.Lin;
        j.grid = grid_for(n_out * 64, kBlock, maxb);
      }
    } else {
      j.variant = 2;
      j.chunk = R;
      j.grid = grid_for(n_out, kBlock, maxb);
    }
    hgpu_buffer* reads[2] = {hold->a, hold->b};
    if (hold_reduction(ctx, j, reads, hold->b ? 2 : 1, hold->out)) return HGPU_OK;
  }
  LaunchGuard lg(ctx, label, bytes, flops);
  if (use_wave && S == 0) {       // one block per output, no partials
    Dims red = red_full;
    int last = red.nd - 1;
    int64_t Lin = red.shape[last], sa = red.st[0][last], sb = red.st[1][last];
    int64_t Q = R / Lin;
    if (red.nd > 1) { red.nd -= 1; } else { red.shape[0] = 1; red.st[0][0] = red.st[1][0] = 0; }
    unsigned g = (unsigned)(n_out < (int64_t)maxb ? n_out : maxb);
    if (b) hipLaunchKernelGGL((k_contract_block<TI, TO, true>), dim3(g), dim3(kBlock), 0, ctx->stream, keep, red, n_out, Q, Lin, sa, sb, (const TI*)a, (const TI*)b, (TO*)out);
    else hipLaunchKernelGGL((k_contract_block<TI, TO, false>), dim3(g), dim3(kBlock), 0, ctx->stream, keep, red, n_out, Q, Lin, sa, sb, (const TI*)a, (const TI*)nullptr, (TO*)out);
  } else if (use_wave) {
    Dims red = red_full;
    int last = red.nd - 1;
    int64_t Lin = red.shape[last], sa = red.st[0][last], sb = red.st[1][last];
    int64_t Q = R / Lin;
    if (red.nd > 1) { red.nd -= 1; } else { red.shape[0] = 1; red.st[0][0] = red.st[1][0] = 0; }
    int64_t span = Q > 1 ? Q : Lin;
    int64_t chunk = (span + S_per - 1) / S_per;
    int64_t items = n_out * S;
    unsigned g = grid_for(items * 64, kBlock, maxb);
    if (b) hipLaunchKernelGGL((k_contract_wave<TI, TO, true>), dim3(g), dim3(kBlock), 0, ctx->stream, keep, red, n_out, Q, Lin, sa, sb, S, chunk, (const TI*)a, (const TI*)b, (TO*)out, tp);
    else hipLaunchKernelGGL((k_contract_wave<TI, TO, false>), dim3(g), dim3(kBlock), 0, ctx->stream, keep, red, n_out, Q, Lin, sa, sb, S, chunk, (const TI*)a, (const TI*)nullptr, (TO*)out, tp);
  } else {
    int64_t chunk = (R + S_per - 1) / S_per;
    unsigned g = grid_for(n_out * S, kBlock, maxb);
    if (b) hipLaunchKernelGGL((k_contract_lane<TI, TO, true>), dim3(g), dim3(kBlock), 0, ctx->stream, keep, red_full, n_out, R, S, chunk, (const TI*)a, (const TI*)b, (TO*)out, tp);
    else hipLaunchKernelGGL((k_contract_lane<TI, TO, false>), dim3(g), dim3(kBlock), 0, ctx->stream, keep, red_full, n_out, R, S, chunk, (const TI*)a, (const TI*)nullptr, (TO*)out, tp);
  }
  HG_CHECK_LAUNCH(ctx, "contract");
  return HGPU_OK;
}

}  // namespace

namespace hg {
hipError_t launch_reduction_group(hgpu_ctx* ctx, const RedJob* const* jobs, int n) {
  RedGroup g;
  memset(&g, 0, sizeof g);
  g.n = n;
  unsigned grid = 0;
  for (int i = 0; i < n; ++i) {
    const RedJob& j = *jobs[i];
    RedArgs& r = g.j[i];
    r.keep = j.keep;
    r.red = j.red;
    r.n_out = j.n_out;
    r.R = j.R;
    r.Q = j.Q;
    r.Lin = j.Lin;
    r.sa = j.sa;
    r.sb = j.sb;
    r.chunk = j.chunk;
    r.variant = j.variant;
    r.hasb = j.hasb;
    r.grid = j.grid;
    r.a = j.a;
    r.b = j.b;
    r.out = j.out;
    grid += j.grid;
  }
  if (jobs[0]->dtype == HGPU_F64) hipLaunchKernelGGL((k_contract_group<double>), dim3(grid), dim3(kBlock), 0, ctx->stream, g);
  else hipLaunchKernelGGL((k_contract_group<float>), dim3(grid), dim3(kBlock), 0, ctx->stream, g);
  return hipGetLastError();
}
}  // namespace hg

namespace {

int64_t min_abs_nonzero(const Dims& d, int dim) {
  int64_t m = INT64_MAX;
  for (int k = 0; k < 2; ++k) {
    int64_t s = d.st[k][dim];
    if (s < 0) s = -s;
    if (s != 0 && s < m) m = s;
  }
  return m;
}

// The HBM-bound path of hgpu_contract: out[o] = sum_r a[o,r] * b[o,r] (b may be
// null) written densely at `out`.  Long reductions with few outputs are split
// into S chunks whose partial sums a second launch adds up.  The partial sums
// live in `scratch` when the caller brings one (then nothing is allocated here,
// and a request whose partial sums exceed scratch_bytes is refused), else in a
// block from the context's allocator.
int reduce_views(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, void* out, void* scratch, size_t scratch_bytes, hgpu_buffer* out_buf = nullptr) {
  int64_t n_out = 1, R = 1;
  for (int i = 0; i < n_keep; ++i) n_out *= a->shape[i];
  for (int i = n_keep; i < a->rank; ++i) R *= a->shape[i];
  int64_t zero[HGPU_MAX_RANK] = {0};
  const int64_t* bst = b ? b->strides : zero;
  const int64_t* ks[2] = {a->strides, bst};
  const int64_t* rs[2] = {a->strides + n_keep, bst + n_keep};
  Dims keep, red;
  if (!collapse(n_keep, a->shape, 2, ks, &keep) || !collapse(a->rank - n_keep, a->shape + n_keep, 2, rs, &red))
    return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract: more than %d merged dims", HG_KDIMS);
  // Which way is memory contiguous: along the kept or along the reduced index?
  int64_t sr = min_abs_nonzero(red, red.nd - 1);
  int64_t sk = min_abs_nonzero(keep, keep.nd - 1);
  int64_t Lin = red.shape[red.nd - 1];
  bool use_wave;
  if (n_out < 2048) use_wave = true;
  else if (sr <= sk && Lin >= 16) use_wave = true;
  else use_wave = false;
  // Enough work items to fill the device, chunks of at least 512 elements.
  int64_t want_items = (int64_t)ctx->num_cu * (use_wave ? 16 : 1024);
  int64_t S = 1;
  if (n_out < want_items) {
    S = (want_items + n_out - 1) / n_out;
    int64_t span = use_wave ? ((R / Lin) > 1 ? (R / Lin) : Lin) : R;
    int64_t per = use_wave ? ((R / Lin) > 1 ? 512 / (Lin < 512 ? Lin : 512) : 1024) : 256;
    if (per < 1) per = 1;
    int64_t maxS = span / per;
    if (maxS < 1) maxS = 1;
    if (S > maxS) S = maxS;
    if (S > 4096) S = 4096;
  }
  // A caller's scratch bounds the partial sums: fewer chunks when they would not
  // fit, none (one launch, every output summed whole) when not even two do.
  if (scratch && S > 1 && (size_t)n_out * (size_t)S * 8 > scratch_bytes) {
    S = (int64_t)(scratch_bytes / ((size_t)n_out * 8));
    if (S < 2) S = 1;
  }
  const void* pa = data_ptr(a);
  const void* pb = b ? data_ptr(b) : nullptr;
  int rc = HGPU_OK;
  // (a caller that brings its own scratch wants its result written by the time the call returns to the stream: not held)
  HoldBufs hb{a->buf, b ? b->buf : nullptr, out_buf};
  const HoldBufs* hold = (out_buf && !scratch && a->buf && (!b || b->buf) && (a->dtype == HGPU_F64 || a->dtype == HGPU_F32)) ? &hb : nullptr;
  if (use_wave && ((n_out >= 64 && n_out <= 1024 && R >= 1024 && R <= 65536) || (n_out < 64 && S > 1 && R >= 1024 && R <= 16384))) {
    // a few hundred outputs of a few thousand elements (or a handful of outputs that would otherwise take a
    // launch for partial sums and a second one to add them): a block per output, one launch
    HG_DISPATCH_DTYPE(a->dtype, T, rc = (launch_stage<T, T>(ctx, true, keep, red, n_out, R, 0, pa, pb, out, nullptr, hold, a->dtype)));
  } else if (S == 1) {
    HG_DISPATCH_DTYPE(a->dtype, T, rc = (launch_stage<T, T>(ctx, use_wave, keep, red, n_out, R, 1, pa, pb, out, nullptr, hold, a->dtype)));
  } else {
    // stage 1: partials [n_out, S] in the accumulator type; stage 2 sums them.
    const size_t need = (size_t)n_out * (size_t)S * 8;
    hgpu_buffer* part = nullptr;
    void* pp = scratch;
    if (scratch) {
      if (need > scratch_bytes)   // cannot happen after the clamp above; kept as the guard of the fixed array
        return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract: %lld outputs in %lld chunks need %zu bytes of partial sums, the fixed scratch holds %zu",
                    (long long)n_out, (long long)S, need, scratch_bytes);
    } else {
      rc = buffer_alloc(ctx, need, &part);
      if (rc) return rc;
      pp = part->ptr;
    }
    int64_t psh[2] = {n_out, S}, pst[2] = {S, 1};
    HG_DISPATCH_DTYPE(a->dtype, T, { using A = typename acc_of<T>::type; rc = (launch_stage<T, A>(ctx, use_wave, keep, red, n_out, R, (int)S, pa, pb, pp)); });
    if (!rc) {
      Dims k2, r2;
      int64_t z1[1] = {0};
      const int64_t* ks2[2] = {pst, z1};
      const int64_t* rs2[2] = {pst + 1, z1};
      collapse(1, psh, 2, ks2, &k2);
      collapse(1, psh + 1, 2, rs2, &r2);
      bool wave2 = n_out < 65536;
      HG_DISPATCH_DTYPE(a->dtype, T, { using A = typename acc_of<T>::type; rc = (launch_stage<A, T>(ctx, wave2, k2, r2, n_out, S, 1, pp, nullptr, out)); });
    }
    if (part) buffer_release(part);
  }
  return rc;
}

// Partial sums of hgpu_contract_noalloc: one array per device, held until the
// process ends.  In host code the name below is only a stand-in for the symbol:
// the device address comes from hipGetSymbolAddress, once per device.
constexpr size_t kScratchBytes = 1u << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mu;

int scratch_of(hgpu_ctx* ctx, void** out) {
  if (ctx->device < 0 || ctx->device >= kMaxDevices) return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract_noalloc: device %d", ctx->device);
  std::lock_guard<std::mutex> g(g_scratch_mu);
  if (!g_scratch_ptr[ctx->device]) {
    hipError_t e = hipSetDevice(ctx->device);
    void* p = nullptr;
    if (e == hipSuccess) e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return check_hip(ctx, e == hipSuccess ? hipErrorInvalidSymbol : e, "hipGetSymbolAddress(scratch)");
    g_scratch_ptr[ctx->device] = p;
  }
  *out = g_scratch_ptr[ctx->device];
  return HGPU_OK;
}

// *acc += x, taking over x (the first term becomes the accumulator).
int add_into(hgpu_ctx* ctx, hgpu_array** acc, hgpu_array* x) {
  if (!*acc) { *acc = x; return HGPU_OK; }
  hgpu_array* sum = nullptr;
  int rc = hgpu_ewise2(ctx, HGPU_ADD, *acc, x, &sum);
  hgpu_release(*acc);
  hgpu_release(x);
  *acc = rc ? nullptr : sum;
  return rc;
}

// out = sum_t contract(as[t], bs[t]) for terms of one layout that are not a
// matrix product: the terms' chunks are reduced by one launch into partials
// [n_out, n * S], a second launch adds the partials up.
int contract_terms(hgpu_ctx* ctx, int n, const hgpu_array* const* as, const hgpu_array* const* bs, int n_keep, hgpu_array* o) {
  const hgpu_array* a = as[0];
  const hgpu_array* b = bs[0];
  int64_t n_out = nelem(o), R = 1;
  for (int i = n_keep; i < a->rank; ++i) R *= a->shape[i];
  const int64_t* ks[2] = {a->strides, b->strides};
  const int64_t* rs[2] = {a->strides + n_keep, b->strides + n_keep};
  Dims keep, red;
  if (!collapse(n_keep, a->shape, 2, ks, &keep) || !collapse(a->rank - n_keep, a->shape + n_keep, 2, rs, &red))
    return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract_sum: more than %d merged dims", HG_KDIMS);
  int64_t sr = min_abs_nonzero(red, red.nd - 1), sk = min_abs_nonzero(keep, keep.nd - 1);
  int64_t Lin = red.shape[red.nd - 1];
  bool use_wave = n_out < 2048 || (sr <= sk && Lin >= 16);
  int64_t want_items = (int64_t)ctx->num_cu * (use_wave ? 16 : 1024);
  int64_t S = 1;
  if (n_out * n < want_items) {
    S = (want_items + n_out * n - 1) / (n_out * n);
    int64_t span = use_wave ? ((R / Lin) > 1 ? (R / Lin) : Lin) : R;
    int64_t per = use_wave ? ((R / Lin) > 1 ? 512 / (Lin < 512 ? Lin : 512) : 1024) : 256;
    if (per < 1) per = 1;
    int64_t maxS = span / per;
    if (maxS < 1) maxS = 1;
    if (S > maxS) S = maxS;
    if (S > 128) S = 128;
  }
  TermPtrs tp;
  tp.n = n;
  tp.s_per = (int)S;
  for (int t = 0; t < n; ++t) { tp.a[t] = data_ptr(as[t]); tp.b[t] = data_ptr(bs[t]); }
  const int64_t S_all = S * n;
  int accdt = dtype_is_float(a->dtype) ? HGPU_F64 : HGPU_I64;
  int64_t psh[2] = {n_out, S_all};
  hgpu_array* part = nullptr;
  int rc = new_dense(ctx, accdt, 2, psh, &part);
  if (rc) return rc;
  HG_DISPATCH_DTYPE(a->dtype, T, { using A = typename acc_of<T>::type; rc = (launch_stage<T, A>(ctx, use_wave, keep, red, n_out, R, (int)S_all, tp.a[0], tp.b[0], data_ptr(part), &tp)); });
  if (!rc) {
    Dims k2, r2;
    int64_t z1[1] = {0};
    const int64_t* ks2[2] = {part->strides, z1};
    const int64_t* rs2[2] = {part->strides + 1, z1};
    collapse(1, psh, 2, ks2, &k2);
    collapse(1, psh + 1, 2, rs2, &r2);
    bool wave2 = n_out < 65536;
    HG_DISPATCH_DTYPE(a->dtype, T, { using A = typename acc_of<T>::type; rc = (launch_stage<A, T>(ctx, wave2, k2, r2, n_out, S_all, 1, data_ptr(part), nullptr, data_ptr(o))); });
  }
  hgpu_release(part);
  return rc;
}

}  // namespace

extern "C" {

int hgpu_contract_sum(hgpu_ctx* ctx, int n, const hgpu_array* const* as, const hgpu_array* const* bs, int n_keep, hgpu_array** out) {
  if (!ctx || !as || !bs || !out || n < 1) return HGPU_ERR_INVALID;
  for (int t = 0; t < n; ++t) {
    if (!as[t] || !bs[t]) return HGPU_ERR_INVALID;
    if (as[t]->dtype != as[0]->dtype || bs[t]->dtype != as[0]->dtype) return fail(ctx, HGPU_ERR_INVALID, "contract_sum: dtypes differ");
    if (!same_shape(as[t], as[0]) || !same_shape(bs[t], as[0])) return fail(ctx, HGPU_ERR_INVALID, "contract_sum: shapes differ");
  }
  const hgpu_array* a = as[0];
  if (n_keep < 0 || n_keep > a->rank) return fail(ctx, HGPU_ERR_INVALID, "contract_sum: n_keep %d of rank %d", n_keep, a->rank);
  if (n == 1) return hgpu_contract(ctx, as[0], bs[0], n_keep, out);
  // Terms of one layout go out together, 32 to a launch: when such a group is a
  // matrix product the K chunks of all its terms are summed in one fixed order
  // by one kernel.  Groups are formed in order of first appearance and their
  // results added in that order.
  const bool groupable = nelem(a) > 0 && (a->dtype == HGPU_F64 || a->dtype == HGPU_F32);
  auto same_layout = [&](int s, int t) {
    for (int d = 0; d < a->rank; ++d)
      if (as[s]->strides[d] != as[t]->strides[d] || bs[s]->strides[d] != bs[t]->strides[d]) return false;
    return true;
  };
  std::vector<char> taken((size_t)n, 0);
  hgpu_array* acc = nullptr;
  for (int t0 = 0; t0 < n; ++t0) {
    if (taken[(size_t)t0]) continue;
    std::vector<const hgpu_array*> ga{as[t0]}, gb{bs[t0]};
    taken[(size_t)t0] = 1;
    for (int t = t0 + 1; t < n && groupable && ga.size() < (size_t)kGemmMaxTerms; ++t)
      if (!taken[(size_t)t] && same_layout(t0, t)) { ga.push_back(as[t]); gb.push_back(bs[t]); taken[(size_t)t] = 1; }
    hgpu_array* part = nullptr;
    int rc = HGPU_OK;
    size_t done = 0;
    if (ga.size() > 1) {
      rc = new_dense(ctx, a->dtype, n_keep, a->shape, &part);
      bool handled = false;
      if (!rc) rc = try_gemm(ctx, ga[0], gb[0], n_keep, part, &handled, (int)ga.size(), ga.data(), gb.data());
      if (!rc && !handled && nelem(part) > 0) {   // not a matrix product: the grouped reduction
        rc = contract_terms(ctx, (int)ga.size(), ga.data(), gb.data(), n_keep, part);
        handled = !rc;
      }
      if (rc || !handled) { if (part) hgpu_release(part); part = nullptr; }
      else done = ga.size();
    }
    for (size_t t = done; t < ga.size() && !rc; ++t) {   // not a matrix product (or a single term): one by one
      hgpu_array* one = nullptr;
      rc = hgpu_contract(ctx, ga[t], gb[t], n_keep, &one);
      if (!rc) rc = add_into(ctx, &part, one);
    }
    if (!rc) rc = add_into(ctx, &acc, part), part = nullptr;
    if (rc) { if (part) hgpu_release(part); if (acc) hgpu_release(acc); return rc; }
  }
  *out = acc;
  return HGPU_OK;
}

int hgpu_contract(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (n_keep < 0 || n_keep > a->rank) return fail(ctx, HGPU_ERR_INVALID, "contract: n_keep %d of rank %d", n_keep, a->rank);
  if (b) {
    if (b->dtype != a->dtype) return fail(ctx, HGPU_ERR_INVALID, "contract: dtypes differ");
    if (!same_shape(a, b)) return fail(ctx, HGPU_ERR_INVALID, "contract: shapes differ");
  }
  if (a->dtype == HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "contract: Bool arrays have no sum");
  // A kept dim along which neither operand moves (both replicated) repeats the
  // same values: compute once without it, replicate the result as a view.
  {
    bool repeats = false;
    int64_t sh1[HGPU_MAX_RANK];
    for (int i = 0; i < a->rank; ++i) {
      sh1[i] = a->shape[i];
      if (i < n_keep && a->shape[i] > 1 && a->strides[i] == 0 && (!b || b->strides[i] == 0)) { sh1[i] = 1; repeats = true; }
    }
    bool empty = false;
    for (int i = 0; i < a->rank; ++i) empty = empty || a->shape[i] == 0;
    if (repeats && !empty) {
      hgpu_array* a1 = new_view(ctx, a->buf, a->dtype, a->rank, sh1, a->strides, a->offset);
      hgpu_array* b1 = b ? new_view(ctx, b->buf, b->dtype, b->rank, sh1, b->strides, b->offset) : nullptr;
      hgpu_array* small = nullptr;
      int rc1 = hgpu_contract(ctx, a1, b1, n_keep, &small);
      hgpu_release(a1);
      if (b1) hgpu_release(b1);
      if (rc1) return rc1;
      int64_t st[HGPU_MAX_RANK];
      for (int i = 0; i < n_keep; ++i) st[i] = sh1[i] != a->shape[i] ? 0 : small->strides[i];
      *out = new_view(ctx, small->buf, small->dtype, n_keep, a->shape, st, small->offset);
      hgpu_release(small);
      return HGPU_OK;
    }
  }
  hgpu_array* o = nullptr;
  int64_t n_out = 1, R = 1;
  for (int i = 0; i < n_keep; ++i) n_out *= a->shape[i];
  for (int i = n_keep; i < a->rank; ++i) R *= a->shape[i];
  int rc;
  if (n_out == 0 || R == 0) {
    rc = new_zeros(ctx, a->dtype, n_keep, a->shape, &o);
    if (rc) return rc;
    *out = o;
    return HGPU_OK;
  }
  rc = new_dense(ctx, a->dtype, n_keep, a->shape, &o);
  if (rc) return rc;

  bool handled = false;
  rc = try_gemm(ctx, a, b, n_keep, o, &handled);
  if (rc) { hgpu_release(o); return rc; }
  if (handled) { *out = o; return HGPU_OK; }

  rc = reduce_views(ctx, a, b, n_keep, data_ptr(o), nullptr, 0, o->buf);
  if (rc) { hgpu_release(o); return rc; }
  *out = o;
  return HGPU_OK;
}

int hgpu_contract_noalloc(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array* out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (n_keep < 0 || n_keep > a->rank) return fail(ctx, HGPU_ERR_INVALID, "contract_noalloc: n_keep %d of rank %d", n_keep, a->rank);
  if (b) {
    if (b->dtype != a->dtype) return fail(ctx, HGPU_ERR_INVALID, "contract_noalloc: dtypes differ");
    if (!same_shape(a, b)) return fail(ctx, HGPU_ERR_INVALID, "contract_noalloc: shapes differ");
  }
  if (a->dtype == HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "contract_noalloc: Bool arrays have no sum");
  if (out->dtype != a->dtype || out->rank != n_keep || !is_dense(out)) return fail(ctx, HGPU_ERR_INVALID, "contract_noalloc: the result array must be dense, of the operands' dtype and of the kept shape");
  for (int i = 0; i < n_keep; ++i)
    if (out->shape[i] != a->shape[i]) return fail(ctx, HGPU_ERR_INVALID, "contract_noalloc: the result array must have the kept shape");
  if (out->buf && (out->buf == a->buf || (b && out->buf == b->buf))) return fail(ctx, HGPU_ERR_INVALID, "contract_noalloc: the result shares memory with an operand");
  int64_t n_out = nelem(out), R = 1;
  for (int i = n_keep; i < a->rank; ++i) R *= a->shape[i];
  if (n_out == 0) return HGPU_OK;
  if (R == 0) {   // an empty sum: zeros (the fill rounds up to 16 bytes, which stays inside a block only from its start)
    if (out->offset != 0) return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract_noalloc: an empty sum into a view that does not start its block");
    return zero_fill(ctx, data_ptr(out), (size_t)n_out * dtype_size(out->dtype));
  }
  void* sp = nullptr;
  if (int rc = scratch_of(ctx, &sp)) return rc;
  return reduce_views(ctx, a, b, n_keep, data_ptr(out), sp, kScratchBytes);
}

int hgpu_extremum_last(hgpu_ctx* ctx, const hgpu_array* a, int want_max, hgpu_array** values, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (a->rank < 1) return fail(ctx, HGPU_ERR_INVALID, "argminmax: rank 0");
  int64_t L = a->shape[a->rank - 1];
  if (L < 1) return fail(ctx, HGPU_ERR_INVALID, "argminmax: empty last dim");
  hgpu_array* o = nullptr;
  int rc = new_dense(ctx, HGPU_I64, a->rank - 1, a->shape, &o);
  if (rc) return rc;
  hgpu_array* v = nullptr;
  if (values) {
    rc = new_dense(ctx, a->dtype, a->rank - 1, a->shape, &v);
    if (rc) { hgpu_release(o); return rc; }
  }
  int64_t n_out = nelem(o);
  if (n_out > 0) {
    const int64_t* ks[1] = {a->strides};
    Dims keep;
    if (!collapse(a->rank - 1, a->shape, 1, ks, &keep)) { hgpu_release(o); if (v) hgpu_release(v); return fail(ctx, HGPU_ERR_UNSUPPORTED, "argminmax: too many dims"); }
    LaunchGuard lg(ctx, "argminmax", (double)n_out * (L * dtype_size(a->dtype) + 8 + (v ? dtype_size(a->dtype) : 0)), (double)n_out * L);
    void* vp = v ? data_ptr(v) : nullptr;
    if (L >= 16384 && n_out <= 16) {
      // very few, very long rows: pieces of a row to many blocks, then one pick per row
      const int G = (int)std::min<int64_t>(128, L / 2048);
      const int64_t piece = (L + G - 1) / G;
      hgpu_buffer* scratch = nullptr;
      const size_t vb = ((size_t)n_out * G * dtype_size(a->dtype) + 15) / 16 * 16;
      rc = buffer_alloc(ctx, vb + (size_t)n_out * G * 8, &scratch);
      if (rc) { hgpu_release(o); if (v) hgpu_release(v); return rc; }
      void* pb = scratch->ptr;
      int64_t* pi = (int64_t*)((char*)scratch->ptr + vb);
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_argminmax_pieces<T>, dim3((unsigned)(n_out * G)), dim3(kBlock), 0, ctx->stream, keep, L, a->strides[a->rank - 1], want_max, G, piece, (const T*)data_ptr(a), (T*)pb, pi));
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_argminmax_pick<T>, dim3((unsigned)n_out), dim3(64), 0, ctx->stream, G, want_max, (const T*)pb, (const int64_t*)pi, (int64_t*)data_ptr(o), (T*)vp));
      buffer_release(scratch);
    } else if (L >= 8192 && n_out <= 64) {
      // few long rows: a whole block per row
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_argminmax_block<T>, dim3((unsigned)n_out), dim3(1024), 0, ctx->stream, keep, L, a->strides[a->rank - 1], want_max, (const T*)data_ptr(a), (int64_t*)data_ptr(o), (T*)vp));
    } else if (L >= 256 && n_out < (int64_t)ctx->num_cu * 64) {
      unsigned g = grid_for(n_out * 64, kBlock, ctx->num_cu * 8);
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_argminmax_wave<T>, dim3(g), dim3(kBlock), 0, ctx->stream, keep, n_out, L, a->strides[a->rank - 1], want_max, (const T*)data_ptr(a), (int64_t*)data_ptr(o), (T*)vp));
    } else {
      unsigned g = grid_for(n_out, kBlock, ctx->num_cu * 8);
      HG_DISPATCH_DTYPE(a->dtype, T, hipLaunchKernelGGL(k_argminmax<T>, dim3(g), dim3(kBlock), 0, ctx->stream, keep, n_out, L, a->strides[a->rank - 1], want_max, (const T*)data_ptr(a), (int64_t*)data_ptr(o), (T*)vp));
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { hgpu_release(o); if (v) hgpu_release(v); return check_hip(ctx, e, "argminmax"); }
  }
  *out = o;
  if (values) *values = v;
  return HGPU_OK;
}

int hgpu_argminmax_last(hgpu_ctx* ctx, const hgpu_array* a, int want_max, hgpu_array** out) {
  return hgpu_extremum_last(ctx, a, want_max, nullptr, out);
}

}  // extern "C"
