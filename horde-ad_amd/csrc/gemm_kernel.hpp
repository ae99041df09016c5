// The MFMA kernel behind hgpu_contract's matrix-product path, shared by the
// per-precision translation units (gemm_f32.hip, gemm_f64.hip).
//
// Operands are addressed through separable offset maps,
//     A[m, k] = A0 + offAm(m) + offAk(k),   B[n, k] = B0 + offBn(n) + offBk(k),
//     C[m, n] = C0 + offCm(m) + offCn(n),
// with m, n, k linear indices into merged dim groups (Group).  The K offsets
// come from two tables written by k_koff (or, for a single K dim, from a
// multiplication: see KOff); row offsets are decomposed once per thread.
//
// 256 threads = 4 wavefronts in a WGM x WGN grid; block tile BM x BN with
// K-step 16.  Operand tiles go global -> registers -> LDS ([k][row] order, one
// element of padding per k-row); the global loads of step t+1 are in flight
// while the MFMAs of step t run, and with two LDS buffers a step needs a single
// barrier.  Lanes staging an operand run along whichever of row / k is
// contiguous in memory (run-time choice per operand), with 16-byte loads when
// the host has checked contiguity and alignment.
#pragma once
#include "common.hpp"
#include <type_traits>

namespace hg {
namespace gemm {

constexpr int BK = 16, NT = 256;
constexpr int GD = 5;  // dims per index group after merging
constexpr int kMaxTerms = 32;   // products summed by one launch (hgpu_contract_sum)

struct Group {
  int nd;
  int64_t shape[GD];
  int64_t sa[GD], sb[GD], sc[GD];
};

struct GemmParams {
  Group m, n, k, bt;
  int64_t M, N, K, BT;
  int a_kc, b_kc;     // lanes staging A (B) run along k (1) or along m (n) (0)
  int split;          // K chunks
  int64_t kchunk;     // K elements per chunk (multiple of BK)
  int64_t c_split_stride;  // elements between partial outputs
  // A sum of products of one shape and layout (hgpu_contract_sum): the K chunks
  // of all terms are enumerated together, chunk index = term * term_split + chunk
  // within the term, and term t reads a_term[t] / b_term[t].  n_terms == 0: one
  // product, the operands are the kernel's pointer arguments.
  int n_terms, term_split;
  int term_loop;           // staged kernel: every block walks all terms itself (k_gemm with LOOP)
  const void* a_term[kMaxTerms];
  const void* b_term[kMaxTerms];
  int c_rows_contig;       // staged kernel: the output is contiguous along m (and not along n)
  int64_t kmask, ksa, ksb; // K offsets: table[k & kmask] + k * ks; kmask 0 = no table (see KOff)
};

__device__ __forceinline__ void group_off(const Group& g, int64_t lin, int64_t* oa, int64_t* ob, int64_t* oc) {
  int64_t a = 0, b = 0, c = 0;
  int64_t r = lin;
  for (int i = g.nd - 1; i >= 0; --i) {
    int64_t idx;
    if (i > 0) {
      int64_t q = r / g.shape[i];
      idx = r - q * g.shape[i];
      r = q;
    } else {
      idx = r;
    }
    a += idx * g.sa[i];
    b += idx * g.sb[i];
    c += idx * g.sc[i];
  }
  *oa = a;
  *ob = b;
  *oc = c;
}

// MFMA flavours.  One instruction multiplies a BMR x KI block of A by a KI x NBW
// block of B.  A fragment: lane l supplies A[row = l % BMR][k = l / BMR].
// B fragment: lane l supplies B[k = l / NBW][col = bcol(l)].  Accumulator
// register r of lane l holds D[row(l, r)][col(l)] of a (BMR x NBW) block.
struct MfmaF32 {
  using T = float;
  using Acc = __attribute__((ext_vector_type(4))) float;
  static constexpr int NBW = 16, NR = 4, BMR = 16, KI = 4;
  static __device__ __forceinline__ Acc zero() { return Acc{0, 0, 0, 0}; }
  static __device__ __forceinline__ Acc run(T a, T b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int bcol(int l) { return l & 15; }
  static __device__ __forceinline__ int row(int l, int r) { return 4 * (l >> 4) + r; }
  static __device__ __forceinline__ int col(int l) { return l & 15; }
  static __device__ __forceinline__ T get(const Acc& c, int r) { return c[r]; }
};
// v_mfma_f32_32x32x2_f32: the instruction stream of 32 x 32 blocks sustains
// nearly the published fp32 rate where that of 16 x 16 x 4 blocks stays near
// 0.8 of it (hgpu_mfma_probe measures both); same LDS reads per flop.
struct MfmaF32W {
  using T = float;
  using Acc = __attribute__((ext_vector_type(16))) float;
  static constexpr int NBW = 32, NR = 16, BMR = 32, KI = 2;
  static __device__ __forceinline__ Acc zero() { return Acc{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}; }
  static __device__ __forceinline__ Acc run(T a, T b, Acc c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int bcol(int l) { return l & 31; }
  static __device__ __forceinline__ int row(int l, int r) { return 8 * (r >> 2) + 4 * (l >> 5) + (r & 3); }
  static __device__ __forceinline__ int col(int l) { return l & 31; }
  static __device__ __forceinline__ T get(const Acc& c, int r) { return c[r]; }
};
struct MfmaF64 {
  using T = double;
  using Acc = __attribute__((ext_vector_type(4))) double;
  static constexpr int NBW = 16, NR = 4, BMR = 16, KI = 4;
  static __device__ __forceinline__ Acc zero() { return Acc{0, 0, 0, 0}; }
  static __device__ __forceinline__ Acc run(T a, T b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int bcol(int l) { return l & 15; }
  static __device__ __forceinline__ int row(int l, int r) { return 4 * r + (l >> 4); }
  static __device__ __forceinline__ int col(int l) { return l & 15; }
  static __device__ __forceinline__ T get(const Acc& c, int r) { return c[r]; }
};
template <typename T, int V> struct VecOf;
template <> struct VecOf<double, 1> { using type = double; };
template <> struct VecOf<float, 1> { using type = float; };
// element-aligned vectors: multi-dword global loads need dword alignment only
template <> struct VecOf<double, 2> { using type = double __attribute__((ext_vector_type(2), aligned(8))); };
template <> struct VecOf<float, 4> { using type = float __attribute__((ext_vector_type(4), aligned(4))); };

// K offset of linear index k for one operand: tab[k & kmask] + k * stride.
// Several K dims: a table written by k_koff, kmask all ones, stride 0.  A single
// K dim: kmask 0 on a table of zeros and the dim's stride.
struct KOff {
  const int64_t* __restrict__ tab;
  int64_t stride;
};

// Stages one operand tile (R rows x BK) from global memory into LDS.  A slot is
// V consecutive elements along the direction the lanes run (along k when kc,
// else along the rows); a lane owns NL slots.
//
// The loads of a tile are issued together, unconditionally (rows and k past the
// end are clamped to the last valid slot and zeroed when the tile is stored),
// and nothing between issuing them and storing them to LDS waits on memory: the
// MFMAs of the current tile run under the whole latency.  A load that sits in a
// branch, or whose value is consumed before the MFMAs, makes the compiler wait
// for every load in flight at that point, which serialises the tile's loads.
// For the same reason the K table (TAB) is read one tile ahead and its entries
// are first used when the next tile's addresses are formed; the kernels choose
// TAB once, outside the K loop, so that the loop itself has no table branch.
template <typename T, int R, int V, bool TAB>
struct Stager {
  static constexpr int NL = R * BK / NT / V;
  static_assert(NL >= 1, "tile too small for 256 threads");
  using Vec = typename VecOf<T, V>::type;
  static constexpr int ML = R / V;        // lanes per k-row when running along rows
  static constexpr int KL = BK / V;       // lanes per row when running along k

  // slot i sits at row rl0 + i * drl, k kl0 + i * dkl of the tile
  int rl0, kl0, drl, dkl;
  int dk;
  int64_t klast;                  // last k a slot may start at
  // Where slot i of the next tile to issue starts.  Without a table: the
  // address itself, moved on by one K-step at a time.  With a table: the row's
  // address and, apart, the table entry of the slot's k.
  const T* ptr[NL];
  int64_t tv[TAB ? NL : 1];
  int64_t kstep;                  // BK * stride
  int64_t kfull;                  // K: a tile that ends at or before it needs no clamping
  // LDS element offset of slot i's first element in a [BK][R + 1] tile, and the
  // step from one element of a slot to the next: fixed for the whole K loop
  int so0, dso, dj;

  __device__ __forceinline__ int rl(int i) const { return rl0 + i * drl; }
  __device__ __forceinline__ int kl(int i) const { return kl0 + i * dkl; }
  __device__ __forceinline__ int64_t clamp_k(int64_t k) const {
    k = k < klast ? k : klast;
    return k > 0 ? k : 0;
  }

  // which: 0 = operand A (offsets sa), 1 = operand B (offsets sb)
  __device__ __forceinline__ void init(int t, int kc, int which, const T* base, const Group& g, int64_t r0, int64_t rows,
                                       const KOff& ko, int64_t kbeg, int64_t K) {
    dk = kc ? 1 : 0;
    klast = K - (kc ? V : 1);
    kstep = (int64_t)BK * ko.stride;
    kfull = K;
    if (kc) { rl0 = t / KL; drl = NT / KL; kl0 = (t % KL) * V; dkl = 0; }
    else { rl0 = (t % ML) * V; drl = 0; kl0 = t / ML; dkl = NT / ML; }
    so0 = kl0 * (R + 1) + rl0;
    dso = dkl * (R + 1) + drl;
    dj = kc ? R + 1 : 1;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      if (kc || i == 0) {
        int64_t r = r0 + rl(i);
        if (r >= rows) r = rows - (kc ? 1 : V);   // clamp: the values are never stored
        int64_t oa, ob, oc;
        group_off(g, r, &oa, &ob, &oc);
        ptr[i] = base + (which == 0 ? oa : ob);
      } else {
        ptr[i] = ptr[0];
      }
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int64_t k = clamp_k(kbeg + kl(i));
      if constexpr (TAB) tv[i] = ko.tab[k];
      else ptr[i] += k * ko.stride;
    }
  }

  // the slots move on to the tile that starts at k0
  __device__ __forceinline__ void advance(const KOff& ko, int64_t k0) {
    if (k0 + BK <= kfull) {       // the whole tile lies inside K (uniform): no clamping
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        if constexpr (TAB) tv[i] = ko.tab[k0 + kl(i)];
        else ptr[i] += kstep;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int64_t k = k0 + kl(i);
        if constexpr (TAB) tv[i] = ko.tab[clamp_k(k)];
        else ptr[i] += k <= klast ? kstep : 0;      // a slot past the end stays where it is: still readable, never stored
      }
    }
  }

  __device__ __forceinline__ void issue(Vec* __restrict__ r) const {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      if constexpr (TAB) r[i] = *reinterpret_cast<const Vec*>(ptr[i] + tv[i]);
      else r[i] = *reinterpret_cast<const Vec*>(ptr[i]);
    }
  }

  // r holds the tile that starts at k0
  __device__ __forceinline__ void store(const Vec* __restrict__ r, int64_t k0, int64_t kend, T (*S)[R + 1]) const {
    T* S0 = &S[0][0];
    if (k0 + BK <= kend) {        // a whole tile (uniform): nothing to zero
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        if constexpr (V == 1) S0[so0 + i * dso] = r[i];
        else {
#pragma unroll
          for (int j = 0; j < V; ++j) S0[so0 + i * dso + j * dj] = r[i][j];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const bool ok = k0 + kl(i) < kend;
        if constexpr (V == 1) S0[so0 + i * dso] = ok ? r[i] : T(0);
        else {
#pragma unroll
          for (int j = 0; j < V; ++j) S0[so0 + i * dso + j * dj] = ok ? r[i][j] : T(0);
        }
      }
    }
  }
};

// One block's K loop over [kbeg, kend) of one product: accumulates into acc.
// Ends with a barrier, so the LDS tiles are free when it returns.
template <typename X, int WGM, int WGN, int TM, int TN, int VA, int VB, int NBUF, bool TAB>
__device__ __forceinline__ void k_loop(const GemmParams& p, const typename X::T* A, const typename X::T* B, const int64_t* koffA,
                                       const int64_t* koffB, int64_t m0, int64_t n0, int64_t kbeg, int64_t kend,
                                       typename X::T (*As)[BK][WGM * TM * 16 + 1], typename X::T (*Bs)[BK][WGN * TN * 16 + 1],
                                       typename X::Acc (*acc)[TN * 16 / X::NBW]) {
  using T = typename X::T;
  constexpr int BM = WGM * TM * 16, BN = WGN * TN * 16;
  constexpr int TNB = TN * 16 / X::NBW, TMB = TM * 16 / X::BMR;
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  using SA = Stager<T, BM, VA, TAB>;
  using SB = Stager<T, BN, VB, TAB>;
  SA sa;
  SB sb;
  typename SA::Vec ra[SA::NL];
  typename SB::Vec rb[SB::NL];
  const KOff koa{koffA, p.ksa}, kob{koffB, p.ksb};
  sa.init(t, p.a_kc, 0, A, p.m, m0, p.M, koa, kbeg, p.K);
  sb.init(t, p.b_kc, 1, B, p.n, n0, p.N, kob, kbeg, p.K);
  if (kbeg < kend) {
    sa.issue(ra);
    sb.issue(rb);
    sa.advance(koa, kbeg + BK);
    sb.advance(kob, kbeg + BK);
    sa.store(ra, kbeg, kend, As[0]);
    sb.store(rb, kbeg, kend, Bs[0]);
  }
  __syncthreads();
  int cur = 0;
  for (int64_t k0 = kbeg; k0 < kend; k0 += BK) {
    const bool more = k0 + BK < kend;
    if (more) {
      sa.issue(ra);
      sb.issue(rb);
      sa.advance(koa, k0 + 2 * BK);
      sb.advance(kob, k0 + 2 * BK);
    }
#pragma unroll
    for (int kk = 0; kk < BK; kk += X::KI) {
      const int kr = kk + lane / X::BMR;
      T fa[TMB], fb[TNB];
#pragma unroll
      for (int i = 0; i < TMB; ++i) fa[i] = As[cur][kr][wm * TM * 16 + i * X::BMR + (lane & (X::BMR - 1))];
#pragma unroll
      for (int j = 0; j < TNB; ++j) fb[j] = Bs[cur][kr][wn * TN * 16 + j * X::NBW + X::bcol(lane)];
#pragma unroll
      for (int i = 0; i < TMB; ++i)
#pragma unroll
        for (int j = 0; j < TNB; ++j) acc[i][j] = X::run(fa[i], fb[j], acc[i][j]);
    }
    if constexpr (NBUF == 1) __syncthreads();   // every wavefront is done reading the tile
    const int nxt = NBUF == 2 ? cur ^ 1 : 0;
    if (more) {
      sa.store(ra, k0 + BK, kend, As[nxt]);
      sb.store(rb, k0 + BK, kend, Bs[nxt]);
    }
    __syncthreads();
    cur = nxt;
  }
}

// Block tile BM x BN = (WGM * TM * 16) x (WGN * TN * 16).  NBUF LDS buffers.
// Skinny tiles keep few accumulators: ask for two wavefronts per SIMD there, so
// that a second block on the CU runs through the first one's barriers and LDS
// stores (three would leave the staging registers of the 256-row tiles too few
// VGPRs: they spill).
constexpr int waves_wanted(int tm, int tn, int esize) { return tm * tn * esize <= 32 ? 2 : 1; }

//
// LOOP: a SUM of products of one layout whose tiles fill the device by
// themselves -- every block walks all terms (GemmParams::a_term / b_term) and
// adds them up in its accumulators, so there are no partial outputs and
// blockIdx.y counts K chunks only.  Otherwise a block works on one term, which
// its chunk index selects.
template <typename X, int WGM, int WGN, int TM, int TN, int VA, int VB, int NBUF, bool LOOP = false>
__global__ void __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(waves_wanted(TM, TN, (int)sizeof(typename X::T)), 8))) k_gemm(GemmParams p, const typename X::T* __restrict__ A, const typename X::T* __restrict__ B,
                                             typename X::T* __restrict__ C, const int64_t* __restrict__ koffA,
                                             const int64_t* __restrict__ koffB) {
  using T = typename X::T;
  using Acc = typename X::Acc;
  constexpr int BM = WGM * TM * 16, BN = WGN * TN * 16;
  constexpr int TNB = TN * 16 / X::NBW;     // MFMA blocks per wavefront along n
  constexpr int TMB = TM * 16 / X::BMR;     // and along m
  static_assert(TMB * X::BMR == TM * 16 && TNB * X::NBW == TN * 16, "whole MFMA blocks per wavefront");
  static_assert(WGM * WGN == 4, "four wavefronts");
  __shared__ T As[NBUF][BK][BM + 1];
  __shared__ T Bs[NBUF][BK][BN + 1];

  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  // XCD-aware numbering of (K chunk, tile): blocks b, b+8, b+16, ... of the
  // grid's x-then-y order share an XCD and its L2.  Each XCD gets a contiguous
  // range of the chunk-major order, so the tiles that read the same rows of A
  // or B over the same K chunk run on one XCD and share those rows in its L2.
  const int64_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int64_t ntiles = tiles_m * tiles_n;
  const int64_t nblocks = ntiles * gridDim.y;
  int64_t lin = blockIdx.x + ntiles * (int64_t)blockIdx.y;
  if (nblocks >= 64) {
    const int64_t x = lin & 7, per = nblocks >> 3, rem = nblocks & 7;
    lin = x * per + (x < rem ? x : rem) + (lin >> 3);
  }
  const int s = (int)(lin / ntiles);
  const int64_t bid = lin - s * ntiles;
  const int64_t tile_m = bid / tiles_n, tile_n = bid - tile_m * tiles_n;
  const int64_t m0 = tile_m * BM, n0 = tile_n * BN;

  int64_t bta, btb, btc;
  group_off(p.bt, blockIdx.z, &bta, &btb, &btc);
  int sk = s;                              // chunk within its term
  if constexpr (!LOOP) {
    if (p.n_terms > 0) {
      const int term = s / p.term_split;
      sk = s - term * p.term_split;
      A = (const T*)p.a_term[term];
      B = (const T*)p.b_term[term];
    }
  }
  const int64_t kbeg = (int64_t)sk * p.kchunk;
  int64_t kend = kbeg + p.kchunk;
  if (kend > p.K) kend = p.K;

  Acc acc[TMB][TNB];
#pragma unroll
  for (int i = 0; i < TMB; ++i)
#pragma unroll
    for (int j = 0; j < TNB; ++j) acc[i][j] = X::zero();

  const int nterm = LOOP ? p.n_terms : 1;
  for (int term = 0; term < nterm; ++term) {
    if constexpr (LOOP) {
      A = (const T*)p.a_term[term];
      B = (const T*)p.b_term[term];
    }
    if (p.kmask) k_loop<X, WGM, WGN, TM, TN, VA, VB, NBUF, true>(p, A + bta, B + btb, koffA, koffB, m0, n0, kbeg, kend, As, Bs, acc);
    else k_loop<X, WGM, WGN, TM, TN, VA, VB, NBUF, false>(p, A + bta, B + btb, koffA, koffB, m0, n0, kbeg, kend, As, Bs, acc);
  }

  T* Cout = C + btc + (int64_t)s * p.c_split_stride;
  if constexpr (BN == 16 && BM >= 64) {
    if (p.c_rows_contig) {
      // A 16-column output that is contiguous along m, not n (a convolution
      // writing [image, channel, h, w]): the accumulators, whose lanes run
      // along n, go through LDS once and are stored with lanes along m.
      T (*Cs)[BM + 1] = As[0];
      __shared__ int64_t ccol[16];
#pragma unroll
      for (int i = 0; i < TMB; ++i)
#pragma unroll
        for (int j = 0; j < TNB; ++j)
#pragma unroll
          for (int r = 0; r < X::NR; ++r) Cs[j * X::NBW + X::col(lane)][wm * TM * 16 + i * X::BMR + X::row(lane, r)] = X::get(acc[i][j], r);
      if (t < 16) {
        int64_t n = n0 + t;
        int64_t oa = 0, ob = 0, oc = 0;
        if (n < p.N) group_off(p.n, n, &oa, &ob, &oc);
        ccol[t] = oc;
      }
      __syncthreads();
      constexpr int MG = NT / BM;                           // column groups stored per pass
      const int ml = t % BM, ng = t / BM;
      const int64_t m = m0 + ml;
      if (m < p.M) {
        int64_t oa, ob, oc;
        group_off(p.m, m, &oa, &ob, &oc);
#pragma unroll
        for (int e = 0; e < 16 / MG; ++e) {
          const int nl = ng + MG * e;
          if (n0 + nl < p.N) Cout[oc + ccol[nl]] = Cs[nl][ml];
        }
      }
      return;
    }
  }
  int64_t coln[TNB];
  bool colok[TNB];
#pragma unroll
  for (int j = 0; j < TNB; ++j) {
    int64_t n = n0 + wn * TN * 16 + j * X::NBW + X::col(lane);
    colok[j] = n < p.N;
    int64_t oa = 0, ob = 0, oc = 0;
    if (colok[j]) group_off(p.n, n, &oa, &ob, &oc);
    coln[j] = oc;
  }
#pragma unroll
  for (int i = 0; i < TMB; ++i) {
#pragma unroll
    for (int r = 0; r < X::NR; ++r) {
      int64_t m = m0 + wm * TM * 16 + i * X::BMR + X::row(lane, r);
      if (m < p.M) {
        int64_t oa, ob, oc;
        group_off(p.m, m, &oa, &ob, &oc);
#pragma unroll
        for (int j = 0; j < TNB; ++j)
          if (colok[j]) Cout[oc + coln[j]] = X::get(acc[i][j], r);
      }
    }
  }
}

// Skinny products (N <= 32): one wavefront owns a (16 TM) x (16 TN) block of the
// output over one K chunk and loads its MFMA operand fragments straight from
// global memory.  With so few columns no operand element is shared between
// wavefronts, so staging through LDS (and its barriers) would buy nothing; the
// wavefronts run independently, each with the loads of the next 16 K elements
// in flight while the MFMAs of the current 16 run.
//
// K is walked in groups of 16.  Within a group lane (r, q) -- r = lane % 16 the
// row, q = lane / 16 -- owns k = k0 + 4 q + j at MFMA step j (any assignment of
// k to steps is a valid summation order as long as A and B agree).  The four k
// of a lane are consecutive, so an operand that is contiguous along K is read
// with one 4-element vector load per row block (VA / VB); otherwise with four
// loads at offsets taken from the K table (itself read as one vector).
// The K tables are padded: entries up to K + 32 exist and repeat the last four
// valid k (see k_koff).
// grid.x * 4 wavefronts cover (split, tile_m, tile_n); grid.z is the batch.
template <typename T> struct Vec4Of { using type = T __attribute__((ext_vector_type(4), aligned(16))); };
using Off4 = int64_t __attribute__((ext_vector_type(4), aligned(16)));

template <typename X, int TM, int TN, bool VA, bool VB>
__global__ void __launch_bounds__(NT) k_gemm_direct(GemmParams p, const typename X::T* __restrict__ A, const typename X::T* __restrict__ B,
                                                    typename X::T* __restrict__ C, const int64_t* __restrict__ koffA,
                                                    const int64_t* __restrict__ koffB) {
  using T = typename X::T;
  using Acc = typename X::Acc;
  using V4 = typename Vec4Of<T>::type;
  static_assert(X::NBW == 16, "16-column MFMA blocks");
  const int lane = threadIdx.x & 63;
  const int r = lane & 15, q = lane >> 4;
  const int64_t tiles_m = (p.M + 16 * TM - 1) / (16 * TM), tiles_n = (p.N + 16 * TN - 1) / (16 * TN);
  const int64_t per_split = tiles_m * tiles_n;
  const int64_t item = (int64_t)blockIdx.x * (NT / 64) + (threadIdx.x >> 6);
  if (item >= per_split * p.split) return;
  const int64_t s = item / per_split, tile = item - s * per_split;
  const int64_t tile_m = tile / tiles_n, tile_n = tile - tile_m * tiles_n;
  const int64_t m0 = tile_m * 16 * TM, n0 = tile_n * 16 * TN;

  int64_t bta, btb, btc;
  group_off(p.bt, blockIdx.z, &bta, &btb, &btc);
  int64_t sk = s;                          // chunk within its term
  if (p.n_terms > 0) {
    const int64_t term = s / p.term_split;
    sk = s - term * p.term_split;
    A = (const T*)p.a_term[term];
    B = (const T*)p.b_term[term];
  }
  const int64_t kbeg = sk * p.kchunk;
  int64_t kend = kbeg + p.kchunk;
  if (kend > p.K) kend = p.K;

  const T* ra[TM];
  const T* rb[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    int64_t m = m0 + 16 * i + r;
    if (m >= p.M) m = p.M - 1;              // clamp: the values are never stored
    int64_t oa, ob, oc;
    group_off(p.m, m, &oa, &ob, &oc);
    ra[i] = A + bta + oa;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int64_t n = n0 + 16 * j + r;
    if (n >= p.N) n = p.N - 1;
    int64_t oa, ob, oc;
    group_off(p.n, n, &oa, &ob, &oc);
    rb[j] = B + btb + ob;
  }

  Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = X::zero();

  // offsets of this lane's four k of the next group to load (vector operands
  // need only the first), and two buffers of operand values
  Off4 oa4, ob4;
  V4 va[2][TM], vb[2][TN];
  // first k of the lane in the group at k0; past the end the group is masked and
  // any valid position will do
  const int64_t klast = ((p.K + 15) / 16) * 16;       // the tables reach klast + 16
  auto fetch_off = [&](int64_t k0) {
    const int64_t k = (k0 < klast ? k0 : klast) + 4 * q;
    const int64_t kt = k & p.kmask;
    oa4 = *reinterpret_cast<const Off4*>(koffA + kt);
    ob4 = *reinterpret_cast<const Off4*>(koffB + kt);
    // past K: the last four valid k, so that a vector load there stays inside
    const int64_t base = k < p.K ? k : (p.K >= 4 ? p.K - 4 : 0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int64_t kj = base + j < p.K ? base + j : p.K - 1;
      oa4[j] += kj * p.ksa;
      ob4[j] += kj * p.ksb;
    }
  };
  auto fetch = [&](int buf, int64_t k0) {
    const int64_t k = k0 + 4 * q;
    bool ok[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) ok[j] = k + j < kend;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      V4 x;
      if constexpr (VA) x = *reinterpret_cast<const V4*>(ra[i] + oa4[0]);
      else {
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = ra[i][oa4[j]];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) va[buf][i][j] = ok[j] ? x[j] : T(0);
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      V4 x;
      if constexpr (VB) x = *reinterpret_cast<const V4*>(rb[i] + ob4[0]);
      else {
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = rb[i][ob4[j]];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) vb[buf][i][j] = ok[j] ? x[j] : T(0);
    }
  };
  auto compute = [&](int buf) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = X::run(va[buf][i][u], vb[buf][j][u], acc[i][j]);
  };
  fetch_off(kbeg);
  fetch(0, kbeg);
  fetch_off(kbeg + 16);
  for (int64_t k0 = kbeg; k0 < kend; k0 += 32) {
    fetch(1, k0 + 16);
    fetch_off(k0 + 32);
    compute(0);
    fetch(0, k0 + 32);
    fetch_off(k0 + 48);
    compute(1);
  }

  T* Cout = C + btc + s * p.c_split_stride;
  int64_t coln[TN];
  bool colok[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int64_t n = n0 + 16 * j + X::col(lane);
    colok[j] = n < p.N;
    int64_t oa = 0, ob = 0, oc = 0;
    if (colok[j]) group_off(p.n, n, &oa, &ob, &oc);
    coln[j] = oc;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int w = 0; w < X::NR; ++w) {
      int64_t m = m0 + 16 * i + X::row(lane, w);
      if (m < p.M) {
        int64_t oa, ob, oc;
        group_off(p.m, m, &oa, &ob, &oc);
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (colok[j]) Cout[oc + coln[j]] = X::get(acc[i][j], w);
      }
    }
  }
}

struct TileCfg { int wgm, wgn, tm, tn; double eff; };
// Candidate tiles, with a rough relative efficiency (operand reuse from LDS).
constexpr TileCfg kTiles[] = {
    {2, 2, 4, 4, 1.00},  // 128 x 128
    {2, 2, 4, 2, 0.85},  // 128 x 64
    {2, 2, 2, 4, 0.85},  // 64 x 128
    {4, 1, 4, 2, 0.70},  // 256 x 32
    {1, 4, 2, 4, 0.70},  // 32 x 256
    {4, 1, 4, 1, 0.50},  // 256 x 16
    {1, 4, 1, 4, 0.50},  // 16 x 256
    {2, 2, 2, 2, 0.65},  // 64 x 64
    {2, 2, 1, 1, 0.35},  // 32 x 32
    {4, 1, 1, 1, 0.30},  // 64 x 16
    {1, 4, 1, 1, 0.30},  // 16 x 64
    {2, 2, 8, 4, 1.15},  // 256 x 128, fp32 only (the accumulators of an fp64 tile this size do not fit)
    {2, 2, 4, 8, 1.15},  // 128 x 256, fp32 only
};
constexpr int kFirstF32OnlyTile = 11;
constexpr int kNumTiles = sizeof(kTiles) / sizeof(kTiles[0]);

struct LaunchArgs {
  hipStream_t stream;
  int cfg;            // index into kTiles, or -1: the direct kernel with direct_tm x direct_tn blocks per wavefront
  int direct_tm, direct_tn;
  bool va, vb;
  dim3 grid;
  const void *A, *B;
  void* C;
  const int64_t *ka, *kb;
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;   // while the profiler is on: events that the launch carries (the kernel's own begin and end)
};

// Blocks that walk the terms of a sum themselves exist for tiles up to 64 x 64
// (small products whose tiles fill the device).
constexpr bool term_loop_tile(int wgm, int wgn, int tm, int tn) { return wgm * tm * 16 * wgn * tn * 16 <= 64 * 64; }

// The MFMA flavour a tile runs on: fp32 tiles whose wavefronts hold whole
// 32 x 32 blocks take the 32x32x2 instruction.
// One launch: plain, or carrying the profiler's events (then they hold the kernel's own begin and end).
template <typename F, typename... Args>
inline void launch_kernel(const LaunchArgs& a, F kernel, Args... args) {
  if (a.ev_start || a.ev_stop) hipExtLaunchKernelGGL(kernel, a.grid, dim3(NT), 0, a.stream, a.ev_start, a.ev_stop, 0, args...);
  else hipLaunchKernelGGL(kernel, a.grid, dim3(NT), 0, a.stream, args...);
}

template <typename X0, int TM, int TN> struct FlavourOf { using type = X0; };
template <int TM, int TN> struct FlavourOf<MfmaF32, TM, TN> {
  using type = typename std::conditional<TM % 2 == 0 && TN % 2 == 0, MfmaF32W, MfmaF32>::type;
};

template <typename X0, int WGM, int WGN, int TM, int TN>
void launch_cfg(const GemmParams& p, const LaunchArgs& a) {
  using X = typename FlavourOf<X0, TM, TN>::type;
  using T = typename X::T;
  constexpr int V = 16 / sizeof(T);
  constexpr int BM = WGM * TM * 16, BN = WGN * TN * 16;
  // two LDS buffers where they still leave room for two blocks per CU next to
  // the accumulators' registers; skinny tiles keep one buffer and more blocks
  constexpr int NBUF = (BM >= 64 && BN >= 64 && BM + BN >= 192) ? 2 : 1;
  if constexpr (term_loop_tile(WGM, WGN, TM, TN)) {
    if (p.term_loop) {
      const T* A = (const T*)a.A;
      const T* B = (const T*)a.B;
      T* C = (T*)a.C;
      constexpr bool CA = BM >= 64, CB = BN >= 64;
      const bool va = CA && a.va, vb = CB && a.vb;
      if constexpr (CA && CB) {
        if (va && vb) { launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, V, V, 1, true>), p, A, B, C, a.ka, a.kb); return; }
      }
      if constexpr (CA) {
        if (va) { launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, V, 1, 1, true>), p, A, B, C, a.ka, a.kb); return; }
      }
      if constexpr (CB) {
        if (vb) { launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, 1, V, 1, true>), p, A, B, C, a.ka, a.kb); return; }
      }
      launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, 1, 1, 1, true>), p, A, B, C, a.ka, a.kb);
      return;
    }
  }
  const T* A = (const T*)a.A;
  const T* B = (const T*)a.B;
  T* C = (T*)a.C;
  // 16-byte loads only on a side of the tile long enough to share a load's lanes sensibly
  constexpr bool CA = BM >= 64, CB = BN >= 64;
  const bool va = CA && a.va, vb = CB && a.vb;
  if constexpr (CA && CB) {
    if (va && vb) { launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, V, V, NBUF>), p, A, B, C, a.ka, a.kb); return; }
  }
  if constexpr (CA) {
    if (va) { launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, V, 1, NBUF>), p, A, B, C, a.ka, a.kb); return; }
  }
  if constexpr (CB) {
    if (vb) { launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, 1, V, NBUF>), p, A, B, C, a.ka, a.kb); return; }
  }
  launch_kernel(a, (k_gemm<X, WGM, WGN, TM, TN, 1, 1, NBUF>), p, A, B, C, a.ka, a.kb);
}

template <typename X, int TM, int TN>
void launch_direct_cfg(const GemmParams& p, const LaunchArgs& a) {
  using T = typename X::T;
  const T* A = (const T*)a.A;
  const T* B = (const T*)a.B;
  T* C = (T*)a.C;
  if (a.va && a.vb) launch_kernel(a, (k_gemm_direct<X, TM, TN, true, true>), p, A, B, C, a.ka, a.kb);
  else if (a.va) launch_kernel(a, (k_gemm_direct<X, TM, TN, true, false>), p, A, B, C, a.ka, a.kb);
  else if (a.vb) launch_kernel(a, (k_gemm_direct<X, TM, TN, false, true>), p, A, B, C, a.ka, a.kb);
  else launch_kernel(a, (k_gemm_direct<X, TM, TN, false, false>), p, A, B, C, a.ka, a.kb);
}

template <typename X>
void launch(const GemmParams& p, const LaunchArgs& a) {
  if (a.cfg < 0) {
    if (a.direct_tn == 2) {
      if (a.direct_tm == 1) launch_direct_cfg<X, 1, 2>(p, a);
      else if (a.direct_tm == 2) launch_direct_cfg<X, 2, 2>(p, a);
      else launch_direct_cfg<X, 4, 2>(p, a);
    } else {
      if (a.direct_tm == 1) launch_direct_cfg<X, 1, 1>(p, a);
      else if (a.direct_tm == 2) launch_direct_cfg<X, 2, 1>(p, a);
      else launch_direct_cfg<X, 4, 1>(p, a);
    }
    return;
  }
  switch (a.cfg) {
    case 0: launch_cfg<X, 2, 2, 4, 4>(p, a); break;
    case 1: launch_cfg<X, 2, 2, 4, 2>(p, a); break;
    case 2: launch_cfg<X, 2, 2, 2, 4>(p, a); break;
    case 3: launch_cfg<X, 4, 1, 4, 2>(p, a); break;
    case 4: launch_cfg<X, 1, 4, 2, 4>(p, a); break;
    case 5: launch_cfg<X, 4, 1, 4, 1>(p, a); break;
    case 6: launch_cfg<X, 1, 4, 1, 4>(p, a); break;
    case 7: launch_cfg<X, 2, 2, 2, 2>(p, a); break;
    case 8: launch_cfg<X, 2, 2, 1, 1>(p, a); break;
    case 9: launch_cfg<X, 4, 1, 1, 1>(p, a); break;
    case 10: launch_cfg<X, 1, 4, 1, 1>(p, a); break;
    case 11:
      if constexpr (sizeof(typename X::T) == 4) launch_cfg<X, 2, 2, 8, 4>(p, a);
      break;
    default:
      if constexpr (sizeof(typename X::T) == 4) launch_cfg<X, 2, 2, 4, 8>(p, a);
      break;
  }
}

// defined in gemm_f32.hip / gemm_f64.hip
void launch_f32(const GemmParams& p, const LaunchArgs& a);
void launch_f64(const GemmParams& p, const LaunchArgs& a);

}  // namespace gemm
}  // namespace hg
