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

#include "common.hpp"

using namespace hg;

namespace {

constexpr int BK = 16, NT = 256;
constexpr int GD = 5;  // dims per index group after merging

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

__global__ void k_koff(Group k, int64_t K, int64_t* __restrict__ ka, int64_t* __restrict__ kb) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < K) {
    int64_t a, b, c;
    group_off(k, i, &a, &b, &c);
    ka[i] = a;
    kb[i] = b;
  }
}

template <typename T> struct Mfma;
template <> struct Mfma<double> {
  using V4 = __attribute__((ext_vector_type(4))) double;
  static __device__ __forceinline__ V4 run(double a, double b, V4 c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  // accumulator register r of a lane holds D[4 r + lane / 16][lane % 16]
  static __device__ __forceinline__ int row(int lane, int r) { return 4 * r + (lane >> 4); }
};
template <> struct Mfma<float> {
  using V4 = __attribute__((ext_vector_type(4))) float;
  static __device__ __forceinline__ V4 run(float a, float b, V4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  // accumulator register r of a lane holds D[4 (lane / 16) + r][lane % 16]
  static __device__ __forceinline__ int row(int lane, int r) { return 4 * (lane >> 4) + r; }
};

template <typename T, int V> struct VecOf;
template <> struct VecOf<double, 1> { using type = double; };
template <> struct VecOf<float, 1> { using type = float; };
template <> struct VecOf<double, 2> { using type = __attribute__((ext_vector_type(2))) double; };
template <> struct VecOf<float, 4> { using type = __attribute__((ext_vector_type(4))) float; };

// Block tile BM x BN = (WGM * TM * 16) x (WGN * TN * 16): the 4 wavefronts form a
// WGM x WGN grid and each owns TM x TN MFMA tiles.  p.a_kc / p.b_kc: the lanes
// that stage an operand tile run along k (the operand's innermost K dim is the
// contiguous one) or along m / n.  VA / VB: elements per global load (16-byte
// vectors when the host has checked contiguity and alignment, else 1).
template <typename T, int WGM, int WGN, int TM, int TN, int VA, int VB>
__global__ void __launch_bounds__(NT) k_gemm(GemmParams p, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                             const int64_t* __restrict__ koffA, const int64_t* __restrict__ koffB) {
  using V4 = typename Mfma<T>::V4;
  using VecA = typename VecOf<T, VA>::type;
  using VecB = typename VecOf<T, VB>::type;
  constexpr int BM = WGM * TM * 16, BN = WGN * TN * 16;
  constexpr int NA = BM * BK / NT / VA, NB = BN * BK / NT / VB;   // loads each thread issues per K-step
  static_assert(WGM * WGN == 4 && NA >= 1 && NB >= 1, "tile shape");
  __shared__ T As[BK][BM + 1];
  __shared__ T Bs[BK][BN + 1];

  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  // XCD-aware tile numbering: blocks b, b+8, b+16, ... share an XCD; give each
  // XCD a contiguous range of tiles.
  const int64_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  const int64_t ntiles = tiles_m * tiles_n;
  int64_t bid = blockIdx.x;
  if (ntiles >= 64 && (ntiles & 7) == 0) bid = (bid & 7) * (ntiles >> 3) + (bid >> 3);
  const int64_t tile_m = bid / tiles_n, tile_n = bid - tile_m * tiles_n;
  const int64_t m0 = tile_m * BM, n0 = tile_n * BN;

  int64_t bta, btb, btc;
  group_off(p.bt, blockIdx.z, &bta, &btb, &btc);
  const int s = blockIdx.y;
  const int64_t kbeg = (int64_t)s * p.kchunk;
  int64_t kend = kbeg + p.kchunk;
  if (kend > p.K) kend = p.K;

  // this thread's (row, k) slots of each operand tile; a slot covers VA (VB)
  // consecutive elements along the direction the lanes run
  int aml[NA], akl[NA], bnl[NB], bkl[NB];
  int64_t aoff[NA], boff[NB];
  bool aok[NA], bok[NB];
  const int adk = p.a_kc ? 1 : 0, adm = 1 - adk, bdk = p.b_kc ? 1 : 0, bdn = 1 - bdk;
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    if (p.a_kc) { constexpr int KL = BK / VA; aml[i] = t / KL + (NT / KL) * i; akl[i] = (t % KL) * VA; }
    else { constexpr int ML = BM / VA; aml[i] = (t % ML) * VA; akl[i] = t / ML + (NT / ML) * i; }
    int64_t m = m0 + aml[i];
    aok[i] = m < p.M;
    if (p.a_kc || i == 0) {
      int64_t oa = 0, ob = 0, oc = 0;
      if (aok[i]) group_off(p.m, m, &oa, &ob, &oc);
      aoff[i] = oa + bta;
    } else {
      aoff[i] = aoff[0];
    }
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    if (p.b_kc) { constexpr int KL = BK / VB; bnl[i] = t / KL + (NT / KL) * i; bkl[i] = (t % KL) * VB; }
    else { constexpr int NL = BN / VB; bnl[i] = (t % NL) * VB; bkl[i] = t / NL + (NT / NL) * i; }
    int64_t n = n0 + bnl[i];
    bok[i] = n < p.N;
    if (p.b_kc || i == 0) {
      int64_t oa = 0, ob = 0, oc = 0;
      if (bok[i]) group_off(p.n, n, &oa, &ob, &oc);
      boff[i] = ob + btb;
    } else {
      boff[i] = boff[0];
    }
  }

  V4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = V4{0, 0, 0, 0};

  VecA ra[NA];
  VecB rb[NB];
  auto load_tile = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      int64_t ka = k0 + akl[i];
      if (aok[i] && ka < kend) ra[i] = *reinterpret_cast<const VecA*>(A + aoff[i] + koffA[ka]);
      else ra[i] = VecA{};
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int64_t kb = k0 + bkl[i];
      if (bok[i] && kb < kend) rb[i] = *reinterpret_cast<const VecB*>(B + boff[i] + koffB[kb]);
      else rb[i] = VecB{};
    }
  };

  if (kbeg < kend) load_tile(kbeg);
  for (int64_t k0 = kbeg; k0 < kend; k0 += BK) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      if constexpr (VA == 1) As[akl[i]][aml[i]] = ra[i];
      else {
#pragma unroll
        for (int j = 0; j < VA; ++j) As[akl[i] + j * adk][aml[i] + j * adm] = ra[i][j];
      }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      if constexpr (VB == 1) Bs[bkl[i]][bnl[i]] = rb[i];
      else {
#pragma unroll
        for (int j = 0; j < VB; ++j) Bs[bkl[i] + j * bdk][bnl[i] + j * bdn] = rb[i][j];
      }
    }
    __syncthreads();
    if (k0 + BK < kend) load_tile(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 4) {
      const int kr = kk + (lane >> 4);
      T fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = As[kr][(wm * TM + i) * 16 + (lane & 15)];
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = Bs[kr][(wn * TN + j) * 16 + (lane & 15)];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<T>::run(fa[i], fb[j], acc[i][j]);
    }
    __syncthreads();
  }

  // each lane holds 4 rows of one column of every 16x16 tile (Mfma<T>::row)
  T* Cout = C + btc + (int64_t)s * p.c_split_stride;
  int64_t coln[TN];
  bool colok[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int64_t n = n0 + (wn * TN + j) * 16 + (lane & 15);
    colok[j] = n < p.N;
    int64_t oa = 0, ob = 0, oc = 0;
    if (colok[j]) group_off(p.n, n, &oa, &ob, &oc);
    coln[j] = oc;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      int64_t m = m0 + (wm * TM + i) * 16 + Mfma<T>::row(lane, r);
      if (m < p.M) {
        int64_t oa, ob, oc;
        group_off(p.m, m, &oa, &ob, &oc);
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (colok[j]) Cout[oc + coln[j]] = acc[i][j][r];
      }
    }
  }
}

// Sums the split-K partials: out[i] = sum_s part[s * stride + i].  A block owns
// 32 consecutive outputs; its 8 groups of 32 lanes each take every 8th partial
// (coalesced rows of 32 elements) and combine through LDS in a fixed order.
template <typename T>
__global__ void __launch_bounds__(256) k_sum_partials(int64_t n, int S, int64_t stride, const T* __restrict__ part, T* __restrict__ out) {
  __shared__ T red[8][33];
  const int ol = threadIdx.x & 31, g = threadIdx.x >> 5;
  for (int64_t base = (int64_t)blockIdx.x * 32; base < n; base += (int64_t)gridDim.x * 32) {
    int64_t i = base + ol;
    T acc = T(0);
    if (i < n)
      for (int s = g; s < S; s += 8) acc += part[(int64_t)s * stride + i];
    red[g][ol] = acc;
    __syncthreads();
    if (g == 0 && i < n) {
      T t = red[0][ol];
#pragma unroll
      for (int k = 1; k < 8; ++k) t += red[k][ol];
      out[i] = t;
    }
    __syncthreads();
  }
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

struct TileCfg { int wgm, wgn, tm, tn; double eff; };
// Candidate tiles, with a rough relative efficiency (operand reuse from LDS).
const TileCfg kTiles[] = {
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
};
constexpr int kNumTiles = sizeof(kTiles) / sizeof(kTiles[0]);

template <typename T, int WGM, int WGN, int TM, int TN>
void launch_cfg(hgpu_ctx* ctx, const GemmParams& p, bool va, bool vb, dim3 grid, const T* A, const T* B, T* C, const int64_t* ka, const int64_t* kb) {
  constexpr int V = 16 / sizeof(T);
  constexpr int BM = WGM * TM * 16, BN = WGN * TN * 16;
  // 16-byte loads only for tiles whose rows are long enough to share a load's lanes sensibly
  if constexpr (BM >= 64 && BN >= 64) {
    if (va && vb) { hipLaunchKernelGGL((k_gemm<T, WGM, WGN, TM, TN, V, V>), grid, dim3(NT), 0, ctx->stream, p, A, B, C, ka, kb); return; }
    if (va) { hipLaunchKernelGGL((k_gemm<T, WGM, WGN, TM, TN, V, 1>), grid, dim3(NT), 0, ctx->stream, p, A, B, C, ka, kb); return; }
    if (vb) { hipLaunchKernelGGL((k_gemm<T, WGM, WGN, TM, TN, 1, V>), grid, dim3(NT), 0, ctx->stream, p, A, B, C, ka, kb); return; }
  }
  hipLaunchKernelGGL((k_gemm<T, WGM, WGN, TM, TN, 1, 1>), grid, dim3(NT), 0, ctx->stream, p, A, B, C, ka, kb);
}

template <typename T>
void launch(hgpu_ctx* ctx, int cfg, const GemmParams& p, bool va, bool vb, dim3 grid, const T* A, const T* B, T* C, const int64_t* ka, const int64_t* kb) {
  switch (cfg) {
    case 0: launch_cfg<T, 2, 2, 4, 4>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 1: launch_cfg<T, 2, 2, 4, 2>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 2: launch_cfg<T, 2, 2, 2, 4>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 3: launch_cfg<T, 4, 1, 4, 2>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 4: launch_cfg<T, 1, 4, 2, 4>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 5: launch_cfg<T, 4, 1, 4, 1>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 6: launch_cfg<T, 1, 4, 1, 4>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 7: launch_cfg<T, 2, 2, 2, 2>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 8: launch_cfg<T, 2, 2, 1, 1>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    case 9: launch_cfg<T, 4, 1, 1, 1>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
    default: launch_cfg<T, 1, 4, 1, 1>(ctx, p, va, vb, grid, A, B, C, ka, kb); break;
  }
}

// True when 16-byte loads along the direction the staging lanes run are safe
// for one operand: unit stride and an extent that is a multiple of the vector
// there, every other stride and the base address a multiple of the vector.
bool vector_ok(const void* base, size_t es, const Group& run, int run_dim, const int64_t* run_st,
               const Group* others[3], const int64_t* const other_st[3]) {
  const int64_t v = (int64_t)(16 / es);
  if (((uintptr_t)base & 15) != 0) return false;
  if (run_st[run_dim] != 1 || run.shape[run_dim] % v != 0) return false;
  for (int i = 0; i < run.nd; ++i)
    if (i != run_dim && run_st[i] % v != 0) return false;
  for (int g = 0; g < 3; ++g)
    for (int i = 0; i < others[g]->nd; ++i)
      if (other_st[g][i] % v != 0) return false;
  return true;
}

}  // namespace

namespace hg {

int try_gemm(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array* out, bool* handled) {
  *handled = false;
  if (!b) return HGPU_OK;
  if (a->dtype != HGPU_F64 && a->dtype != HGPU_F32) return HGPU_OK;
  GemmParams p;
  p.m.nd = p.n.nd = p.k.nd = p.bt.nd = 0;
  // Classify the dims.  The dims of a group are an index SET: any order works
  // as long as A, B and C agree, so each group is sorted with the dim that is
  // most contiguous in memory last (innermost) -- that is the dim the lanes of
  // a load run along -- and only then merged.
  struct DimRec { int64_t e, sa, sb, sc; };
  std::vector<DimRec> gm, gn, gk, gb;
  for (int i = 0; i < n_keep; ++i) {
    int64_t e = a->shape[i], sa = a->strides[i], sb = b->strides[i], sc = out->strides[i];
    if (e == 1) continue;
    if (sa != 0 && sb == 0) gm.push_back({e, sa, 0, sc});
    else if (sa == 0 && sb != 0) gn.push_back({e, 0, sb, sc});
    else if (sa != 0 && sb != 0) gb.push_back({e, sa, sb, sc});
    else return HGPU_OK;  // an output dim neither operand depends on
  }
  for (int i = n_keep; i < a->rank; ++i) {
    int64_t e = a->shape[i], sa = a->strides[i], sb = b->strides[i];
    if (e == 1) continue;
    if (sa == 0 || sb == 0) return HGPU_OK;  // a plain sum hidden in the contraction
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
  for (auto& d : gm) if (!push_dim(p.m, d.e, d.sa, d.sb, d.sc)) return HGPU_OK;
  for (auto& d : gn) if (!push_dim(p.n, d.e, d.sa, d.sb, d.sc)) return HGPU_OK;
  for (auto& d : gk) if (!push_dim(p.k, d.e, d.sa, d.sb, d.sc)) return HGPU_OK;
  for (auto& d : gb) if (!push_dim(p.bt, d.e, d.sa, d.sb, d.sc)) return HGPU_OK;
  finish(p.m);
  finish(p.n);
  finish(p.k);
  finish(p.bt);
  p.M = total(p.m);
  p.N = total(p.n);
  p.K = total(p.k);
  p.BT = total(p.bt);
  // Worth the matrix cores only when there is reuse on both sides.
  if (p.K < 4 || p.M * p.N < 256) return HGPU_OK;
  if (p.BT > 65535) return HGPU_OK;
  if ((double)p.M * p.N * p.K * p.BT < 2.0e6) return HGPU_OK;

  // tile shape: least padded work per unit of efficiency
  int cfg = 0;
  double best = 1e300;
  for (int c = 0; c < kNumTiles; ++c) {
    int64_t bm = kTiles[c].wgm * kTiles[c].tm * 16, bn = kTiles[c].wgn * kTiles[c].tn * 16;
    double padded = (double)((p.M + bm - 1) / bm * bm) * (double)((p.N + bn - 1) / bn * bn);
    double cost = padded / kTiles[c].eff;
    // a tile shape that cannot occupy the device even with K split pays for the idle CUs
    double blocks = (double)((p.M + bm - 1) / bm) * (double)((p.N + bn - 1) / bn) * (double)p.BT;
    double can_split = (double)(p.K / (4 * BK));
    double cap0 = (double)(p.M + p.N) * p.K / (2.0 * p.M * p.N);
    if (can_split > cap0) can_split = cap0;
    if (can_split > 512) can_split = 512;
    if (can_split < 1) can_split = 1;
    if (blocks * can_split < ctx->num_cu) cost *= ctx->num_cu / (blocks * can_split);
    if (cost < best * 0.999) { best = cost; cfg = c; }
  }
  const int64_t BM = kTiles[cfg].wgm * kTiles[cfg].tm * 16, BN = kTiles[cfg].wgn * kTiles[cfg].tn * 16;
  int64_t tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  if (tiles > 0x7fffffff) return HGPU_OK;
  // split K when the tiles alone cannot fill the device
  int split = 1;
  int64_t want = (int64_t)ctx->num_cu * 2;
  int64_t out_elems = p.M * p.N * p.BT;
  if (tiles * p.BT < want && p.K >= 8 * BK) {
    split = (int)((want + tiles * p.BT - 1) / (tiles * p.BT));
    int64_t max_split = p.K / (4 * BK);
    if (split > max_split) split = (int)max_split;
    // the partial products must stay small next to the operands
    int64_t cap = out_elems > 0 ? (int64_t)((double)(p.M + p.N) * p.K * p.BT / (2.0 * out_elems)) : 1;
    if (cap > 512) cap = 512;
    if (cap < 1) cap = 1;
    if (split > cap) split = (int)cap;
    if (split < 1) split = 1;
  }
  p.split = split;
  p.kchunk = ((p.K + split - 1) / split + BK - 1) / BK * BK;
  p.split = (int)((p.K + p.kchunk - 1) / p.kchunk);
  split = p.split;

  size_t es = dtype_size(a->dtype);
  int64_t out_n = nelem(out);
  hgpu_buffer* koff = nullptr;
  int rc = buffer_alloc(ctx, (size_t)p.K * 16, &koff);
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
  bool va, vb;
  {
    const Group* oa[3] = {akc ? &p.m : &p.k, &p.bt, &p.bt};
    const int64_t* const osa[3] = {akc ? p.m.sa : p.k.sa, p.bt.sa, p.bt.sa};
    va = vector_ok(data_ptr(a), dtype_size(a->dtype), akc ? p.k : p.m, (akc ? p.k.nd : p.m.nd) - 1, akc ? p.k.sa : p.m.sa, oa, osa);
    const Group* ob[3] = {bkc ? &p.n : &p.k, &p.bt, &p.bt};
    const int64_t* const osb[3] = {bkc ? p.n.sb : p.k.sb, p.bt.sb, p.bt.sb};
    vb = vector_ok(data_ptr(b), dtype_size(b->dtype), bkc ? p.k : p.n, (bkc ? p.k.nd : p.n.nd) - 1, bkc ? p.k.sb : p.n.sb, ob, osb);
  }
  dim3 grid((unsigned)tiles, (unsigned)split, (unsigned)p.BT);
  {
    double flops = 2.0 * p.M * p.N * p.K * p.BT;
    double bytes = ((double)p.M * p.K + (double)p.N * p.K + (double)p.M * p.N) * p.BT * es;
    const char* label = a->dtype == HGPU_F64 ? "gemm_f64" : "gemm_f32";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[128];
      snprintf(buf, sizeof buf, "%s[M%lldxN%lldxK%lldxB%lld,s%d,%s%s,t%lldx%lld]", label, (long long)p.M, (long long)p.N, (long long)p.K, (long long)p.BT, split, akc ? (va ? "K" : "k") : (va ? "M" : "m"), bkc ? (vb ? "K" : "k") : (vb ? "N" : "n"), (long long)BM, (long long)BN);
      label = ctx->label_pool.insert(buf).first->c_str();
    }
    LaunchGuard lg(ctx, label, bytes, flops);
    hipLaunchKernelGGL(k_koff, dim3((unsigned)((p.K + 255) / 256)), dim3(256), 0, ctx->stream, p.k, p.K, ka, kb);
    if (a->dtype == HGPU_F64) {
      double* cdst = split > 1 ? (double*)part->ptr : (double*)data_ptr(out);
      launch<double>(ctx, cfg, p, va, vb, grid, (const double*)data_ptr(a), (const double*)data_ptr(b), cdst, ka, kb);
      if (split > 1)
        hipLaunchKernelGGL(k_sum_partials<double>, dim3(grid_for(out_n, 32, ctx->num_cu * 8)), dim3(256), 0, ctx->stream, out_n, split, out_n, (const double*)part->ptr, (double*)data_ptr(out));
    } else {
      float* cdst = split > 1 ? (float*)part->ptr : (float*)data_ptr(out);
      launch<float>(ctx, cfg, p, va, vb, grid, (const float*)data_ptr(a), (const float*)data_ptr(b), cdst, ka, kb);
      if (split > 1)
        hipLaunchKernelGGL(k_sum_partials<float>, dim3(grid_for(out_n, 32, ctx->num_cu * 8)), dim3(256), 0, ctx->stream, out_n, split, out_n, (const float*)part->ptr, (float*)data_ptr(out));
    }
  }
  hipError_t e = hipGetLastError();
  buffer_release(koff);
  if (part) buffer_release(part);
  if (e != hipSuccess) return check_hip(ctx, e, "gemm");
  *handled = true;
  return HGPU_OK;
}

}  // namespace hg
