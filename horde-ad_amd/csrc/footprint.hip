// Matrix products whose operands are windows into small footprints.
//
// A contraction C[m, n] = sum_k A[moff(m) + koff(k)] * B[noff(n) + koff'(k)]
// whose index sets split into an outer "chunk" index (an image of a batch) and
// inner indices that address only a few tens of KB of each operand per chunk:
// the convolution, its weight gradient and its input gradient written as
// products over overlapping windows.  A general GEMM kernel fetches every
// window element from the vector cache again; here a block copies the chunk's
// footprint of each operand into LDS once, contiguously, and all MFMA operands
// are LDS reads whose addresses are a per-lane register plus an immediate.
//
// Shapes, strides and the K enumeration are compiled into the kernel (hiprtc,
// cached per context by source text), so the inner loop is ds_read + v_mfma
// only.  One block of four wavefronts per CU walks chunks grid-stride; the
// next chunk's footprint is fetched while the current one is multiplied (two
// LDS buffers).  Row blocks (16 rows) are dealt to the wavefronts; blocks left
// over after an even deal are split along K between them and added up through
// LDS.  Chunk index in K (weight gradient): every block keeps its partial
// product over its chunks, summed afterwards in a fixed order.  Chunk index in
// the rows: each chunk writes its own rows of C.
#include "common.hpp"
#include "gemm_kernel.hpp"

#include <hip/hiprtc.h>

#include <array>
#include <map>
#include <sstream>
#include <string>
#include <vector>

using namespace hg;
using namespace hg::gemm;

namespace {

constexpr int kLdsBudget = 156 * 1024;   // of the CU's 160 KB
constexpr int kMaxGroups = 256;          // K groups of 4 per chunk
constexpr int kMaxMfma = 1400;           // unrolled MFMAs per wavefront and chunk
constexpr int kMaxPatterns = 6;

struct Compiled {
  hipModule_t mod;
  hipFunction_t fn;
};

std::map<std::string, Compiled>& cache_of(hgpu_ctx* ctx) {
  auto it = ctx->jit_cache.find("__footprint__");
  if (it == ctx->jit_cache.end()) it = ctx->jit_cache.emplace("__footprint__", new std::map<std::string, Compiled>()).first;
  return *static_cast<std::map<std::string, Compiled>*>(it->second);
}

int compile(hgpu_ctx* ctx, const std::string& src, const std::string& kname, Compiled* out) {
  std::vector<char> code;
  int rc = rtc_compile(ctx, src, "footprint gemm", &code);
  if (rc) return rc;
  hipError_t e = hipModuleLoadData(&out->mod, code.data());
  if (e != hipSuccess) return check_hip(ctx, e, "hipModuleLoadData");
  e = hipModuleGetFunction(&out->fn, out->mod, kname.c_str());
  if (e != hipSuccess) return check_hip(ctx, e, "hipModuleGetFunction");
  return HGPU_OK;
}

struct Dim { int64_t e, sx, sy, sc; };

// The rows operand is X, the columns operand Y (A and B, or swapped).
struct Plan {
  bool f64;
  int mode;            // 0: chunk index in K, partial products per block; 1: chunk index in the rows
  int64_t nch, chx, chy, chc;
  int min_rows, nin;   // inner rows, inner columns (<= 16)
  std::vector<int> row_x, row_c, col_y, col_c;
  std::vector<int> gx, gy, gp;                 // per K group: base offsets, pattern
  std::vector<std::array<int, 4>> px, py;      // per pattern: lane offsets
  int kvalid;                                  // valid lanes of the last group
  int64_t span_x, span_y, shift_x, shift_y;
  int vx, vy;                                  // elements per staging vector
  // Y in LDS: element e of the footprint sits at e + (e / ys) * ypad, so that
  // the 16 columns of a B fragment fall into different banks (ypad 0: a plain copy)
  int64_t ys;
  int ypad;
  int addr_regs;   // per-lane address registers of the kernel
  int nbufs;   // LDS chunk buffers: 2, or 1 when two do not fit (the prefetch then waits in registers)
  bool cvec;   // groups of four rows are adjacent in C and 16-byte aligned: vector stores
};

int64_t prod(const std::vector<Dim>& d) {
  int64_t p = 1;
  for (auto& x : d) p *= x.e;
  return p;
}

// Offsets of every flat index over dims (row-major, last dim fastest).
void enumerate(const std::vector<Dim>& d, std::vector<int64_t>* ox, std::vector<int64_t>* oy, std::vector<int64_t>* oc) {
  int64_t n = prod(d);
  ox->assign((size_t)n, 0);
  oy->assign((size_t)n, 0);
  oc->assign((size_t)n, 0);
  for (int64_t i = 0; i < n; ++i) {
    int64_t r = i, x = 0, y = 0, c = 0;
    for (int k = (int)d.size() - 1; k >= 0; --k) {
      int64_t idx = r % d[(size_t)k].e;
      r /= d[(size_t)k].e;
      x += idx * d[(size_t)k].sx;
      y += idx * d[(size_t)k].sy;
      c += idx * d[(size_t)k].sc;
    }
    (*ox)[(size_t)i] = x;
    (*oy)[(size_t)i] = y;
    (*oc)[(size_t)i] = c;
  }
}

// rows / cols / kd: the index groups seen from X and Y; chunk_in_k and ci pick
// the chunk dim.  Returns false when the shape does not suit the kernel.
bool make_plan(bool f64, std::vector<Dim> rows, std::vector<Dim> cols, std::vector<Dim> kd, bool chunk_in_k, size_t ci,
               int num_cu, Plan* pl) {
  const int es = f64 ? 8 : 4;
  pl->f64 = f64;
  pl->mode = chunk_in_k ? 0 : 1;
  Dim ch = chunk_in_k ? kd[ci] : rows[ci];
  if (chunk_in_k) kd.erase(kd.begin() + (long)ci);
  else rows.erase(rows.begin() + (long)ci);
  pl->nch = ch.e;
  pl->chx = ch.sx;
  pl->chy = ch.sy;
  pl->chc = ch.sc;
  if (pl->nch < num_cu / 2) return false;
  int64_t R = prod(rows), Cn = prod(cols), Kin = prod(kd);
  if (R < 16 || R > 64 * 16 || Cn < 4 || Cn > 16 || Kin < 8 || Kin > 4 * kMaxGroups) return false;
  // K: a dim whose extent is a multiple of 4 goes innermost, so that the four
  // lanes of a group differ by one stride
  for (size_t i = kd.size(); i-- > 0;)
    if (kd[i].e % 4 == 0) { Dim d = kd[i]; kd.erase(kd.begin() + (long)i); kd.push_back(d); break; }
  std::vector<int64_t> rx, ry, rc, cx, cy, cc, kx, ky, kc;
  enumerate(rows, &rx, &ry, &rc);
  enumerate(cols, &cx, &cy, &cc);
  enumerate(kd, &kx, &ky, &kc);
  auto minmax = [](const std::vector<int64_t>& v, int64_t* lo, int64_t* hi) {
    *lo = *hi = v[0];
    for (int64_t x : v) { if (x < *lo) *lo = x; if (x > *hi) *hi = x; }
  };
  int64_t rlo, rhi, klo, khi, clo, chi, k2lo, k2hi;
  minmax(rx, &rlo, &rhi);
  minmax(kx, &klo, &khi);
  minmax(cy, &clo, &chi);
  minmax(ky, &k2lo, &k2hi);
  pl->shift_x = rlo + klo;
  pl->shift_y = clo + k2lo;
  pl->span_x = (rhi - rlo) + (khi - klo) + 1;
  pl->span_y = (chi - clo) + (k2hi - k2lo) + 1;
  if (pl->span_x > (1 << 20) || pl->span_y > (1 << 20)) return false;
  pl->min_rows = (int)R;
  pl->nin = (int)Cn;
  for (int64_t i = 0; i < R; ++i) { pl->row_x.push_back((int)(rx[(size_t)i] - rlo)); pl->row_c.push_back((int)rc[(size_t)i]); }
  for (int64_t i = 0; i < Cn; ++i) { pl->col_y.push_back((int)(cy[(size_t)i] - clo)); pl->col_c.push_back((int)cc[(size_t)i]); }
  for (auto v : rc) if (v < 0 || v > INT32_MAX) return false;
  for (auto v : cc) if (v < 0 || v > INT32_MAX) return false;
  int64_t ng = (Kin + 3) / 4;
  pl->kvalid = (int)(Kin - 4 * (ng - 1));
  for (int64_t g = 0; g < ng; ++g) {
    std::array<int, 4> dx{}, dy{};
    int64_t k0 = 4 * g, bx = INT64_MAX, byy = INT64_MAX;
    for (int q = 0; q < 4; ++q) {
      int64_t k = k0 + q < Kin ? k0 + q : Kin - 1;
      if (kx[(size_t)k] < bx) bx = kx[(size_t)k];
      if (ky[(size_t)k] < byy) byy = ky[(size_t)k];
    }
    for (int q = 0; q < 4; ++q) {   // lane offsets from the group's smallest offset: never negative
      int64_t k = k0 + q < Kin ? k0 + q : Kin - 1;
      dx[(size_t)q] = (int)(kx[(size_t)k] - bx);
      dy[(size_t)q] = (int)(ky[(size_t)k] - byy);
    }
    size_t pi = 0;
    for (; pi < pl->px.size(); ++pi)
      if (pl->px[pi] == dx && pl->py[pi] == dy) break;
    if (pi == pl->px.size()) { pl->px.push_back(dx); pl->py.push_back(dy); }
    pl->gx.push_back((int)(bx - klo));
    pl->gy.push_back((int)(byy - k2lo));
    pl->gp.push_back((int)pi);
  }
  if ((int)pl->px.size() > kMaxPatterns) return false;
  // LDS immediates are 16 bits of bytes
  for (size_t g = 0; g < pl->gx.size(); ++g)
    if ((int64_t)pl->gx[g] * es > 65000 || (int64_t)pl->gy[g] * es > 65000) return false;
  const int MB = (int)((R + 15) / 16), NBF = MB / 4, REM = MB % 4, NG = (int)ng, NSLOT = (NG + 3) / 4;
  if (NBF * NG + REM * NSLOT > kMaxMfma) return false;
  if (NBF + REM > 20) return false;                       // accumulators
  pl->addr_regs = NBF * (int)pl->px.size() + REM * NSLOT * 2 + 8 * (NBF + REM);
  if (pl->addr_regs > 300) return false;   // address registers and accumulators
  return true;
}

std::string table(const char* qual, const char* name, const std::vector<int>& v) {
  std::ostringstream s;
  s << qual << " int " << name << "[" << (v.empty() ? 1 : v.size()) << "] = {";
  for (size_t i = 0; i < v.size(); ++i) s << (i ? "," : "") << v[i];
  if (v.empty()) s << "0";
  s << "};\n";
  return s.str();
}

const char* kBody = R"HG(
typedef long long i64;
template <int I> struct IC { static constexpr int v = I; };
#if F64
typedef double T;
typedef __attribute__((ext_vector_type(4))) double Acc;
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0)
// Register j of a lane holds row 4 j + lane / 16 of the block's A fragment.  A
// lane r of the A fragment reads matrix row ROW_OF(r) of the block, chosen so
// that the four registers of a lane are four consecutive matrix rows.
#define ROW_OF(r) (4 * ((r) & 3) + ((r) >> 2))
#else
typedef float T;
typedef __attribute__((ext_vector_type(4))) float Acc;
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0)
#define ROW_OF(r) (r)   // register j of a lane holds row 4 (lane / 16) + j already
#endif
template <int N> struct VT { typedef T type __attribute__((ext_vector_type(N))); };
template <> struct VT<1> { typedef T type; };
template <int N> using Vec = typename VT<N>::type;

constexpr int MB = (MIN + 15) / 16, NBF = MB / 4, REM = MB % 4, NSLOT = (NG + 3) / 4;
constexpr int NACC = NBF + REM > 0 ? NBF + REM : 1;
// staging: vectors per operand and loads per thread
constexpr int XV = (SPANX + VX - 1) / VX, YV = (SPANY + VY - 1) / VY;
constexpr int NLX = (XV + 255) / 256, NLY = (YV + 255) / 256;
constexpr int LX = XV * VX, LY = YV * VY + (YPAD ? (YV * VY / YS) * YPAD : 0);   // LDS elements per buffer
// where vector v of the Y footprint sits in LDS (in vectors)
__device__ __forceinline__ int ypos(int v) { return YPAD ? v + (v * VY / YS) * (YPAD / VY) : v; }
constexpr int NLD = MODE == 0 ? NLX + NLY : NLX;        // loads per thread and chunk
constexpr int PH = NG >= 12 ? 3 : 1;                    // prefetch phases
constexpr int LPP = (NLD + PH - 1) / PH;
constexpr int BUF = MODE == 0 ? LX + LY : LX;           // elements per chunk buffer
constexpr int RED0 = NBUFS * BUF + (MODE == 0 ? 0 : LY);    // scratch for adding up split row blocks
constexpr int LDS_ELEMS = RED0 + (REM > 0 ? REM * 4 * 256 : 0);

// The four registers of a lane are rows m0 .. m0 + 3 of column col.  Where
// they go inside a chunk's output comes from two tables in memory; a kernel that
// stores once per chunk looks them up before its loop over the chunks, because a
// wait for such a lookup is also a wait for every store issued before it.
struct OutPos { int o[CVEC ? 1 : 4]; };
__device__ __forceinline__ OutPos out_pos(int m0, int col) {
  OutPos p;
  const int cc = kColC[col < NIN ? col : NIN - 1];
#pragma unroll
  for (int j = 0; j < (CVEC ? 1 : 4); ++j) p.o[j] = kRowC[m0 + j < MIN ? m0 + j : MIN - 1] + cc;
  return p;
}
__device__ __forceinline__ void store_rows(T* __restrict__ out, const OutPos& p, int m0, int col, T v0, T v1, T v2, T v3) {
  if (col >= NIN) return;
  if (CVEC) {      // the four rows are adjacent in memory and 16-byte aligned
    if (m0 < MIN) {
      T* dst = out + p.o[0];
#if F64
      reinterpret_cast<Vec<2>*>(dst)[0] = Vec<2>{v0, v1};
      reinterpret_cast<Vec<2>*>(dst)[1] = Vec<2>{v2, v3};
#else
      reinterpret_cast<Vec<4>*>(dst)[0] = Vec<4>{v0, v1, v2, v3};
#endif
    }
  } else {
    if (m0 < MIN) out[p.o[0]] = v0;
    if (m0 + 1 < MIN) out[p.o[CVEC ? 0 : 1]] = v1;
    if (m0 + 2 < MIN) out[p.o[CVEC ? 0 : 2]] = v2;
    if (m0 + 3 < MIN) out[p.o[CVEC ? 0 : 3]] = v3;
  }
}

extern "C" __global__ void __launch_bounds__(256, 1)
KNAME(const T* __restrict__ X, const T* __restrict__ Y, T* __restrict__ C, i64 nch, i64 chx, i64 chy, i64 chc, i64 part_stride) {
  __shared__ T lds[LDS_ELEMS];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q4 = lane >> 4;
  // per-lane addresses: row base + lane offset of each K pattern
  int ax[NBF > 0 ? NBF : 1][NPAT];
#pragma unroll
  for (int t = 0; t < NBF; ++t) {
    int m = (wave + 4 * t) * 16 + ROW_OF(r);
    int ro = kRowX[m < MIN ? m : MIN - 1];
#pragma unroll
    for (int p = 0; p < NPAT; ++p) ax[t][p] = ro + kPatX[p * 4 + q4];
  }
  const int cn = r < NIN ? r : NIN - 1;
  int by[NPAT];
#pragma unroll
  for (int p = 0; p < NPAT; ++p) by[p] = YOFF + kColY[cn] + kPatY[p * 4 + q4];
  // split row blocks: block rb, slot s: this wavefront's K group is 4 s + (wave + rb) % 4
  int remx[REM > 0 ? REM * NSLOT : 1], remy[REM > 0 ? REM * NSLOT : 1];
#pragma unroll
  for (int rb = 0; rb < REM; ++rb) {
    int m = (4 * NBF + rb) * 16 + ROW_OF(r);
    int ro = kRowX[m < MIN ? m : MIN - 1];
#pragma clang loop unroll(full)
    for (int s = 0; s < NSLOT; ++s) {
      int gi = 4 * s + ((wave + rb) & 3);
      if (gi >= NG) gi = NG - 1;
      int p = kGrpPd[gi];
      remx[rb * NSLOT + s] = ro + kGrpXd[gi] + kPatX[p * 4 + q4];
      remy[rb * NSLOT + s] = YOFF + kColY[cn] + kGrpYd[gi] + kPatY[p * 4 + q4];
    }
  }
  // lanes past the end of K in the last group contribute zero
  const bool tail_lane = q4 >= KVALID;
  OutPos pos[MODE == 1 ? NACC : 1];
  if (MODE == 1) {
#pragma unroll
    for (int t = 0; t < NBF; ++t) pos[t] = out_pos((wave + 4 * t) * 16 + 4 * q4, r);
    if (REM > 0) pos[NBF] = out_pos((4 * NBF + (wave < REM ? wave : 0)) * 16 + 4 * q4, r);
  }
  Acc acc[NACC];
#pragma unroll
  for (int t = 0; t < NACC; ++t) acc[t] = Acc{0, 0, 0, 0};

  // j-th staging vector of this thread; the tail repeats the last vector
  auto vidx = [&](int j) -> int { int v = tid + 256 * (j < NLX ? j : j - NLX); int lim = (j < NLX ? XV : YV) - 1; return v < lim ? v : lim; };
  // The first chunk, and the columns operand of mode 1, go to LDS eight vectors
  // at a time: eight loads in flight, then eight stores.  Copied one by one,
  // every vector would wait out its own trip to memory.
  constexpr int kFill = 8;
  i64 ch = blockIdx.x;
  if (ch < nch) {
#pragma unroll
    for (int j0 = 0; j0 < NLD; j0 += kFill) {
      Vec<VX> fx[kFill];
      Vec<VY> fy[kFill];
#pragma unroll
      for (int j = j0; j < j0 + kFill && j < NLD; ++j) {
        if (j < NLX) fx[j - j0] = reinterpret_cast<const Vec<VX>*>(X + ch * chx)[vidx(j)];
        else fy[j - j0] = reinterpret_cast<const Vec<VY>*>(Y + ch * chy)[vidx(j)];
      }
#pragma unroll
      for (int j = j0; j < j0 + kFill && j < NLD; ++j) {
        if (j < NLX) reinterpret_cast<Vec<VX>*>(lds)[vidx(j)] = fx[j - j0];
        else reinterpret_cast<Vec<VY>*>(lds + LX)[ypos(vidx(j))] = fy[j - j0];
      }
    }
  }
  if (MODE == 1) {   // the columns operand does not change with the chunk
    for (int v0 = tid; v0 < YV; v0 += 256 * kFill) {
      Vec<VY> fy[kFill];
#pragma unroll
      for (int u = 0; u < kFill; ++u) {
        const int v = v0 + 256 * u;
        fy[u] = reinterpret_cast<const Vec<VY>*>(Y)[v < YV ? v : YV - 1];
      }
#pragma unroll
      for (int u = 0; u < kFill; ++u) {
        const int v = v0 + 256 * u;
        if (v < YV) reinterpret_cast<Vec<VY>*>(lds + NBUFS * BUF)[ypos(v)] = fy[u];
      }
    }
  }
  int cur = 0;
  for (; ch < nch; ch += gridDim.x) {
    __syncthreads();
    const T* L = lds + cur * BUF;
    T* Ln = lds + (NBUFS == 2 ? cur ^ 1 : 0) * BUF;
    const T* LYp = MODE == 0 ? L : lds + NBUFS * BUF - LX;   // so that YOFF = LX addresses Y in both modes
    // the next chunk's footprint on its way from memory: with two buffers a
    // phase's share goes to LDS when the phase ends, with one buffer everything
    // waits in registers until this chunk has been multiplied
    Vec<VX> prex[PH * LPP];
    Vec<VY> prey[PH * LPP];
    i64 chn = ch + gridDim.x;
    if (chn >= nch) chn = nch - 1;    // the last prefetch is not used
    if (MODE == 1) {
#pragma unroll
      for (int t = 0; t < NACC; ++t) acc[t] = Acc{0, 0, 0, 0};
    }
    auto phase = [&](auto PHI) {
      constexpr int ph = decltype(PHI)::v;
      constexpr int g0 = ph < PH ? NG * ph / PH : NG, g1 = ph < PH ? NG * (ph + 1) / PH : NG;
#pragma unroll
      for (int j = 0; j < LPP; ++j) {
        int jj = ph * LPP + j;
        if (jj < NLD) {
          if (jj < NLX) prex[jj] = reinterpret_cast<const Vec<VX>*>(X + chn * chx)[vidx(jj)];
          else prey[jj] = reinterpret_cast<const Vec<VY>*>(Y + chn * chy)[vidx(jj)];
        }
      }
      auto groups = [&](auto self, auto GI) -> void {
        constexpr int gi = decltype(GI)::v;
        if constexpr (gi < g1) {
          constexpr int p = kGrpP[gi], gx = kGrpX[gi], gy = kGrpY[gi];
          constexpr bool tail = gi == NG - 1 && KVALID < 4;
          T bv = LYp[by[p] + gy];
          if (tail && tail_lane) bv = T(0);
#pragma unroll
          for (int t = 0; t < NBF; ++t) {
            T av = L[ax[t][p] + gx];
            if (tail && tail_lane) av = T(0);
            acc[t] = MFMA(av, bv, acc[t]);
          }
          if constexpr (REM > 0 && ((gi & 3) == 3 || gi == NG - 1)) {
            constexpr int s = gi >> 2;
#pragma unroll
            for (int rb = 0; rb < REM; ++rb) {
              const int g2 = 4 * s + ((wave + rb) & 3);
              if (s < NSLOT - 1 || g2 < NG) {
                T a2 = L[remx[rb * NSLOT + s]], b2 = LYp[remy[rb * NSLOT + s]];
                if (KVALID < 4 && g2 == NG - 1 && tail_lane) { a2 = T(0); b2 = T(0); }
                acc[NBF + rb] = MFMA(a2, b2, acc[NBF + rb]);
              }
            }
          }
          self(self, IC<gi + 1>{});
        }
      };
      groups(groups, IC<g0>{});
      if (NBUFS == 2) {
#pragma unroll
        for (int j = 0; j < LPP; ++j) {
          int jj = ph * LPP + j;
          if (jj < NLD) {
            if (jj < NLX) reinterpret_cast<Vec<VX>*>(Ln)[vidx(jj)] = prex[jj];
            else reinterpret_cast<Vec<VY>*>(Ln + LX)[ypos(vidx(jj))] = prey[jj];
          }
        }
      }
    };
    phase(IC<0>{});
    if constexpr (PH > 1) phase(IC<1>{});
    if constexpr (PH > 2) phase(IC<2>{});
    if (NBUFS == 2) {
      cur ^= 1;
    } else {
      __syncthreads();    // everyone has finished reading this chunk
#pragma unroll
      for (int jj = 0; jj < NLD; ++jj) {
        if (jj < NLX) reinterpret_cast<Vec<VX>*>(Ln)[vidx(jj)] = prex[jj];
        else reinterpret_cast<Vec<VY>*>(Ln + LX)[ypos(vidx(jj))] = prey[jj];
      }
    }
    if (MODE == 1) {
      T* out = C + ch * chc;
#pragma unroll
      for (int t = 0; t < NBF; ++t) store_rows(out, pos[t], (wave + 4 * t) * 16 + 4 * q4, r, acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
      if (REM > 0) {
        T* red = lds + RED0;
#pragma unroll
        for (int rb = 0; rb < REM; ++rb)
#pragma unroll
          for (int j = 0; j < 4; ++j) red[((rb * 4 + wave) * 4 + j) * 64 + lane] = acc[NBF + rb][j];
        __syncthreads();
        if (wave < REM) {
          const int rb = wave;
          T s[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            s[j] = T(0);
#pragma unroll
            for (int w = 0; w < 4; ++w) s[j] += red[((rb * 4 + w) * 4 + j) * 64 + lane];
          }
          store_rows(out, pos[MODE == 1 ? NBF : 0], (4 * NBF + rb) * 16 + 4 * q4, r, s[0], s[1], s[2], s[3]);
        }
      }
    }
  }
  if (MODE == 0) {
    T* out = C + (i64)blockIdx.x * part_stride;
#pragma unroll
    for (int t = 0; t < NBF; ++t) store_rows(out, out_pos((wave + 4 * t) * 16 + 4 * q4, r), (wave + 4 * t) * 16 + 4 * q4, r, acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
    if (REM > 0) {
      T* red = lds + RED0;
      __syncthreads();
#pragma unroll
      for (int rb = 0; rb < REM; ++rb)
#pragma unroll
        for (int j = 0; j < 4; ++j) red[((rb * 4 + wave) * 4 + j) * 64 + lane] = acc[NBF + rb][j];
      __syncthreads();
      if (wave < REM) {
        const int rb = wave;
        T s[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          s[j] = T(0);
#pragma unroll
          for (int w = 0; w < 4; ++w) s[j] += red[((rb * 4 + w) * 4 + j) * 64 + lane];
        }
        store_rows(out, out_pos((4 * NBF + rb) * 16 + 4 * q4, r), (4 * NBF + rb) * 16 + 4 * q4, r, s[0], s[1], s[2], s[3]);
      }
    }
  }
}
)HG";

std::string generate(const Plan& pl, const std::string& kname) {
  std::ostringstream s;
  s << "#define KNAME " << kname << "\n";
  const int es = pl.f64 ? 8 : 4;
  s << "#define F64 " << (pl.f64 ? 1 : 0) << "\n";
  s << "#define MODE " << pl.mode << "\n";
  s << "#define MIN " << pl.min_rows << "\n#define NIN " << pl.nin << "\n#define NG " << pl.gx.size() << "\n";
  s << "#define NPAT " << pl.px.size() << "\n#define KVALID " << pl.kvalid << "\n";
  s << "#define SPANX " << pl.span_x << "\n#define SPANY " << pl.span_y << "\n";
  s << "#define VX " << pl.vx << "\n#define VY " << pl.vy << "\n";
  s << "#define NBUFS " << pl.nbufs << "\n";
  s << "#define CVEC " << (pl.cvec ? 1 : 0) << "\n";
  s << "#define YS " << (pl.ypad ? pl.ys : 1) << "\n#define YPAD " << pl.ypad << "\n";
  // Y sits behind X in a chunk buffer
  int64_t xv = (pl.span_x + pl.vx - 1) / pl.vx;
  s << "#define YOFF " << xv * pl.vx << "\n";
  (void)es;
  std::vector<int> patx, paty;
  for (size_t p = 0; p < pl.px.size(); ++p)
    for (int q = 0; q < 4; ++q) { patx.push_back(pl.px[p][(size_t)q]); paty.push_back(pl.py[p][(size_t)q]); }
  s << table("constexpr", "kGrpX", pl.gx) << table("constexpr", "kGrpY", pl.gy) << table("constexpr", "kGrpP", pl.gp);
  s << table("__device__ const", "kGrpXd", pl.gx) << table("__device__ const", "kGrpYd", pl.gy) << table("__device__ const", "kGrpPd", pl.gp);
  s << table("__device__ const", "kPatX", patx) << table("__device__ const", "kPatY", paty);
  s << table("__device__ const", "kRowX", pl.row_x) << table("__device__ const", "kRowC", pl.row_c);
  std::vector<int> col_y = pl.col_y;
  if (pl.ypad)
    for (auto& c : col_y) c += (int)(c / pl.ys) * pl.ypad;
  s << table("__device__ const", "kColY", col_y) << table("__device__ const", "kColC", pl.col_c);
  s << kBody;
  return s.str();
}

int lds_bytes(const Plan& pl) {
  const int es = pl.f64 ? 8 : 4;
  int64_t lx = (pl.span_x + pl.vx - 1) / pl.vx * pl.vx, ly = (pl.span_y + pl.vy - 1) / pl.vy * pl.vy;
  if (pl.ypad) ly += (ly / pl.ys) * pl.ypad;
  int64_t buf = pl.mode == 0 ? lx + ly : lx;
  int MB = (pl.min_rows + 15) / 16, REM = MB % 4;
  int64_t total = pl.nbufs * buf + (pl.mode == 0 ? 0 : ly) + (REM > 0 ? REM * 4 * 256 : 0);
  total *= es;
  return total > INT32_MAX ? INT32_MAX : (int)total;
}

}  // namespace

namespace hg {

// gemm.hip: out[i] = sum over the `parts` partial outputs of part[s * n + i], in a fixed order.
int sum_partials(hgpu_ctx* ctx, int dtype, int64_t n, int parts, const void* part, void* out);

// Runs the contraction described by p with the footprint kernel when its shape
// suits it (*handled), else leaves it to the caller's other kernels.
int try_footprint(hgpu_ctx* ctx, const GemmParams& p, int dtype, const void* pa, const void* pb, hgpu_array* out, bool* handled) {
  *handled = false;
  if (p.BT != 1 || p.n_terms > 0) return HGPU_OK;
  if (dtype != HGPU_F64 && dtype != HGPU_F32) return HGPU_OK;
  const bool f64 = dtype == HGPU_F64;
  const int es = f64 ? 8 : 4;
  // too little work to pay for a kernel of its own
  if ((double)p.M * p.N * p.K < 1.0e7) return HGPU_OK;
  auto dims = [](const Group& g, int who) {   // who: 0 rows of A / k as (x = a, y = b); 1 swapped
    std::vector<Dim> v;
    for (int i = 0; i < g.nd; ++i) v.push_back(who == 0 ? Dim{g.shape[i], g.sa[i], g.sb[i], g.sc[i]} : Dim{g.shape[i], g.sb[i], g.sa[i], g.sc[i]});
    return v;
  };
  Plan best;
  bool found = false, best_swapped = false;
  for (int swapped = 0; swapped < 2 && !found; ++swapped) {
    // columns: the side with at most 16 inner indices
    const Group& gr = swapped ? p.n : p.m;
    const Group& gc = swapped ? p.m : p.n;
    int64_t cols = swapped ? p.M : p.N;
    if (cols > 16) continue;
    std::vector<Dim> rows = dims(gr, swapped), colsd = dims(gc, swapped), kd = dims(p.k, swapped);
    // for the columns operand sx of a column dim is its own stride: dims() put
    // the strides of the rows operand in sx, of the columns operand in sy
    for (int in_k = 1; in_k >= 0 && !found; --in_k) {
      const std::vector<Dim>& cand = in_k ? kd : rows;
      for (size_t ci = 0; ci < cand.size() && !found; ++ci) {
        if (cand[ci].e < 64) continue;
        Plan pl;
        if (!make_plan(f64, rows, colsd, kd, in_k != 0, ci, ctx->num_cu, &pl)) continue;
        // staging vectors: 16 bytes when bases, chunk strides and buffers allow
        const char* xp = (const char*)(swapped ? pb : pa) + pl.shift_x * es;
        const char* yp = (const char*)(swapped ? pa : pb) + pl.shift_y * es;
        const int V = 16 / es;
        pl.vx = (((uintptr_t)xp & 15) == 0 && (pl.chx * es) % 16 == 0) ? V : 1;
        pl.vy = (((uintptr_t)yp & 15) == 0 && (pl.chy * es) % 16 == 0) ? V : 1;
        // columns a constant stride apart, each with its K offsets inside the
        // stride: pad the stride in LDS until 16 columns hit 16 different banks
        pl.ys = 1;
        pl.ypad = 0;
        if (pl.col_y.size() >= 2 && pl.col_y[1] > 0) {
          const int64_t S = pl.col_y[1];
          bool regular = S % pl.vy == 0 && pl.span_y <= S * (int64_t)pl.col_y.size();
          for (size_t c = 0; c < pl.col_y.size() && regular; ++c) regular = pl.col_y[c] == (int64_t)c * S;
          int64_t inner = pl.span_y - S * ((int64_t)pl.col_y.size() - 1);
          if (regular && inner <= S) {
            const int dw = es / 4;
            // a column stride of 4 (or 2) dwords modulo 8 (4) walks 16 lanes over all 64 banks
            for (int pad = 0; pad <= 16; pad += pl.vy) {
              int64_t sdw = (S + pad) * dw;
              if (sdw % 8 == 4 || sdw % 4 == 2) { pl.ys = S; pl.ypad = pad; break; }
            }
          }
        }
        {
          const int V16 = 16 / es;
          const char* cp = (const char*)data_ptr(out);
          bool ok = pl.min_rows % 4 == 0 && ((uintptr_t)cp & 15) == 0 && pl.chc % V16 == 0;
          for (size_t m = 0; m < pl.row_c.size() && ok; m += 4)
            ok = pl.row_c[m] % V16 == 0 && pl.row_c[m + 1] == pl.row_c[m] + 1 && pl.row_c[m + 2] == pl.row_c[m] + 2 && pl.row_c[m + 3] == pl.row_c[m] + 3;
          for (size_t c = 0; c < pl.col_c.size() && ok; ++c) ok = pl.col_c[c] % V16 == 0;
          if (pl.mode == 0) ok = ok && nelem(out) % V16 == 0;   // partial outputs lie nelem(out) apart
          pl.cvec = ok;
        }
        // scalar staging of a large footprint would need too many loads in flight
        int64_t loads = (pl.span_x / pl.vx + 255) / 256 + (pl.mode == 0 ? (pl.span_y / pl.vy + 255) / 256 : 0);
        if (loads > 48) continue;
        pl.nbufs = 2;
        if (lds_bytes(pl) > kLdsBudget) {
          pl.nbufs = 1;
          if (lds_bytes(pl) > kLdsBudget || loads * 4 + pl.addr_regs > 330) continue;   // the prefetch must fit the register file
        }
        best = pl;
        best_swapped = swapped != 0;
        found = true;
      }
    }
  }
  if (!found) return HGPU_OK;
  const Plan& pl = best;
  // the kernel's name tells a profiler which product it is
  char kname[128];
  snprintf(kname, sizeof kname, "footprint_gemm_%s_m%lld_n%lld_k%lld_%s%s", f64 ? "f64" : "f32", (long long)p.M, (long long)p.N, (long long)p.K,
           pl.mode == 0 ? "chunkK" : "chunkM", best_swapped ? "_swapped" : "");
  std::string src = generate(pl, kname);
  auto& cache = cache_of(ctx);
  auto it = cache.find(src);
  if (it == cache.end()) {
    Compiled c{nullptr, nullptr};
    // a shape the compiler rejects is remembered and left to the other kernels
    if (compile(ctx, src, kname, &c) != HGPU_OK) c = Compiled{nullptr, nullptr};
    it = cache.emplace(src, c).first;
  }
  if (!it->second.fn) return HGPU_OK;
  const char* xp = (const char*)(best_swapped ? pb : pa) + pl.shift_x * es;
  const char* yp = (const char*)(best_swapped ? pa : pb) + pl.shift_y * es;
  int64_t out_n = nelem(out);
  int64_t grid = pl.nch < ctx->num_cu ? pl.nch : ctx->num_cu;
  hgpu_buffer* part = nullptr;
  void* cdst = data_ptr(out);
  int64_t part_stride = 0;
  if (pl.mode == 0) {
    int rc = buffer_alloc(ctx, (size_t)out_n * (size_t)grid * es, &part);
    if (rc) return rc;
    cdst = part->ptr;
    part_stride = out_n;
  }
  int64_t nch = pl.nch, chx = pl.chx, chy = pl.chy, chc = pl.chc;
  void* args[] = {(void*)&xp, (void*)&yp, (void*)&cdst, (void*)&nch, (void*)&chx, (void*)&chy, (void*)&chc, (void*)&part_stride};
  {
    double flops = 2.0 * p.M * p.N * p.K;
    double bytes = ((double)p.M * p.K + (double)p.N * p.K + (double)p.M * p.N) * es;
    const char* label = f64 ? "gemm_f64" : "gemm_f32";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[160];
      snprintf(buf, sizeof buf, "%s[M%lldxN%lldxK%lldxB1,footprint,%s%s,chunks%lld,rows%d,kgroups%d,lds%dK]", label, (long long)p.M, (long long)p.N,
               (long long)p.K, pl.mode == 0 ? "chunkK" : "chunkM", best_swapped ? ",swapped" : "", (long long)pl.nch, pl.min_rows, (int)pl.gx.size(), lds_bytes(pl) / 1024);
      label = ctx->label_pool.insert(buf).first->c_str();
    }
    {
      LaunchGuard lg(ctx, label, bytes, flops);
      hipError_t e = hipModuleLaunchKernel(it->second.fn, (unsigned)grid, 1, 1, 256, 1, 1, 0, ctx->stream, args, nullptr);
      if (e != hipSuccess) { if (part) buffer_release(part); return check_hip(ctx, e, "footprint gemm launch"); }
    }
    if (pl.mode == 0) {
      int rc = sum_partials(ctx, dtype, out_n, (int)grid, (const void*)part->ptr, data_ptr(out));
      buffer_release(part);
      if (rc) return rc;
    }
  }
  *handled = true;
  return HGPU_OK;
}

}  // namespace hg
