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
#include "fused_gen.hpp"
#include "gemm_kernel.hpp"

#include <hip/hiprtc.h>

#include <array>
#include <map>
#include <string>
#include <unordered_map>
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
  // callers leave a shape the compiler rejects to the other kernels: say so when asked
  if (rc && getenv("HORDEAD_GPU_DEBUG")) fprintf(stderr, "hordead_gpu: %s rejected: %s\n", kname.c_str(), hgpu_last_error(ctx));
  if (rc) return rc;
  hipError_t e = hipModuleLoadData(&out->mod, code.data());
  if (e != hipSuccess) return check_hip(ctx, e, "hipModuleLoadData");
  e = hipModuleGetFunction(&out->fn, out->mod, kname.c_str());
  if (e != hipSuccess) return check_hip(ctx, e, "hipModuleGetFunction");
  return HGPU_OK;
}

// A kernel found again by what its text depends on; the text is written (and
// looked up, and compiled) the first time only.  source() writes it.
struct KnownKernel { Compiled c; std::string text; };
template <typename F>
int known_kernel(hgpu_ctx* ctx, const hg::fusedgen::Key& key, const std::string& kname, F&& source, Compiled* out) {
  auto kit = ctx->jit_cache.find("__footprint_known__");
  if (kit == ctx->jit_cache.end()) kit = ctx->jit_cache.emplace("__footprint_known__", new std::unordered_map<std::string, KnownKernel>()).first;
  auto& known = *static_cast<std::unordered_map<std::string, KnownKernel>*>(kit->second);
  auto it = known.find(key.bytes);
  if (it != known.end() && !hg::fusedgen::check_keys()) { *out = it->second.c; return HGPU_OK; }
  std::string src = source();
  if (it != known.end()) {
    if (it->second.text != src) return fail(ctx, HGPU_ERR_DEVICE, "%s: two different kernels under one key", kname.c_str());
    *out = it->second.c;
    return HGPU_OK;
  }
  auto& cache = cache_of(ctx);
  auto ct = cache.find(src);
  if (ct == cache.end()) {
    Compiled c{nullptr, nullptr};
    // a shape the compiler rejects is remembered and left to the other kernels
    if (compile(ctx, src, kname, &c) != HGPU_OK) c = Compiled{nullptr, nullptr};
    ct = cache.emplace(src, c).first;
  }
  *out = ct->second;
  known.emplace(key.bytes, KnownKernel{ct->second, hg::fusedgen::check_keys() ? src : std::string()});
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
  int ks = 1;  // wavefronts per SIMD: the block's 4 ks wavefronts split the K groups of a chunk ks ways
  int64_t colsum_at = -1;   // >= 0: the kernel also sums the columns operand over K, into these elements of its partial result (mode 0)
  int bpc = 1; // blocks that share a CU (their LDS fits together): one's loads and stores run under the other's multiplications
  bool cvec;   // groups of four rows are adjacent in C and 16-byte aligned: vector stores
};

// (a field added to Plan changes its size: it belongs in put_plan too)
static_assert(sizeof(Plan) == 352, "put_plan must cover every field of Plan");
void put_plan(hg::fusedgen::Key& k, const Plan& pl) {
  k.put(pl.f64).put(pl.mode).put(pl.nch).put(pl.chx).put(pl.chy).put(pl.chc).put(pl.min_rows).put(pl.nin);
  k.put(pl.row_x).put(pl.row_c).put(pl.col_y).put(pl.col_c).put(pl.gx).put(pl.gy).put(pl.gp);
  k.put(pl.px.size());
  for (size_t p = 0; p < pl.px.size(); ++p)
    for (int q = 0; q < 4; ++q) k.put(pl.px[p][(size_t)q]).put(pl.py[p][(size_t)q]);
  k.put(pl.kvalid).put(pl.span_x).put(pl.span_y).put(pl.shift_x).put(pl.shift_y).put(pl.vx).put(pl.vy).put(pl.ys).put(pl.ypad);
  k.put(pl.addr_regs).put(pl.nbufs).put(pl.ks).put(pl.colsum_at).put(pl.bpc).put(pl.cvec);
}

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
  hg::fusedgen::Src s;
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

// KS wavefronts per SIMD: the block has 4 KS wavefronts, wavefront 4 h + w takes the row blocks of w
// and the h-th part of the K groups (half h); the parts' products are added through LDS.
constexpr int NT = 256 * KS;
constexpr int MB = (MIN + 15) / 16, NBF = MB / 4, REM = MB % 4, NSLOT = (NG + 3) / 4;
constexpr int NACC = NBF + REM > 0 ? NBF + REM : 1;
// staging: vectors per operand and loads per thread
constexpr int XV = (SPANX + VX - 1) / VX, YV = (SPANY + VY - 1) / VY;
constexpr int NLX = (XV + NT - 1) / NT, NLY = (YV + NT - 1) / NT;
constexpr int LX = XV * VX, LY = YV * VY + (YPAD ? (YV * VY / YS) * YPAD : 0);   // LDS elements per buffer
// where vector v of the Y footprint sits in LDS (in vectors)
__device__ __forceinline__ int ypos(int v) { return YPAD ? v + (v * VY / YS) * (YPAD / VY) : v; }
constexpr int NLD = MODE == 0 ? NLX + NLY : NLX;        // loads per thread and chunk
constexpr int PH = (NG + KS - 1) / KS >= 12 ? 3 : 1;    // prefetch phases
constexpr int LPP = (NLD + PH - 1) / PH;
constexpr int BUF = MODE == 0 ? LX + LY : LX;           // elements per chunk buffer
// split row blocks: slots whose turn comes before K group g (slot s runs after group min(4 s + 3, NG - 1))
constexpr int rem_slots_before(int g) {
  int c = 0;
  for (int sl = 0; sl < NSLOT; ++sl) c += (sl == NSLOT - 1 ? NG - 1 : 4 * sl + 3) < g ? 1 : 0;
  return c;
}
constexpr int RGB = REM > 0 ? (4 / REM > 1 ? 4 / REM : 1) : 1;     // slots per batch of LDS reads
struct RemOps { T a[RGB][REM > 0 ? REM : 1], b[RGB][REM > 0 ? REM : 1]; };
constexpr int RED0 = NBUFS * BUF + (MODE == 0 ? 0 : LY);    // scratch for adding up split row blocks
constexpr int CS0 = RED0 + (REM > 0 && KS == 1 ? REM * 4 * 256 : 0);   // where the parts' column sums meet
constexpr int LDS_ELEMS = CS0 + (COLSUM && KS > 1 ? 16 * KS : 0);
// where the parts' partial products meet (KS > 1): a chunk buffer that has been multiplied; the whole
// row blocks first, the split ones behind them
constexpr int XCH = 4 * NBF * (KS - 1) * 256;
static_assert(KS == 1 || XCH + REM * 4 * KS * 256 <= (MODE == 0 ? RED0 : BUF), "the exchange area must fit a chunk buffer");

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

//@EPILOGUE@
// An operand that is an unevaluated expression is computed where a stored one
// is loaded, in three steps: the element's place in the expression's inputs
// (once per lane and staging slot, before the loop over the chunks), the loads
// (issued like a stored operand's, ahead of the multiplications), and the
// program on the loaded values (when the vector goes to LDS).
#if VIRT_X
typedef VRaw_x RawX;
#define LOAD_X(ch_, j_) vfetch_x(vax, vpx[j_], ch_)
#define FIN_X(j_, r_) vfinish_x(hsx, vpx[j_], r_)
#else
typedef Vec<VX> RawX;
#define LOAD_X(ch_, j_) reinterpret_cast<const Vec<VX>*>(X + (ch_) * chx)[vidx(j_)]
#define FIN_X(j_, r_) (r_)
#endif
#if VIRT_Y
typedef VRaw_y RawY;
#define LOAD_Y(ch_, j_) vfetch_y(vay, vpy[(j_) - NLX], ch_)
#define FIN_Y(j_, r_) vfinish_y(hsy, vpy[(j_) - NLX], r_)
#else
typedef Vec<VY> RawY;
#define LOAD_Y(ch_, j_) reinterpret_cast<const Vec<VY>*>(Y + (ch_) * chy)[vidx(j_)]
#define FIN_Y(j_, r_) (r_)
#endif
extern "C" __global__ void __launch_bounds__(NT, BPC)
KNAME(const T* __restrict__ X, const T* __restrict__ Y, T* __restrict__ C, i64 nch, i64 chx, i64 chy, i64 chc, i64 part_stride
#if EPI
      , EpiArgs ea
#endif
#if VIRT_X
      , VArgs_x vax
#endif
#if VIRT_Y
      , VArgs_y vay
#endif
      ) {
#if VIRT_X
  const VHoist_x hsx = vhoist_x(vax);
#endif
#if VIRT_Y
  const VHoist_y hsy = vhoist_y(vay);
#endif
  __shared__ T lds[LDS_ELEMS];
#if EPI_STAGE
  // the chunk's results in the layout they have in memory, written out with whole vectors once the chunk is done
  __shared__ __attribute__((aligned(16))) unsigned char stage[EPI_STAGE];
#else
  unsigned char* const stage = nullptr;
#endif
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave = wave_all & 3;
  const int r = lane & 15, q4 = lane >> 4;
  // everything below is compiled once per part of K (KH): its K groups, hence the LDS offsets of its loop, are constants
  auto run = [&](auto KHI) {
  constexpr int KH = decltype(KHI)::v;
  if constexpr (KH < KS) {
  constexpr int GA = NG * KH / KS, GB = NG * (KH + 1) / KS;        // this part's K groups
  constexpr bool kRemOwner = KH == KS - 1;                          // its wavefronts 0 .. REM - 1 finish the split row blocks
  // j-th staging vector of this thread; the tail repeats the last vector.  The last vector of a footprint may reach up to
  // VX - 1 elements past it: still inside the operand's block, which the allocator ends with 16 spare bytes.
  auto vidx = [&](int j) -> int { int v = tid + NT * (j < NLX ? j : j - NLX); int lim = (j < NLX ? XV : YV) - 1; return v < lim ? v : lim; };
  // The first chunk, and the columns operand of mode 1, go to LDS up to 32
  // vectors at a time: the loads in flight together, then the stores.  Copied
  // one by one, every vector would wait out its own trip to memory.  The first
  // batch of each is asked for here, before the address tables below are looked
  // up: the three trips to memory (tables, first chunk, columns operand) then
  // run side by side instead of one after the other.
  constexpr int kFill = NLD < 32 ? (NLD > 0 ? NLD : 1) : 32;
#if VIRT_X
  VPre_x vpx[NLX];
#pragma unroll
  for (int j = 0; j < NLX; ++j) vpx[j] = vpre_x(XBASE + (i64)vidx(j) * VX);
#endif
#if VIRT_Y
  VPre_y vpy[NLY];
#pragma unroll
  for (int j = 0; j < NLY; ++j) vpy[j] = vpre_y(YBASE + (i64)vidx(NLX + j) * VY);
#endif
  i64 ch = blockIdx.x;
  RawX fx0[kFill];
  RawY fy0[kFill];
  if (ch < nch) {
#pragma unroll
    for (int j = 0; j < kFill && j < NLD; ++j) {
      if (j < NLX) fx0[j] = LOAD_X(ch, j);
      else fy0[j] = LOAD_Y(ch, j);
    }
  }
  Vec<VY> fyc0[MODE == 1 ? kFill : 1];
  if (MODE == 1) {
#pragma unroll
    for (int u = 0; u < kFill; ++u) {
      const int v = tid + NT * u;
      fyc0[u] = reinterpret_cast<const Vec<VY>*>(Y)[v < YV ? v : YV - 1];
    }
  }
  // per-lane addresses: row base + lane offset of each K pattern.  Two blocks on a CU (BPC 2) have half the
  // registers each: the sums are then made where they are used, from NBF + NPAT registers instead of NBF * NPAT.
#if BPC == 2
  int axr[NBF > 0 ? NBF : 1], axp[NPAT];
#pragma unroll
  for (int t = 0; t < NBF; ++t) {
    int m = (wave + 4 * t) * 16 + ROW_OF(r);
    axr[t] = kRowX[m < MIN ? m : MIN - 1];
  }
#pragma unroll
  for (int p = 0; p < NPAT; ++p) axp[p] = kPatX[p * 4 + q4];
#define AX(t_, p_) (axr[t_] + axp[p_])
#else
  int ax[NBF > 0 ? NBF : 1][NPAT];
#pragma unroll
  for (int t = 0; t < NBF; ++t) {
    int m = (wave + 4 * t) * 16 + ROW_OF(r);
    int ro = kRowX[m < MIN ? m : MIN - 1];
#pragma unroll
    for (int p = 0; p < NPAT; ++p) ax[t][p] = ro + kPatX[p * 4 + q4];
  }
#define AX(t_, p_) ax[t_][p_]
#endif
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
      const int trig = s == NSLOT - 1 ? NG - 1 : 4 * s + 3;     // the slot runs after this K group: in the part that holds it
      if (trig < GA || trig >= GB) continue;
      int gi = 4 * s + ((wave + rb) & 3);
      if (gi >= NG) gi = NG - 1;
      int p = kGrpPd[gi];
      remx[rb * NSLOT + s] = ro + kGrpXd[gi] + kPatX[p * 4 + q4];
      remy[rb * NSLOT + s] = YOFF + kColY[cn] + kGrpYd[gi] + kPatY[p * 4 + q4];
    }
  }
  // lanes past the end of K in the last group contribute zero
  const bool tail_lane = q4 >= KVALID;
#if EPI
  // where a lane's rows and windows go, and the program inputs that do not change with the row
#if BPC == 2
  // (half the registers: the places are looked up when a chunk is finished, in copies of the tables in LDS --
  // a lookup in memory would wait for every store issued before it)
  epi_tables_to_lds(tid);
#define EPOS(t_, m0_) epi_pos(m0_, r)
#else
  EPos epos[NACC];
#pragma unroll
  for (int t = 0; t < NBF; ++t)
    if (t % KS == KH) epos[t] = epi_pos((wave + 4 * t) * 16 + 4 * q4, r);     // row block t is finished by part t % KS
  if (REM > 0 && kRemOwner) epos[NBF] = epi_pos((4 * NBF + (wave < REM ? wave : 0)) * 16 + 4 * q4, r);
#define EPOS(t_, m0_) epos[t_]
#endif
  const Hoist hz = epi_hoist(ea, r < NIN ? r : NIN - 1);
#else
  OutPos pos[MODE == 1 ? NACC : 1];
  if (MODE == 1) {
#pragma unroll
    for (int t = 0; t < NBF; ++t)
      if (t % KS == KH) pos[t] = out_pos((wave + 4 * t) * 16 + 4 * q4, r);
    if (REM > 0 && kRemOwner) pos[NBF] = out_pos((4 * NBF + (wave < REM ? wave : 0)) * 16 + 4 * q4, r);
  }
#endif
  Acc acc[NACC];
#pragma unroll
  for (int t = 0; t < NACC; ++t) acc[t] = Acc{0, 0, 0, 0};
  // The parts' partial products of whole row block t go to the part t % KS, which adds them to its own
  // (xch: an area of LDS nobody reads any more); the partial products of the split row blocks, of all
  // 4 KS wavefronts, are added by wavefronts 0 .. REM - 1 of the last part into srem.
  T srem[4] = {T(0), T(0), T(0), T(0)};
  // COLSUM: wavefront 0 of every part adds up the column operand's fragments as it reads them: lane (r, q4)
  // the elements k = 4 g + q4 of column r, over the part's K groups g and all the block's chunks
  T colacc = T(0);
  auto meet = [&](T* xch) {
    if (KS > 1) {
#pragma unroll
      for (int t = 0; t < NBF; ++t) {
        if (t % KS != KH) {
          const int slot = KH < t % KS ? KH : KH - 1;
#pragma unroll
          for (int j = 0; j < 4; ++j) xch[(((wave * NBF + t) * (KS - 1) + slot) * 4 + j) * 64 + lane] = acc[t][j];
        }
      }
    }
    T* red = KS > 1 ? xch + XCH : lds + RED0;
    if (REM > 0) {
#pragma unroll
      for (int rb = 0; rb < REM; ++rb)
#pragma unroll
        for (int j = 0; j < 4; ++j) red[((rb * 4 * KS + wave_all) * 4 + j) * 64 + lane] = acc[NBF + rb][j];
    }
    if ((KS > 1 && NBF > 0) || REM > 0) __syncthreads();
    if (KS > 1) {
#pragma unroll
      for (int t = 0; t < NBF; ++t) {
        if (t % KS == KH) {
#pragma unroll
          for (int sl = 0; sl < KS - 1; ++sl)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[t][j] += xch[(((wave * NBF + t) * (KS - 1) + sl) * 4 + j) * 64 + lane];
        }
      }
    }
    if (REM > 0 && kRemOwner && wave < REM) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        T sum = T(0);
#pragma unroll
        for (int w = 0; w < 4 * KS; ++w) sum += red[((wave * 4 * KS + w) * 4 + j) * 64 + lane];
        srem[j] = sum;
      }
    }
  };

  // the first batches arrive in LDS; what is left of the first chunk and of the columns operand follows, a batch at a time
  if (ch < nch) {
#pragma unroll
    for (int j = 0; j < kFill && j < NLD; ++j) {
      if (j < NLX) reinterpret_cast<Vec<VX>*>(lds)[vidx(j)] = FIN_X(j, fx0[j]);
      else reinterpret_cast<Vec<VY>*>(lds + LX)[ypos(vidx(j))] = FIN_Y(j, fy0[j]);
    }
#pragma unroll
    for (int j0 = kFill; j0 < NLD; j0 += kFill) {
      RawX fx[kFill];
      RawY fy[kFill];
#pragma unroll
      for (int j = j0; j < j0 + kFill && j < NLD; ++j) {
        if (j < NLX) fx[j - j0] = LOAD_X(ch, j);
        else fy[j - j0] = LOAD_Y(ch, j);
      }
#pragma unroll
      for (int j = j0; j < j0 + kFill && j < NLD; ++j) {
        if (j < NLX) reinterpret_cast<Vec<VX>*>(lds)[vidx(j)] = FIN_X(j, fx[j - j0]);
        else reinterpret_cast<Vec<VY>*>(lds + LX)[ypos(vidx(j))] = FIN_Y(j, fy[j - j0]);
      }
    }
  }
  if (MODE == 1) {   // the columns operand does not change with the chunk
#pragma unroll
    for (int u = 0; u < kFill; ++u) {
      const int v = tid + NT * u;
      if (v < YV) reinterpret_cast<Vec<VY>*>(lds + NBUFS * BUF)[ypos(v)] = fyc0[u];
    }
    for (int v0 = tid + NT * kFill; v0 < YV; v0 += NT * kFill) {
      Vec<VY> fy[kFill];
#pragma unroll
      for (int u = 0; u < kFill; ++u) {
        const int v = v0 + NT * u;
        fy[u] = reinterpret_cast<const Vec<VY>*>(Y)[v < YV ? v : YV - 1];
      }
#pragma unroll
      for (int u = 0; u < kFill; ++u) {
        const int v = v0 + NT * u;
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
    RawX prex[PH * LPP];
    RawY prey[PH * LPP];
    // one buffer and an expression operand: a phase's loads are turned into values
    // when the phase ends, so that only one phase's raw loads are alive at a time
    Vec<VX> finx[(NBUFS == 1 && VIRT_X) ? PH * LPP : 1];
    Vec<VY> finy[(NBUFS == 1 && VIRT_Y) ? PH * LPP : 1];
    i64 chn = ch + gridDim.x;
    if (chn >= nch) chn = nch - 1;    // the last prefetch is not used
    if (MODE == 1) {
#pragma unroll
      for (int t = 0; t < NACC; ++t) acc[t] = Acc{0, 0, 0, 0};
    }
    auto phase = [&](auto PHI) {
      constexpr int ph = decltype(PHI)::v;
      constexpr int g0 = ph < PH ? GA + (GB - GA) * ph / PH : GB, g1 = ph < PH ? GA + (GB - GA) * (ph + 1) / PH : GB;
#pragma unroll
      for (int j = 0; j < LPP; ++j) {
        int jj = ph * LPP + j;
        if (jj < NLD) {
          if (jj < NLX) prex[jj] = LOAD_X(chn, jj);
          else prey[jj] = LOAD_Y(chn, jj);
        }
      }
      auto groups = [&](auto self, auto GI) -> void {
        constexpr int gi = decltype(GI)::v;
        if constexpr (gi < g1) {
          constexpr int p = kGrpP[gi], gx = kGrpX[gi], gy = kGrpY[gi];
          constexpr bool tail = gi == NG - 1 && KVALID < 4;
          T bv = LYp[by[p] + gy];
          if (tail && tail_lane) bv = T(0);
#if COLSUM
          if (wave == 0) colacc += bv;
#endif
#pragma unroll
          for (int t = 0; t < NBF; ++t) {
            T av = L[AX(t, p) + gx];
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
      if constexpr (NBF == 0 && REM > 0) {
        // Nothing but split row blocks: every multiplication has LDS operands of
        // its own.  They are read a batch of slots ahead of the batch being
        // multiplied (the fences keep the compiler from sinking each read to
        // its use, where every MFMA would wait out a trip to LDS).
        constexpr int S0 = rem_slots_before(g0), S1 = rem_slots_before(g1);
        auto rem_load = [&](auto SI) {
          constexpr int sb = decltype(SI)::v;
          RemOps o;
#pragma unroll
          for (int u = 0; u < RGB; ++u)
#pragma unroll
            for (int rb = 0; rb < REM; ++rb) {
              const int sl = sb + u < S1 ? sb + u : S1 - 1;
              o.a[u][rb] = L[remx[rb * NSLOT + sl]];
              o.b[u][rb] = LYp[remy[rb * NSLOT + sl]];
            }
          return o;
        };
        auto rem_run = [&](auto self, auto SI, const RemOps& cur) -> void {
          constexpr int sb = decltype(SI)::v;
          if constexpr (sb < S1) {
            constexpr int sn = sb + RGB;
            RemOps nxt;
            if constexpr (sn < S1) nxt = rem_load(IC<sn>{});
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < RGB; ++u) {
              if (sb + u < S1) {
#pragma unroll
                for (int rb = 0; rb < REM; ++rb) {
                  const int sl = sb + u;
                  const int g2 = 4 * sl + ((wave + rb) & 3);
                  if (sl < NSLOT - 1 || g2 < NG) {
                    T a2 = cur.a[u][rb], b2 = cur.b[u][rb];
                    if (KVALID < 4 && g2 == NG - 1 && tail_lane) { a2 = T(0); b2 = T(0); }
                    acc[NBF + rb] = MFMA(a2, b2, acc[NBF + rb]);
                  }
                }
              }
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (sn < S1) self(self, IC<sn>{}, nxt);
          }
        };
        if constexpr (S0 < S1) rem_run(rem_run, IC<S0>{}, rem_load(IC<S0>{}));
      } else {
        groups(groups, IC<g0>{});
      }
      if (NBUFS == 2) {
#pragma unroll
        for (int j = 0; j < LPP; ++j) {
          int jj = ph * LPP + j;
          if (jj < NLD) {
            if (jj < NLX) reinterpret_cast<Vec<VX>*>(Ln)[vidx(jj)] = FIN_X(jj, prex[jj]);
            else reinterpret_cast<Vec<VY>*>(Ln + LX)[ypos(vidx(jj))] = FIN_Y(jj, prey[jj]);
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < LPP; ++j) {
          int jj = ph * LPP + j;
          if (jj < NLD) {
            if (VIRT_X && jj < NLX) finx[VIRT_X ? jj : 0] = FIN_X(jj, prex[jj]);
            if (VIRT_Y && jj >= NLX) finy[VIRT_Y ? jj : 0] = FIN_Y(jj, prey[jj]);
          }
        }
      }
    };
    phase(IC<0>{});
    if constexpr (PH > 1) phase(IC<1>{});
    if constexpr (PH > 2) phase(IC<2>{});
    // ---- the parts' products meet (KS > 1), the split row blocks are added up
    if (MODE == 1) {
      if (KS > 1) __syncthreads();     // everyone has multiplied this chunk: its buffer becomes the exchange area
      meet(const_cast<T*>(L));
    }
    if (NBUFS == 2) {
      cur ^= 1;
    } else {
      __syncthreads();    // everyone has finished reading this chunk
#pragma unroll
      for (int jj = 0; jj < NLD; ++jj) {
#if VIRT_X
        if (jj < NLX) reinterpret_cast<Vec<VX>*>(Ln)[vidx(jj)] = finx[jj];
#else
        if (jj < NLX) reinterpret_cast<Vec<VX>*>(Ln)[vidx(jj)] = prex[jj];
#endif
#if VIRT_Y
        if (jj >= NLX) reinterpret_cast<Vec<VY>*>(Ln + LX)[ypos(vidx(jj))] = finy[jj];
#else
        if (jj >= NLX) reinterpret_cast<Vec<VY>*>(Ln + LX)[ypos(vidx(jj))] = prey[jj];
#endif
      }
    }
    if (MODE == 1) {
#if EPI
#pragma unroll
      for (int t = 0; t < NBF; ++t)
        if (t % KS == KH) epi_tile(ea, hz, EPOS(t, (wave + 4 * t) * 16 + 4 * q4), stage, ch, (wave + 4 * t) * 16 + 4 * q4, r, acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
      if (REM > 0 && kRemOwner && wave < REM) epi_tile(ea, hz, EPOS(NBF, (4 * NBF + wave) * 16 + 4 * q4), stage, ch, (4 * NBF + wave) * 16 + 4 * q4, r, srem[0], srem[1], srem[2], srem[3]);
#else
      T* out = C + ch * chc;
#pragma unroll
      for (int t = 0; t < NBF; ++t)
        if (t % KS == KH) store_rows(out, pos[t], (wave + 4 * t) * 16 + 4 * q4, r, acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
      if (REM > 0 && kRemOwner && wave < REM) store_rows(out, pos[MODE == 1 ? NBF : 0], (4 * NBF + wave) * 16 + 4 * q4, r, srem[0], srem[1], srem[2], srem[3]);
#endif
#if EPI_STAGE
      __syncthreads();
      epi_flush(ea, stage, ch, tid);
#endif
    }
  }
#if !EPI
  if (MODE == 0) {
#if COLSUM
    if (wave == 0) {
      colacc += __shfl_xor(colacc, 16);
      colacc += __shfl_xor(colacc, 32);
      if (KS > 1 && q4 == 0) lds[CS0 + KH * 16 + r] = colacc;
    }
#endif
    if (KS > 1 || REM > 0) __syncthreads();      // all multiplications are done: the chunk buffers are free
    meet(lds);
    T* out = C + (i64)blockIdx.x * part_stride;
#if COLSUM
    if (KH == 0 && wave == 0 && q4 == 0 && r < NIN) {
      T tot = colacc;
#pragma unroll
      for (int h = 1; h < KS; ++h) tot += lds[CS0 + h * 16 + r];
      out[COLSUM + r - 1] = tot;       // COLSUM - 1: where the column sums start in a block's partial result
    }
#endif
#pragma unroll
    for (int t = 0; t < NBF; ++t)
      if (t % KS == KH) store_rows(out, out_pos((wave + 4 * t) * 16 + 4 * q4, r), (wave + 4 * t) * 16 + 4 * q4, r, acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
    if (REM > 0 && kRemOwner && wave < REM) store_rows(out, out_pos((4 * NBF + wave) * 16 + 4 * q4, r), (4 * NBF + wave) * 16 + 4 * q4, r, srem[0], srem[1], srem[2], srem[3]);
  }
#endif
  }
  };   // run
  if constexpr (KS == 1) {
    run(IC<0>{});
  } else if constexpr (KS == 2) {
    if (wave_all < 4) run(IC<0>{}); else run(IC<1>{});
  } else {
    switch (wave_all >> 2) {
      case 0: run(IC<0>{}); break;
      case 1: run(IC<1>{}); break;
      case 2: run(IC<2>{}); break;
      default: run(IC<3>{}); break;
    }
  }
}
)HG";

int lds_bytes(const Plan& pl) {
  const int es = pl.f64 ? 8 : 4;
  int64_t lx = (pl.span_x + pl.vx - 1) / pl.vx * pl.vx, ly = (pl.span_y + pl.vy - 1) / pl.vy * pl.vy;
  if (pl.ypad) ly += (ly / pl.ys) * pl.ypad;
  int64_t buf = pl.mode == 0 ? lx + ly : lx;
  int MB = (pl.min_rows + 15) / 16, REM = MB % 4;
  int64_t total = pl.nbufs * buf + (pl.mode == 0 ? 0 : ly) + (REM > 0 && pl.ks == 1 ? REM * 4 * 256 : 0);
  total *= es;
  return total > INT32_MAX ? INT32_MAX : (int)total;
}

std::string generate(const Plan& pl, const std::string& kname, const std::string& epilogue = std::string(), int stage_bytes = 0,
                     const std::string& virt_x = std::string(), int64_t xbase = 0, const std::string& virt_y = std::string(), int64_t ybase = 0) {
  hg::fusedgen::Src s;
  s << "#define KNAME " << kname << "\n";
  s << "#define VIRT_X " << (virt_x.empty() ? 0 : 1) << "\n#define XBASE " << xbase << "ll\n";
  s << "#define VIRT_Y " << (virt_y.empty() ? 0 : 1) << "\n#define YBASE " << ybase << "ll\n";
  s << "#define EPI " << (epilogue.empty() ? 0 : 1) << "\n#define EPI_STAGE " << stage_bytes << "\n#define BPC " << pl.bpc << "\n";
  const int es = pl.f64 ? 8 : 4;
  s << "#define F64 " << (pl.f64 ? 1 : 0) << "\n#define KS " << pl.ks << "\n#define COLSUM " << (pl.colsum_at >= 0 ? pl.colsum_at + 1 : 0) << "\n";
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
  std::string body = kBody;
  const std::string mark = "//@EPILOGUE@";
  std::string pre = epilogue;
  if (epilogue.empty() && (!virt_x.empty() || !virt_y.empty())) pre = fusedgen::kPrelude;
  body.replace(body.find(mark), mark.size(), pre + virt_x + virt_y);
  s << body;
  return s.str();
}

// An operand that is an elementwise program's result, its dims merged to M,
// zero-extended to P = M + lo + hi, seen through a strided view of P's dense
// row-major layout.  The kernels address it by element offsets in that layout.
struct VirtualOp {
  int n_in = 0, n_instr = 0, slot = 0, dtype = 0;
  const hgpu_array* const* in = nullptr;
  const hgpu_fused_instr* prog = nullptr;
  std::vector<int> dt;                       // type of every slot
  std::vector<int64_t> E, M, lo, hi, P;      // shape of the inputs; merged; extension; extended
  int64_t total = 0;                         // elements of P
  bool padded = false;
};

// true when V consecutive elements of the layout, starting at a multiple of V,
// are V consecutive elements of the innermost dim of the inputs (all valid or all padding)
bool vector_ok(const VirtualOp& v, int V) {
  if (V == 1) return true;
  if (v.E.empty() || v.M.empty()) return false;
  return v.E.back() % V == 0 && v.P.back() % V == 0 && v.lo.back() % V == 0 && v.total % V == 0;
}

// Everything vops_source reads.
static_assert(sizeof(VirtualOp) == 192, "put_virtual must cover every field of VirtualOp");
void put_virtual(hg::fusedgen::Key& k, const VirtualOp& v, int V, int64_t chunk_stride, int64_t max_elem) {
  k.put(v.n_in).put(v.n_instr, v.prog).put(v.slot).put(v.dtype).put(v.dt).put(v.E).put(v.M).put(v.lo).put(v.hi).put(v.P).put(v.total).put(v.padded);
  for (int i = 0; i < v.n_in; ++i) {
    const hgpu_array* a = v.in[i];
    k.put(a->dtype).put(a->rank, a->shape).put(a->rank, a->strides).put((int)((uintptr_t)data_ptr(a) & 63));
  }
  k.put(V).put(chunk_stride).put(max_elem);
}

// Source of the three steps that stand in for the load of V consecutive
// elements of an expression operand (tag "x" or "y"):
//   VPre  vpre(w)                the place of element offset w (the chunk's own
//                                offset left out) in the inputs of the expression;
//   VRaw  vfetch(args, pre, ch)  the loads for chunk ch;
//   Vec   vfinish(hoisted, pre, raw)   the program on the loaded values; elements
//                                in the zero-extension, or past the end, are zero.
// chunk_stride: elements of the layout between chunks.  When a chunk is a step
// along the outermost dim of the layout, and that dim is one of the inputs' own
// (not merged, not extended), the place is decoded once, before the loop over
// the chunks, and a chunk only adds a constant to every input offset; else the
// offset is decoded for every chunk.  Divisors are constants of the kernel.
std::string vops_source(const VirtualOp& v, const char* tag_, int V, int64_t chunk_stride, int64_t max_elem = INT64_MAX) {
  using namespace hg::fusedgen;
  Src s;
  const std::string tag = tag_;
  const std::string T_ = ctype(v.dtype);
  const size_t rm = v.M.size(), re = v.E.size();
  // per input: one broadcast element; no move along the innermost dim (one load
  // serves a vector); V neighbours there that one aligned load fetches
  std::vector<char> scalar((size_t)v.n_in, 0), shared((size_t)v.n_in, 0), vecload((size_t)v.n_in, 0), wide((size_t)v.n_in, 0);
  std::vector<int> rep((size_t)v.n_in, -1);   // the first input with the same strides: they share their offsets
  for (int i = 0; i < v.n_in; ++i) {
    const hgpu_array* a = v.in[i];
    bool all0 = true;
    int64_t reach = 0;
    for (int d = 0; d < a->rank; ++d) {
      if (a->shape[d] != 1 && a->strides[d] != 0) all0 = false;
      reach += (a->shape[d] - 1) * (a->strides[d] < 0 ? -a->strides[d] : a->strides[d]);
    }
    scalar[(size_t)i] = all0;
    wide[(size_t)i] = reach >= (1LL << 31);
    shared[(size_t)i] = !all0 && V > 1 && (v.E[re - 1] == 1 || a->strides[re - 1] == 0);
    if (!all0 && V > 1 && !shared[(size_t)i] && a->strides[re - 1] == 1) {
      bool ok = ((uintptr_t)data_ptr(a) % (dtype_size(a->dtype) * (size_t)V)) == 0;
      for (size_t j = 0; j + 1 < re && ok; ++j) ok = v.E[j] == 1 || a->strides[j] % V == 0;
      vecload[(size_t)i] = ok;
    }
    rep[(size_t)i] = i;
    for (int k = 0; k < i && !all0; ++k) {
      if (scalar[(size_t)k]) continue;
      bool same = true;
      for (size_t j = 0; j < re && same; ++j) same = v.E[j] == 1 || v.in[k]->strides[j] == a->strides[j];
      if (same) { rep[(size_t)i] = rep[(size_t)k]; break; }
    }
  }
  auto own = [&](int i) { return !scalar[(size_t)i] && rep[(size_t)i] == i; };   // carries offsets of its own
  auto oty = [&](int i) { return wide[(size_t)i] ? "i64" : "int"; };
  std::vector<int64_t> PS(rm), MS(rm), ES(re);
  { int64_t a = 1, b = 1; for (size_t k = rm; k-- > 0;) { PS[k] = a; a *= v.P[k]; MS[k] = b; b *= v.M[k]; } }
  { int64_t a = 1; for (size_t j = re; j-- > 0;) { ES[j] = a; a *= v.E[j]; } }
  // first dims with more than one element
  size_t k0 = 0, j0 = 0;
  while (k0 < rm && v.P[k0] == 1) ++k0;
  while (j0 < re && v.E[j0] == 1) ++j0;
  const bool separable = chunk_stride != 0 && k0 < rm && j0 < re && chunk_stride % PS[k0] == 0 && v.lo[k0] == 0 && v.hi[k0] == 0 && v.E[j0] == v.M[k0] &&
                         ES[j0] == MS[k0] && !(V > 1 && j0 == re - 1);
  const int64_t chunk_step = separable ? chunk_stride / PS[k0] : 0;   // coordinates along the outermost dim per chunk
  const bool range_check = max_elem > v.total;        // some lane of some chunk may address past the layout's end
  const bool has_ok = range_check || v.padded;
  auto gp = [&](int i, const std::string& ty) { return std::string("const __attribute__((address_space(1))) ") + ty + "*"; };

  s << "struct VArgs_" << tag << " {\n";
  for (int i = 0; i < v.n_in; ++i) s << "  const " << ctype(v.dt[(size_t)i]) << "* i" << i << ";\n";
  s << "};\nstruct VHoist_" << tag << " {\n";
  for (int i = 0; i < v.n_in; ++i)
    if (scalar[(size_t)i]) s << "  " << ctype(v.dt[(size_t)i]) << " s" << i << ";\n";
  s << "  int unused;\n};\n";
  s << "__device__ __forceinline__ VHoist_" << tag << " vhoist_" << tag << "(const VArgs_" << tag << "& va) {\n  VHoist_" << tag << " h;\n  h.unused = 0;\n";
  for (int i = 0; i < v.n_in; ++i)
    if (scalar[(size_t)i]) s << "  h.s" << i << " = va.i" << i << "[0];\n";
  s << "  return h;\n}\n";
  for (int i = 0; i < v.n_in; ++i)
    if (vecload[(size_t)i]) s << "struct alignas(" << dtype_size(v.dt[(size_t)i]) * (size_t)V << ") VPack_" << tag << i << " { " << ctype(v.dt[(size_t)i]) << " v[" << V << "]; };\n";

  // decode: element offset `e` (unsigned, in range) -> ok, input offsets o<i>
  auto emit_decode = [&](const char* ind) {
    if (v.padded) {
      s << ind << "unsigned flat = 0;\n";
      for (size_t k = 0; k < rm; ++k) {
        if (v.P[k] == 1) continue;
        s << ind << "{\n" << ind << "  const unsigned c = " << (k == k0 ? "e / " + std::to_string(PS[k]) + "u" : "(e / " + std::to_string(PS[k]) + "u) % " + std::to_string(v.P[k]) + "u") << ";\n";
        if (v.lo[k] != 0 || v.hi[k] != 0) s << ind << "  ok = ok && c >= " << v.lo[k] << "u && c < " << v.lo[k] + v.M[k] << "u;\n";
        s << ind << "  flat += (c - " << v.lo[k] << "u) * " << MS[k] << "u;\n" << ind << "}\n";
      }
      s << ind << "if (!ok) flat = 0;\n";
    } else {
      s << ind << "const unsigned flat = e;\n";
    }
    for (size_t j = 0; j < re; ++j) {
      bool used = false;
      for (int i = 0; i < v.n_in; ++i) used = used || (!scalar[(size_t)i] && v.in[i]->strides[j] != 0);
      if (!used || v.E[j] == 1) continue;
      if (V > 1 && j == re - 1) s << ind << "const unsigned x" << j << " = flat % " << v.E[j] << "u;\n";
      else s << ind << "const unsigned x" << j << " = " << (j == j0 ? "flat / " + std::to_string(ES[j]) + "u" : "(flat / " + std::to_string(ES[j]) + "u) % " + std::to_string(v.E[j]) + "u") << ";\n";
    }
    for (int i = 0; i < v.n_in; ++i) {
      if (!own(i)) continue;
      s << ind << "const " << oty(i) << " o" << i << " = 0";
      for (size_t j = 0; j < re; ++j)
        if (v.E[j] != 1 && v.in[i]->strides[j] != 0) s << " + (" << oty(i) << ")x" << j << " * " << v.in[i]->strides[j] << (wide[(size_t)i] ? "ll" : "");
      s << ";\n";
    }
  };

  s << "struct VPre_" << tag << " {\n";
  if (separable) {
    for (int i = 0; i < v.n_in; ++i)
      if (own(i)) s << "  " << oty(i) << " o" << i << ";\n";
    if (v.padded) s << "  bool ok;\n";
  }
  if (!separable || range_check) s << "  i64 w;\n";
  s << "  int unused[0];\n};\n";
  s << "__device__ __forceinline__ VPre_" << tag << " vpre_" << tag << "(i64 w) {\n  VPre_" << tag << " p;\n";
  if (separable) {
    s << "  bool ok = w >= 0 && w < " << v.total << "ll;\n";
    s << "  const unsigned e = ok ? (unsigned)w : 0u;\n";
    emit_decode("  ");
    for (int i = 0; i < v.n_in; ++i)
      if (own(i)) s << "  p.o" << i << " = o" << i << ";\n";
    if (v.padded) s << "  p.ok = ok;\n";
  }
  if (!separable || range_check) s << "  p.w = w;\n";
  s << "  return p;\n}\n";

  s << "struct VRaw_" << tag << " {\n";
  for (int i = 0; i < v.n_in; ++i) {
    if (scalar[(size_t)i]) continue;
    if (vecload[(size_t)i]) s << "  VPack_" << tag << i << " r" << i << ";\n";
    else s << "  " << ctype(v.dt[(size_t)i]) << " r" << i << (shared[(size_t)i] ? "" : "[" + std::to_string(V) + "]") << ";\n";
  }
  if (has_ok) s << "  bool ok;\n";
  s << "  int unused[0];\n};\n";
  s << "__device__ __forceinline__ VRaw_" << tag << " vfetch_" << tag << "(const VArgs_" << tag << "& va, const VPre_" << tag << "& p, i64 ch) {\n  VRaw_" << tag << " r;\n";
  if (separable) {
    // the chunk moves every input by a constant; an element past the layout's end reads the first one's place (its value is dropped)
    if (has_ok) {
      s << "  bool ok = " << (v.padded ? "p.ok" : "true") << (range_check ? " && p.w + ch * " + std::to_string(chunk_stride) + "ll < " + std::to_string(v.total) + "ll" : "") << ";\n";
      s << "  const i64 cq = ok ? ch * " << chunk_step << "ll : 0;\n";
    } else {
      s << "  const i64 cq = ch * " << chunk_step << "ll;\n";
    }
    for (int i = 0; i < v.n_in; ++i)
      if (own(i)) s << "  const i64 o" << i << " = (i64)" << (has_ok ? "(ok ? p.o" + std::to_string(i) + " : 0)" : "p.o" + std::to_string(i)) << " + cq * " << v.in[i]->strides[j0] << "ll;\n";
  } else {
    s << "  const i64 e0 = p.w + ch * " << chunk_stride << "ll;\n";
    s << "  bool ok = e0 >= 0 && e0 < " << v.total << "ll;\n";
    s << "  const unsigned e = ok ? (unsigned)e0 : 0u;\n";
    emit_decode("  ");
  }
  for (int i = 0; i < v.n_in; ++i) {
    if (scalar[(size_t)i]) continue;
    const std::string ct = ctype(v.dt[(size_t)i]);
    const std::string off = "o" + std::to_string(rep[(size_t)i]);
    if (vecload[(size_t)i]) {
      const std::string pk = "VPack_" + tag + std::to_string(i);
      s << "  r.r" << i << " = *(" << gp(i, pk) << ")((" << gp(i, ct) << ")va.i" << i << " + " << off << ");\n";
    } else {
      s << "  {\n    " << gp(i, ct) << " g = (" << gp(i, ct) << ")va.i" << i << ";\n";
      if (shared[(size_t)i]) s << "    r.r" << i << " = g[" << off << "];\n";
      else for (int el = 0; el < V; ++el) s << "    r.r" << i << "[" << el << "] = g[" << off << " + " << (int64_t)el * (re > 0 ? v.in[i]->strides[re - 1] : 0) << "ll];\n";
      s << "  }\n";
    }
  }
  if (has_ok) s << "  r.ok = ok;\n";
  s << "  return r;\n}\n";

  s << "__device__ __forceinline__ Vec<" << V << "> vfinish_" << tag << "(const VHoist_" << tag << "& hs, const VPre_" << tag << "&, const VRaw_" << tag << "& raw) {\n";
  s << "  Vec<" << V << "> r;\n";
  for (int el = 0; el < V; ++el) {
    std::string suf = "_" + std::to_string(el);
    s << "  {\n";
    for (int i = 0; i < v.n_in; ++i) {
      s << "    const " << ctype(v.dt[(size_t)i]) << " v" << i << suf << " = ";
      if (scalar[(size_t)i]) s << "hs.s" << i;
      else if (vecload[(size_t)i]) s << "raw.r" << i << ".v[" << el << "]";
      else if (shared[(size_t)i]) s << "raw.r" << i;
      else s << "raw.r" << i << "[" << el << "]";
      s << ";\n";
    }
    emit_program(s, v.n_in, v.n_instr, v.prog, v.dt, "    ", suf);
    const std::string val = has_ok ? "raw.ok ? v" + std::to_string(v.slot) + suf + " : " + T_ + "(0)" : "v" + std::to_string(v.slot) + suf;
    if (V > 1) s << "    r[" << el << "] = " << val << ";\n";
    else s << "    r = " << val << ";\n";
    s << "  }\n";
  }
  s << "  return r;\n}\n";
  return s.str();
}

// Staging vectors, LDS padding of the columns operand, output vectors and the
// number of chunk buffers of a plan whose operands sit at xp / yp; false when
// the plan does not fit the CU.
bool finish_plan(Plan& pl, const char* xp, const char* yp, const char* cp, int64_t out_n, int extra_lds_bytes, const VirtualOp* virt_x = nullptr,
                 const VirtualOp* virt_y = nullptr) {
  const int es = pl.f64 ? 8 : 4;
  const int V = 16 / es;
  pl.vx = (((uintptr_t)xp & 15) == 0 && (pl.chx * es) % 16 == 0) ? V : 1;
  pl.vy = (((uintptr_t)yp & 15) == 0 && (pl.chy * es) % 16 == 0) ? V : 1;
  if (virt_x && !vector_ok(*virt_x, pl.vx)) pl.vx = 1;
  if (virt_y && !vector_ok(*virt_y, pl.vy)) pl.vy = 1;
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
    bool ok = cp != nullptr && pl.min_rows % 4 == 0 && ((uintptr_t)cp & 15) == 0 && pl.chc % V == 0;
    for (size_t m = 0; m < pl.row_c.size() && ok; m += 4)
      ok = pl.row_c[m] % V == 0 && pl.row_c[m + 1] == pl.row_c[m] + 1 && pl.row_c[m + 2] == pl.row_c[m] + 2 && pl.row_c[m + 3] == pl.row_c[m] + 3;
    for (size_t c = 0; c < pl.col_c.size() && ok; ++c) ok = pl.col_c[c] % V == 0;
    if (pl.mode == 0) ok = ok && out_n % V == 0;   // partial outputs lie out_n apart
    pl.cvec = ok;
  }
  // scalar staging of a large footprint would need too many loads in flight; a
  // staging slot of an expression operand costs one load per input that is not a
  // single broadcast element (the kernel is bound by the number of loads a
  // wavefront can have in flight, not by their size)
  auto per_slot = [](const VirtualOp* v) {
    if (!v) return (int64_t)1;
    int64_t n = 0;
    for (int i = 0; i < v->n_in; ++i) {
      bool all0 = true;
      for (int d = 0; d < v->in[i]->rank; ++d)
        if (v->in[i]->shape[d] != 1 && v->in[i]->strides[d] != 0) all0 = false;
      if (!all0) ++n;
    }
    return n > 0 ? n : (int64_t)1;
  };
  // Two wavefronts per SIMD, each multiplying half of a chunk's K groups, keep the matrix cores busier
  // than one (a wavefront's LDS reads and waits hide behind the other's multiplications).  That needs K
  // groups to share out and room for the halves' partial products in a chunk buffer.
  static const int ks_env = getenv("HORDEAD_FOOTPRINT_KS") ? atoi(getenv("HORDEAD_FOOTPRINT_KS")) : 0;
  const int MB = (pl.min_rows + 15) / 16, NBF = MB / 4, REM = MB % 4, NG = (int)pl.gx.size();
  auto staged_loads = [&](int nt) {
    return (pl.span_x / pl.vx + nt - 1) / nt * per_slot(virt_x) + (pl.mode == 0 ? (pl.span_y / pl.vy + nt - 1) / nt * per_slot(virt_y) : 0);
  };
  for (int ks : {ks_env == 1 ? 1 : 2, 1}) {
    if (ks == 2 && NG < 16) continue;
    pl.ks = ks;
    const int64_t loads = staged_loads(256 * ks);
    if (loads > 48) continue;
    const int64_t lx = (pl.span_x + pl.vx - 1) / pl.vx * pl.vx;
    int64_t ly = (pl.span_y + pl.vy - 1) / pl.vy * pl.vy;
    if (pl.ypad) ly += (ly / pl.ys) * pl.ypad;
    const int64_t exchange = (int64_t)4 * NBF * (ks - 1) * 256 + (int64_t)REM * 4 * ks * 256;
    pl.nbufs = 2;
    if (lds_bytes(pl) + extra_lds_bytes > kLdsBudget) {
      pl.nbufs = 1;
      // the prefetch must fit the register file (half of it with two wavefronts per SIMD)
      if (lds_bytes(pl) + extra_lds_bytes > kLdsBudget || loads * 4 + pl.addr_regs > (ks == 1 ? 330 : 170)) continue;
    }
    if (ks > 1 && exchange > (pl.mode == 0 ? pl.nbufs * (lx + ly) : lx)) continue;
    return true;
  }
  return false;
}

}  // namespace

namespace {
void remember_sum(hgpu_ctx* ctx, const VirtualOp& v, const std::vector<int>& kept, hgpu_array* sum);
}

namespace hg {

// gemm.hip: out[i] = sum over the `parts` partial outputs of part[s * n + i], in a fixed order.
int sum_partials(hgpu_ctx* ctx, int dtype, int64_t n, int parts, const void* part, void* out);
int sum_partials_split(hgpu_ctx* ctx, int dtype, int64_t n1, int64_t n2, int parts, const void* part, void* out1, void* out2);

int try_footprint_virtual(hgpu_ctx* ctx, const GemmParams& p, int dtype, const void* pa, const void* pb, hgpu_array* out, bool* handled,
                          const void* va_, const void* vb_);

// Runs the contraction described by p with the footprint kernel when its shape
// suits it (*handled), else leaves it to the caller's other kernels.
int try_footprint(hgpu_ctx* ctx, const GemmParams& p, int dtype, const void* pa, const void* pb, hgpu_array* out, bool* handled) {
  return try_footprint_virtual(ctx, p, dtype, pa, pb, out, handled, nullptr, nullptr);
}

// The same with operands that may be unevaluated expressions (va / vb not null:
// pa / pb are then the element offset of the operand's view in the layout of
// its expression, times the element size, as a pointer from address 0).
int try_footprint_virtual(hgpu_ctx* ctx, const GemmParams& p, int dtype, const void* pa, const void* pb, hgpu_array* out, bool* handled,
                          const void* va_, const void* vb_) {
  const VirtualOp* va = static_cast<const VirtualOp*>(va_);
  const VirtualOp* vb = static_cast<const VirtualOp*>(vb_);
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
        const char* xp = (const char*)(swapped ? pb : pa) + pl.shift_x * es;
        const char* yp = (const char*)(swapped ? pa : pb) + pl.shift_y * es;
        if (!finish_plan(pl, xp, yp, (const char*)data_ptr(out), nelem(out), 0, swapped ? vb : va, swapped ? va : vb)) continue;
        if (pl.mode == 1 && (swapped ? va : vb)) continue;   // the columns operand of this mode is staged once, from memory
        best = pl;
        best_swapped = swapped != 0;
        found = true;
      }
    }
  }
  if (!found) return HGPU_OK;
  Plan& pl = best;
  // the kernel's name tells a profiler which product it is
  char kname[128];
  const VirtualOp* vx = best_swapped ? vb : va;
  const VirtualOp* vy = best_swapped ? va : vb;
  // The columns operand an expression, summed over K by the same kernel: the sum of the expression over
  // every merged dim but the columns' (a bias's cotangent next to the kernel's), for the caller who asks next.
  std::vector<int> colsum_dims;
  std::vector<int64_t> colsum_shape;
  if (vy && pl.mode == 0 && (pl.min_rows + 15) / 16 >= 4 && (best_swapped ? pa : pb) == nullptr && !vy->padded) {
    const std::vector<Dim> cd = dims(best_swapped ? p.m : p.n, best_swapped), kd = dims(p.k, best_swapped);
    const size_t rm = vy->M.size();
    std::vector<int64_t> DM(rm, 1);
    for (size_t k = rm; k-- > 1;) DM[k - 1] = DM[k] * vy->M[k];
    std::vector<char> covered(rm, 0);
    bool ok = true;
    auto match = [&](const std::vector<Dim>& ds, bool keep) {
      for (auto& d : ds) {
        if (d.e == 1) continue;
        int hit = -1;
        for (size_t k = 0; k < rm; ++k)
          if (vy->M[k] > 1 && !covered[k] && DM[k] == d.sy && vy->M[k] == d.e) { hit = (int)k; break; }
        if (hit < 0) { ok = false; return; }
        covered[(size_t)hit] = 1;
        if (keep) { colsum_dims.push_back(hit); colsum_shape.push_back(d.e); }
      }
    };
    match(cd, true);
    if (ok) match(kd, false);
    for (size_t k = 0; k < rm && ok; ++k)
      if (vy->M[k] > 1 && !covered[k]) ok = false;
    if (ok && !colsum_dims.empty()) pl.colsum_at = nelem(out);
    else { colsum_dims.clear(); colsum_shape.clear(); }
  }
  snprintf(kname, sizeof kname, "footprint_gemm_%s_m%lld_n%lld_k%lld_%s%s%s%s%s", f64 ? "f64" : "f32", (long long)p.M, (long long)p.N, (long long)p.K,
           pl.mode == 0 ? "chunkK" : "chunkM", best_swapped ? "_swapped" : "", vx ? "_xmap" : "", vy ? "_ymap" : "", pl.ks == 2 ? "_w8" : "");
  const int64_t xbase = (int64_t)((uintptr_t)((const char*)(best_swapped ? pb : pa) + pl.shift_x * es) / (uintptr_t)es);
  const int64_t ybase = (int64_t)((uintptr_t)((const char*)(best_swapped ? pa : pb) + pl.shift_y * es) / (uintptr_t)es);
  // the last staging vector of the last chunk may reach past its footprint: how far at most
  const int64_t xmax = xbase + (pl.nch - 1) * pl.chx + (pl.span_x + pl.vx - 1) / pl.vx * pl.vx;
  const int64_t ymax = ybase + (pl.nch - 1) * pl.chy + (pl.span_y + pl.vy - 1) / pl.vy * pl.vy;
  Compiled kernel{nullptr, nullptr};
  {
    fusedgen::Key key;
    key.put(std::string(kname));
    put_plan(key, pl);
    key.put(vx != nullptr).put(vy != nullptr);
    if (vx) { put_virtual(key, *vx, pl.vx, pl.chx, xmax); key.put(xbase); }
    if (vy) { put_virtual(key, *vy, pl.vy, pl.chy, ymax); key.put(ybase); }
    int rc = known_kernel(ctx, key, kname, [&] {
      return generate(pl, kname, std::string(), 0, vx ? vops_source(*vx, "x", pl.vx, pl.chx, xmax) : std::string(), vx ? xbase : 0,
                      vy ? vops_source(*vy, "y", pl.vy, pl.chy, ymax) : std::string(), vy ? ybase : 0);
    }, &kernel);
    if (rc) return rc;
  }
  if (!kernel.fn) return HGPU_OK;
  const char* xp = (const char*)(best_swapped ? pb : pa) + pl.shift_x * es;
  const char* yp = (const char*)(best_swapped ? pa : pb) + pl.shift_y * es;
  int64_t out_n = nelem(out);
  int64_t grid = pl.nch < ctx->num_cu ? pl.nch : ctx->num_cu;
  hgpu_buffer* part = nullptr;
  void* cdst = data_ptr(out);
  int64_t part_stride = 0;
  const int64_t n_colsum = pl.colsum_at >= 0 ? pl.nin : 0;
  hgpu_array* colsum = nullptr;
  if (pl.mode == 0) {
    if (n_colsum > 0) {
      int rc = new_dense(ctx, dtype, (int)colsum_shape.size(), colsum_shape.data(), &colsum);
      if (rc) return rc;
    }
    int rc = buffer_alloc(ctx, (size_t)(out_n + n_colsum) * (size_t)grid * es, &part);
    if (rc) { if (colsum) hgpu_release(colsum); return rc; }
    cdst = part->ptr;
    part_stride = out_n + n_colsum;
  }
  int64_t nch = pl.nch, chx = pl.chx, chy = pl.chy, chc = pl.chc;
  // the inputs of an expression operand follow as one struct of pointers each
  std::vector<const void*> vxa, vya;
  if (vx) { xp = nullptr; for (int i = 0; i < vx->n_in; ++i) vxa.push_back(data_ptr(vx->in[i])); }
  if (vy) { yp = nullptr; for (int i = 0; i < vy->n_in; ++i) vya.push_back(data_ptr(vy->in[i])); }
  std::vector<void*> args = {(void*)&xp, (void*)&yp, (void*)&cdst, (void*)&nch, (void*)&chx, (void*)&chy, (void*)&chc, (void*)&part_stride};
  if (vx) args.push_back((void*)vxa.data());
  if (vy) args.push_back((void*)vya.data());
  {
    double flops = 2.0 * p.M * p.N * p.K;
    double bytes = ((double)p.M * p.K + (double)p.N * p.K + (double)p.M * p.N) * es;
    const char* label = f64 ? "gemm_f64" : "gemm_f32";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[160];
      snprintf(buf, sizeof buf, "%s[M%lldxN%lldxK%lldxB1,footprint,%s%s,chunks%lld,rows%d,kgroups%d,lds%dK,waves%d%s%s]", label, (long long)p.M, (long long)p.N,
               (long long)p.K, pl.mode == 0 ? "chunkK" : "chunkM", best_swapped ? ",swapped" : "", (long long)pl.nch, pl.min_rows, (int)pl.gx.size(), lds_bytes(pl) / 1024,
               4 * pl.ks, vx ? ",xmap" : "", vy ? ",ymap" : "");
      label = intern_label(ctx, buf);
    }
    {
      LaunchGuard lg(ctx, label, bytes, flops);
      hipError_t e = launch_module(lg, kernel.fn, (unsigned)grid, 256u * (unsigned)pl.ks, args.data());
      if (e != hipSuccess) { if (part) buffer_release(part); if (colsum) hgpu_release(colsum); return check_hip(ctx, e, "footprint gemm launch"); }
    }
    if (pl.mode == 0) {
      int rc = colsum ? sum_partials_split(ctx, dtype, out_n, n_colsum, (int)grid, (const void*)part->ptr, data_ptr(out), data_ptr(colsum))
                      : sum_partials(ctx, dtype, out_n, (int)grid, (const void*)part->ptr, data_ptr(out));
      buffer_release(part);
      if (rc) { if (colsum) hgpu_release(colsum); return rc; }
      if (colsum) remember_sum(ctx, *vy, colsum_dims, colsum);
    }
  }
  *handled = true;
  return HGPU_OK;
}

}  // namespace hg

// ---------------------------------------------------------------------------
// hgpu_contract_map: a contraction, an elementwise program over its result and
// an extremum over windows of that, as one footprint kernel.
//
// The view (the windows) refines the kept dims: every view dim walks ONE kept
// dim with a constant step, and together the view dims of a kept dim count
// through it exactly once (h = 2 h2 + p).  The product's rows are then
// enumerated over the view dims, the reduced ones innermost, so that the four
// accumulator registers of a lane -- four consecutive rows of one column -- hold
// whole windows: the program and the extremum need no data from another lane.
namespace {

using namespace hg::fusedgen;

struct EpiSpec {
  int n_in = 0, c_slot = -1, n_instr = 0;
  const hgpu_fused_instr* prog = nullptr;
  std::vector<int> dt;                 // type of every slot
  std::vector<char> cls;               // per input: 'C' the contraction, 's' one element, 'c' moves with the column only, 'g' general
  std::vector<std::vector<int>> in_row, in_col;   // per input: offsets of every inner row / column
  std::vector<int64_t> in_chs;         // per input: chunk stride
  std::vector<int> out_slots;
  bool has_ext = false, want_max = true;
  int ext_slot = 0, L = 1;             // window = L consecutive rows
  std::vector<int> win_row, win_col;   // offsets of every window / column in values and indices
  int64_t win_chs = 0, out_chs = 0;
  // Staged: a chunk's part of every result is one dense block of memory; the
  // block is put together in LDS and written with 16-byte vectors.
  bool staged = false;
  std::vector<int> out_off;            // per output: byte offset of its block in the stage buffer
  int val_off = 0, idx_off = 0, stage_bytes = 0;
};

static_assert(sizeof(EpiSpec) == 296, "put_epilogue must cover every field of EpiSpec");
void put_epilogue(hg::fusedgen::Key& k, const EpiSpec& e) {
  k.put(e.n_in).put(e.c_slot).put(e.n_instr, e.prog).put(e.dt).put(e.cls).put(e.in_row).put(e.in_col).put(e.in_chs).put(e.out_slots);
  k.put(e.has_ext).put(e.want_max).put(e.ext_slot).put(e.L).put(e.win_row).put(e.win_col).put(e.win_chs).put(e.out_chs);
  k.put(e.staged).put(e.out_off).put(e.val_off).put(e.idx_off).put(e.stage_bytes);
}

std::string epilogue_source(const Plan& pl, const EpiSpec& e) {
  Src s;
  s << kPrelude;
  const int WPL = 4 / e.L;
  for (int i = 0; i < e.n_in; ++i) {
    if (e.cls[(size_t)i] == 'g') s << table("__device__ const", ("kRowI" + std::to_string(i)).c_str(), e.in_row[(size_t)i]);
    if (e.cls[(size_t)i] == 'g' || e.cls[(size_t)i] == 'c') s << table("__device__ const", ("kColI" + std::to_string(i)).c_str(), e.in_col[(size_t)i]);
  }
  if (e.has_ext) s << table("__device__ const", "kWinO", e.win_row) << table("__device__ const", "kColO", e.win_col);
  s << "struct EpiArgs {\n";
  for (int i = 0; i < e.n_in; ++i)
    if (i != e.c_slot) s << "  const " << ctype(e.dt[(size_t)i]) << "* i" << i << ";\n";
  for (size_t o = 0; o < e.out_slots.size(); ++o) s << "  " << ctype(e.dt[(size_t)e.out_slots[o]]) << "* o" << o << ";\n";
  if (e.has_ext) s << "  " << ctype(e.dt[(size_t)e.ext_slot]) << "* ov;\n  i64* oi;\n";
  s << "  int unused;\n};\n";
  s << "struct Hoist {\n";
  for (int i = 0; i < e.n_in; ++i)
    if (e.cls[(size_t)i] == 's' || e.cls[(size_t)i] == 'c') s << "  " << ctype(e.dt[(size_t)i]) << " h" << i << ";\n";
  s << "  int unused;\n};\n";
  s << "__device__ __forceinline__ Hoist epi_hoist(const EpiArgs& ea, int col) {\n  Hoist z;\n  z.unused = 0;\n";
  for (int i = 0; i < e.n_in; ++i) {
    if (e.cls[(size_t)i] == 's') s << "  z.h" << i << " = ea.i" << i << "[0];\n";
    if (e.cls[(size_t)i] == 'c') s << "  z.h" << i << " = ea.i" << i << "[kColI" << i << "[col]];\n";
  }
  s << "  return z;\n}\n";
  // positions of a lane's four rows (outputs of the kept shape, general inputs) and of its windows
  s << "struct EPos {\n  int o[4];\n  int w[" << WPL << "];\n";
  for (int i = 0; i < e.n_in; ++i)
    if (e.cls[(size_t)i] == 'g') s << "  int g" << i << "[4];\n";
  s << "};\n";
  // Two blocks on a CU: the tables epi_pos reads are copied to LDS when the block starts (E_ROWC ... name the copies).
  s << "#if BPC == 2\n__shared__ int sRowC[MIN], sColC[NIN];\n";
  if (e.has_ext) s << "__shared__ int sWinO[MIN / " << e.L << "], sColO[NIN];\n";
  s << "__device__ __forceinline__ void epi_tables_to_lds(int tid) {\n";
  s << "  for (int i = tid; i < MIN; i += NT) sRowC[i] = kRowC[i];\n  if (tid < NIN) sColC[tid] = kColC[tid];\n";
  if (e.has_ext) s << "  for (int i = tid; i < MIN / " << e.L << "; i += NT) sWinO[i] = kWinO[i];\n  if (tid < NIN) sColO[tid] = kColO[tid];\n";
  s << "}\n#define E_ROWC sRowC\n#define E_COLC sColC\n#define E_WINO sWinO\n#define E_COLO sColO\n";
  s << "#else\n#define E_ROWC kRowC\n#define E_COLC kColC\n#define E_WINO kWinO\n#define E_COLO kColO\n#endif\n";
  s << "__device__ __forceinline__ EPos epi_pos(int m0, int col) {\n  EPos p;\n";
  s << "  const int cc = col < NIN ? col : NIN - 1;\n";
  s << "#pragma unroll\n  for (int j = 0; j < 4; ++j) {\n    const int m = m0 + j < MIN ? m0 + j : MIN - 1;\n";
  s << "    p.o[j] = E_ROWC[m] + E_COLC[cc];\n";
  for (int i = 0; i < e.n_in; ++i)
    if (e.cls[(size_t)i] == 'g') s << "    p.g" << i << "[j] = kRowI" << i << "[m] + kColI" << i << "[cc];\n";
  s << "  }\n";
  s << "#pragma unroll\n  for (int w = 0; w < " << WPL << "; ++w) {\n";
  if (e.has_ext) s << "    const int wi = m0 / " << e.L << " + w;\n    p.w[w] = E_WINO[wi < MIN / " << e.L << " ? wi : MIN / " << e.L << " - 1] + E_COLO[cc];\n";
  else s << "    p.w[w] = 0;\n";
  s << "  }\n  return p;\n}\n";
  s << "__device__ __forceinline__ void epi_tile(const EpiArgs& ea, const Hoist& hz, const EPos& ep, unsigned char* stage, i64 ch, int m0, int col, T c0, T c1, T c2, T c3) {\n";
  s << "  if (col >= NIN || m0 >= MIN) return;\n";
  s << "  const T cv[4] = {c0, c1, c2, c3};\n";
  if (e.has_ext) s << "  " << ctype(e.dt[(size_t)e.ext_slot]) << " ev[4];\n";
  for (int j = 0; j < 4; ++j) {
    std::string suf = "_" + std::to_string(j);
    s << "  {\n";
    for (int i = 0; i < e.n_in; ++i) {
      s << "    const " << ctype(e.dt[(size_t)i]) << " v" << i << suf << " = ";
      switch (e.cls[(size_t)i]) {
        case 'C': s << "cv[" << j << "]"; break;
        case 's': case 'c': s << "hz.h" << i; break;
        default: s << "ea.i" << i << "[ch * " << e.in_chs[(size_t)i] << "ll + ep.g" << i << "[" << j << "]]"; break;
      }
      s << ";\n";
    }
    emit_program(s, e.n_in, e.n_instr, e.prog, e.dt, "    ", suf);
    for (size_t o = 0; o < e.out_slots.size(); ++o) {
      if (e.staged) s << "    reinterpret_cast<" << ctype(e.dt[(size_t)e.out_slots[o]]) << "*>(stage + " << e.out_off[o] << ")[ep.o[" << j << "]] = v" << e.out_slots[o] << suf << ";\n";
      else s << "    ea.o" << o << "[ch * " << e.out_chs << "ll + ep.o[" << j << "]] = v" << e.out_slots[o] << suf << ";\n";
    }
    if (e.has_ext) s << "    ev[" << j << "] = v" << e.ext_slot << suf << ";\n";
    s << "  }\n";
  }
  if (e.has_ext) {
    for (int w = 0; w < WPL; ++w) {
      s << "  {\n    " << ctype(e.dt[(size_t)e.ext_slot]) << " best = ev[" << w * e.L << "];\n    i64 bi = 0;\n";
      for (int u = 1; u < e.L; ++u)
        s << "    if (ev[" << w * e.L + u << "] " << (e.want_max ? ">" : "<") << " best) { best = ev[" << w * e.L + u << "]; bi = " << u << "; }\n";
      if (e.staged) {
        s << "    reinterpret_cast<" << ctype(e.dt[(size_t)e.ext_slot]) << "*>(stage + " << e.val_off << ")[ep.w[" << w << "]] = best;\n";
        s << "    (stage + " << e.idx_off << ")[ep.w[" << w << "]] = (unsigned char)bi;\n  }\n";
      } else {
        s << "    const i64 at = ch * " << e.win_chs << "ll + ep.w[" << w << "];\n    ea.ov[at] = best;\n    ea.oi[at] = bi;\n  }\n";
      }
    }
  }
  s << "}\n";
  if (e.staged) {
    // every block of the stage buffer to its place in memory, 16 bytes per lane and step
    s << "struct alignas(16) V16 { unsigned int w[4]; };\n";
    s << "__device__ __forceinline__ void epi_flush(const EpiArgs& ea, const unsigned char* stage, i64 ch, int tid) {\n";
    auto block = [&](const std::string& ptr, const char* ct, int64_t chs, int off, int64_t elems, size_t es) {
      const int64_t nv = elems * (int64_t)es / 16;
      s << "  {\n    V16* dst = reinterpret_cast<V16*>(" << ptr << " + ch * " << chs << "ll);\n";
      s << "    const V16* src = reinterpret_cast<const V16*>(stage + " << off << ");\n";
      s << "#pragma unroll 4\n    for (int v = tid; v < " << nv << "; v += NT) dst[v] = src[v];\n  }\n";
      (void)ct;
    };
    const int64_t n_el = (int64_t)pl.min_rows * pl.nin;
    for (size_t o = 0; o < e.out_slots.size(); ++o) block("ea.o" + std::to_string(o), ctype(e.dt[(size_t)e.out_slots[o]]), e.out_chs, e.out_off[o], n_el, dtype_size(e.dt[(size_t)e.out_slots[o]]));
    if (e.has_ext) {
      block("ea.ov", ctype(e.dt[(size_t)e.ext_slot]), e.win_chs, e.val_off, n_el / e.L, dtype_size(e.dt[(size_t)e.ext_slot]));
      // the places within the windows wait in LDS as bytes and are widened on their way out, two per lane and step
      s << "  {\n    V16* dst = reinterpret_cast<V16*>(ea.oi + ch * " << e.win_chs << "ll);\n";
      s << "    const unsigned char* src = stage + " << e.idx_off << ";\n";
      s << "#pragma unroll 4\n    for (int v = tid; v < " << n_el / e.L / 2 << "; v += NT) dst[v] = V16{{src[2 * v], 0u, src[2 * v + 1], 0u}};\n  }\n";
    }
    s << "}\n";
  }
  (void)pl;
  return s.str();
}

// offsets of every flat index over dims with the given strides (row-major, last dim fastest)
std::vector<int> offsets_of(const std::vector<int64_t>& ext, const std::vector<int64_t>& st, bool* fits) {
  int64_t n = 1;
  for (auto e : ext) n *= e;
  std::vector<int> out((size_t)n, 0);
  for (int64_t i = 0; i < n; ++i) {
    int64_t r = i, o = 0;
    for (int k = (int)ext.size() - 1; k >= 0; --k) { o += (r % ext[(size_t)k]) * st[(size_t)k]; r /= ext[(size_t)k]; }
    if (o < 0 || o > INT32_MAX) *fits = false;
    out[(size_t)i] = (int)o;
  }
  return out;
}

struct ViewDim { int64_t e; int kd; int64_t coef; };

// Every view dim as a constant step along one kept dim; the view dims of a kept
// dim must count through it exactly once.
bool refine_view(int n_keep, const int64_t* kshape, int view_rank, const int64_t* vshape, const int64_t* vstrides, std::vector<ViewDim>* out) {
  int64_t D[HGPU_MAX_RANK];
  dense_strides(n_keep, kshape, D);
  int64_t nk = 1, nv = 1;
  for (int k = 0; k < n_keep; ++k) nk *= kshape[k];
  for (int j = 0; j < view_rank; ++j) nv *= vshape[j];
  if (nk != nv || nk == 0) return false;
  out->clear();
  for (int j = 0; j < view_rank; ++j) {
    ViewDim v{vshape[j], -1, 0};
    if (v.e > 1) {
      if (vstrides[j] <= 0) return false;
      for (int k = 0; k < n_keep; ++k)
        if (kshape[k] > 1 && D[k] <= vstrides[j] && (v.kd < 0 || D[k] > D[v.kd])) v.kd = k;
      if (v.kd < 0 || vstrides[j] % D[v.kd] != 0) return false;
      v.coef = vstrides[j] / D[v.kd];
    }
    out->push_back(v);
  }
  for (int k = 0; k < n_keep; ++k) {
    if (kshape[k] <= 1) continue;
    std::vector<std::pair<int64_t, int64_t>> digits;   // (step, extent)
    for (auto& v : *out)
      if (v.kd == k) digits.push_back({v.coef, v.e});
    std::sort(digits.begin(), digits.end());
    int64_t reach = 1;
    for (auto& d : digits) {
      if (d.first != reach) return false;
      reach *= d.second;
    }
    if (reach != kshape[k]) return false;
  }
  return true;
}

int try_contract_map(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, int n_in, const hgpu_array* const* in, int c_slot, int n_instr,
                     const hgpu_fused_instr* prog, const std::vector<int>& dt, int n_out, const int* out_slots, hgpu_array** outs, int ext_slot, int view_rank,
                     const int64_t* view_shape, const int64_t* view_strides, int n_reduce, int want_max, hgpu_array** values, hgpu_array** indices, bool* handled) {
  *handled = false;
  if (a->dtype != HGPU_F64 && a->dtype != HGPU_F32) return HGPU_OK;
  const bool f64 = a->dtype == HGPU_F64;
  const int es = f64 ? 8 : 4;
  const bool has_ext = values != nullptr;
  // without windows the "view" is the kept shape itself
  int64_t dshape[HGPU_MAX_RANK], dstrides[HGPU_MAX_RANK];
  if (!has_ext) {
    view_rank = n_keep;
    for (int k = 0; k < n_keep; ++k) dshape[k] = a->shape[k];
    dense_strides(n_keep, dshape, dstrides);
    view_shape = dshape;
    view_strides = dstrides;
    n_reduce = 0;
  }
  std::vector<ViewDim> vd;
  if (!refine_view(n_keep, a->shape, view_rank, view_shape, view_strides, &vd)) return HGPU_OK;
  int64_t L = 1;
  for (int j = view_rank - n_reduce; j < view_rank; ++j) L *= view_shape[j];
  if (L != 1 && L != 2 && L != 4) return HGPU_OK;
  // strides of the operands and outputs along every view dim
  struct VS { int64_t e, sa, sb, sc, so; bool red; std::vector<int64_t> sin; };
  std::vector<VS> dims;
  {
    int64_t lead[HGPU_MAX_RANK], lst[HGPU_MAX_RANK];
    const int rl = view_rank - n_reduce;
    for (int j = 0; j < rl; ++j) lead[j] = view_shape[j];
    dense_strides(rl, lead, lst);
    for (int j = 0; j < view_rank; ++j) {
      if (vd[(size_t)j].e <= 1) continue;
      const int k = vd[(size_t)j].kd;
      const int64_t c = vd[(size_t)j].coef;
      VS v{vd[(size_t)j].e, c * a->strides[k], c * b->strides[k], view_strides[j], j < rl ? lst[j] : 0, j >= rl, {}};
      for (int i = 0; i < n_in; ++i) v.sin.push_back(i == c_slot ? 0 : c * in[i]->strides[k]);
      dims.push_back(v);
    }
  }
  // rows: the side the reduced dims are on (else the larger side); columns: the other one, at most 16
  int side_of_red = -1;   // 0: a, 1: b
  int64_t Ma = 1, Nb = 1;
  for (auto& v : dims) {
    const bool ma = v.sa != 0 && v.sb == 0, nb = v.sa == 0 && v.sb != 0;
    if (!ma && !nb) return HGPU_OK;   // a batch dim, or a dim neither operand moves along
    if (ma) Ma *= v.e; else Nb *= v.e;
    if (v.red) {
      int sd = ma ? 0 : 1;
      if (side_of_red >= 0 && side_of_red != sd) return HGPU_OK;
      side_of_red = sd;
    }
  }
  const bool swapped = side_of_red >= 0 ? side_of_red == 1 : Nb > Ma;   // rows operand is b
  if ((swapped ? Ma : Nb) > 16) return HGPU_OK;
  std::vector<Dim> rows, cols, kd;
  std::vector<size_t> row_ix, col_ix;   // indices into dims, in the order of rows / cols
  {
    std::vector<size_t> plain, red;
    for (size_t i = 0; i < dims.size(); ++i) {
      const bool on_a = dims[i].sa != 0;
      if (on_a == !swapped) (dims[i].red ? red : plain).push_back(i);
      else col_ix.push_back(i);
    }
    auto mag = [](int64_t v) { return v < 0 ? -v : v; };
    std::stable_sort(plain.begin(), plain.end(), [&](size_t x, size_t y) { return mag(swapped ? dims[x].sb : dims[x].sa) > mag(swapped ? dims[y].sb : dims[y].sa); });
    row_ix = plain;
    row_ix.insert(row_ix.end(), red.begin(), red.end());
    for (size_t i : row_ix) rows.push_back(Dim{dims[i].e, swapped ? dims[i].sb : dims[i].sa, 0, dims[i].sc});
    for (size_t i : col_ix) cols.push_back(Dim{dims[i].e, 0, swapped ? dims[i].sa : dims[i].sb, dims[i].sc});
  }
  double K = 1;
  for (int i = n_keep; i < a->rank; ++i) {
    if (a->shape[i] == 1) continue;
    if (a->strides[i] == 0 || b->strides[i] == 0) return HGPU_OK;
    kd.push_back(Dim{a->shape[i], swapped ? b->strides[i] : a->strides[i], swapped ? a->strides[i] : b->strides[i], 0});
    K *= (double)a->shape[i];
  }
  if (kd.empty() || cols.empty() || rows.empty()) return HGPU_OK;
  if ((double)Ma * (double)Nb * K < 1.0e7) return HGPU_OK;
  const char* pa = (const char*)data_ptr(a);
  const char* pb = (const char*)data_ptr(b);
  Plan pl;
  size_t chunk = 0;
  bool found = false;
  for (size_t ci = 0; ci < rows.size() && !found; ++ci) {
    if (rows[ci].e < 64 || dims[row_ix[ci]].red) continue;
    Plan p2;
    if (!make_plan(f64, rows, cols, kd, false, ci, ctx->num_cu, &p2)) continue;
    if (p2.min_rows % 4 != 0) continue;
    const char* xp = (swapped ? pb : pa) + p2.shift_x * es;
    const char* yp = (swapped ? pa : pb) + p2.shift_y * es;
    if (!finish_plan(p2, xp, yp, nullptr, 0, 0)) continue;
    pl = p2;
    chunk = ci;
    found = true;
  }
  if (!found) return HGPU_OK;

  // ---- the epilogue's tables
  EpiSpec e;
  e.n_in = n_in;
  e.c_slot = c_slot;
  e.n_instr = n_instr;
  e.prog = prog;
  e.dt = dt;
  e.out_slots.assign(out_slots, out_slots + n_out);
  e.has_ext = has_ext;
  e.want_max = want_max != 0;
  e.ext_slot = ext_slot;
  e.L = (int)L;
  bool fits = true;
  std::vector<int64_t> rext, cext;
  for (size_t i = 0; i < row_ix.size(); ++i)
    if (i != chunk) rext.push_back(dims[row_ix[i]].e);
  for (size_t i : col_ix) cext.push_back(dims[i].e);
  auto row_strides = [&](auto get) { std::vector<int64_t> st; for (size_t i = 0; i < row_ix.size(); ++i) if (i != chunk) st.push_back(get(dims[row_ix[i]])); return st; };
  auto col_strides = [&](auto get) { std::vector<int64_t> st; for (size_t i : col_ix) st.push_back(get(dims[i])); return st; };
  e.out_chs = dims[row_ix[chunk]].sc;
  e.win_chs = dims[row_ix[chunk]].so;
  e.cls.assign((size_t)n_in, 'g');
  e.in_row.resize((size_t)n_in);
  e.in_col.resize((size_t)n_in);
  e.in_chs.assign((size_t)n_in, 0);
  for (int i = 0; i < n_in; ++i) {
    if (i == c_slot) { e.cls[(size_t)i] = 'C'; continue; }
    bool any = false, any_row = false;
    for (size_t d = 0; d < dims.size(); ++d) any = any || dims[d].sin[(size_t)i] != 0;
    for (size_t q = 0; q < row_ix.size(); ++q) any_row = any_row || dims[row_ix[q]].sin[(size_t)i] != 0;
    if (!any) { e.cls[(size_t)i] = 's'; continue; }
    e.in_col[(size_t)i] = offsets_of(cext, col_strides([&](const VS& v) { return v.sin[(size_t)i]; }), &fits);
    if (!any_row) { e.cls[(size_t)i] = 'c'; continue; }
    e.in_row[(size_t)i] = offsets_of(rext, row_strides([&](const VS& v) { return v.sin[(size_t)i]; }), &fits);
    e.in_chs[(size_t)i] = dims[row_ix[chunk]].sin[(size_t)i];
  }
  if (has_ext) {
    // windows: the rows without the reduced dims
    std::vector<int64_t> wext, wst;
    for (size_t i = 0; i < row_ix.size(); ++i)
      if (i != chunk && !dims[row_ix[i]].red) { wext.push_back(dims[row_ix[i]].e); wst.push_back(dims[row_ix[i]].so); }
    e.win_row = offsets_of(wext, wst, &fits);
    e.win_col = offsets_of(cext, col_strides([&](const VS& v) { return v.so; }), &fits);
    if ((int64_t)e.win_row.size() * L != pl.min_rows) return HGPU_OK;
  }
  if (!fits) return HGPU_OK;
  // A chunk's share of every result one dense block (the offsets of its rows
  // and columns count through 0 .. n-1), blocks and chunk strides whole 16-byte
  // vectors: the blocks are put together in LDS.
  {
    auto dense_block = [](const std::vector<int>& rowo, const std::vector<int>& colo) {
      const size_t n = rowo.size() * colo.size();
      std::vector<char> hit(n, 0);
      for (int r0 : rowo)
        for (int c0 : colo) {
          const int64_t o = (int64_t)r0 + c0;
          if (o < 0 || o >= (int64_t)n || hit[(size_t)o]) return false;
          hit[(size_t)o] = 1;
        }
      return true;
    };
    bool ok = n_out == 0 || dense_block(pl.row_c, pl.col_c);
    if (has_ext) ok = ok && dense_block(e.win_row, e.win_col);
    const int64_t n_el = (int64_t)pl.min_rows * pl.nin;
    int off = 0;
    auto place = [&](int64_t elems, size_t esz, int64_t chs) {
      if ((elems * (int64_t)esz) % 16 != 0 || (chs * (int64_t)esz) % 16 != 0) ok = false;
      int at = off;
      off += (int)((elems * (int64_t)esz + 15) / 16 * 16);
      return at;
    };
    for (int o = 0; o < n_out; ++o) e.out_off.push_back(place(n_el, dtype_size(dt[(size_t)out_slots[o]]), e.out_chs));
    if (has_ext) {
      e.val_off = place(n_el / L, dtype_size(dt[(size_t)ext_slot]), e.win_chs);
      if ((n_el / L) % 2 != 0 || (e.win_chs * 8) % 16 != 0) ok = false;
      e.idx_off = place(n_el / L, 1, 16);     // one byte per window in LDS, 8 in memory
    }
    e.stage_bytes = off;
    Plan p3 = pl;
    const char* xp3 = (swapped ? pb : pa) + pl.shift_x * es;
    const char* yp3 = (swapped ? pa : pb) + pl.shift_y * es;
    if (ok && off > 0 && finish_plan(p3, xp3, yp3, nullptr, 0, off) && p3.nbufs == pl.nbufs) { e.staged = true; pl = p3; }
    else e.stage_bytes = 0;
  }
  // For measurements (HORDEAD_FOOTPRINT_BPC=2): two blocks to a CU when their LDS fits together.  The first
  // CNN layer (784 rows x 16 x K 25 per chunk) runs 40 us that way against 34 us with one block per CU.
  // Two blocks on a CU where their LDS fits twice (with the copies of the epilogue's tables) and no input of the
  // program is looked up per row: one block's loads, stores and program then run under the other's multiplications.
  // (HORDEAD_FOOTPRINT_BPC=1: one block per CU.)
  static const int bpc_env = getenv("HORDEAD_FOOTPRINT_BPC") ? atoi(getenv("HORDEAD_FOOTPRINT_BPC")) : 0;
  bool rows_looked_up = false;
  for (char c : e.cls) rows_looked_up = rows_looked_up || c == 'g';
  const int64_t tables_lds = 4 * ((int64_t)pl.min_rows + pl.nin + (e.has_ext ? pl.min_rows / e.L + pl.nin : 0));
  pl.bpc = (pl.ks == 1 && e.staged && !rows_looked_up && 2 * (lds_bytes(pl) + e.stage_bytes + tables_lds + 512) <= 160 * 1024 &&
            pl.nch >= 3 * (int64_t)ctx->num_cu && bpc_env != 1) ? 2 : 1;

  // ---- results
  std::vector<hgpu_array*> res((size_t)n_out, nullptr);
  hgpu_array *v = nullptr, *ix = nullptr;
  auto release_all = [&] { for (auto* r : res) if (r) hgpu_release(r); if (v) hgpu_release(v); if (ix) hgpu_release(ix); };
  for (int o = 0; o < n_out; ++o) {
    int rc = new_dense(ctx, dt[(size_t)out_slots[o]], n_keep, a->shape, &res[(size_t)o]);
    if (rc) { release_all(); return rc; }
  }
  if (has_ext) {
    int rc = new_dense(ctx, dt[(size_t)ext_slot], view_rank - n_reduce, view_shape, &v);
    if (!rc) rc = new_dense(ctx, HGPU_I64, view_rank - n_reduce, view_shape, &ix);
    if (rc) { release_all(); return rc; }
  }

  char kname[160];
  snprintf(kname, sizeof kname, "footprint_gemm_%s_m%lld_n%lld_k%lld_chunkM%s_map%d%s%s", f64 ? "f64" : "f32", (long long)(swapped ? Nb : Ma), (long long)(swapped ? Ma : Nb),
           (long long)K, swapped ? "_swapped" : "", n_instr, has_ext ? (want_max ? "_max" : "_min") : "", pl.ks == 2 ? "_w8" : "");
  Compiled kernel{nullptr, nullptr};
  {
    Key key;
    key.put(std::string(kname));
    put_plan(key, pl);
    put_epilogue(key, e);
    int rc = known_kernel(ctx, key, kname, [&] { return generate(pl, kname, epilogue_source(pl, e), e.staged ? e.stage_bytes : 0); }, &kernel);
    if (rc) { release_all(); return rc; }
  }
  if (!kernel.fn) { release_all(); return HGPU_OK; }

  // kernel arguments: the footprint kernel's own, then the EpiArgs struct (pointers in declaration order)
  const char* xp = (swapped ? pb : pa) + pl.shift_x * es;
  const char* yp = (swapped ? pa : pb) + pl.shift_y * es;
  void* cnull = nullptr;
  int64_t nch = pl.nch, chx = pl.chx, chy = pl.chy, chc = 0, part_stride = 0;
  std::vector<const void*> ea;
  for (int i = 0; i < n_in; ++i)
    if (i != c_slot) ea.push_back(data_ptr(in[i]));
  for (int o = 0; o < n_out; ++o) ea.push_back(data_ptr(res[(size_t)o]));
  if (has_ext) { ea.push_back(data_ptr(v)); ea.push_back(data_ptr(ix)); }
  ea.push_back(nullptr);   // the int at the end, padded to a pointer
  void* args[] = {(void*)&xp, (void*)&yp, (void*)&cnull, (void*)&nch, (void*)&chx, (void*)&chy, (void*)&chc, (void*)&part_stride, (void*)ea.data()};
  int64_t grid = std::min<int64_t>(pl.nch, (int64_t)ctx->num_cu * pl.bpc);
  {
    const double M = (double)(swapped ? Nb : Ma), N = (double)(swapped ? Ma : Nb);
    double flops = 2.0 * M * N * K;
    double bytes = (M * K + N * K) * es;   // as for the plain product: operands once ...
    for (int o = 0; o < n_out; ++o) bytes += M * N * (double)dtype_size(res[(size_t)o]->dtype);   // ... and what is written
    if (has_ext) bytes += M * N / (double)L * (dtype_size(v->dtype) + 8.0);
    const char* label = f64 ? "gemm_f64" : "gemm_f32";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[200];
      snprintf(buf, sizeof buf, "%s[M%lldxN%lldxK%lldxB1,footprint,chunkM%s,chunks%lld,rows%d,kgroups%d,lds%dK,waves%d,map(instr%d,out%d%s)]", label, (long long)M, (long long)N,
               (long long)K, swapped ? ",swapped" : "", (long long)pl.nch, pl.min_rows, (int)pl.gx.size(), lds_bytes(pl) / 1024, 4 * pl.ks, n_instr, n_out,
               has_ext ? (L == 4 ? ",ext4" : (L == 2 ? ",ext2" : ",ext1")) : "");
      label = intern_label(ctx, buf);
    }
    LaunchGuard lg(ctx, label, bytes, flops);
    hipError_t err = launch_module(lg, kernel.fn, (unsigned)grid, 256u * (unsigned)pl.ks, args);
    if (err != hipSuccess) { release_all(); return check_hip(ctx, err, "contract_map launch"); }
  }
  for (int o = 0; o < n_out; ++o) outs[o] = res[(size_t)o];
  if (has_ext) { *values = v; *indices = ix; }
  *handled = true;
  return HGPU_OK;
}

}  // namespace

extern "C" int hgpu_contract_map(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, int n_in, const hgpu_array* const* in, int n_instr,
                                 const hgpu_fused_instr* prog, int n_out, const int* out_slots, hgpu_array** outs, int ext_slot, int view_rank,
                                 const int64_t* view_shape, const int64_t* view_strides, int n_reduce, int want_max, hgpu_array** values, hgpu_array** indices) {
  if (!ctx || !a || !b || !in || (n_instr > 0 && !prog) || (n_out > 0 && (!out_slots || !outs))) return HGPU_ERR_INVALID;
  if ((values == nullptr) != (indices == nullptr)) return HGPU_ERR_INVALID;
  if (n_keep < 1 || n_keep > a->rank) return fail(ctx, HGPU_ERR_INVALID, "contract_map: n_keep %d of rank %d", n_keep, a->rank);
  if (b->dtype != a->dtype || !same_shape(a, b)) return fail(ctx, HGPU_ERR_INVALID, "contract_map: operands differ in dtype or shape");
  if (n_in < 1 || n_in > 12 || n_instr < 0 || n_instr > 96 || n_out < 0 || n_out > 6) return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract_map: %d inputs, %d instructions, %d outputs", n_in, n_instr, n_out);
  int c_slot = -1;
  for (int i = 0; i < n_in; ++i) {
    if (!in[i]) {
      if (c_slot >= 0) return fail(ctx, HGPU_ERR_INVALID, "contract_map: more than one input stands for the contraction");
      c_slot = i;
      continue;
    }
    bool ok = in[i]->rank == n_keep;
    for (int d = 0; d < n_keep && ok; ++d) ok = in[i]->shape[d] == a->shape[d];
    if (!ok) return fail(ctx, HGPU_ERR_INVALID, "contract_map: input %d does not have the kept shape", i);
  }
  if (c_slot < 0) return fail(ctx, HGPU_ERR_INVALID, "contract_map: no input stands for the contraction");
  // slot types: the contraction's slot has the operands' dtype
  std::vector<int> dt;
  {
    std::vector<const hgpu_array*> tin(in, in + n_in);
    tin[(size_t)c_slot] = a;   // only the dtype is read
    if (int rc = check_program(ctx, n_in, tin.data(), n_instr, prog, &dt)) return rc;
  }
  for (int o = 0; o < n_out; ++o)
    if (out_slots[o] < 0 || out_slots[o] >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "contract_map: bad output slot");
  int64_t n_kept = 1;
  for (int d = 0; d < n_keep; ++d) n_kept *= a->shape[d];
  if (values) {
    if (ext_slot < 0 || ext_slot >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "contract_map: bad extremum slot");
    if (view_rank < 1 || view_rank > HGPU_MAX_RANK || !view_shape || !view_strides || n_reduce < 1 || n_reduce > view_rank)
      return fail(ctx, HGPU_ERR_INVALID, "contract_map: bad view");
    int64_t hi = 0;
    for (int j = 0; j < view_rank; ++j) {
      if (view_shape[j] < 1 || view_strides[j] < 0) return fail(ctx, HGPU_ERR_INVALID, "contract_map: the view must have positive extents and no negative strides");
      hi += (view_shape[j] - 1) * view_strides[j];
    }
    if (hi >= n_kept) return fail(ctx, HGPU_ERR_INVALID, "contract_map: the view leaves the result");
  }
  if (n_kept > 0) {
    bool handled = false;
    int rc = try_contract_map(ctx, a, b, n_keep, n_in, in, c_slot, n_instr, prog, dt, n_out, out_slots, outs, ext_slot, view_rank, view_shape, view_strides, n_reduce,
                              want_max, values, indices, &handled);
    if (rc || handled) return rc;
  }
  // one entry point after another
  hgpu_array* c = nullptr;
  int rc = hgpu_contract(ctx, a, b, n_keep, &c);
  if (rc) return rc;
  std::vector<const hgpu_array*> ins(in, in + n_in);
  ins[(size_t)c_slot] = c;
  std::vector<int> slots(out_slots, out_slots + n_out);
  if (values) slots.push_back(ext_slot);
  std::vector<hgpu_array*> res(slots.size(), nullptr);
  auto release_res = [&] { for (auto*& r : res) if (r) { hgpu_release(r); r = nullptr; } };
  // slots that are inputs are copied, the others come out of one fused pass
  std::vector<int> fslots;
  std::vector<size_t> fpos;
  for (size_t i = 0; i < slots.size() && !rc; ++i) {
    if (slots[i] < n_in) rc = hgpu_materialize(ctx, ins[(size_t)slots[i]], &res[i]);
    else { fslots.push_back(slots[i]); fpos.push_back(i); }
  }
  if (!rc && !fslots.empty()) {
    std::vector<hgpu_array*> fres(fslots.size(), nullptr);
    rc = hgpu_fused_map(ctx, n_in, ins.data(), n_instr, prog, (int)fslots.size(), fslots.data(), fres.data());
    if (!rc) for (size_t i = 0; i < fpos.size(); ++i) res[fpos[i]] = fres[i];
  }
  hgpu_release(c);
  if (rc) { release_res(); return rc; }
  if (values) {
    hgpu_array *vw = nullptr, *flat = nullptr;
    rc = hgpu_as_strided(ctx, res.back(), view_rank, view_shape, view_strides, 0, &vw);
    if (!rc) {
      int64_t sh[HGPU_MAX_RANK];
      const int rl = view_rank - n_reduce;
      int64_t L = 1;
      for (int j = 0; j < rl; ++j) sh[j] = view_shape[j];
      for (int j = rl; j < view_rank; ++j) L *= view_shape[j];
      sh[rl] = L;
      rc = hgpu_reshape(ctx, vw, rl + 1, sh, &flat);
      hgpu_release(vw);
    }
    if (!rc) {
      rc = hgpu_extremum_last(ctx, flat, want_max, values, indices);
      hgpu_release(flat);
    }
    hgpu_release(res.back());
    res.back() = nullptr;
    if (rc) { release_res(); return rc; }
  }
  for (int o = 0; o < n_out; ++o) outs[o] = res[(size_t)o];
  return HGPU_OK;
}

// ---------------------------------------------------------------------------
// hgpu_contract_operands: contractions whose operands may be unevaluated
// elementwise expressions (see VirtualOp).
namespace {

// Checks the description of an expression operand and fills in v.
int virtual_from_operand(hgpu_ctx* ctx, const hgpu_operand* o, VirtualOp* v) {
  if (o->n_in < 1 || o->n_in > 12 || o->n_instr < 0 || o->n_instr > 96 || !o->in || (o->n_instr > 0 && !o->prog))
    return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract_operands: %d inputs, %d instructions", o->n_in, o->n_instr);
  for (int i = 0; i < o->n_in; ++i) {
    if (!o->in[i]) return HGPU_ERR_INVALID;
    if (!same_shape(o->in[i], o->in[0])) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: input %d has another shape", i);
  }
  if (int rc = hg::fusedgen::check_program(ctx, o->n_in, o->in, o->n_instr, o->prog, &v->dt)) return rc;
  if (o->slot < 0 || o->slot >= o->n_in + o->n_instr) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: bad slot");
  if (o->rank_m < 0 || o->rank_m > HGPU_MAX_RANK || o->rank < 0 || o->rank > HGPU_MAX_RANK || (o->rank_m > 0 && !o->mshape) || (o->rank > 0 && (!o->shape || !o->strides)))
    return fail(ctx, HGPU_ERR_INVALID, "contract_operands: bad ranks");
  if ((o->lo == nullptr) != (o->hi == nullptr)) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: lo and hi go together");
  v->n_in = o->n_in;
  v->in = o->in;
  v->n_instr = o->n_instr;
  v->prog = o->prog;
  v->slot = o->slot;
  v->dtype = v->dt[(size_t)o->slot];
  v->E.assign(o->in[0]->shape, o->in[0]->shape + o->in[0]->rank);
  int64_t ne = 1, nm = 1;
  for (auto e : v->E) ne *= e;
  v->total = 1;
  v->padded = false;
  for (int k = 0; k < o->rank_m; ++k) {
    const int64_t lo = o->lo ? o->lo[k] : 0, hi = o->hi ? o->hi[k] : 0;
    if (o->mshape[k] < 0 || lo < 0 || hi < 0) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: negative extent");
    v->M.push_back(o->mshape[k]);
    v->lo.push_back(lo);
    v->hi.push_back(hi);
    v->P.push_back(o->mshape[k] + lo + hi);
    nm *= o->mshape[k];
    v->total *= v->P.back();
    v->padded = v->padded || lo != 0 || hi != 0;
  }
  if (ne != nm) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: %lld elements seen as %lld", (long long)ne, (long long)nm);
  // the view must stay inside the extended layout
  int64_t lo = o->offset, hi = o->offset;
  bool empty = false;
  for (int d = 0; d < o->rank; ++d) {
    if (o->shape[d] < 0) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: negative extent");
    if (o->shape[d] == 0) { empty = true; continue; }
    const int64_t span = (o->shape[d] - 1) * o->strides[d];
    if (span > 0) hi += span; else lo += span;
  }
  if (!empty && (lo < 0 || hi >= v->total)) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: the view leaves the layout");
  return HGPU_OK;
}

// The operand as an array: program, merged dims, zero-extension, view.
int write_out(hgpu_ctx* ctx, const hgpu_operand* o, hgpu_array** out) {
  if (o->array) { hgpu_retain(const_cast<hgpu_array*>(o->array)); *out = const_cast<hgpu_array*>(o->array); return HGPU_OK; }
  hgpu_array *e = nullptr, *m = nullptr, *p = nullptr;
  int rc;
  if (o->slot < o->n_in) rc = hgpu_materialize(ctx, o->in[o->slot], &e);
  else rc = hgpu_fused_map(ctx, o->n_in, o->in, o->n_instr, o->prog, 1, &o->slot, &e);
  if (rc) return rc;
  rc = hgpu_reshape(ctx, e, o->rank_m, o->mshape, &m);
  hgpu_release(e);
  if (rc) return rc;
  if (o->lo) {
    rc = hgpu_pad(ctx, m, o->lo, o->hi, &p);
    hgpu_release(m);
    if (rc) return rc;
  } else {
    p = m;
  }
  rc = hgpu_as_strided(ctx, p, o->rank, o->shape, o->strides, o->offset, out);
  hgpu_release(p);
  return rc;
}

// ---- sums that another kernel has made on its way ---------------------------
// The sum of an expression over all merged dims but a few (a bias's cotangent:
// the layer's cotangent summed over batch, height and width) costs nothing in
// a kernel that evaluates the expression anyway (onehot_contract).  Such a sum
// is remembered under the expression -- program, inputs (held, so that their
// blocks stay theirs), merged shape, the dims kept -- for the caller that asks
// for exactly it next.  Arrays are written once; the two entry points that
// write into existing arrays end everything remembered (hgpu_ctx::write_epoch).
struct MemoSum {
  std::string key;
  hgpu_array* sum;
  std::vector<hgpu_buffer*> held;
  uint64_t epoch;
};
struct MemoSums { std::vector<MemoSum> items; };

MemoSums& memo_of(hgpu_ctx* ctx) {
  auto it = ctx->jit_cache.find("__memo_sums__");
  if (it == ctx->jit_cache.end()) it = ctx->jit_cache.emplace("__memo_sums__", new MemoSums()).first;
  return *static_cast<MemoSums*>(it->second);
}

std::string expression_key(const VirtualOp& v, const std::vector<int>& kept) {
  std::string k;
  auto put = [&](const void* p, size_t n) { k.append((const char*)p, n); };
  put(&v.n_in, sizeof v.n_in);
  put(&v.n_instr, sizeof v.n_instr);
  put(&v.slot, sizeof v.slot);
  if (v.n_instr > 0) put(v.prog, sizeof(hgpu_fused_instr) * (size_t)v.n_instr);
  for (int i = 0; i < v.n_in; ++i) {
    const hgpu_array* a = v.in[i];
    put(&a->buf, sizeof a->buf);
    put(&a->dtype, sizeof a->dtype);
    put(&a->rank, sizeof a->rank);
    put(a->shape, sizeof(int64_t) * (size_t)a->rank);
    put(a->strides, sizeof(int64_t) * (size_t)a->rank);
    put(&a->offset, sizeof a->offset);
  }
  for (int64_t m : v.M) put(&m, sizeof m);
  k += "|";
  for (int d : kept) put(&d, sizeof d);
  return k;
}

void forget(MemoSum& m) {
  hgpu_release(m.sum);
  for (auto* b : m.held) buffer_release(b);
}

// Takes over the caller's reference to `sum`.
void remember_sum(hgpu_ctx* ctx, const VirtualOp& v, const std::vector<int>& kept, hgpu_array* sum) {
  MemoSum m{expression_key(v, kept), sum, {}, 0};
  for (int i = 0; i < v.n_in; ++i)
    if (v.in[i]->buf) { buffer_retain(v.in[i]->buf); m.held.push_back(v.in[i]->buf); }
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  m.epoch = ctx->write_epoch;
  MemoSums& ms = memo_of(ctx);
  for (size_t i = 0; i < ms.items.size();)
    if (ms.items[i].key == m.key || ms.items[i].epoch != m.epoch) { forget(ms.items[i]); ms.items.erase(ms.items.begin() + (long)i); } else ++i;
  if (ms.items.size() >= 2) { forget(ms.items.front()); ms.items.erase(ms.items.begin()); }
  ms.items.push_back(std::move(m));
}

// The remembered sum (a new reference), or nullptr.
hgpu_array* recall_sum(hgpu_ctx* ctx, const VirtualOp& v, const std::vector<int>& kept) {
  const std::string key = expression_key(v, kept);
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  MemoSums& ms = memo_of(ctx);
  for (auto& m : ms.items)
    if (m.epoch == ctx->write_epoch && m.key == key) { hgpu_retain(m.sum); return m.sum; }
  return nullptr;
}

// The merged dims that the first n_keep dims of an operand's view walk whole, in order, when the view as
// a whole walks every merged dim exactly once (no zero-extension, no offset): the sum over the other
// dims of the view is then the sum over all other merged dims.  false: the view is something else.
bool kept_merged_dims(const VirtualOp& v, const hgpu_operand* o, int n_keep, std::vector<int>* kept) {
  if (v.padded || o->offset != 0) return false;
  const size_t rm = v.M.size();
  std::vector<int64_t> DM(rm, 1);
  for (size_t k = rm; k-- > 1;) DM[k - 1] = DM[k] * v.M[k];
  std::vector<char> covered(rm, 0);
  kept->clear();
  for (int d = 0; d < o->rank; ++d) {
    if (o->shape[d] == 1) continue;
    int found = -1;
    for (size_t k = 0; k < rm; ++k)
      if (v.M[k] > 1 && !covered[k] && DM[k] == o->strides[d] && v.M[k] == o->shape[d]) { found = (int)k; break; }
    if (found < 0) return false;
    covered[(size_t)found] = 1;
    if (d < n_keep) kept->push_back(found);
  }
  for (size_t k = 0; k < rm; ++k)
    if (v.M[k] > 1 && !covered[k]) return false;
  return true;
}

// out[o] = sum over the dims behind the first n_keep of the view of an
// expression: blocks take (output, chunk of the summed index range), lanes
// evaluate the expression at their elements, partial sums are added up in a
// fixed order by a second launch.
int try_mapped_sum(hgpu_ctx* ctx, const VirtualOp& v, const hgpu_operand* o, int n_keep, hgpu_array* out, bool* handled) {
  *handled = false;
  if (v.dtype != HGPU_F64 && v.dtype != HGPU_F32) return HGPU_OK;
  if (v.total >= (1LL << 31)) return HGPU_OK;
  const int es = v.dtype == HGPU_F64 ? 8 : 4;
  // dims of the view, each group merged where contiguous
  struct D2 { int64_t e, s; };
  auto merged = [&](int from, int to) {
    std::vector<D2> g;
    for (int d = from; d < to; ++d) {
      if (o->shape[d] == 1) continue;
      if (!g.empty() && g.back().s == o->strides[d] * o->shape[d]) { g.back().e *= o->shape[d]; g.back().s = o->strides[d]; }
      else g.push_back({o->shape[d], o->strides[d]});
    }
    return g;
  };
  std::vector<D2> kd = merged(0, n_keep), rd = merged(n_keep, o->rank);
  int64_t n_out = 1, R = 1;
  for (auto& d : kd) n_out *= d.e;
  for (auto& d : rd) R *= d.e;
  if (n_out > 4096 || R < 16384 || rd.empty()) return HGPU_OK;   // few outputs under long sums: what this kernel is for
  int W = 16 / es;
  {
    bool ok = rd.back().s == 1 && rd.back().e % W == 0 && o->offset % W == 0 && vector_ok(v, W);
    for (size_t i = 0; i + 1 < rd.size(); ++i) ok = ok && rd[i].s % W == 0;
    for (auto& d : kd) ok = ok && d.s % W == 0;
    if (!ok) W = 1;
  }
  int64_t S = ((int64_t)ctx->num_cu * 8 + n_out - 1) / n_out;
  if (S > R / 4096) S = R / 4096;
  if (S < 1) S = 1;
  int64_t CH = ((R + S - 1) / S + W - 1) / W * W;
  S = (R + CH - 1) / CH;
  Src s;
  s << "typedef long long i64;\n";
  s << "typedef " << (es == 8 ? "double" : "float") << " T;\n";
  s << "template <int N> struct VT { typedef T type __attribute__((ext_vector_type(N))); };\ntemplate <> struct VT<1> { typedef T type; };\ntemplate <int N> using Vec = typename VT<N>::type;\n";
  s << hg::fusedgen::kPrelude;
  s << vops_source(v, "x", W, 0);
  s << "extern \"C\" __global__ void __launch_bounds__(256) mapped_sum(VArgs_x vax, T* __restrict__ part) {\n";
  s << "  __shared__ double red[4];\n";
  s << "  const VHoist_x hsx = vhoist_x(vax);\n";
  s << "  const unsigned o = blockIdx.x % " << n_out << "u, sc = blockIdx.x / " << n_out << "u;\n";
  s << "  i64 base = " << o->offset << "ll;\n  {\n    unsigned r = o;\n";
  for (size_t i = kd.size(); i-- > 0;) {
    if (i > 0) s << "    base += (i64)(r % " << kd[i].e << "u) * " << kd[i].s << "ll; r /= " << kd[i].e << "u;\n";
    else s << "    base += (i64)r * " << kd[i].s << "ll;\n";
  }
  s << "  }\n";
  s << "  const i64 r0 = (i64)sc * " << CH << "ll, r1 = r0 + " << CH << "ll < " << R << "ll ? r0 + " << CH << "ll : " << R << "ll;\n";
  s << "  double acc = 0;\n";
  s << "  for (i64 rr = r0 + (i64)threadIdx.x * " << W << "; rr < r1; rr += 256 * " << W << ") {\n";
  s << "    unsigned r = (unsigned)rr;\n    i64 e = base;\n";
  for (size_t i = rd.size(); i-- > 0;) {
    if (i > 0) s << "    e += (i64)(r % " << rd[i].e << "u) * " << rd[i].s << "ll; r /= " << rd[i].e << "u;\n";
    else s << "    e += (i64)r * " << rd[i].s << "ll;\n";
  }
  s << "    const VPre_x pre = vpre_x(e);\n    const Vec<" << W << "> x = vfinish_x(hsx, pre, vfetch_x(vax, pre, 0));\n";
  if (W == 1) s << "    acc += (double)x;\n";
  else for (int k = 0; k < W; ++k) s << "    acc += (double)x[" << k << "];\n";
  s << "  }\n";
  s << "  for (int off = 32; off > 0; off >>= 1) {\n"
       "    unsigned long long u = *reinterpret_cast<unsigned long long*>(&acc);\n"
       "    unsigned lo = __shfl_down((unsigned)(u & 0xffffffffu), off, 64), hi = __shfl_down((unsigned)(u >> 32), off, 64);\n"
       "    unsigned long long w = ((unsigned long long)hi << 32) | lo;\n"
       "    acc += *reinterpret_cast<double*>(&w);\n  }\n";
  s << "  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;\n  __syncthreads();\n";
  s << "  if (threadIdx.x == 0) part[(i64)sc * " << n_out << "ll + o] = (T)((red[0] + red[1]) + (red[2] + red[3]));\n}\n";
  std::string src = s.str();
  auto& cache = cache_of(ctx);
  auto it = cache.find(src);
  if (it == cache.end()) {
    Compiled c{nullptr, nullptr};
    if (compile(ctx, src, "mapped_sum", &c) != HGPU_OK) c = Compiled{nullptr, nullptr};
    it = cache.emplace(src, c).first;
  }
  if (!it->second.fn) return HGPU_OK;
  hgpu_buffer* part = nullptr;
  void* dst = data_ptr(out);
  if (S > 1) {
    int rc = buffer_alloc(ctx, (size_t)(n_out * S) * es, &part);
    if (rc) return rc;
    dst = part->ptr;
  }
  std::vector<const void*> vxa;
  for (int i = 0; i < v.n_in; ++i) vxa.push_back(data_ptr(v.in[i]));
  void* args[] = {(void*)vxa.data(), (void*)&dst};
  {
    double bytes = 0;
    for (int i = 0; i < v.n_in; ++i) {
      int64_t distinct = 1;
      for (int d = 0; d < v.in[i]->rank; ++d)
        if (v.in[i]->strides[d] != 0) distinct *= v.in[i]->shape[d];
      if (distinct > 1) bytes += (double)distinct * dtype_size(v.in[i]->dtype);
    }
    const char* label = "mapped_sum";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[160];
      snprintf(buf, sizeof buf, "mapped_sum[out%lld,R%lld,S%lld,in%d,instr%d,vec%d%s]", (long long)n_out, (long long)R, (long long)S, v.n_in, v.n_instr, W, v.padded ? ",padded" : "");
      label = intern_label(ctx, buf);
    }
    LaunchGuard lg(ctx, label, bytes, (double)n_out * R * (v.n_instr + 1));
    hipError_t e = launch_module(lg, it->second.fn, (unsigned)(n_out * S), 256, args);
    if (e != hipSuccess) { if (part) buffer_release(part); return check_hip(ctx, e, "mapped_sum launch"); }
  }
  if (part) {
    int rc = hg::sum_partials(ctx, v.dtype, n_out, (int)S, part->ptr, data_ptr(out));
    buffer_release(part);
    if (rc) return rc;
  }
  *handled = true;
  return HGPU_OK;
}


// ---------------------------------------------------------------------------
// A contraction with an expression operand that is ONE-HOT along some of the
// contracted dims: the expression is `select (which == where) u 0` (times other
// factors) with `which` counting through those dims -- what the adjoint of
// "gather at kargMax" (max-pooling, External/CommonShapedOps.hs:241-260) puts
// into the cotangent of a convolution: one non-zero per pooling window, at the
// window's argument.  Summing over the one-hot dims then takes ONE term per
// position of the other dims: the expression is evaluated there only, its
// values meet the other operand's rows (a few tens, read from LDS) in the
// vector units, and the dense cotangent -- three quarters structural zeros
// for 2 x 2 windows -- is neither written nor read.
//
// The structure is proved from the program and from what the library knows of
// its input blocks without reading them (hgpu_buffer::known): `which` is a
// view of an index vector, the else-branch a zero constant.

// An instruction slot that can be non-zero only where input `which_in` (a view of an index vector)
// equals input `where_in`.
bool onehot_gate(const VirtualOp& v, int slot, int* which_in, int* where_in) {
  if (slot < v.n_in) return false;
  const hgpu_fused_instr& q = v.prog[slot - v.n_in];
  auto zero_const = [&](int s0) {
    if (s0 >= v.n_in) return false;
    const hgpu_array* a = v.in[s0];
    if (!a->buf || a->buf->known != hgpu_buffer::kZeroScalar) return false;
    for (int d = 0; d < a->rank; ++d)
      if (a->shape[d] != 1 && a->strides[d] != 0) return false;
    return true;
  };
  auto index_vector = [&](int s0) {
    return s0 < v.n_in && v.in[s0]->dtype == HGPU_I64 && v.in[s0]->buf && v.in[s0]->buf->known == hgpu_buffer::kIotaI64;
  };
  switch (q.kind) {
    case HGPU_FUSED_OP2:
      if (q.op == HGPU_MUL) return onehot_gate(v, q.a, which_in, where_in) || onehot_gate(v, q.b, which_in, where_in);
      return false;
    case HGPU_FUSED_OP1:
      return q.op == HGPU_NEG && onehot_gate(v, q.a, which_in, where_in);
    case HGPU_FUSED_SELECT: {
      if (zero_const(q.b)) return onehot_gate(v, q.c, which_in, where_in);      // select c 0 u
      if (!zero_const(q.c)) return false;
      if (q.a >= v.n_in) {                                                       // select (x == y) u 0
        const hgpu_fused_instr& c = v.prog[q.a - v.n_in];
        if (c.kind == HGPU_FUSED_CMP && c.op == HGPU_EQ) {
          for (int sw = 0; sw < 2; ++sw) {
            const int x = sw ? c.b : c.a, y = sw ? c.a : c.b;
            if (index_vector(x) && y < v.n_in && v.in[y]->dtype == HGPU_I64 && !index_vector(y)) { *which_in = x; *where_in = y; return true; }
          }
        }
      }
      return onehot_gate(v, q.b, which_in, where_in);
    }
    default:
      return false;
  }
}

// What a call of the one-hot kernel needs besides its operands: worked out once per kind of call
// (shapes, strides, program), found again by those.
struct OnehotKnown {
  bool taken = false;      // false: the kernel does not take this kind of call
  Compiled c{nullptr, nullptr};
  std::string kname, text; // (the text is kept with HORDEAD_GPU_CHECK_KEYS only)
  int which_in = -1, MR = 0, NC = 0;
  int64_t nch = 0, G = 0, EH = 0, span = 0, lo = 0;
  std::vector<int64_t> colshape;   // the column sums' shape, and the merged dims of the expression they keep
  std::vector<int> colk;
};

// The plan and the kernel's text for x (an array) times the expression v seen through yo; kn->taken stays false when the kernel does not fit.
void plan_onehot(const hgpu_array* x, const VirtualOp& v, const hgpu_operand* yo, int n_keep, int64_t out_n, int which_in, int where_in, OnehotKnown* kn, std::string* text) {
  const int rank = yo->rank;
  const size_t re = v.E.size(), rm = v.M.size();
  // ---- the one-hot dims of the inputs' shape: where `which` moves; `where` must stand still there
  const hgpu_array* wh = v.in[which_in];
  const hgpu_array* wr = v.in[where_in];
  std::vector<char> oh(re, 0);
  std::vector<std::pair<int64_t, size_t>> digits;      // (stride of which, dim)
  for (size_t j = 0; j < re; ++j) {
    if (v.E[j] == 1 || wh->strides[j] == 0) continue;
    if (wh->strides[j] < 0 || wr->strides[j] != 0) return;
    oh[j] = 1;
    digits.push_back({wh->strides[j], j});
  }
  if (digits.empty()) return;
  std::sort(digits.begin(), digits.end());
  int64_t EH = 1;                                        // values `which` takes: which.offset + 0 .. EH - 1, as a mixed-radix number of the one-hot dims
  for (auto& d : digits) {
    if (d.first != EH) return;
    EH *= v.E[d.second];
  }
  if (EH < 2 || EH > 64) return;
  // ---- the inputs' dims as parts of the merged dims; one-hot dims must be the innermost parts of theirs
  std::vector<int> group_of(re, -1);
  std::vector<int64_t> inner_oh(rm, 1);                  // product of the one-hot parts of merged dim k
  std::vector<int64_t> unit(re, 1);                      // coordinate of merged dim k per step of input dim j
  {
    size_t j = 0;
    for (size_t k = 0; k < rm; ++k) {
      int64_t got = 1;
      const size_t j_first = j;
      while (j < re && (got < v.M[k] || (j < re && v.E[j] == 1))) { group_of[j] = (int)k; got *= v.E[j]; ++j; }
      if (got != v.M[k]) return;
      int64_t u = 1;
      bool below_all_onehot = true;
      for (size_t q = j; q-- > j_first;) {
        unit[q] = u;
        u *= v.E[q];
        if (v.E[q] == 1) continue;
        if (oh[q]) { if (!below_all_onehot) return; inner_oh[k] *= v.E[q]; }
        else below_all_onehot = false;
      }
    }
    for (; j < re; ++j) if (v.E[j] != 1) return;
  }
  // ---- the view's dims: each walks one whole merged dim (or none: the operand stands still)
  std::vector<int64_t> DM(rm, 1);
  for (size_t k = rm; k-- > 1;) DM[k - 1] = DM[k] * v.M[k];
  struct VD { int64_t e, sx, sy, so; int k; bool kept; };
  std::vector<VD> vd;
  std::vector<char> covered(rm, 0);
  int64_t ostr[HGPU_MAX_RANK];
  dense_strides(n_keep, yo->shape, ostr);
  for (int d = 0; d < rank; ++d) {
    if (yo->shape[d] == 1) continue;
    VD q{yo->shape[d], x->strides[d], yo->strides[d], d < n_keep ? ostr[d] : 0, -1, d < n_keep};
    if (q.sy != 0) {
      for (size_t k = 0; k < rm; ++k)
        if (v.M[k] > 1 && DM[k] == q.sy && v.M[k] == q.e && !covered[k]) { q.k = (int)k; covered[k] = 1; break; }
      if (q.k < 0) return;
    }
    vd.push_back(q);
  }
  for (size_t k = 0; k < rm; ++k) if (v.M[k] > 1 && !covered[k]) return;
  // ---- rows (the array's kept dims), columns (the expression's), contracted dims; the chunk dim
  std::vector<int64_t> rx{0}, rco{0}, cy{0}, cco{0};
  auto extend = [](std::vector<int64_t>& a, std::vector<int64_t>& b, int64_t e, int64_t sa, int64_t sb) {
    std::vector<int64_t> a2, b2;
    for (size_t i = 0; i < a.size(); ++i)
      for (int64_t t = 0; t < e; ++t) { a2.push_back(a[i] + t * sa); b2.push_back(b[i] + t * sb); }
    a.swap(a2); b.swap(b2);
  };
  int chunk = -1;
  for (size_t i = 0; i < vd.size(); ++i) {
    const VD& q = vd[i];
    if (q.kept) {
      if (q.sx != 0 && q.sy == 0) { if ((int64_t)rx.size() * q.e > 32) return; extend(rx, rco, q.e, q.sx, q.so); }
      else if (q.sx == 0 && q.sy != 0) { if (inner_oh[(size_t)q.k] != 1 || (int64_t)cy.size() * q.e > 64) return; extend(cy, cco, q.e, q.sy, q.so); }
      else return;
    } else {
      if (q.sx == 0 || q.sy == 0) return;
      if (inner_oh[(size_t)q.k] == 1 && (chunk < 0 || q.e > vd[(size_t)chunk].e)) chunk = (int)i;
    }
  }
  for (size_t k = 0; k < rm; ++k) {
    if (inner_oh[k] == 1) continue;
    bool contracted = false;
    for (auto& q : vd) contracted = contracted || (q.k == (int)k && !q.kept);
    if (!contracted) return;                     // a one-hot dim that is kept: nothing to skip
  }
  if (chunk < 0 || vd[(size_t)chunk].e < 64) return;
  const int MR = (int)rx.size(), NC = (int)cy.size();
  if (MR < 2) return;
  // ---- the other contracted positions of a chunk (one-hot parts left out), and where the one-hot parts lead
  std::vector<int64_t> gx{0}, gy{0};
  std::vector<int64_t> ohx((size_t)EH, 0), ohy((size_t)EH, 0);
  for (size_t i = 0; i < vd.size(); ++i) {
    const VD& q = vd[i];
    if (q.kept || (int)i == chunk) continue;
    const int64_t io = inner_oh[(size_t)q.k];
    if (q.e / io > 1) {
      if ((int64_t)gx.size() * (q.e / io) > 65536) return;
      extend(gx, gy, q.e / io, q.sx * io, q.sy * io);
    }
  }
  for (int64_t e = 0; e < EH; ++e) {
    int64_t r = e;
    for (size_t t = digits.size(); t-- > 0;) {            // the largest stride is the first digit
      const size_t j = digits[t].second;
      const int64_t c = r / digits[t].first;
      r -= c * digits[t].first;
      for (auto& q : vd)
        if (q.k == group_of[j]) { ohx[(size_t)e] += c * unit[j] * q.sx; ohy[(size_t)e] += c * unit[j] * q.sy; }
    }
  }
  const int64_t G = (int64_t)gx.size();
  if ((double)G * NC * (double)vd[(size_t)chunk].e * MR < 1.0e7) return;     // too little work for a kernel of its own
  int64_t lo = 0, hi = 0;
  {
    int64_t rlo = rx[0], rhi = rx[0], glo = gx[0], ghi = gx[0], olo = ohx[0], ohi = ohx[0];
    for (int64_t a : rx) { rlo = std::min(rlo, a); rhi = std::max(rhi, a); }
    for (int64_t a : gx) { glo = std::min(glo, a); ghi = std::max(ghi, a); }
    for (int64_t a : ohx) { olo = std::min(olo, a); ohi = std::max(ohi, a); }
    lo = rlo + glo + olo;
    hi = rhi + ghi + ohi;
  }
  const int64_t span = hi - lo + 1;
  const int es = v.dtype == HGPU_F64 ? 8 : 4;
  if (span * es > 64 * 1024 || span < 1) return;
  for (int64_t a : gy) if (a < 0 || a > INT32_MAX) return;
  const VD& chd = vd[(size_t)chunk];
  const int64_t nch = chd.e, chx = chd.sx, chy = chd.sy;
  // threads per column, a power of two: 256 threads share the columns out
  int TPC = 256;
  while (TPC * NC > 256) TPC >>= 1;
  if (TPC < 1) return;
  // ---- where every input of the expression is read: the offset of (chunk, column, position, one-hot place)
  // is a sum of four parts, tabulated here from the inputs' strides; nothing is decoded in the kernel
  std::vector<char> scalar((size_t)v.n_in, 0);
  std::vector<int> rep((size_t)v.n_in, -1);
  for (int i = 0; i < v.n_in; ++i) {
    bool all0 = true;
    for (size_t j = 0; j < re; ++j) all0 = all0 && (v.E[j] == 1 || v.in[i]->strides[j] == 0);
    scalar[(size_t)i] = all0;
    rep[(size_t)i] = i;
    for (int k = 0; k < i && !all0; ++k) {
      if (scalar[(size_t)k]) continue;
      bool same = true;
      for (size_t j = 0; j < re && same; ++j) same = v.E[j] == 1 || v.in[k]->strides[j] == v.in[i]->strides[j];
      if (same) { rep[(size_t)i] = rep[(size_t)k]; break; }
    }
  }
  auto in_off = [&](int i, int64_t yoff) {       // input i's offset at the element of the layout yoff elements in
    int64_t o = 0;
    size_t j = 0;
    for (size_t k = 0; k < rm; ++k) {
      const int64_t ck = (yoff / DM[k]) % v.M[k];
      for (; j < re && group_of[j] == (int)k; ++j)
        if (v.E[j] > 1) o += ((ck / unit[j]) % v.E[j]) * v.in[i]->strides[j];
    }
    return o;
  };
  std::vector<int64_t> chs((size_t)v.n_in, 0);
  bool fits32 = true;
  for (int i = 0; i < v.n_in; ++i) {
    if (scalar[(size_t)i] || rep[(size_t)i] != i) continue;
    chs[(size_t)i] = in_off(i, chy);
    if (in_off(i, chy * (nch - 1)) != chs[(size_t)i] * (nch - 1)) return;     // the chunk dim is one dim of the inputs
    int64_t reach = 0;
    for (size_t j = 0; j < re; ++j) reach += (v.E[j] - 1) * (v.in[i]->strides[j] < 0 ? -v.in[i]->strides[j] : v.in[i]->strides[j]);
    fits32 = fits32 && reach < (1LL << 31);
  }
  if (!fits32) return;
  Src s;
  char kname[160];
  snprintf(kname, sizeof kname, "onehot_contract_%s_m%d_n%d_k%lldx%lld_onehot%lld", es == 8 ? "f64" : "f32", MR, NC, (long long)nch, (long long)G, (long long)EH);
  s << "typedef long long i64;\n";
  s << "typedef " << (es == 8 ? "double" : "float") << " T;\n";
  s << hg::fusedgen::kPrelude;
  auto itab = [&](const std::string& name, const std::vector<int64_t>& t, int64_t shift) {
    std::vector<int> t2;
    for (int64_t a : t) t2.push_back((int)(a - shift));
    return table("__device__ const", name.c_str(), t2);
  };
  int64_t rlo = rx[0], glo = gx[0], olo = ohx[0];
  for (int64_t a : rx) rlo = std::min(rlo, a);
  for (int64_t a : gx) glo = std::min(glo, a);
  for (int64_t a : ohx) olo = std::min(olo, a);
  s << itab("kGX", gx, glo) << itab("kOhX", ohx, olo) << itab("kColC", cco, 0) << itab("kRowC", rco, 0);
  for (int i = 0; i < v.n_in; ++i) {
    if (scalar[(size_t)i] || rep[(size_t)i] != i) continue;
    std::vector<int64_t> tc, tg, to;
    for (int64_t y : cy) tc.push_back(in_off(i, y));
    for (int64_t y : gy) tg.push_back(in_off(i, y));
    for (int64_t y : ohy) to.push_back(in_off(i, y));
    const std::string n = std::to_string(i);
    s << itab("kCol" + n, tc, 0) << itab("kG" + n, tg, 0) << itab("kOh" + n, to, 0);
  }
  s << "struct Ins {\n";
  for (int i = 0; i < v.n_in; ++i) s << "  const " << ctype(v.dt[(size_t)i]) << "* i" << i << ";\n";
  s << "};\n";
  static const int knob_batch = getenv("HORDEAD_ONEHOT_BATCH") ? atoi(getenv("HORDEAD_ONEHOT_BATCH")) : 16;
  const int RB = 4;       // rows of the result added up per round at the end
  const int MA = MR + 1;  // the rows, and the plain sum of the expression's values per column
  s << "extern \"C\" __global__ void __launch_bounds__(256) " << kname << "(const T* __restrict__ X, Ins ins, T* __restrict__ part) {\n";
  s << "  __shared__ T xs[" << span << "];\n  __shared__ T red[" << RB * 256 << "];\n";
  s << "  const int tid = threadIdx.x, col = tid / " << TPC << ", li = tid % " << TPC << ";\n  const int cq = col < " << NC << " ? col : 0;\n";
  for (int i = 0; i < v.n_in; ++i) {
    if (scalar[(size_t)i]) s << "  const " << ctype(v.dt[(size_t)i]) << " h" << i << " = ins.i" << i << "[0];\n";
    else if (rep[(size_t)i] == i) s << "  const int c" << i << " = kCol" << i << "[cq];\n";
  }
  s << "  T acc[" << MA << "];\n#pragma unroll\n  for (int m = 0; m < " << MA << "; ++m) acc[m] = T(0);\n";
  // A thread's positions of a chunk are taken a batch at a time: all the loads of `where`, then all the loads
  // of the expression's inputs at the places they name, then the multiplications -- each step's trips to memory overlap.
  // When one batch holds all of a thread's positions, its loads of `where` are issued before the chunk's footprint
  // is copied to LDS: that trip to memory then runs under the copy's.
  const int NI = (int)((G + TPC - 1) / TPC);
  const int BATCH = NI < knob_batch ? NI : knob_batch;
  const bool early_where = BATCH == NI;
  const int rw = rep[(size_t)where_in];
  auto where_loads = [&](const char* g0) {
    s << "        int gg[" << BATCH << "], ee[" << BATCH << "];\n        bool ok[" << BATCH << "];\n        i64 wv[" << BATCH << "];\n";
    s << "#pragma unroll\n        for (int it = 0; it < " << BATCH << "; ++it) {\n";
    s << "          const int g = " << g0 << " + it * " << TPC << ";\n          ok[it] = g < " << G << ";\n          gg[it] = ok[it] ? g : 0;\n";
    s << "          wv[it] = ins.i" << where_in << "[ch * " << chs[(size_t)rw] << "ll + (c" << rw << " + kG" << rw << "[gg[it]])];\n        }\n";
  };
  s << "  for (i64 ch = blockIdx.x; ch < " << nch << "ll; ch += gridDim.x) {\n";
  if (early_where) where_loads("li");
  s << "    __syncthreads();\n";
  s << "    for (int u = tid; u < " << span << "; u += 256) xs[u] = X[ch * " << chx << "ll + u];\n";
  s << "    __syncthreads();\n";
  s << "    if (col < " << NC << ") {\n";
  if (early_where) {
    s << "      {\n";
  } else {
    s << "      for (int g0 = li; g0 < " << G << "; g0 += " << TPC * BATCH << ") {\n";
    where_loads("g0");
  }
  for (int i = 0; i < v.n_in; ++i)
    if (!scalar[(size_t)i] && i != which_in && i != where_in) s << "        " << ctype(v.dt[(size_t)i]) << " r" << i << "[" << BATCH << "];\n";
  s << "#pragma unroll\n        for (int it = 0; it < " << BATCH << "; ++it) {\n";
  s << "          const i64 e = wv[it] - " << wh->offset << "ll;\n";
  s << "          ok[it] = ok[it] && e >= 0 && e < " << EH << ";\n          ee[it] = ok[it] ? (int)e : 0;\n";
  for (int i = 0; i < v.n_in; ++i) {
    if (scalar[(size_t)i] || i == which_in || i == where_in) continue;
    const int r = rep[(size_t)i];
    s << "          r" << i << "[it] = ins.i" << i << "[ch * " << chs[(size_t)r] << "ll + (c" << r << " + kG" << r << "[gg[it]] + kOh" << r << "[ee[it]])];\n";
  }
  s << "        }\n";
  s << "#pragma unroll\n        for (int it = 0; it < " << BATCH << "; ++it) {\n";
  for (int i = 0; i < v.n_in; ++i) {
    s << "          const " << ctype(v.dt[(size_t)i]) << " v" << i << "_ = ";
    if (scalar[(size_t)i]) s << "h" << i;
    else if (i == which_in) s << "(i64)ee[it] + " << wh->offset << "ll";       // the index vector holds its own offsets
    else if (i == where_in) s << "wv[it]";
    else s << "r" << i << "[it]";
    s << ";\n";
  }
  emit_program(s, v.n_in, v.n_instr, v.prog, v.dt, "          ", "_");
  s << "          const T val = ok[it] ? v" << v.slot << "_ : T(0);\n";
  s << "          const T* xp = xs + kGX[gg[it]] + kOhX[ee[it]];\n";
  for (int m = 0; m < MR; ++m) s << "          acc[" << m << "] += val * xp[" << rx[(size_t)m] - rlo << "];\n";
  s << "          acc[" << MR << "] += val;\n";
  s << "        }\n      }\n    }\n  }\n";
  // the threads of a column add up, a few rows of the result per round; thread (row, column) writes the block's partial result
  s << "#pragma unroll\n  for (int m0 = 0; m0 < " << MA << "; m0 += " << RB << ") {\n    __syncthreads();\n";
  s << "#pragma unroll\n    for (int m = m0; m < m0 + " << RB << " && m < " << MA << "; ++m) red[(m - m0) * 256 + tid] = acc[m];\n    __syncthreads();\n";
  s << "    for (int o = tid; o < " << RB * NC << "; o += 256) {\n      const int m = m0 + o / " << NC << ", c = o % " << NC << ";\n";
  s << "      if (m < " << MA << ") {\n        T sum = T(0);\n";
  s << "        for (int l = 0; l < " << TPC << "; ++l) sum += red[(m - m0) * 256 + c * " << TPC << " + l];\n";
  // a block's partial result: the rows of the product, then the columns' plain sums
  s << "        if (m < " << MR << ") part[(i64)blockIdx.x * " << out_n + NC << "ll + kRowC[m] + kColC[c]] = sum;\n";
  s << "        else part[(i64)blockIdx.x * " << out_n + NC << "ll + " << out_n << " + c] = sum;\n      }\n    }\n  }\n}\n";
  *text = s.str();
  kn->taken = true;
  kn->kname = kname;
  kn->which_in = which_in;
  kn->MR = MR;
  kn->NC = NC;
  kn->nch = nch;
  kn->G = G;
  kn->EH = EH;
  kn->span = span;
  kn->lo = lo;
  // the column sums: an array of the columns' shape, kept for a caller that asks for exactly that sum next
  for (auto& q : vd)
    if (q.kept && q.sx == 0) { kn->colshape.push_back(q.e); kn->colk.push_back(q.k); }
}

// x: the operand that is an array; y: the expression operand.  Both seen through views of `rank` dims of one shape.
int try_onehot_contract(hgpu_ctx* ctx, const hgpu_array* x, const VirtualOp& v, const hgpu_operand* yo, int n_keep, hgpu_array* out, bool* handled) {
  *handled = false;
  static const bool disabled = getenv("HORDEAD_NO_ONEHOT") != nullptr;
  if (disabled) return HGPU_OK;
  if (v.dtype != HGPU_F64 && v.dtype != HGPU_F32) return HGPU_OK;
  if (v.padded || yo->offset != 0 || v.total >= (1LL << 31)) return HGPU_OK;
  int which_in = -1, where_in = -1;
  if (!onehot_gate(v, v.slot, &which_in, &where_in)) return HGPU_OK;
  const int64_t out_n = nelem(out);
  Key key;
  key.put(which_in).put(where_in).put(x->dtype).put(x->rank, x->shape).put(x->rank, x->strides).put((int)((uintptr_t)data_ptr(x) & 63));
  put_virtual(key, v, 0, 0, 0);
  for (int i = 0; i < v.n_in; ++i) key.put(v.in[i]->offset);
  key.put(yo->rank, yo->shape).put(yo->rank, yo->strides).put(yo->offset).put(n_keep).put(out_n);
  auto kit = ctx->jit_cache.find("__onehot_known__");
  if (kit == ctx->jit_cache.end()) kit = ctx->jit_cache.emplace("__onehot_known__", new std::unordered_map<std::string, OnehotKnown>()).first;
  auto& known = *static_cast<std::unordered_map<std::string, OnehotKnown>*>(kit->second);
  auto found = known.find(key.bytes);
  if (found == known.end() || check_keys()) {
    OnehotKnown fresh;
    std::string text;
    plan_onehot(x, v, yo, n_keep, out_n, which_in, where_in, &fresh, &text);
    if (found != known.end()) {
      if (fresh.taken != found->second.taken || (fresh.taken && text != found->second.text)) return fail(ctx, HGPU_ERR_DEVICE, "onehot_contract: two different kernels under one key");
    } else {
      if (fresh.taken) {
        auto& cache = cache_of(ctx);
        auto it = cache.find(text);
        if (it == cache.end()) {
          Compiled c{nullptr, nullptr};
          if (compile(ctx, text, fresh.kname, &c) != HGPU_OK) c = Compiled{nullptr, nullptr};
          it = cache.emplace(text, c).first;
        }
        fresh.c = it->second;
        if (check_keys()) fresh.text = text;
      }
      found = known.emplace(key.bytes, std::move(fresh)).first;
    }
  }
  const OnehotKnown& kn = found->second;
  if (!kn.taken || !kn.c.fn) return HGPU_OK;
  const hgpu_array* wh = v.in[kn.which_in];
  const int es = v.dtype == HGPU_F64 ? 8 : 4;
  const int MR = kn.MR, NC = kn.NC;
  const int64_t nch = kn.nch, G = kn.G, EH = kn.EH, span = kn.span, lo = kn.lo;
  const std::vector<int64_t>& colshape = kn.colshape;
  const std::vector<int>& colk = kn.colk;
  wh->buf->known_relied_on = true;
  for (int i = 0; i < v.n_in; ++i)
    if (v.in[i]->buf && v.in[i]->buf->known == hgpu_buffer::kZeroScalar) v.in[i]->buf->known_relied_on = true;
  static const int knob_grid = getenv("HORDEAD_ONEHOT_GRID") ? atoi(getenv("HORDEAD_ONEHOT_GRID")) : 2;
  const int64_t grid = std::min<int64_t>(nch, (int64_t)ctx->num_cu * knob_grid);
  hgpu_array* colsum = nullptr;
  int rc = new_dense(ctx, v.dtype, (int)colshape.size(), colshape.data(), &colsum);
  if (rc) return rc;
  hgpu_buffer* part = nullptr;
  rc = buffer_alloc(ctx, (size_t)((out_n + NC) * grid) * es, &part);
  if (rc) { hgpu_release(colsum); return rc; }
  const char* xp = (const char*)data_ptr(x) + lo * es;
  void* pdst = part->ptr;
  std::vector<const void*> ia;
  for (int i = 0; i < v.n_in; ++i) ia.push_back(data_ptr(v.in[i]));
  void* args[] = {(void*)&xp, (void*)ia.data(), (void*)&pdst};
  {
    double bytes = (double)nch * span * es;
    for (int i = 0; i < v.n_in; ++i) {
      if (i == kn.which_in) continue;
      int64_t distinct = 1;
      for (int d = 0; d < v.in[i]->rank; ++d)
        if (v.in[i]->strides[d] != 0) distinct *= v.in[i]->shape[d];
      if (distinct > 1) bytes += (double)distinct * dtype_size(v.in[i]->dtype);
    }
    const char* label = "onehot_contract";
    if (ctx->profiling && ctx->profile_shapes) {
      char buf[200];
      snprintf(buf, sizeof buf, "onehot_contract[rows%d,cols%d,chunks%lld,positions%lld,onehot%lld,in%d,instr%d,es%d]", MR, NC, (long long)nch, (long long)G, (long long)EH, v.n_in, v.n_instr, es);
      label = intern_label(ctx, buf);
    }
    LaunchGuard lg(ctx, label, bytes, 2.0 * MR * NC * (double)G * (double)nch);
    hipError_t e = launch_module(lg, kn.c.fn, (unsigned)grid, 256, args);
    if (e != hipSuccess) { buffer_release(part); hgpu_release(colsum); return check_hip(ctx, e, "onehot_contract launch"); }
  }
  rc = hg::sum_partials_split(ctx, v.dtype, out_n, NC, (int)grid, part->ptr, data_ptr(out), data_ptr(colsum));
  buffer_release(part);
  if (rc) { hgpu_release(colsum); return rc; }
  remember_sum(ctx, v, colk, colsum);
  *handled = true;
  return HGPU_OK;
}

}  // namespace

namespace hg {
bool classify_contraction(int rank, const int64_t* shape, const int64_t* st_a, const int64_t* st_b, const int64_t* st_c, int n_keep, gemm::GemmParams* p);

void forget_remembered_sums(hgpu_ctx* ctx) {
  std::vector<MemoSum> gone;
  {
    std::lock_guard<std::mutex> lk(ctx->launch_mu);
    gone.swap(memo_of(ctx).items);
  }
  for (auto& m : gone) forget(m);
}
}

extern "C" int hgpu_contract_operands(hgpu_ctx* ctx, const hgpu_operand* a, const hgpu_operand* b, int n_keep, int flags, hgpu_array** out) {
  if (!ctx || !a || !out) return HGPU_ERR_INVALID;
  if (a->array && (!b || b->array)) {   // nothing to evaluate on the way: the plain contraction
    return hgpu_contract(ctx, a->array, b ? b->array : nullptr, n_keep, out);
  }
  VirtualOp va, vb;
  if (!a->array) if (int rc = virtual_from_operand(ctx, a, &va)) return rc;
  if (b && !b->array) if (int rc = virtual_from_operand(ctx, b, &vb)) return rc;
  // shape, strides and dtype of both operands
  auto rank_of = [](const hgpu_operand* o) { return o->array ? o->array->rank : o->rank; };
  auto shape_of = [](const hgpu_operand* o) { return o->array ? o->array->shape : o->shape; };
  auto strides_of = [](const hgpu_operand* o) { return o->array ? o->array->strides : o->strides; };
  const int rank = rank_of(a);
  const int dtype = a->array ? a->array->dtype : va.dtype;
  if (n_keep < 0 || n_keep > rank) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: n_keep %d of rank %d", n_keep, rank);
  if (b) {
    if (rank_of(b) != rank) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: ranks differ");
    for (int d = 0; d < rank; ++d)
      if (shape_of(b)[d] != shape_of(a)[d]) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: shapes differ");
    if ((b->array ? b->array->dtype : vb.dtype) != dtype) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: dtypes differ");
  }
  if (dtype == HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "contract_operands: Bool values have no sum");
  int64_t n_all = 1;
  for (int d = 0; d < rank; ++d) n_all *= shape_of(a)[d];
  if (n_all > 0 && (dtype == HGPU_F64 || dtype == HGPU_F32)) {
    hgpu_array* o = nullptr;
    int rc = new_dense(ctx, dtype, n_keep, shape_of(a), &o);
    if (rc) return rc;
    bool handled = false;
    if (!b) {
      std::vector<int> kept;
      if (kept_merged_dims(va, a, n_keep, &kept)) {
        if (hgpu_array* known = recall_sum(ctx, va, kept)) {     // a kernel that evaluated the expression has left this sum behind
          hgpu_release(o);
          rc = hgpu_reshape(ctx, known, n_keep, shape_of(a), out);
          hgpu_release(known);
          return rc;
        }
      }
      rc = try_mapped_sum(ctx, va, a, n_keep, o, &handled);
    } else if ((a->array || va.total < (1LL << 31)) && (b->array || vb.total < (1LL << 31))) {
      // one operand an array, the other an expression that is one-hot along contracted dims
      if (a->array && !b->array) rc = try_onehot_contract(ctx, a->array, vb, b, n_keep, o, &handled);
      else if (b->array && !a->array) rc = try_onehot_contract(ctx, b->array, va, a, n_keep, o, &handled);
      if (rc || handled) {
        if (rc) hgpu_release(o); else *out = o;
        return rc;
      }
      GemmParams p;
      if (hg::classify_contraction(rank, shape_of(a), strides_of(a), strides_of(b), o->strides, n_keep, &p)) {
        p.n_terms = 0;
        p.term_loop = 0;
        const size_t es = dtype_size(dtype);
        const void* pa = a->array ? data_ptr(a->array) : (const void*)(uintptr_t)(a->offset * (int64_t)es);
        const void* pb = b->array ? data_ptr(b->array) : (const void*)(uintptr_t)(b->offset * (int64_t)es);
        rc = hg::try_footprint_virtual(ctx, p, dtype, pa, pb, o, &handled, a->array ? nullptr : &va, b->array ? nullptr : &vb);
      }
    }
    if (rc || handled) {
      if (rc) hgpu_release(o); else *out = o;
      return rc;
    }
    hgpu_release(o);
  }
  if (flags & 1) return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract_operands: no kernel takes these operands unevaluated");
  hgpu_array *aa = nullptr, *bb = nullptr;
  int rc = write_out(ctx, a, &aa);
  if (!rc && b) rc = write_out(ctx, b, &bb);
  if (!rc) rc = hgpu_contract(ctx, aa, bb, n_keep, out);
  if (aa) hgpu_release(aa);
  if (bb) hgpu_release(bb);
  return rc;
}
