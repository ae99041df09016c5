// hgpu_contract_sum_map: a sum of matrix products with short contracted dims and
// an elementwise program over the sum, as ONE kernel compiled for the shapes.
//
//     outs = program( sum_t  X_t[p, k] * Y_t[q, k]  , other inputs at [q, p] )
//
// This is the layer of the reference's recurrent example,
// `tanh (wX `rmatmul2` x + wS `rmatmul2` s + rtr (rreplicate batch_size b))`
// (example/MnistRnnRanked2.hs:62-75), and the head of its cotangent,
// `(wX2^T dz2 + wS^T dz1) * (1 - h * h)`: products whose whole contracted dim
// (28 or 128 elements) fits into LDS next to a tile of the result, so that a
// kernel with a K loop, a K table and a separate pass for `+ b`, `tanh` spends
// most of its time on fixed costs.
//
// The kernel (256 threads = 4 wavefronts, tile BP x BQ of the result):
//   * P is the kept dim that is contiguous in the results, Q the other one; X_t
//     is whichever factor of term t moves along P, Y_t the one along Q.
//   * The contracted dims of all terms are cut into chunks of at most 128 (fp32)
//     or 64 (fp64) elements.  A chunk's two operand tiles are loaded with
//     16-byte loads into registers, stored to LDS, and the loads of the NEXT
//     chunk are issued before the MFMAs of this one start, so a chunk's memory
//     latency hides behind the previous chunk's arithmetic; a single chunk (one
//     product with K <= 128) has no loop at all.  Extents, strides and chunk
//     bounds are compile-time constants: addresses are immediates.
//   * LDS layouts are chosen per operand by which of (row, k) is contiguous in
//     memory, with row pitches that make the 64 lanes of a fragment read hit 64
//     different banks.
//   * fp32: v_mfma_f32_16x16x4 with X as the A operand, so the four accumulator
//     registers of a lane are four CONSECUTIVE p of one q: inputs of the
//     program and its results move as 16-byte vectors.  fp64: X as the B
//     operand, so the 16 lanes of an accumulator row are 16 consecutive p.
//   * The program runs on the accumulators in registers; only its results are
//     written.
//
// Shapes the kernel does not cover (long K, batched or higher-rank products,
// too many terms) are computed by the other entry points one after another.
//
// A problem of this size cannot fill the device and pays a launch and a round
// of memory latency for a few microseconds of arithmetic, so launches are held
// back (DeferredQueue) until something else needs the stream, and held-back
// problems that do not read one another's results run as one kernel: each
// problem's code in a namespace of its own, the first blocks of the grid for
// problem 0, the next for problem 1, ...
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.hpp"
#include "fused_gen.hpp"

using namespace hg;
using namespace hg::fusedgen;

namespace hg {
int try_gemm(hgpu_ctx* ctx, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array* out, bool* handled,
             int n_terms, const hgpu_array* const* as, const hgpu_array* const* bs, hgpu_array** partials_out = nullptr);
}

namespace {

constexpr int kMaxTermsSmallK = 4;
constexpr int64_t kMaxKTotal = 512;        // contracted elements of all terms together ...
constexpr int64_t kMaxKSmallOut = 1024;    // ... and when the result is small (a staged product would split K to fill the device and add partial results)
constexpr int64_t kSmallOut = 160000;

struct Compiled {
  hipModule_t mod;
  hipFunction_t fn;
};

std::map<std::string, Compiled>& cache_of(hgpu_ctx* ctx) {
  auto it = ctx->jit_cache.find("__smallk__");
  if (it == ctx->jit_cache.end()) it = ctx->jit_cache.emplace("__smallk__", new std::map<std::string, Compiled>()).first;
  return *static_cast<std::map<std::string, Compiled>*>(it->second);
}

// A problem's kernel, found again by what its text depends on (the text itself
// is only written the first time), and the kernels over sets of problems, found
// by their members.
struct Known {
  std::string body;    // the problem's device code
  int id = 0;          // stands for the body where sets of problems are keyed
  std::string kname;
  hipFunction_t fn = nullptr, finish_fn = nullptr;
};
struct KnownKernels {
  std::unordered_map<std::string, Known> problems;
  std::unordered_map<std::string, hipFunction_t> groups;   // by the members' ids, grids and LDS bytes in the order of the kernel's text
};
KnownKernels& known_of(hgpu_ctx* ctx) {
  auto it = ctx->jit_cache.find("__smallk_known__");
  if (it == ctx->jit_cache.end()) it = ctx->jit_cache.emplace("__smallk_known__", new KnownKernels()).first;
  return *static_cast<KnownKernels*>(it->second);
}

struct Term {
  const void *x, *y;
  int64_t K, sxp, sxk, syq, syk;
};

struct Operand {       // one operand tile of one chunk
  int rows;            // BP or BQ
  int layout;          // 0: LDS [k][row], 1: LDS [row][k]
  int V;               // elements per load
  int pitch;           // LDS elements between k rows (layout 0) or rows (layout 1)
  int64_t sr, sk;      // element strides in memory
  int64_t extent;      // rows of the whole operand (P or Q)
};

struct Chunk {
  int term, k0, kc, kcp;   // valid k, rounded up to 4
  Operand x, y;
};

struct Spec {
  bool f64;
  int64_t P, Q;
  int BP, BQ, WP, WQ;
  std::vector<Term> terms;
  std::vector<Chunk> chunks;
  int n_in, c_slot, n_instr;
  const hgpu_fused_instr* prog;
  std::vector<int> dt;
  std::vector<int64_t> in_sp, in_sq;
  std::vector<int> out_slots;
  int x_elems, y_elems;    // LDS elements of the largest X / Y tile
  // K shared out between `splits` blocks per tile (few tiles, long K: the blocks of one tile run side by side
  // instead of one block walking all of K); each block writes its partial tile, and a second launch of one block
  // per tile adds the partial tiles up in the order of K and runs the program
  int splits = 1, chunks_per_split = 0;
};

// LDS pitch of a tile: the fragment reads of 16 rows x 4 k must not collide.
int pitch_for(int layout, int rows, int kcp, bool f64) {
  if (layout == 0) {           // [k][row]: lanes of one k are adjacent, the four k of a fragment sit `pitch` apart
    int p = rows;
    while (p % 32 != 16) p += 4;
    return p;
  }
  int p = kcp;                 // [row][k]: the 16 rows of a fragment sit `pitch` apart
  if (f64) { while (p % 4 != 2) p += 2; }
  else { while (p % 8 != 4) p += 4; }
  return p;
}

Operand make_operand(bool f64, int rows, int64_t extent, int64_t sr, int64_t sk, int kc, int kcp) {
  Operand o;
  o.rows = rows;
  o.extent = extent;
  o.sr = sr;
  o.sk = sk;
  const int vmax = f64 ? 2 : 4;
  if (sk == 1 && kc % vmax == 0 && kc >= vmax) {          // k contiguous
    o.layout = 1;
    o.V = vmax;
  } else if (sr == 1 && extent % vmax == 0 && extent >= vmax) {   // rows contiguous
    o.layout = 0;
    o.V = vmax;
  } else {
    o.layout = 0;
    o.V = 1;
  }
  o.pitch = pitch_for(o.layout, rows, kcp, f64);
  return o;
}

int tile_elems(const Operand& o, int kcp) { return o.layout == 0 ? kcp * o.pitch : o.rows * o.pitch; }

void emit_stage_fn(Src& s, const char* name, const Operand& o, const Chunk& c, const char* ptr, const char* r0) {
  // registers of the next chunk's tile: load_<name>() issues the loads, store_<name>() puts them into LDS
  const int slots = o.rows * c.kcp / o.V;
  const int ns = (slots + 255) / 256;
  const bool ragged = slots % 256 != 0;
  const char* vec = o.V == 1 ? "T" : (o.V == 2 ? "V2" : "V4");
  const char* veca = o.V == 1 ? "T" : (o.V == 2 ? "A2" : "A4");
  auto decode = [&](const char* ind) {
    s << ind << "int s = tid + 256 * i;\n";
    if (ragged) s << ind << "const bool live = s < " << slots << ";\n" << ind << "s = live ? s : " << slots - 1 << ";\n";
    if (o.layout == 0) s << ind << "const int k = s / " << o.rows / o.V << ", r = (s % " << o.rows / o.V << ") * " << o.V << ";\n";
    else s << ind << "const int r = s / " << c.kcp / o.V << ", k = (s % " << c.kcp / o.V << ") * " << o.V << ";\n";
  };
  s << "struct Regs_" << name << " { " << vec << " v[" << ns << "]; };\n";
  s << "__device__ __forceinline__ void load_" << name << "(Regs_" << name << "& rg, const T* __restrict__ base, i64 r0, int tid) {\n";
  s << "#pragma unroll\n  for (int i = 0; i < " << ns << "; ++i) {\n";
  decode("    ");
  // rows past the end read the last valid vector (never stored to a result); k past the end reads a valid k (zeroed in LDS)
  s << "    i64 rr = r0 + r;\n    rr = rr > " << o.extent - (o.layout == 0 ? o.V : 1) << "LL ? " << o.extent - (o.layout == 0 ? o.V : 1) << "LL : rr;\n";
  s << "    int kk = k > " << c.kc - (o.layout == 1 ? o.V : 1) << " ? " << c.kc - (o.layout == 1 ? o.V : 1) << " : k;\n";
  s << "    rg.v[i] = *reinterpret_cast<const " << vec << "*>(base + rr * " << o.sr << "LL + (i64)(" << c.k0 << " + kk) * " << o.sk << "LL);\n";
  s << "  }\n}\n";
  s << "__device__ __forceinline__ void store_" << name << "(const Regs_" << name << "& rg, T* lds, int tid) {\n";
  s << "#pragma unroll\n  for (int i = 0; i < " << ns << "; ++i) {\n";
  decode("    ");
  if (ragged) s << "    if (!live) continue;\n";
  s << "    " << vec << " v = rg.v[i];\n";
  if (c.kcp != c.kc) {
    if (o.V == 1) s << "    if (k >= " << c.kc << ") v = T(0);\n";
    else {
      s << "    if (k >= " << c.kc << ") {";
      for (int e = 0; e < o.V; ++e) s << " v[" << e << "] = T(0);";
      s << " }\n";
    }
  }
  if (o.layout == 0) s << "    *reinterpret_cast<" << veca << "*>(lds + k * " << o.pitch << " + r) = v;\n";
  else s << "    *reinterpret_cast<" << veca << "*>(lds + r * " << o.pitch << " + k) = v;\n";
  s << "  }\n}\n";
  (void)ptr;
  (void)r0;
}

// The device code of one problem, ending in
// `body(const Args&, unsigned block, T* lds)`: what one block of 256 threads
// does.  It names nothing outside itself but the prelude, so several problems'
// code can sit in one source file, each in a namespace of its own.
std::string generate_body(const Spec& sp) {
  Src s;
  const int TP = sp.BP / (16 * sp.WP), TQ = sp.BQ / (16 * sp.WQ);
  const int64_t nbp = (sp.P + sp.BP - 1) / sp.BP, nbq = (sp.Q + sp.BQ - 1) / sp.BQ;
  const int S = sp.splits;
  const int64_t nblk = nbp * nbq, per_xcd = (nblk * S + 7) / 8;
  const bool vec_epi = !sp.f64 && sp.P % 4 == 0;
  s << "typedef " << (sp.f64 ? "double" : "float") << " T;\n";
  s << "typedef T V2 __attribute__((ext_vector_type(2), aligned(" << (sp.f64 ? 8 : 4) << ")));\n";
  s << "typedef T V4 __attribute__((ext_vector_type(4), aligned(" << (sp.f64 ? 8 : 4) << ")));\n";
  s << "typedef T A2 __attribute__((ext_vector_type(2)));\ntypedef T A4 __attribute__((ext_vector_type(4)));\n";
  s << "typedef T Acc __attribute__((ext_vector_type(4)));\n";
  // vectors of four for every type the program reads or writes
  s << "template <typename E> struct Vec4 { typedef E type __attribute__((ext_vector_type(4), aligned(sizeof(E)))); };\n";
  s << "struct Args {\n";
  for (size_t t = 0; t < sp.terms.size(); ++t) s << "  const T* x" << t << ";\n  const T* y" << t << ";\n";
  for (int i = 0; i < sp.n_in; ++i)
    if (i != sp.c_slot) s << "  const " << ctype(sp.dt[(size_t)i]) << "* i" << i << ";\n";
  for (size_t o = 0; o < sp.out_slots.size(); ++o) s << "  " << ctype(sp.dt[(size_t)sp.out_slots[o]]) << "* o" << o << ";\n";
  if (sp.splits > 1) s << "  T* part;\n";
  s << "};\n";
  for (size_t c = 0; c < sp.chunks.size(); ++c) {
    emit_stage_fn(s, ("x" + std::to_string(c)).c_str(), sp.chunks[c].x, sp.chunks[c], "", "");
    emit_stage_fn(s, ("y" + std::to_string(c)).c_str(), sp.chunks[c].y, sp.chunks[c], "", "");
  }
  // The MFMAs of one chunk.  Fragments are read from LDS a group of four k-steps
  // ahead of the MFMAs that use them (two register sets, alternating): left to
  // itself the compiler reads a step's fragments right before its MFMAs and
  // waits out the whole LDS latency at every step.
  s << "template <int KCP, int LX, int PX, int LY, int PY>\n";
  s << "__device__ __forceinline__ void compute(const T* __restrict__ xs, const T* __restrict__ ys, Acc (&acc)[" << TP << "][" << TQ << "], int r, int g, int wp, int wq) {\n";
  s << "  constexpr int NS = KCP / 4, G = 4;\n";
  s << "  T xf[2][G][" << TP << "], yf[2][G][" << TQ << "];\n";
  s << "  auto rd = [&](int buf, int j0) {\n";
  s << "#pragma unroll\n    for (int u = 0; u < G; ++u) {\n      const int j = j0 + u;\n      if (j >= NS) break;\n";
  s << "#pragma unroll\n      for (int a = 0; a < " << TP << "; ++a) xf[buf][u][a] = LX == 0 ? xs[(4 * j + g) * PX + (wp * " << TP << " + a) * 16 + r] : xs[((wp * " << TP
    << " + a) * 16 + r) * PX + 4 * j + g];\n";
  s << "#pragma unroll\n      for (int b = 0; b < " << TQ << "; ++b) yf[buf][u][b] = LY == 0 ? ys[(4 * j + g) * PY + (wq * " << TQ << " + b) * 16 + r] : ys[((wq * " << TQ
    << " + b) * 16 + r) * PY + 4 * j + g];\n";
  s << "    }\n  };\n";
  s << "  rd(0, 0);\n";
  // (the scheduling barriers keep the compiler from moving the reads back down to their uses)
  s << "#pragma unroll\n  for (int j0 = 0; j0 < NS; j0 += G) {\n    const int cur = (j0 / G) & 1;\n    if (j0 + G < NS) rd(cur ^ 1, j0 + G);\n    __builtin_amdgcn_sched_barrier(0);\n";
  s << "#pragma unroll\n    for (int u = 0; u < G; ++u) {\n      if (j0 + u >= NS) break;\n";
  s << "#pragma unroll\n      for (int a = 0; a < " << TP << "; ++a)\n#pragma unroll\n        for (int b = 0; b < " << TQ << "; ++b)\n";
  if (sp.f64) s << "          acc[a][b] = __builtin_amdgcn_mfma_f64_16x16x4f64(yf[cur][u][b], xf[cur][u][a], acc[a][b], 0, 0, 0);\n";
  else s << "          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(xf[cur][u][a], yf[cur][u][b], acc[a][b], 0, 0, 0);\n";
  s << "    }\n    __builtin_amdgcn_sched_barrier(0);\n  }\n}\n";
  // The program over one accumulator block.  What it reads besides the
  // accumulators is loaded by epi_load (rows past the end read a valid place
  // and are never written), which the kernel calls before the first chunk's
  // MFMAs when the registers allow: the loads then wait behind the arithmetic.
  s << "struct EpiIn {\n";
  for (int i = 0; i < sp.n_in; ++i) {
    if (i == sp.c_slot) continue;
    const char* ct = ctype(sp.dt[(size_t)i]);
    if (vec_epi && sp.in_sp[(size_t)i] == 1) s << "  Vec4<" << ct << ">::type w" << i << ";\n";
    else if (sp.in_sp[(size_t)i] == 0 && !sp.f64) s << "  " << ct << " w" << i << ";\n";      // one q per lane
    else if (sp.in_sp[(size_t)i] == 0) s << "  " << ct << " w" << i << "x[4];\n";                  // fp64: a lane's four values are four q
    else s << "  " << ct << " w" << i << "[4];\n";
  }
  s << "  int unused;\n};\n";
  s << "__device__ __forceinline__ EpiIn epi_load(const Args& ar, i64 pb, i64 qb, int r, int g) {\n  EpiIn z;\n  z.unused = 0;\n";
  if (vec_epi) {
    s << "  i64 p = pb + 4 * g, q = qb + r;\n  p = p > " << sp.P - 4 << "LL ? " << sp.P - 4 << "LL : p;\n  q = q > " << sp.Q - 1 << "LL ? " << sp.Q - 1 << "LL : q;\n";
    for (int i = 0; i < sp.n_in; ++i) {
      if (i == sp.c_slot) continue;
      const char* ct = ctype(sp.dt[(size_t)i]);
      if (sp.in_sp[(size_t)i] == 1) s << "  z.w" << i << " = *reinterpret_cast<const Vec4<" << ct << ">::type*>(ar.i" << i << " + q * " << sp.in_sq[(size_t)i] << "LL + p);\n";
      else if (sp.in_sp[(size_t)i] == 0) s << "  z.w" << i << " = ar.i" << i << "[q * " << sp.in_sq[(size_t)i] << "LL];\n";
      else
        for (int e = 0; e < 4; ++e) s << "  z.w" << i << "[" << e << "] = ar.i" << i << "[q * " << sp.in_sq[(size_t)i] << "LL + (p + " << e << ") * " << sp.in_sp[(size_t)i] << "LL];\n";
    }
  } else {
    bool any_q = false;
    for (int i = 0; i < sp.n_in; ++i) any_q = any_q || (i != sp.c_slot);
    if (any_q) {
      s << "#pragma unroll\n  for (int e = 0; e < 4; ++e) {\n";
      if (sp.f64) s << "    i64 p = pb + r, q = qb + 4 * e + g;\n";
      else s << "    i64 p = pb + 4 * g + e, q = qb + r;\n";
      s << "    p = p > " << sp.P - 1 << "LL ? " << sp.P - 1 << "LL : p;\n    q = q > " << sp.Q - 1 << "LL ? " << sp.Q - 1 << "LL : q;\n";
      for (int i = 0; i < sp.n_in; ++i) {
        if (i == sp.c_slot) continue;
        if (sp.in_sp[(size_t)i] == 0 && !sp.f64) s << "    if (e == 0) z.w" << i << " = ar.i" << i << "[q * " << sp.in_sq[(size_t)i] << "LL];\n";
        else if (sp.in_sp[(size_t)i] == 0) s << "    z.w" << i << "x[e] = ar.i" << i << "[q * " << sp.in_sq[(size_t)i] << "LL];\n";
        else s << "    z.w" << i << "[e] = ar.i" << i << "[q * " << sp.in_sq[(size_t)i] << "LL + p * " << sp.in_sp[(size_t)i] << "LL];\n";
      }
      s << "  }\n";
    }
  }
  s << "  return z;\n}\n";
  s << "__device__ __forceinline__ void epilogue(const Args& ar, i64 pb, i64 qb, int r, int g, const Acc& c, const EpiIn& z) {\n";
  if (vec_epi) {
    // four consecutive p of one q
    s << "  const i64 p = pb + 4 * g, q = qb + r;\n  if (p >= " << sp.P << "LL || q >= " << sp.Q << "LL) return;\n";
    for (int i = 0; i < sp.n_in; ++i) {
      const char* ct = ctype(sp.dt[(size_t)i]);
      for (int e = 0; e < 4; ++e) {
        s << "  const " << ct << " v" << i << "_" << e << " = ";
        if (i == sp.c_slot) s << "c[" << e << "];\n";
        else if (sp.in_sp[(size_t)i] == 0) s << "z.w" << i << ";\n";
        else s << "z.w" << i << "[" << e << "];\n";
      }
    }
    for (int e = 0; e < 4; ++e) emit_program(s, sp.n_in, sp.n_instr, sp.prog, sp.dt, "  ", "_" + std::to_string(e));
    for (size_t o = 0; o < sp.out_slots.size(); ++o) {
      const char* ct = ctype(sp.dt[(size_t)sp.out_slots[o]]);
      s << "  {\n    Vec4<" << ct << ">::type w;\n";
      for (int e = 0; e < 4; ++e) s << "    w[" << e << "] = v" << sp.out_slots[o] << "_" << e << ";\n";
      s << "    *reinterpret_cast<Vec4<" << ct << ">::type*>(ar.o" << o << " + q * " << sp.P << "LL + p) = w;\n  }\n";
    }
  } else {
    s << "#pragma unroll\n  for (int e = 0; e < 4; ++e) {\n";
    if (sp.f64) s << "    const i64 p = pb + r, q = qb + 4 * e + g;\n";
    else s << "    const i64 p = pb + 4 * g + e, q = qb + r;\n";
    s << "    if (p >= " << sp.P << "LL || q >= " << sp.Q << "LL) continue;\n";
    for (int i = 0; i < sp.n_in; ++i) {
      const char* ct = ctype(sp.dt[(size_t)i]);
      if (i == sp.c_slot) s << "    const T v" << i << " = c[e];\n";
      else if (sp.in_sp[(size_t)i] == 0 && !sp.f64) s << "    const " << ct << " v" << i << " = z.w" << i << ";\n";
      else if (sp.in_sp[(size_t)i] == 0) s << "    const " << ct << " v" << i << " = z.w" << i << "x[e];\n";
      else s << "    const " << ct << " v" << i << " = z.w" << i << "[e];\n";
    }
    emit_program(s, sp.n_in, sp.n_instr, sp.prog, sp.dt, "    ", "");
    for (size_t o = 0; o < sp.out_slots.size(); ++o) s << "    ar.o" << o << "[q * " << sp.P << "LL + p] = v" << sp.out_slots[o] << ";\n";
    s << "  }\n";
  }
  s << "}\n";
  s << "__device__ __forceinline__ void body(const Args& ar, unsigned bid, T* __restrict__ lds) {\n";
  s << "  T* const xs = lds;\n  T* const ys = lds + " << sp.x_elems << ";\n";
  // consecutive block ids go round the eight XCDs: blocks that share operand tiles get ids of one XCD
  if (S == 1) {
    s << "  const i64 blk = (i64)(bid % 8) * " << per_xcd << "LL + bid / 8;\n";
    s << "  if (blk >= " << nblk << "LL) return;\n";
  } else {
    s << "  const i64 blk_all = (i64)(bid % 8) * " << per_xcd << "LL + bid / 8;\n";
    s << "  if (blk_all >= " << nblk * S << "LL) return;\n";
    s << "  const i64 blk = blk_all / " << S << ";\n  const int sidx = (int)(blk_all % " << S << ");\n";
  }
  s << "  const i64 q0 = (blk % " << nbq << "LL) * " << sp.BQ << ", p0 = (blk / " << nbq << "LL) * " << sp.BP << ";\n";
  s << "  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r = lane & 15, g = lane >> 4;\n";
  s << "  const int wp = w % " << sp.WP << ", wq = w / " << sp.WP << ";\n";
  s << "  Acc acc[" << TP << "][" << TQ << "];\n";
  s << "#pragma unroll\n  for (int a = 0; a < " << TP << "; ++a)\n#pragma unroll\n    for (int b = 0; b < " << TQ << "; ++b) acc[a][b] = Acc{0, 0, 0, 0};\n";
  const size_t nc = sp.chunks.size();
  for (size_t c = 0; c < nc; ++c) s << "  Regs_x" << c << " rx" << c << ";\n  Regs_y" << c << " ry" << c << ";\n";
  auto load = [&](size_t c) {
    int t = sp.chunks[c].term;
    s << "  load_x" << c << "(rx" << c << ", ar.x" << t << ", p0, tid);\n  load_y" << c << "(ry" << c << ", ar.y" << t << ", q0, tid);\n";
  };
  int n_read = 0;
  for (int i = 0; i < sp.n_in; ++i) n_read += i != sp.c_slot;
  const bool prefetch = S == 1 && n_read > 0 && n_read * TP * TQ <= 16;
  if (n_read > 0) s << "  EpiIn ei[" << TP << "][" << TQ << "];\n";
  auto epi_loads = [&]() {
    s << "#pragma unroll\n  for (int a = 0; a < " << TP << "; ++a)\n#pragma unroll\n    for (int b = 0; b < " << TQ << "; ++b)\n";
    s << "      ei[a][b] = epi_load(ar, p0 + (wp * " << TP << " + a) * 16, q0 + (wq * " << TQ << " + b) * 16, r, g);\n";
  };
  auto run_chunks = [&](size_t c0, size_t c1) {
    load(c0);
    if (prefetch) epi_loads();
    for (size_t c = c0; c < c1; ++c) {
      const Chunk& ch = sp.chunks[c];
      s << "  store_x" << c << "(rx" << c << ", xs, tid);\n  store_y" << c << "(ry" << c << ", ys, tid);\n  __syncthreads();\n";
      if (c + 1 < c1) load(c + 1);
      s << "  compute<" << ch.kcp << ", " << ch.x.layout << ", " << ch.x.pitch << ", " << ch.y.layout << ", " << ch.y.pitch << ">(xs, ys, acc, r, g, wp, wq);\n";
      if (c + 1 < c1) s << "  __syncthreads();\n";
    }
  };
  if (S == 1) {
    run_chunks(0, nc);
  } else {
    for (int sp_i = 0; sp_i < S; ++sp_i) {
      const size_t c0 = (size_t)sp_i * (size_t)sp.chunks_per_split, c1 = std::min(nc, c0 + (size_t)sp.chunks_per_split);
      s << (sp_i ? "  else if" : "  if") << " (sidx == " << sp_i << ") {\n";
      run_chunks(c0, c1);
      s << "  }\n";
    }
    // hand the partial tile over: the registers of a lane side by side for the block's 256 lanes
    const int nreg = TP * TQ * 4;
    s << "  {\n    T* mine = ar.part + ((blk * " << S << " + sidx) * " << nreg << "LL) * 256 + tid;\n";
    s << "#pragma unroll\n    for (int a = 0; a < " << TP << "; ++a)\n#pragma unroll\n      for (int b = 0; b < " << TQ << "; ++b)\n#pragma unroll\n        for (int e = 0; e < 4; ++e) {\n";
    s << "          mine[((a * " << TQ << " + b) * 4 + e) * 256] = acc[a][b][e];\n        }\n  }\n";
    s << "}\n";
    // The second launch: one block per tile adds the partial tiles up, in the order of K, and runs the program.
    s << "__device__ __forceinline__ void finish(const Args& ar, unsigned bid) {\n";
    s << "  const i64 blk = (i64)(bid % 8) * " << (nblk + 7) / 8 << "LL + bid / 8;\n";
    s << "  if (blk >= " << nblk << "LL) return;\n";
    s << "  const i64 q0 = (blk % " << nbq << "LL) * " << sp.BQ << ", p0 = (blk / " << nbq << "LL) * " << sp.BP << ";\n";
    s << "  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r = lane & 15, g = lane >> 4;\n";
    s << "  const int wp = w % " << sp.WP << ", wq = w / " << sp.WP << ";\n";
    s << "  Acc acc[" << TP << "][" << TQ << "];\n";
    if (n_read > 0) s << "  EpiIn ei[" << TP << "][" << TQ << "];\n";
    s << "#pragma unroll\n  for (int a = 0; a < " << TP << "; ++a)\n#pragma unroll\n    for (int b = 0; b < " << TQ << "; ++b) acc[a][b] = Acc{0, 0, 0, 0};\n";
    s << "  for (int sj = 0; sj < " << S << "; ++sj) {\n    const T* theirs = ar.part + ((blk * " << S << " + sj) * " << nreg << "LL) * 256 + tid;\n";
    s << "#pragma unroll\n    for (int a = 0; a < " << TP << "; ++a)\n#pragma unroll\n      for (int b = 0; b < " << TQ << "; ++b)\n#pragma unroll\n        for (int e = 0; e < 4; ++e)\n";
    s << "          acc[a][b][e] += theirs[((a * " << TQ << " + b) * 4 + e) * 256];\n  }\n";
  }
  if (n_read > 0 && !prefetch) epi_loads();
  s << "#pragma unroll\n  for (int a = 0; a < " << TP << "; ++a)\n#pragma unroll\n    for (int b = 0; b < " << TQ << "; ++b)\n";
  if (n_read > 0) s << "      epilogue(ar, p0 + (wp * " << TP << " + a) * 16, q0 + (wq * " << TQ << " + b) * 16, r, g, acc[a][b], ei[a][b]);\n";
  else s << "      epilogue(ar, p0 + (wp * " << TP << " + a) * 16, q0 + (wq * " << TQ << " + b) * 16, r, g, acc[a][b], EpiIn{0});\n";
  s << "}\n";
  return s.str();
}

// One kernel over several problems that do not depend on one another: the
// first blocks run problem 0, the next ones problem 1, ...  (`grids[k]` blocks
// each, multiples of 8 so that every problem's block ids keep their place in
// the round of the XCDs).  A single problem gives the kernel of that problem.
std::string kernel_source(const std::vector<const std::string*>& bodies, const std::vector<unsigned>& grids, const std::vector<int>& lds_bytes, const std::string& kname,
                          bool with_finish = false) {
  Src s;
  s << kPrelude;
  int lds = 16;
  for (size_t k = 0; k < bodies.size(); ++k) {
    s << "namespace g" << k << " {\n" << *bodies[k] << "}\n";
    lds = std::max(lds, lds_bytes[k]);
  }
  s << "struct GroupArgs {\n";
  for (size_t k = 0; k < bodies.size(); ++k) s << "  g" << k << "::Args a" << k << ";\n";
  s << "};\n";
  s << "extern \"C\" __global__ void __launch_bounds__(256) " << kname << "(GroupArgs ar) {\n";
  s << "  __shared__ __attribute__((aligned(16))) double lds[" << (lds + 7) / 8 << "];\n";
  unsigned first = 0;
  for (size_t k = 0; k < bodies.size(); ++k) {
    s << "  ";
    if (k + 1 < bodies.size()) s << "if (blockIdx.x < " << first + grids[k] << "u) ";
    s << "{ g" << k << "::body(ar.a" << k << ", blockIdx.x - " << first << "u, reinterpret_cast<g" << k << "::T*>(lds)); return; }\n";
    first += grids[k];
  }
  s << "}\n";
  // a single problem whose K is shared out between blocks: the launch that adds the partial tiles up
  if (with_finish) s << "extern \"C\" __global__ void __launch_bounds__(256) " << kname << "_finish(GroupArgs ar) { g0::finish(ar.a0, blockIdx.x); }\n";
  return s.str();
}

// Tile shape by a small model of the busiest CU: its blocks are resident
// together (as far as LDS allows), so after the first block's loads have
// arrived the loads of one block hide behind the MFMAs of another; a CU with a
// single block pays load latency, loads and arithmetic one after the other.
// Measured on the recurrent layer (128 x 5000, K 128, fp32): 16 x 64 tiles
// 4.9 us per launch, 64 x 64 5.5, 64 x 128 7.8 -- the model's order.
void choose_tile(hgpu_ctx* ctx, Spec& sp, int64_t ktot) {
  static const int cand[][4] = {{16, 64, 1, 4}, {64, 16, 4, 1}, {32, 32, 2, 2}, {32, 64, 2, 2}, {64, 32, 2, 2}, {16, 128, 1, 4},
                                {64, 64, 2, 2}, {32, 128, 2, 2}, {128, 32, 2, 2}, {64, 128, 2, 2}, {128, 64, 2, 2}};
  const double es = sp.f64 ? 8 : 4;
  const double cu_flops = (sp.f64 ? 78.6e12 : 157.3e12) / ctx->num_cu;
  const double cu_load = 150e9, latency = 1.0e-6;
  const int kc = (int)std::min<int64_t>(ktot, 64);
  double best = 1e300;
  for (auto& c : cand) {
    double blocks = (double)((sp.P + c[0] - 1) / c[0]) * (double)((sp.Q + c[1] - 1) / c[1]);
    double n = std::ceil(blocks / ctx->num_cu);
    double comp = 2.0 * c[0] * c[1] * (double)ktot / cu_flops, load = (c[0] + c[1]) * (double)ktot * es / cu_load;
    double lds = (c[0] + c[1] + 20) * (double)kc * es;
    double resident = std::max(1.0, std::min(n, std::floor(160.0 * 1024 / lds)));
    double t = std::ceil(n / resident) * (latency + load + comp + (resident - 1) * std::max(load, comp));
    if (t < best) { best = t; sp.BP = c[0]; sp.BQ = c[1]; sp.WP = c[2]; sp.WQ = c[3]; }
  }
  if (const char* e = getenv("HORDEAD_SMALLK_TILE")) {   // for measurements: BPxBQxWPxWQ
    int bp, bq, wp, wq;
    if (sscanf(e, "%dx%dx%dx%d", &bp, &bq, &wp, &wq) == 4 && wp * wq == 4 && bp % (16 * wp) == 0 && bq % (16 * wq) == 0 && bp >= 16 && bq >= 16 &&
        bp / (16 * wp) * (bq / (16 * wq)) <= 16) {
      sp.BP = bp; sp.BQ = bq; sp.WP = wp; sp.WQ = wq;
    }
  }
}

// Cuts the contracted dims of the terms into chunks and lays their tiles out in LDS.
bool plan_chunks(Spec& sp) {
  // K elements per chunk: 64 (the recurrent layer's grouped step products, fp32, K 28 + 128 and 128 + 128: the
  // gradient takes 0.938 ms with chunks of 64, 0.977 with 128, 0.957 with 32)
  int kcmax = 64;
  if (const char* e = getenv("HORDEAD_SMALLK_KC")) {   // for measurements
    int v = atoi(e);
    if (v >= 8 && v <= 256 && v % 4 == 0) kcmax = v;
  }
  sp.x_elems = sp.y_elems = 0;
  sp.chunks.clear();
  for (int t = 0; t < (int)sp.terms.size(); ++t) {
    const Term& tm = sp.terms[(size_t)t];
    int n = (int)((tm.K + kcmax - 1) / kcmax);
    int per = (int)((tm.K + n - 1) / n);
    per = (per + 3) / 4 * 4;
    for (int k0 = 0; k0 < tm.K; k0 += per) {
      Chunk c;
      c.term = t;
      c.k0 = k0;
      c.kc = (int)std::min<int64_t>(per, tm.K - k0);
      c.kcp = (c.kc + 3) / 4 * 4;
      c.x = make_operand(sp.f64, sp.BP, sp.P, tm.sxp, tm.sxk, c.kc, c.kcp);
      c.y = make_operand(sp.f64, sp.BQ, sp.Q, tm.syq, tm.syk, c.kc, c.kcp);
      sp.x_elems = std::max(sp.x_elems, tile_elems(c.x, c.kcp));
      sp.y_elems = std::max(sp.y_elems, tile_elems(c.y, c.kcp));
      sp.chunks.push_back(c);
    }
  }
  sp.x_elems = (sp.x_elems + 3) / 4 * 4;
  if (sp.chunks.size() > 16) return false;
  return (size_t)(sp.x_elems + sp.y_elems) * (sp.f64 ? 8 : 4) <= 150 * 1024;
}

// Everything generate_body reads.
static_assert(sizeof(Spec) == 224 && sizeof(Chunk) == 96 && sizeof(Term) == 56, "spec_key must cover every field of Spec, Chunk, Operand and Term");
Key spec_key(const Spec& sp) {
  Key k;
  k.put(sp.f64).put(sp.P).put(sp.Q).put(sp.BP).put(sp.BQ).put(sp.WP).put(sp.WQ).put(sp.terms.size());
  for (const Term& t : sp.terms) k.put(t.K).put(t.sxp).put(t.sxk).put(t.syq).put(t.syk);
  k.put(sp.chunks.size());
  for (const Chunk& c : sp.chunks) {
    k.put(c.term).put(c.k0).put(c.kc).put(c.kcp);
    for (const Operand* o : {&c.x, &c.y}) k.put(o->rows).put(o->layout).put(o->V).put(o->pitch).put(o->sr).put(o->sk).put(o->extent);
  }
  k.put(sp.n_in).put(sp.c_slot).put(sp.n_instr, sp.prog).put(sp.dt).put(sp.in_sp).put(sp.in_sq).put(sp.out_slots);
  k.put(sp.x_elems).put(sp.y_elems).put(sp.splits).put(sp.chunks_per_split);
  return k;
}

// The non-unit kept dims of the terms must be two: P (contiguous in a dense
// result: the later one) and Q.
struct KeptDims { int dp, dq; int64_t P, Q; };

bool kept_dims(int n_keep, const int64_t* shape, KeptDims* kd) {
  int found[2], n = 0;
  for (int d = 0; d < n_keep; ++d) {
    if (shape[d] == 1) continue;
    if (n == 2) return false;
    found[n++] = d;
  }
  if (n != 2) return false;
  kd->dq = found[0];
  kd->dp = found[1];
  kd->Q = shape[found[0]];
  kd->P = shape[found[1]];
  return true;
}

// One term: which factor moves along P, and the single contracted dim.
bool term_of(const hgpu_array* a, const hgpu_array* b, int n_keep, const KeptDims& kd, Term* t) {
  const hgpu_array *x = nullptr, *y = nullptr;
  // (a factor that moves along neither -- the broadcast zero a recurrence starts from -- fits both places)
  if (a->strides[kd.dq] == 0 && b->strides[kd.dp] == 0 && (a->strides[kd.dp] != 0 || b->strides[kd.dq] != 0)) { x = a; y = b; }
  else if (b->strides[kd.dq] == 0 && a->strides[kd.dp] == 0 && (b->strides[kd.dp] != 0 || a->strides[kd.dq] != 0)) { x = b; y = a; }
  else return false;
  // contracted dims: merge what merges in both factors; one dim must remain
  int64_t K = 1, sxk = 0, syk = 0;
  bool have = false;
  for (int d = a->rank - 1; d >= n_keep; --d) {
    int64_t e = a->shape[d];
    if (e == 1) continue;
    if (!have) { K = e; sxk = x->strides[d]; syk = y->strides[d]; have = true; continue; }
    if (x->strides[d] == sxk * K && y->strides[d] == syk * K) { K *= e; continue; }
    return false;
  }
  if (!have) return false;
  t->x = data_ptr(x);
  t->y = data_ptr(y);
  t->K = K;
  t->sxp = x->strides[kd.dp];
  t->sxk = sxk;
  t->syq = y->strides[kd.dq];
  t->syk = syk;
  return true;
}

bool fits_int(int64_t v) { return v > -(1LL << 40) && v < (1LL << 40); }

// The kernel over the given problems, compiled once per source text; nullptr when the compiler refuses it.
hipFunction_t compiled_kernel(hgpu_ctx* ctx, const std::vector<const std::string*>& bodies, const std::vector<unsigned>& grids, const std::vector<int>& lds_bytes,
                              const std::string& kname, hipFunction_t* finish_fn = nullptr) {
  std::string src = kernel_source(bodies, grids, lds_bytes, kname, finish_fn != nullptr);
  auto& cache = cache_of(ctx);
  auto it = cache.find(src);
  if (it == cache.end()) {
    Compiled c{nullptr, nullptr};
    std::vector<char> code;
    int rc = rtc_compile(ctx, src, "small-K product", &code);
    if (rc && getenv("HORDEAD_GPU_DEBUG")) fprintf(stderr, "hordead_gpu: %s rejected: %s\n", kname.c_str(), hgpu_last_error(ctx));
    if (!rc) {
      hipError_t e = hipModuleLoadData(&c.mod, code.data());
      if (e == hipSuccess) e = hipModuleGetFunction(&c.fn, c.mod, kname.c_str());
      if (e != hipSuccess) c = Compiled{nullptr, nullptr};
    }
    it = cache.emplace(src, c).first;
  }
  if (finish_fn) {
    *finish_fn = nullptr;
    if (it->second.fn && hipModuleGetFunction(finish_fn, it->second.mod, (kname + "_finish").c_str()) != hipSuccess) return nullptr;
  }
  return it->second.fn;
}

constexpr size_t kMaxHeld = 256;          // launches held back at most
constexpr size_t kMaxGroup = 4;           // problems in one kernel at most
constexpr int64_t kGroupBlocksPerCu = 4;  // a problem with more blocks than this per CU fills the device alone

}  // namespace

namespace hg {
// A launch that is held back: everything the kernel needs, and the buffers it
// reads and writes (retained, so that none is handed out again before the launch).
struct Deferred {
  bool is_reduction = false;   // a reduction of contract.hip (`red`) instead of a small product
  RedJob red;
  const std::string* body = nullptr;   // the problem's device code (kept with the known kernels) and the number that stands for it
  int body_id = -1;
  std::string kname;
  hipFunction_t fn = nullptr;
  unsigned grid = 0;
  int lds_bytes = 0;
  std::vector<const void*> args;
  std::vector<hgpu_buffer*> reads, writes;
  const char* label = nullptr;
  double bytes = 0, flops = 0;
  int level = 0;
};

struct DeferredQueue {
  std::vector<Deferred> items;
  std::map<size_t, int> seen;        // how often a set of problems came up together, by the hash of their ids, grids and LDS bytes
  long n_launches = 0, n_grouped = 0;
};
}  // namespace hg

namespace hg {

// outs[i] (dense, of the kept shape, allocated by the caller) = slot
// out_slots[i] of the program over sum_t contract(as[t], bs[t]).  *handled says
// whether the kernel took the case.
int try_smallk(hgpu_ctx* ctx, int n_terms, const hgpu_array* const* as, const hgpu_array* const* bs, int n_keep, int n_in, const hgpu_array* const* in, int c_slot,
               int n_instr, const hgpu_fused_instr* prog, const std::vector<int>& dt, int n_out, const int* out_slots, hgpu_array* const* outs, bool* handled) {
  *handled = false;
  const hgpu_array* a0 = as[0];
  if (a0->dtype != HGPU_F64 && a0->dtype != HGPU_F32) return HGPU_OK;
  if (n_terms < 1 || n_terms > kMaxTermsSmallK || n_out < 1) return HGPU_OK;
  static const bool disabled = getenv("HORDEAD_NO_SMALLK") != nullptr;
  if (disabled) return HGPU_OK;
  KeptDims kd;
  if (!kept_dims(n_keep, a0->shape, &kd)) return HGPU_OK;
  Spec sp;
  sp.f64 = a0->dtype == HGPU_F64;
  sp.P = kd.P;
  sp.Q = kd.Q;
  int64_t ktot = 0;
  for (int t = 0; t < n_terms; ++t) {
    Term tm;
    if (!as[t]->buf || !bs[t]->buf) return HGPU_OK;
    if (!term_of(as[t], bs[t], n_keep, kd, &tm)) return HGPU_OK;
    if (!fits_int(tm.sxp * sp.P) || !fits_int(tm.syq * sp.Q) || !fits_int(tm.sxk * tm.K) || !fits_int(tm.syk * tm.K)) return HGPU_OK;
    ktot += tm.K;
    sp.terms.push_back(tm);
  }
  if (ktot < 4 || ktot > (sp.P * sp.Q <= kSmallOut ? kMaxKSmallOut : kMaxKTotal)) return HGPU_OK;
  // below about a million multiply-adds the wave-per-output kernels are as fast; from there on this kernel wins, the more so with a program to
  // run over the result (the CNN's readout layer and its cotangent, 10 x 1000 x 128 each: the gradient 0.453 -> 0.430 ms with them in)
  if (sp.P < 16 || sp.Q < 4 || (double)sp.P * sp.Q * ktot < 1.0e6) return HGPU_OK;
  for (int o = 0; o < n_out; ++o) {
    if (out_slots[o] < n_in && out_slots[o] != c_slot) return HGPU_OK;   // a copy of an input: not this kernel's business
    if (!outs[o]->buf) return HGPU_OK;
  }
  sp.n_in = n_in;
  sp.c_slot = c_slot;
  sp.n_instr = n_instr;
  sp.prog = prog;
  sp.dt = dt;
  sp.in_sp.assign((size_t)n_in, 0);
  sp.in_sq.assign((size_t)n_in, 0);
  for (int i = 0; i < n_in; ++i) {
    if (i == c_slot) continue;
    if (!in[i]->buf) return HGPU_OK;
    sp.in_sp[(size_t)i] = in[i]->strides[kd.dp];
    sp.in_sq[(size_t)i] = in[i]->strides[kd.dq];
    if (!fits_int(sp.in_sp[(size_t)i] * sp.P) || !fits_int(sp.in_sq[(size_t)i] * sp.Q)) return HGPU_OK;
  }
  sp.out_slots.assign(out_slots, out_slots + n_out);
  choose_tile(ctx, sp, ktot);
  if (!plan_chunks(sp)) return HGPU_OK;
  const int64_t ntiles = ((sp.P + sp.BP - 1) / sp.BP) * ((sp.Q + sp.BQ - 1) / sp.BQ);
  {
    // Fewer tiles than three quarters of the CUs and a long K (a dense layer's weight gradient, 784 x 128 over
    // a batch of 1000: 98 tiles of 16 chunks): K is shared out so that about two blocks per CU run.  Short K
    // (the steps of a recurrence) stays whole: those products are held back and grouped instead.
    static const bool no_split = getenv("HORDEAD_SMALLK_NOSPLIT") != nullptr;
    const int nc = (int)sp.chunks.size();
    if (!no_split && ntiles * 4 < (int64_t)ctx->num_cu * 3 && nc >= 8) {
      int want = (int)std::min<int64_t>(nc / 2, (2 * (int64_t)ctx->num_cu + ntiles - 1) / ntiles);
      if (want >= 2) {
        sp.chunks_per_split = (nc + want - 1) / want;
        sp.splits = (nc + sp.chunks_per_split - 1) / sp.chunks_per_split;
      }
    }
  }

  char kname[96];
  snprintf(kname, sizeof kname, "smallk_%s_p%lld_q%lld_k%lld_t%d_in%d_instr%d_out%d", sp.f64 ? "f64" : "f32", (long long)sp.P, (long long)sp.Q, (long long)ktot, n_terms, n_in - 1,
           n_instr, n_out);
  Deferred d;
  hipFunction_t finish_fn = nullptr;
  d.kname = kname;
  const int64_t nblk = ntiles * sp.splits;
  const int64_t grid = (nblk + 7) / 8 * 8;
  if (grid > 0x7fffffff) return HGPU_OK;
  d.grid = (unsigned)grid;
  d.lds_bytes = (sp.x_elems + sp.y_elems) * (sp.f64 ? 8 : 4);
  {
    std::lock_guard<std::mutex> lk(ctx->launch_mu);   // the kernel caches are shared with the thread that launches what is held back
    auto& known = known_of(ctx).problems;
    const Key key = spec_key(sp);
    auto it = known.find(key.bytes);
    if (it == known.end()) {
      Known kn;
      kn.body = generate_body(sp);
      kn.id = (int)known.size();
      kn.kname = kname;
      kn.fn = compiled_kernel(ctx, {&kn.body}, {d.grid}, {d.lds_bytes}, kn.kname, sp.splits > 1 ? &kn.finish_fn : nullptr);
      it = known.emplace(key.bytes, std::move(kn)).first;
    } else if (check_keys() && (it->second.body != generate_body(sp) || it->second.kname != kname)) {
      return fail(ctx, HGPU_ERR_DEVICE, "small-K product: two different kernels under one key (%s)", kname);
    }
    d.body = &it->second.body;
    d.body_id = it->second.id;
    d.fn = it->second.fn;
    finish_fn = it->second.finish_fn;
  }
  if (!d.fn) return HGPU_OK;

  for (auto& tm : sp.terms) { d.args.push_back(tm.x); d.args.push_back(tm.y); }
  for (int i = 0; i < n_in; ++i)
    if (i != c_slot) d.args.push_back(data_ptr(in[i]));
  for (int o = 0; o < n_out; ++o) d.args.push_back(data_ptr(outs[o]));
  const double es = sp.f64 ? 8 : 4;
  hgpu_buffer* part = nullptr;
  if (sp.splits > 1) {
    int rc = buffer_alloc(ctx, (size_t)nblk * (size_t)sp.BP * (size_t)sp.BQ * (size_t)es, &part);
    if (rc) return rc;
    d.args.push_back(part->ptr);
  }
  d.flops = 2.0 * (double)sp.P * sp.Q * ktot;
  d.bytes = ((double)sp.P + sp.Q) * ktot * es;
  for (int i = 0; i < n_in; ++i)
    if (i != c_slot) d.bytes += (sp.in_sp[(size_t)i] ? (double)sp.P : 1.0) * (sp.in_sq[(size_t)i] ? (double)sp.Q : 1.0) * (double)dtype_size(in[i]->dtype);
  for (int o = 0; o < n_out; ++o) d.bytes += (double)sp.P * sp.Q * (double)dtype_size(outs[o]->dtype);
  d.label = sp.f64 ? "gemm_f64" : "gemm_f32";
  if (ctx->profiling && ctx->profile_shapes) {
    char buf[200];
    std::string ks;
    for (auto& tm : sp.terms) ks += (ks.empty() ? "" : "+") + std::to_string(tm.K);
    char splits[24] = "";
    if (sp.splits > 1) snprintf(splits, sizeof splits, ",splits%d", sp.splits);
    snprintf(buf, sizeof buf, "%s[M%lldxN%lldxK%sxB1,wholeK,t%dx%d,chunks%d%s,lds%dK,map(in%d,instr%d,out%d)]", d.label, (long long)sp.Q, (long long)sp.P, ks.c_str(), sp.BQ,
             sp.BP, (int)sp.chunks.size(), splits, (int)((sp.x_elems + sp.y_elems) * (int)es / 1024), n_in - 1, n_instr, n_out);
    d.label = intern_label(ctx, buf);
  }
  static const bool hold = getenv("HORDEAD_NO_GROUPED_LAUNCH") == nullptr;
  if (hold && sp.splits == 1 && nblk <= kGroupBlocksPerCu * ctx->num_cu) {
    // held back: the next small products may be independent of this one
    for (int t = 0; t < n_terms; ++t) { d.reads.push_back(as[t]->buf); d.reads.push_back(bs[t]->buf); }
    for (int i = 0; i < n_in; ++i)
      if (i != c_slot) d.reads.push_back(in[i]->buf);
    for (int o = 0; o < n_out; ++o) d.writes.push_back(outs[o]->buf);
    for (auto* b : d.reads) buffer_retain(b);
    for (auto* b : d.writes) buffer_retain(b);
    std::lock_guard<std::mutex> lk(ctx->launch_mu);
    if (!ctx->dq) ctx->dq = new DeferredQueue;
    if (ctx->dq->items.size() >= kMaxHeld) flush_deferred_locked(ctx);
    ctx->dq->items.push_back(std::move(d));
    ctx->dq_pending = true;
    *handled = true;
    return HGPU_OK;
  }
  LaunchGuard lg(ctx, d.label, d.bytes, d.flops);
  void* args[] = {(void*)d.args.data()};
  hipError_t err = launch_module(lg, d.fn, d.grid, 256, args, true, finish_fn == nullptr);
  if (err == hipSuccess && finish_fn) err = launch_module(lg, finish_fn, (unsigned)((ntiles + 7) / 8 * 8), 256, args, false, true);
  if (part) buffer_release(part);
  if (err != hipSuccess) return check_hip(ctx, err, "small-K product launch");
  *handled = true;
  return HGPU_OK;
}

// Launches what was held back.  Products are levelled by who reads whose
// results (arrays are never written twice, so reads-after-writes are the only
// order there is); the members of one level are independent and go out
// together, the levels one after another.  For an unrolled recurrence of two
// layers, issued layer by layer, level k holds step k + 1 of the first layer
// and step k of the second: the diagonal of the time x layer grid.
void flush_deferred_locked(hgpu_ctx* ctx) {
  ctx->dq_pending = false;
  if (!ctx->dq || ctx->dq->items.empty()) return;
  std::vector<Deferred> items;
  items.swap(ctx->dq->items);
  (void)hipSetDevice(ctx->device);
  std::map<const hgpu_buffer*, int> written_at;
  int top = 0;
  for (auto& d : items) {
    d.level = 0;
    for (auto* b : d.reads) {
      auto it = written_at.find(b);
      if (it != written_at.end()) d.level = std::max(d.level, it->second + 1);
    }
    for (auto* b : d.writes) written_at[b] = d.level;
    top = std::max(top, d.level);
  }
  auto timed_launch = [&](hipFunction_t fn, unsigned grid, const std::vector<const void*>& ar, const char* label, double bytes, double flops) {
    // (timed: the launch carries its record's two events, which then hold the kernel's own begin and end)
    hipEvent_t ea = nullptr, eb = nullptr;
    if (ctx->profiling && !ctx->cap && (uint64_t)grid * 256 <= 0xffffffffull) {
      hgpu_ctx::ProfRec r{label, nullptr, nullptr, bytes, flops};
      if (hipEventCreate(&r.a) == hipSuccess && hipEventCreate(&r.b) == hipSuccess) {
        ctx->prof.push_back(r);
        ea = r.a;
        eb = r.b;
      }
    }
    void* args[] = {(void*)ar.data()};
    hipError_t err = ea ? hipExtModuleLaunchKernel(fn, grid * 256, 1, 1, 256, 1, 1, 0, ctx->stream, args, nullptr, ea, eb, 0)
                        : hipModuleLaunchKernel(fn, grid, 1, 1, 256, 1, 1, 0, ctx->stream, args, nullptr);
    if (err != hipSuccess) {
      int rc = check_hip(ctx, err, "small-K product launch");
      if (!ctx->deferred_rc) ctx->deferred_rc = rc;
    }
  };
  for (int lv = 0; lv <= top; ++lv) {
    // the level's reductions: those of one element type go out together, four at a time
    {
      std::vector<Deferred*> reds;
      for (auto& d : items)
        if (d.level == lv && d.is_reduction) reds.push_back(&d);
      std::stable_sort(reds.begin(), reds.end(), [](const Deferred* a, const Deferred* b) { return a->red.dtype < b->red.dtype; });
      for (size_t g0 = 0; g0 < reds.size();) {
        size_t g1 = g0 + 1;
        while (g1 < reds.size() && g1 - g0 < 4 && reds[g1]->red.dtype == reds[g0]->red.dtype) ++g1;
        const RedJob* jobs[4];
        double bytes = 0, flops = 0;
        for (size_t i = g0; i < g1; ++i) { jobs[i - g0] = &reds[i]->red; bytes += reds[i]->bytes; flops += reds[i]->flops; }
        const char* label = reds[g0]->label;
        if (g1 - g0 > 1) {
          label = "contract_group";
          if (ctx->profiling && ctx->profile_shapes) {
            std::string lab = "contract_group[";
            for (size_t i = g0; i < g1; ++i) lab += (i > g0 ? "|" : "") + std::string(reds[i]->label);
            label = intern_label(ctx, lab + "]");
          }
        }
        bool timed = false;
        if (ctx->profiling && !ctx->cap) {
          hgpu_ctx::ProfRec r{label, nullptr, nullptr, bytes, flops};
          if (hipEventCreate(&r.a) == hipSuccess && hipEventCreate(&r.b) == hipSuccess) {
            (void)hipEventRecord(r.a, ctx->stream);
            ctx->prof.push_back(r);
            timed = true;
          }
        }
        hipError_t err = launch_reduction_group(ctx, jobs, (int)(g1 - g0));
        if (timed) (void)hipEventRecord(ctx->prof.back().b, ctx->stream);
        if (err != hipSuccess) {
          int rc = check_hip(ctx, err, "grouped reduction launch");
          if (!ctx->deferred_rc) ctx->deferred_rc = rc;
        }
        ctx->dq->n_launches += 1;
        if (g1 - g0 > 1) ctx->dq->n_grouped += (long)(g1 - g0);
        g0 = g1;
      }
    }
    std::vector<Deferred*> here;
    for (auto& d : items)
      if (d.level == lv && !d.is_reduction) here.push_back(&d);
    for (size_t g0 = 0; g0 < here.size(); g0 += kMaxGroup) {
      std::vector<Deferred*> grp(here.begin() + (long)g0, here.begin() + (long)std::min(here.size(), g0 + kMaxGroup));
      hipFunction_t fn = nullptr;
      std::string gname;
      if (grp.size() > 1) {
        // one order for a set of problems, whichever way round they were issued
        std::stable_sort(grp.begin(), grp.end(), [](const Deferred* a, const Deferred* b) {
          return a->kname != b->kname ? a->kname < b->kname : (a->body_id != b->body_id && *a->body < *b->body);
        });
        Key key;
        for (auto* d : grp) key.put(d->body_id).put(d->grid).put(d->lds_bytes);
        // a set seen once may never come again (a second or so of compilation): the second time pays
        if (++ctx->dq->seen[std::hash<std::string>()(key.bytes)] >= 2) {
          auto& groups = known_of(ctx).groups;
          auto it = groups.find(key.bytes);
          if (it == groups.end() || check_keys()) {
            gname = "smallk_x" + std::to_string(grp.size());
            std::vector<const std::string*> bodies;
            std::vector<unsigned> grids;
            std::vector<int> lds;
            for (auto* d : grp) { gname += "__" + d->kname.substr(7); bodies.push_back(d->body); grids.push_back(d->grid); lds.push_back(d->lds_bytes); }
            hipFunction_t f = compiled_kernel(ctx, bodies, grids, lds, gname);
            if (it != groups.end() && it->second != f) {
              fprintf(stderr, "hordead_gpu: two different kernels under one key (%s)\n", gname.c_str());
              if (!ctx->deferred_rc) ctx->deferred_rc = HGPU_ERR_DEVICE;
            }
            if (it == groups.end()) it = groups.emplace(key.bytes, f).first;
          }
          fn = it->second;
        }
      }
      if (fn) {
        std::vector<const void*> ar;
        unsigned grid = 0;
        double bytes = 0, flops = 0;
        std::string lab = std::string(grp[0]->label).substr(0, std::string(grp[0]->label).find('[')) + "[group:";   // same family as its members
        for (auto* d : grp) {
          ar.insert(ar.end(), d->args.begin(), d->args.end());
          grid += d->grid;
          bytes += d->bytes;
          flops += d->flops;
          std::string in(d->label);
          size_t at = in.find('[');
          if (at != std::string::npos && in.back() == ']') in = in.substr(at + 1, in.size() - at - 2);
          lab += (d == grp[0] ? "" : "|") + in;
        }
        const char* label = grp[0]->label;
        if (ctx->profiling && ctx->profile_shapes) label = intern_label(ctx, lab + "]");
        timed_launch(fn, grid, ar, label, bytes, flops);
        ctx->dq->n_grouped += (long)grp.size();
      } else {
        for (auto* d : grp) timed_launch(d->fn, d->grid, d->args, d->label, d->bytes, d->flops);
      }
      ctx->dq->n_launches += fn ? 1 : (long)grp.size();
    }
  }
  for (auto& d : items) {
    for (auto* b : d.reads) buffer_release(b);
    for (auto* b : d.writes) buffer_release(b);
  }
}

// A single-launch reduction joins the queue: held back until something else needs the stream, levelled with
// the held products by who reads whose results, and launched together with the other reductions of its level.
bool hold_reduction(hgpu_ctx* ctx, const RedJob& job, hgpu_buffer* const* reads, int n_reads, hgpu_buffer* write) {
  static const bool hold = getenv("HORDEAD_NO_GROUPED_LAUNCH") == nullptr;
  if (!hold || !write) return false;
  Deferred d;
  d.is_reduction = true;
  d.red = job;
  d.label = job.label;
  d.bytes = job.bytes;
  d.flops = job.flops;
  for (int i = 0; i < n_reads; ++i)
    if (reads[i]) d.reads.push_back(reads[i]);
  d.writes.push_back(write);
  for (auto* b : d.reads) buffer_retain(b);
  for (auto* b : d.writes) buffer_retain(b);
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  if (!ctx->dq) ctx->dq = new DeferredQueue;
  if (ctx->dq->items.size() >= kMaxHeld) flush_deferred_locked(ctx);
  ctx->dq->items.push_back(std::move(d));
  ctx->dq_pending = true;
  return true;
}

void flush_deferred(hgpu_ctx* ctx) {
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  if (ctx->dq_pending) flush_deferred_locked(ctx);
}

// Launches what is held back and gives the queue's own memory back (hgpu_shutdown).
void drop_deferred(hgpu_ctx* ctx) {
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  if (ctx->dq_pending) flush_deferred_locked(ctx);
  delete ctx->dq;
  ctx->dq = nullptr;
}

}  // namespace hg

extern "C" int hgpu_contract_sum_map(hgpu_ctx* ctx, int n_terms, const hgpu_array* const* as, const hgpu_array* const* bs, int n_keep, int n_in,
                                     const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int n_out, const int* out_slots, hgpu_array** outs) {
  if (!ctx || !as || !bs || !in || n_terms < 1 || (n_instr > 0 && !prog) || n_out < 1 || !out_slots || !outs) return HGPU_ERR_INVALID;
  for (int t = 0; t < n_terms; ++t)
    if (!as[t] || !bs[t]) return HGPU_ERR_INVALID;
  const hgpu_array* a0 = as[0];
  if (n_keep < 1 || n_keep > a0->rank) return fail(ctx, HGPU_ERR_INVALID, "contract_sum_map: n_keep %d of rank %d", n_keep, a0->rank);
  for (int t = 0; t < n_terms; ++t) {
    if (as[t]->dtype != a0->dtype || bs[t]->dtype != a0->dtype || !same_shape(as[t], bs[t])) return fail(ctx, HGPU_ERR_INVALID, "contract_sum_map: factors differ in dtype or shape");
    bool ok = as[t]->rank >= n_keep;
    for (int d = 0; d < n_keep && ok; ++d) ok = as[t]->shape[d] == a0->shape[d];
    if (!ok) return fail(ctx, HGPU_ERR_INVALID, "contract_sum_map: term %d does not have the kept shape", t);
  }
  if (n_in < 1 || n_in > 12 || n_instr < 0 || n_instr > 96 || n_out > 6) return fail(ctx, HGPU_ERR_UNSUPPORTED, "contract_sum_map: %d inputs, %d instructions, %d outputs", n_in, n_instr, n_out);
  int c_slot = -1;
  for (int i = 0; i < n_in; ++i) {
    if (!in[i]) {
      if (c_slot >= 0) return fail(ctx, HGPU_ERR_INVALID, "contract_sum_map: more than one input stands for the sum");
      c_slot = i;
      continue;
    }
    bool ok = in[i]->rank == n_keep;
    for (int d = 0; d < n_keep && ok; ++d) ok = in[i]->shape[d] == a0->shape[d];
    if (!ok) return fail(ctx, HGPU_ERR_INVALID, "contract_sum_map: input %d does not have the kept shape", i);
  }
  if (c_slot < 0) return fail(ctx, HGPU_ERR_INVALID, "contract_sum_map: no input stands for the sum");
  std::vector<int> dt;
  {
    std::vector<const hgpu_array*> tin(in, in + n_in);
    tin[(size_t)c_slot] = a0;   // only the dtype is read
    if (int rc = check_program(ctx, n_in, tin.data(), n_instr, prog, &dt)) return rc;
  }
  for (int o = 0; o < n_out; ++o)
    if (out_slots[o] < 0 || out_slots[o] >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "contract_sum_map: bad output slot");
  int64_t n_kept = 1;
  for (int d = 0; d < n_keep; ++d) n_kept *= a0->shape[d];
  if (n_kept > 0) {
    std::vector<hgpu_array*> res((size_t)n_out, nullptr);
    auto release_res = [&] { for (auto*& r : res) if (r) { hgpu_release(r); r = nullptr; } };
    int rc = HGPU_OK;
    for (int o = 0; o < n_out && !rc; ++o) rc = new_dense(ctx, dt[(size_t)out_slots[o]], n_keep, a0->shape, &res[(size_t)o]);
    bool handled = false;
    if (!rc) rc = try_smallk(ctx, n_terms, as, bs, n_keep, n_in, in, c_slot, n_instr, prog, dt, n_out, out_slots, res.data(), &handled);
    if (rc || !handled) release_res();
    if (rc) return rc;
    if (handled) {
      for (int o = 0; o < n_out; ++o) outs[o] = res[(size_t)o];
      return HGPU_OK;
    }
  }
  // one entry point after another: the products (terms of one shape together), their sum, the program
  hgpu_array* c = nullptr;
  // A single product that the staged kernel splits in two or three along K
  // leaves partial results to add: the pass that runs the program adds them.
  bool sum_is_output = false;
  for (int o = 0; o < n_out; ++o) sum_is_output = sum_is_output || out_slots[o] == c_slot;
  if (n_terms == 1 && !sum_is_output && n_instr >= 1 && n_in + 2 <= 12 && n_instr + 2 <= 96 && n_kept > 0 && (a0->dtype == HGPU_F64 || a0->dtype == HGPU_F32)) {
    hgpu_array *c0 = nullptr, *parts = nullptr;
    int rc = new_dense(ctx, a0->dtype, n_keep, a0->shape, &c0);
    bool handled = false;
    if (!rc) rc = try_gemm(ctx, as[0], bs[0], n_keep, c0, &handled, 0, nullptr, nullptr, &parts);
    if (rc) { if (c0) hgpu_release(c0); return rc; }
    if (handled && parts) {
      hgpu_release(c0);
      const int S = (int)parts->shape[0], n_in2 = n_in + S - 1, shift = (S - 1) + (S - 1);
      std::vector<hgpu_array*> slices((size_t)S, nullptr);
      for (int s2 = 0; s2 < S && !rc; ++s2) {
        const int64_t ix = s2;
        rc = hgpu_index_prefix(ctx, parts, 1, &ix, &slices[(size_t)s2]);
      }
      std::vector<const hgpu_array*> ins2(in, in + n_in);
      std::vector<hgpu_fused_instr> prog2;
      if (!rc) {
        ins2[(size_t)c_slot] = slices[0];
        for (int s2 = 1; s2 < S; ++s2) ins2.push_back(slices[(size_t)s2]);
        // the sum: (p0 + p1) + p2, then the caller's program with its slots moved
        for (int s2 = 1; s2 < S; ++s2)
          prog2.push_back(hgpu_fused_instr{HGPU_FUSED_OP2, HGPU_ADD, a0->dtype, s2 == 1 ? c_slot : n_in2 + s2 - 2, n_in + s2 - 1, 0});
        const int sum_slot = n_in2 + S - 2;
        auto moved = [&](int v) { return v == c_slot ? sum_slot : (v < n_in ? v : v + shift); };
        for (int k = 0; k < n_instr; ++k) {
          hgpu_fused_instr q = prog[k];
          q.a = moved(q.a);
          if (q.kind == HGPU_FUSED_OP2 || q.kind == HGPU_FUSED_CMP || q.kind == HGPU_FUSED_SELECT) q.b = moved(q.b);
          if (q.kind == HGPU_FUSED_SELECT) q.c = moved(q.c);
          prog2.push_back(q);
        }
        std::vector<int> slots2;
        for (int o = 0; o < n_out; ++o) slots2.push_back(moved(out_slots[o]));
        rc = hgpu_fused_map(ctx, n_in2, ins2.data(), (int)prog2.size(), prog2.data(), n_out, slots2.data(), outs);
      }
      for (auto* sl : slices) if (sl) hgpu_release(sl);
      hgpu_release(parts);
      return rc;
    }
    if (handled) c = c0;            // computed whole: the program below
    else hgpu_release(c0);
  }
  if (!c) {
    std::vector<char> taken((size_t)n_terms, 0);
    for (int t0 = 0; t0 < n_terms; ++t0) {
      if (taken[(size_t)t0]) continue;
      std::vector<const hgpu_array*> ga, gb;
      for (int t = t0; t < n_terms; ++t)
        if (!taken[(size_t)t] && same_shape(as[t], as[t0])) { ga.push_back(as[t]); gb.push_back(bs[t]); taken[(size_t)t] = 1; }
      hgpu_array* part = nullptr;
      int rc = hgpu_contract_sum(ctx, (int)ga.size(), ga.data(), gb.data(), n_keep, &part);
      if (!rc && c) {
        hgpu_array* sum = nullptr;
        rc = hgpu_ewise2(ctx, HGPU_ADD, c, part, &sum);
        hgpu_release(part);
        hgpu_release(c);
        c = sum;
      } else if (!rc) {
        c = part;
      }
      if (rc) { if (c) hgpu_release(c); return rc; }
    }
  }
  std::vector<const hgpu_array*> ins(in, in + n_in);
  ins[(size_t)c_slot] = c;
  std::vector<hgpu_array*> res((size_t)n_out, nullptr);
  int rc = HGPU_OK;
  std::vector<int> fslots;
  std::vector<size_t> fpos;
  for (int o = 0; o < n_out && !rc; ++o) {
    if (out_slots[o] == c_slot) { hgpu_retain(c); res[(size_t)o] = c; }
    else if (out_slots[o] < n_in) rc = hgpu_materialize(ctx, ins[(size_t)out_slots[o]], &res[(size_t)o]);
    else { fslots.push_back(out_slots[o]); fpos.push_back((size_t)o); }
  }
  if (!rc && !fslots.empty()) {
    std::vector<hgpu_array*> fres(fslots.size(), nullptr);
    rc = hgpu_fused_map(ctx, n_in, ins.data(), n_instr, prog, (int)fslots.size(), fslots.data(), fres.data());
    if (!rc) for (size_t i = 0; i < fpos.size(); ++i) res[fpos[i]] = fres[i];
  }
  hgpu_release(c);
  if (rc) {
    for (auto* r : res) if (r) hgpu_release(r);
    return rc;
  }
  for (int o = 0; o < n_out; ++o) outs[o] = res[(size_t)o];
  return HGPU_OK;
}
