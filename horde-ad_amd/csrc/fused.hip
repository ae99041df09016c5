// Fused elementwise maps: a chain of Num / Floating / comparison / conditional
// / conversion operations over same-shaped views evaluated in ONE pass.
//
// horde-ad's interpreter calls `+`, `*`, `sin` ... one at a time
// (src/HordeAd/Core/AstInterpret.hs:187-194) and the `Concrete` backend runs a
// full pass over memory for each.  The host layer instead collects such calls
// into a small straight-line program (inputs = views, one instruction per
// call) and hands it over here; the program is turned into HIP source, compiled
// once with hiprtc for gfx950 (cached by source text) and launched as one
// kernel with any number of outputs, so every input element is read once and
// every output element written once -- the traffic the HBM roofline is
// computed from.
//
// Kernel shape: grid-stride loop, 256 lanes per block; when every non-scalar
// input is dense each lane moves 16-byte vectors, otherwise each lane walks the
// merged index space of the inputs (same decomposition as the eager kernels).
#include <hip/hiprtc.h>

#include <memory>
#include <unordered_map>

#include "common.hpp"
#include "fused_gen.hpp"

using namespace hg;

namespace {

using namespace hg::fusedgen;

struct Compiled {
  hipModule_t mod;
  hipFunction_t fn;
};

std::map<std::string, Compiled>& cache_of(hgpu_ctx* ctx) {
  // one cache per context, kept in the context's generic pointer map
  auto it = ctx->jit_cache.find("__fused__");
  if (it == ctx->jit_cache.end()) it = ctx->jit_cache.emplace("__fused__", new std::map<std::string, Compiled>()).first;
  return *static_cast<std::map<std::string, Compiled>*>(it->second);
}

int compile(hgpu_ctx* ctx, const std::string& src, Compiled* out, const char* kname = "fused_map") {
  std::vector<char> code;
  int rc = rtc_compile(ctx, src, kname, &code);
  if (rc) return rc;
  hipError_t e = hipModuleLoadData(&out->mod, code.data());
  if (e != hipSuccess) return check_hip(ctx, e, "hipModuleLoadData");
  e = hipModuleGetFunction(&out->fn, out->mod, kname);
  if (e != hipSuccess) return check_hip(ctx, e, "hipModuleGetFunction");
  return HGPU_OK;
}

// Kernels found again by what their text depends on (the inputs' layouts and the program).
struct Known { Compiled c; std::string text; };
const Known* find_known(hgpu_ctx* ctx, const Key& key) {
  std::lock_guard<std::mutex> lk(ctx->launch_mu);
  auto kit = ctx->jit_cache.find("__fused_known__");
  if (kit == ctx->jit_cache.end()) return nullptr;
  auto& known = *static_cast<std::unordered_map<std::string, Known>*>(kit->second);
  auto it = known.find(key.bytes);
  return it == known.end() ? nullptr : &it->second;
}
// The kernel of a call: the known one (`hit`; with HORDEAD_GPU_CHECK_KEYS its text is compared with the one just written),
// else the one with the text `src`, compiled if need be and remembered under the key.  Call with launch_mu held.
int kernel_for(hgpu_ctx* ctx, const Key& key, const Known* hit, const std::string& src, const char* kname, Compiled* out) {
  if (hit) {
    if (check_keys() && hit->text != src) return fail(ctx, HGPU_ERR_DEVICE, "%s: two different kernels under one key", kname);
    *out = hit->c;
    return HGPU_OK;
  }
  auto& cache = cache_of(ctx);
  auto it = cache.find(src);
  if (it == cache.end()) {
    Compiled c;
    int rc = compile(ctx, src, &c, kname);
    if (rc) return rc;
    it = cache.emplace(src, c).first;
  }
  auto kit = ctx->jit_cache.find("__fused_known__");
  if (kit == ctx->jit_cache.end()) kit = ctx->jit_cache.emplace("__fused_known__", new std::unordered_map<std::string, Known>()).first;
  static_cast<std::unordered_map<std::string, Known>*>(kit->second)->emplace(key.bytes, Known{it->second, check_keys() ? src : std::string()});
  *out = it->second;
  return HGPU_OK;
}

constexpr int kMaxIn = 12, kMaxOut = 6, kMaxInstr = 96;

struct FDims {
  int nd;
  int64_t shape[HG_KDIMS];
  int64_t st[kMaxIn][HG_KDIMS];
};

}  // namespace

namespace hg {
int sum_partials(hgpu_ctx* ctx, int dtype, int64_t n, int parts, const void* part, void* out);
}

// hgpu_fused_map, and with sum_slot >= 0 hgpu_fused_map_dimsum: the same pass
// also adds up slot sum_slot over every dim but keep_dim.
static int fused_map_impl(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int n_out, const int* out_slots,
                          hgpu_array** outs, int sum_slot, int keep_dim, hgpu_array** sum) {
  if (!ctx || !in || !prog || !out_slots || !outs) return HGPU_ERR_INVALID;
  if (n_in < 1 || n_in > kMaxIn || n_out < 1 || n_out > kMaxOut || n_instr < 1 || n_instr > kMaxInstr)
    return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_map: %d inputs, %d instructions, %d outputs", n_in, n_instr, n_out);
  const hgpu_array* a0 = in[0];
  for (int i = 0; i < n_in; ++i) {
    if (!in[i]) return HGPU_ERR_INVALID;
    if (!same_shape(in[i], a0)) return fail(ctx, HGPU_ERR_INVALID, "fused_map: input %d has another shape", i);
  }
  std::vector<int> dt;
  if (int rc = check_program(ctx, n_in, in, n_instr, prog, &dt)) return rc;
  for (int o = 0; o < n_out; ++o)
    if (out_slots[o] < 0 || out_slots[o] >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "fused_map: bad output slot");

  int64_t n = nelem(a0);
  std::vector<hgpu_array*> res((size_t)n_out, nullptr);
  auto release_all = [&] { for (auto* r : res) if (r) hgpu_release(r); };
  for (int o = 0; o < n_out; ++o) {
    int rc = new_dense(ctx, dt[(size_t)out_slots[o]], a0->rank, a0->shape, &res[(size_t)o]);
    if (rc) { release_all(); return rc; }
  }
  if (n == 0) {
    for (int o = 0; o < n_out; ++o) outs[o] = res[(size_t)o];
    return HGPU_OK;
  }

  // the sum over all dims but keep_dim: blocks take (element of keep_dim, chunk of the rest)
  int64_t dsO = 1, dsC = 1, dsI = 1;
  if (sum_slot >= 0) {
    if (sum_slot >= n_in + n_instr || keep_dim < 0 || keep_dim >= a0->rank || !sum) { release_all(); return fail(ctx, HGPU_ERR_INVALID, "fused_map_dimsum: bad sum slot or dim"); }
    if (dt[(size_t)sum_slot] != HGPU_F64 && dt[(size_t)sum_slot] != HGPU_F32) { release_all(); return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_map_dimsum: sums of floating-point values only"); }
    for (int d = 0; d < keep_dim; ++d) dsO *= a0->shape[d];
    dsC = a0->shape[keep_dim];
    for (int d = keep_dim + 1; d < a0->rank; ++d) dsI *= a0->shape[d];
  }

  // layout class of every input: 'd' dense, 's' one element broadcast, 'g' general
  std::string layout((size_t)n_in, 'g');
  bool all_simple = true;
  int vec = 16;
  for (int i = 0; i < n_in; ++i) {
    bool all0 = true;
    for (int d = 0; d < in[i]->rank; ++d)
      if (in[i]->shape[d] != 1 && in[i]->strides[d] != 0) all0 = false;
    if (all0) layout[(size_t)i] = 's';
    else if (is_dense(in[i]) && ((uintptr_t)data_ptr(in[i]) & 15) == 0) layout[(size_t)i] = 'd';
    else all_simple = false;
  }
  // vector width: 16 bytes of the widest type involved
  size_t widest = 1;
  for (int i = 0; i < n_in; ++i) widest = std::max(widest, dtype_size(in[i]->dtype));
  for (int o = 0; o < n_out; ++o) widest = std::max(widest, dtype_size(res[(size_t)o]->dtype));
  vec = (int)(16 / widest);
  if (sum_slot >= 0) all_simple = false;     // the summing kernel wants coordinates
  if (!all_simple) vec = 1;

  // general views: the dims merged jointly over all inputs.  For large arrays
  // the merged shape and strides are compiled into the kernel (a division by a
  // constant is a multiplication; 32-bit index arithmetic), one kernel per
  // layout; small ones share a kernel that takes them as an argument.
  FDims fd;
  fd.nd = 0;
  if (!all_simple) {
    const int64_t* sts[kMaxIn];
    for (int i = 0; i < n_in; ++i) sts[i] = in[i]->strides;
    // merge dims jointly over all inputs
    fd.nd = 0;
    for (int d = 0; d < a0->rank; ++d) {
      if (a0->shape[d] == 1) continue;
      bool merged = false;
      if (fd.nd > 0) {
        int p = fd.nd - 1;
        bool ok = true;
        for (int k = 0; k < n_in; ++k)
          if (fd.st[k][p] != sts[k][d] * a0->shape[d]) { ok = false; break; }
        if (ok) {
          fd.shape[p] *= a0->shape[d];
          for (int k = 0; k < n_in; ++k) fd.st[k][p] = sts[k][d];
          merged = true;
        }
      }
      if (!merged) {
        if (fd.nd == HG_KDIMS) { release_all(); return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_map: more than %d merged dims", HG_KDIMS); }
        fd.shape[fd.nd] = a0->shape[d];
        for (int k = 0; k < n_in; ++k) fd.st[k][fd.nd] = sts[k][d];
        fd.nd++;
      }
    }
    if (fd.nd == 0) {
      fd.nd = 1;
      fd.shape[0] = 1;
      for (int k = 0; k < n_in; ++k) fd.st[k][0] = 0;
    }
  }
  const bool bake = !all_simple && n >= (1 << 18) && n < (1LL << 31);
  // A compiled-in layout whose innermost dim holds whole 16-byte groups of the
  // widest type: a lane takes one group.  An input that does not move along that
  // dim is loaded once for the group, one that runs along it (and whose other
  // strides and address keep the groups aligned) with one vector load.
  int gvec = 1;
  std::string inner((size_t)n_in, 'x');   // per input: '0' broadcast, 'v' vector load, 'x' one load per element
  if (bake) {
    const int W = (int)(16 / widest);
    const int in_d = fd.nd - 1;
    if (W > 1 && fd.shape[in_d] % W == 0) {
      gvec = W;
      for (int i = 0; i < n_in; ++i) {
        if (layout[(size_t)i] == 's') continue;
        if (fd.st[i][in_d] == 0) { inner[(size_t)i] = '0'; continue; }
        if (fd.st[i][in_d] != 1) continue;
        bool ok = ((uintptr_t)data_ptr(in[i]) % (dtype_size(in[i]->dtype) * W)) == 0;
        for (int q = 0; q < in_d && ok; ++q) ok = fd.st[i][q] % W == 0;
        if (ok) inner[(size_t)i] = 'v';
      }
    }
  }

  const int dsum_es = sum_slot >= 0 ? (int)dtype_size(dt[(size_t)sum_slot]) : 0;
  int64_t ds_chunks = 1, ds_ch = 0;     // chunks of the summed index range per kept element, vector groups per chunk
  if (sum_slot >= 0) {
    if (!bake || dsC > 65536) { release_all(); return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_map_dimsum: array too small, too large or too many sums"); }
    if (dsI % gvec != 0) {
      gvec = 1;
      std::fill(inner.begin(), inner.end(), 'x');
    }
    const int64_t groups = dsO * (dsI / gvec);      // per kept element
    // 32 blocks per CU: measured on the first convolution layer's cotangent (16 x 784,000 fp64), 8 / 16 / 32 / 64 per CU: 42 / 39 / 36 / 38 us
    ds_chunks = std::max<int64_t>(1, std::min<int64_t>(((int64_t)ctx->num_cu * 32 + dsC - 1) / dsC, groups / 512));
    ds_ch = (groups + ds_chunks - 1) / ds_chunks;
    ds_chunks = (groups + ds_ch - 1) / ds_ch;
  }

  // ---- source
  const char* kernel_name = sum_slot >= 0 ? "fused_map_dimsum" : "fused_map";
  Key key;
  key.put(std::string(kernel_name)).put(n_out).put(sum_slot).put(keep_dim);
  for (int o = 0; o < n_out; ++o) key.put(out_slots[o]);
  put_inputs(key, n_in, in, n_instr, prog);
  const Known* hit = find_known(ctx, key);
  Src s(!hit || check_keys());
  s << kPrelude;
  if (!all_simple) s << "struct FDims { int nd; i64 shape[" << HG_KDIMS << "]; i64 st[" << kMaxIn << "][" << HG_KDIMS << "]; };\n";
  s << "template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };\n";
  s << "extern \"C\" __global__ void __launch_bounds__(256) " << kernel_name << "(i64 n";
  if (!all_simple && !bake) s << ", FDims d";
  for (int i = 0; i < n_in; ++i) s << ", const " << ctype(in[i]->dtype) << "* __restrict__ i" << i;
  for (int o = 0; o < n_out; ++o) s << ", " << ctype(res[(size_t)o]->dtype) << "* __restrict__ o" << o;
  if (sum_slot >= 0) s << ", " << ctype(dt[(size_t)sum_slot]) << "* __restrict__ part";
  s << ") {\n";
  s << "  const i64 step = (i64)gridDim.x * 256;\n";
  for (int i = 0; i < n_in; ++i)
    if (layout[(size_t)i] == 's') s << "  const " << ctype(in[i]->dtype) << " s" << i << " = i" << i << "[0];\n";
  auto emit_program = [&](const char* ind, const std::string& lane_suffix) {
    for (int k = 0; k < n_instr; ++k) {
      const hgpu_fused_instr& q = prog[k];
      int self = n_in + k;
      auto v = [&](int slot) { return "v" + std::to_string(slot) + lane_suffix; };
      s << ind << "const " << ctype(dt[(size_t)self]) << " " << v(self) << " = ";
      switch (q.kind) {
        case HGPU_FUSED_OP1: s << "op1<" << q.op << ">(" << v(q.a) << ")"; break;
        case HGPU_FUSED_OP2: s << "op2<" << q.op << ">(" << v(q.a) << ", " << v(q.b) << ")"; break;
        case HGPU_FUSED_CMP: s << "cmp2<" << q.op << ">(" << v(q.a) << ", " << v(q.b) << ")"; break;
        case HGPU_FUSED_SELECT: s << "(" << v(q.a) << " ? " << v(q.b) << " : " << v(q.c) << ")"; break;
        default: s << "conv<" << q.op << ", " << ctype(q.dtype) << ">(" << v(q.a) << ")"; break;
      }
      s << ";\n";
    }
  };
  if (all_simple) {
    s << "  const i64 nv = n / " << vec << ";\n";
    s << "  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < nv; i += step) {\n";
    for (int i = 0; i < n_in; ++i)
      if (layout[(size_t)i] == 'd') s << "    const Vec<" << ctype(in[i]->dtype) << ", " << vec << "> l" << i << " = reinterpret_cast<const Vec<" << ctype(in[i]->dtype) << ", " << vec << ">*>(i" << i << ")[i];\n";
    for (int o = 0; o < n_out; ++o) s << "    Vec<" << ctype(res[(size_t)o]->dtype) << ", " << vec << "> r" << o << ";\n";
    for (int e = 0; e < vec; ++e) {
      std::string suf = "_" + std::to_string(e);
      s << "    {\n";
      for (int i = 0; i < n_in; ++i) {
        s << "      const " << ctype(in[i]->dtype) << " v" << i << suf << " = ";
        if (layout[(size_t)i] == 's') s << "s" << i; else s << "l" << i << ".v[" << e << "]";
        s << ";\n";
      }
      emit_program("      ", suf);
      for (int o = 0; o < n_out; ++o) s << "      r" << o << ".v[" << e << "] = v" << out_slots[o] << suf << ";\n";
      s << "    }\n";
    }
    for (int o = 0; o < n_out; ++o) s << "    reinterpret_cast<Vec<" << ctype(res[(size_t)o]->dtype) << ", " << vec << ">*>(o" << o << ")[i] = r" << o << ";\n";
    s << "  }\n";
    // tail
    s << "  const i64 t = nv * " << vec << " + (i64)blockIdx.x * 256 + threadIdx.x;\n";
    s << "  if (t < n) {\n";
    for (int i = 0; i < n_in; ++i) {
      s << "    const " << ctype(in[i]->dtype) << " v" << i << "_t = ";
      if (layout[(size_t)i] == 's') s << "s" << i; else s << "i" << i << "[t]";
      s << ";\n";
    }
    emit_program("    ", "_t");
    for (int o = 0; o < n_out; ++o) s << "    o" << o << "[t] = v" << out_slots[o] << "_t;\n";
    s << "  }\n";
  } else if (bake && (gvec > 1 || sum_slot >= 0)) {
    const int W = gvec, in_d = fd.nd - 1;
    if (sum_slot >= 0) {
      // a block adds up one chunk of one kept element; a lane's groups lie 256 apart in the chunk
      const long long IV = dsI / W, groups = dsO * IV;
      s << "  __shared__ double red[4];\n";
      s << "  const unsigned ck = blockIdx.x % " << dsC << "u, chunk = blockIdx.x / " << dsC << "u;\n";
      s << "  const unsigned j1 = (chunk + 1u) * " << ds_ch << "u < " << groups << "u ? (chunk + 1u) * " << ds_ch << "u : " << groups << "u;\n";
      s << "  double acc = 0;\n";
      s << "  for (unsigned j = chunk * " << ds_ch << "u + threadIdx.x; j < j1; j += 256u) {\n";
      s << "    const unsigned jo = j / " << IV << "u;\n";
      s << "    const i64 i = ((i64)jo * " << dsC << " + ck) * " << IV << " + (j - jo * " << IV << "u);\n";
    } else {
      s << "  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n / " << W << "; i += step) {\n";
    }
    s << "    unsigned r = (unsigned)i;\n";
    for (int q = in_d; q >= 0; --q) {
      const long long ext = q == in_d ? fd.shape[q] / W : fd.shape[q];
      if (q > 0) s << "    const unsigned c" << q << " = (r % " << ext << "u)" << (q == in_d ? " * " + std::to_string(W) + "u" : std::string()) << "; r /= " << ext << "u;\n";
      else s << "    const unsigned c0 = r" << (q == in_d ? " * " + std::to_string(W) + "u" : std::string()) << ";\n";
    }
    for (int i = 0; i < n_in; ++i) {
      if (layout[(size_t)i] == 's') continue;
      s << "    const i64 off" << i << " = 0";
      for (int q = 0; q < fd.nd; ++q)
        if (fd.st[i][q] != 0) s << " + (i64)c" << q << " * " << fd.st[i][q] << "ll";
      s << ";\n";
      const char* ct = ctype(in[i]->dtype);
      if (inner[(size_t)i] == 'v') s << "    const Vec<" << ct << ", " << W << "> l" << i << " = *reinterpret_cast<const Vec<" << ct << ", " << W << ">*>(i" << i << " + off" << i << ");\n";
      else if (inner[(size_t)i] == '0') s << "    const " << ct << " b" << i << " = i" << i << "[off" << i << "];\n";
    }
    for (int o = 0; o < n_out; ++o) s << "    Vec<" << ctype(res[(size_t)o]->dtype) << ", " << W << "> r" << o << ";\n";
    for (int e = 0; e < W; ++e) {
      std::string suf = "_" + std::to_string(e);
      s << "    {\n";
      for (int i = 0; i < n_in; ++i) {
        s << "      const " << ctype(in[i]->dtype) << " v" << i << suf << " = ";
        if (layout[(size_t)i] == 's') s << "s" << i;
        else if (inner[(size_t)i] == 'v') s << "l" << i << ".v[" << e << "]";
        else if (inner[(size_t)i] == '0') s << "b" << i;
        else s << "i" << i << "[off" << i << " + " << (long long)e * fd.st[i][in_d] << "ll]";
        s << ";\n";
      }
      emit_program("      ", suf);
      for (int o = 0; o < n_out; ++o) s << "      r" << o << ".v[" << e << "] = v" << out_slots[o] << suf << ";\n";
      if (sum_slot >= 0) s << "      acc += (double)v" << sum_slot << suf << ";\n";
      s << "    }\n";
    }
    for (int o = 0; o < n_out; ++o) s << "    reinterpret_cast<Vec<" << ctype(res[(size_t)o]->dtype) << ", " << W << ">*>(o" << o << ")[i] = r" << o << ";\n";
    s << "  }\n";
    if (sum_slot >= 0) {
      s << "  for (int off = 32; off > 0; off >>= 1) {\n"
           "    unsigned long long u = *reinterpret_cast<unsigned long long*>(&acc);\n"
           "    unsigned lo = __shfl_down((unsigned)(u & 0xffffffffu), off, 64), hi = __shfl_down((unsigned)(u >> 32), off, 64);\n"
           "    unsigned long long w = ((unsigned long long)hi << 32) | lo;\n"
           "    acc += *reinterpret_cast<double*>(&w);\n  }\n";
      s << "  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;\n  __syncthreads();\n";
      s << "  if (threadIdx.x == 0) part[(i64)chunk * " << dsC << " + ck] = (" << ctype(dt[(size_t)sum_slot]) << ")((red[0] + red[1]) + (red[2] + red[3]));\n";
    }
  } else if (bake) {
    s << "  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {\n";
    s << "    unsigned r = (unsigned)i;\n";
    for (int q = fd.nd - 1; q >= 0; --q) {
      if (q > 0) s << "    const unsigned c" << q << " = r % " << fd.shape[q] << "u; r /= " << fd.shape[q] << "u;\n";
      else s << "    const unsigned c0 = r;\n";
    }
    for (int i = 0; i < n_in; ++i) {
      if (layout[(size_t)i] == 's') continue;
      s << "    const i64 off" << i << " = 0";
      for (int q = 0; q < fd.nd; ++q)
        if (fd.st[i][q] != 0) s << " + (i64)c" << q << " * " << fd.st[i][q] << "ll";
      s << ";\n";
    }
    for (int i = 0; i < n_in; ++i) {
      s << "    const " << ctype(in[i]->dtype) << " v" << i << "_g = ";
      if (layout[(size_t)i] == 's') s << "s" << i; else s << "i" << i << "[off" << i << "]";
      s << ";\n";
    }
    emit_program("    ", "_g");
    for (int o = 0; o < n_out; ++o) s << "    o" << o << "[i] = v" << out_slots[o] << "_g;\n";
    s << "  }\n";
  } else {
    s << "  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {\n";
    s << "    i64 off[" << n_in << "];\n";
    s << "    for (int k = 0; k < " << n_in << "; ++k) off[k] = 0;\n";
    s << "    i64 r = i;\n";
    s << "    for (int q = d.nd - 1; q >= 0; --q) {\n";
    s << "      i64 c = r;\n";
    s << "      if (q > 0) { i64 w = r / d.shape[q]; c = r - w * d.shape[q]; r = w; }\n";
    s << "      for (int k = 0; k < " << n_in << "; ++k) off[k] += c * d.st[k][q];\n";
    s << "    }\n";
    for (int i = 0; i < n_in; ++i) {
      s << "    const " << ctype(in[i]->dtype) << " v" << i << "_g = ";
      if (layout[(size_t)i] == 's') s << "s" << i; else s << "i" << i << "[off[" << i << "]]";
      s << ";\n";
    }
    emit_program("    ", "_g");
    for (int o = 0; o < n_out; ++o) s << "    o" << o << "[i] = v" << out_slots[o] << "_g;\n";
    s << "  }\n";
  }
  s << "}\n";
  std::string src = s.str();

  const char* label = kernel_name;
  if (ctx->profiling && ctx->profile_shapes) {
    std::string sh;
    for (int d = 0; d < a0->rank; ++d) sh += (d ? "x" : "") + std::to_string(a0->shape[d]);
    // strides of the first input that is a general view
    std::string gst;
    for (int i = 0; i < n_in && gst.empty(); ++i)
      if (layout[(size_t)i] == 'g')
        for (int d = 0; d < in[i]->rank; ++d) gst += (d ? ":" : ",g") + std::to_string(in[i]->strides[d]);
    char buf[200];
    snprintf(buf, sizeof buf, "%s[%s,in%d(%s),instr%d(k%d.op%d..),out%d,vec%d,dt%d%s]", kernel_name, sh.c_str(), n_in, layout.c_str(), n_instr, prog[0].kind, prog[0].op, n_out, all_simple ? vec : gvec, a0->dtype, gst.c_str());
    label = intern_label(ctx, buf);
  }
  std::unique_ptr<LaunchGuard> guard(new LaunchGuard(ctx, label, 0, 0));   // ends before the partial sums' own launch
  LaunchGuard& lg = *guard;
  Compiled kernel;
  if (int rc = kernel_for(ctx, key, hit, src, kernel_name, &kernel)) { release_all(); return rc; }
  // algorithmic traffic: every distinct non-broadcast input once, every output once
  double bytes = 0;
  for (int i = 0; i < n_in; ++i) {
    if (layout[(size_t)i] == 's') continue;
    bool dup = false;
    for (int j = 0; j < i; ++j)
      if (data_ptr(in[j]) == data_ptr(in[i]) && layout[(size_t)j] != 's') dup = true;
    int64_t distinct = 1;
    for (int d = 0; d < in[i]->rank; ++d)
      if (in[i]->strides[d] != 0) distinct *= in[i]->shape[d];
    if (!dup) bytes += (double)distinct * dtype_size(in[i]->dtype);
  }
  for (int o = 0; o < n_out; ++o) bytes += (double)n * dtype_size(res[(size_t)o]->dtype);
  if (lg.timed) { ctx->prof.back().bytes = bytes; ctx->prof.back().flops = (double)n * n_instr; }

  std::vector<void*> args;
  int64_t nn = n;
  args.push_back(&nn);
  std::vector<const void*> ptrs((size_t)n_in);
  std::vector<void*> optrs((size_t)n_out);
  if (!all_simple && !bake) args.push_back(&fd);
  for (int i = 0; i < n_in; ++i) { ptrs[(size_t)i] = data_ptr(in[i]); args.push_back(&ptrs[(size_t)i]); }
  for (int o = 0; o < n_out; ++o) { optrs[(size_t)o] = data_ptr(res[(size_t)o]); args.push_back(&optrs[(size_t)o]); }
  int64_t work = all_simple ? (n + vec - 1) / vec : n / gvec;
  unsigned grid = grid_for(work, 256, ctx->num_cu * 16);
  hgpu_array* sums = nullptr;
  hgpu_buffer* part = nullptr;
  void* part_ptr = nullptr;
  if (sum_slot >= 0) {
    int rc = new_dense(ctx, dt[(size_t)sum_slot], 1, &dsC, &sums);
    if (!rc && ds_chunks > 1) rc = buffer_alloc(ctx, (size_t)(dsC * ds_chunks) * (size_t)dsum_es, &part);
    if (rc) { if (sums) hgpu_release(sums); release_all(); return rc; }
    part_ptr = part ? part->ptr : data_ptr(sums);
    args.push_back(&part_ptr);
    grid = (unsigned)(dsC * ds_chunks);
  }
  hipError_t e = launch_module(lg, kernel.fn, grid, 256, args.data());
  if (e != hipSuccess) { if (part) buffer_release(part); if (sums) hgpu_release(sums); release_all(); return check_hip(ctx, e, "fused_map launch"); }
  guard.reset();
  if (part) {
    int rc = hg::sum_partials(ctx, dt[(size_t)sum_slot], dsC, (int)ds_chunks, part->ptr, data_ptr(sums));
    buffer_release(part);
    if (rc) { hgpu_release(sums); release_all(); return rc; }
  }
  for (int o = 0; o < n_out; ++o) outs[o] = res[(size_t)o];
  if (sum_slot >= 0) *sum = sums;
  return HGPU_OK;
}

extern "C" int hgpu_fused_map(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog,
                              int n_out, const int* out_slots, hgpu_array** outs) {
  return fused_map_impl(ctx, n_in, in, n_instr, prog, n_out, out_slots, outs, -1, 0, nullptr);
}

extern "C" int hgpu_fused_map_dimsum(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int n_out, const int* out_slots,
                                     hgpu_array** outs, int sum_slot, int keep_dim, hgpu_array** sum) {
  if (!sum || sum_slot < 0) return HGPU_ERR_INVALID;
  return fused_map_impl(ctx, n_in, in, n_instr, prog, n_out, out_slots, outs, sum_slot, keep_dim, sum);
}

// The first extremum of an elementwise program's result along its trailing
// `n_reduce` dims (taken together, row-major), evaluated on the fly: the
// program's result is never written.  values / indices have the leading dims'
// shape; the index counts positions within the reduced dims.
extern "C" int hgpu_fused_extremum(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int slot,
                                   int n_reduce, int want_max, hgpu_array** values, hgpu_array** indices) {
  if (!ctx || !in || (!prog && n_instr > 0) || !values || !indices) return HGPU_ERR_INVALID;
  if (n_in < 1 || n_in > kMaxIn || n_instr < 0 || n_instr > kMaxInstr) return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_extremum: %d inputs, %d instructions", n_in, n_instr);
  const hgpu_array* a0 = in[0];
  for (int i = 0; i < n_in; ++i) {
    if (!in[i]) return HGPU_ERR_INVALID;
    if (!same_shape(in[i], a0)) return fail(ctx, HGPU_ERR_INVALID, "fused_extremum: input %d has another shape", i);
  }
  if (n_reduce < 1 || n_reduce > a0->rank) return fail(ctx, HGPU_ERR_INVALID, "fused_extremum: %d reduced dims of rank %d", n_reduce, a0->rank);
  std::vector<int> dt;
  if (int rc = check_program(ctx, n_in, in, n_instr, prog, &dt)) return rc;
  if (slot < 0 || slot >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "fused_extremum: bad slot");
  const int rank_o = a0->rank - n_reduce;
  int64_t L = 1, n_out = 1;
  for (int d = rank_o; d < a0->rank; ++d) L *= a0->shape[d];
  for (int d = 0; d < rank_o; ++d) n_out *= a0->shape[d];
  if (L < 1) return fail(ctx, HGPU_ERR_INVALID, "fused_extremum: empty reduced dims");
  if (L > 64 || n_out >= (1LL << 31)) return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_extremum: %lld reduced elements per result", (long long)L);
  hgpu_array *v = nullptr, *ix = nullptr;
  int rc = new_dense(ctx, dt[(size_t)slot], rank_o, a0->shape, &v);
  if (rc) return rc;
  rc = new_dense(ctx, HGPU_I64, rank_o, a0->shape, &ix);
  if (rc) { hgpu_release(v); return rc; }
  if (n_out == 0) { *values = v; *indices = ix; return HGPU_OK; }

  std::string layout((size_t)n_in, 'g');
  for (int i = 0; i < n_in; ++i) {
    bool all0 = true;
    for (int d = 0; d < in[i]->rank; ++d)
      if (in[i]->shape[d] != 1 && in[i]->strides[d] != 0) all0 = false;
    if (all0) layout[(size_t)i] = 's';
  }
  // leading dims merged jointly over all inputs
  FDims fd;
  fd.nd = 0;
  for (int d = 0; d < rank_o; ++d) {
    if (a0->shape[d] == 1) continue;
    bool merged = false;
    if (fd.nd > 0) {
      int p = fd.nd - 1;
      bool ok = true;
      for (int k = 0; k < n_in; ++k)
        if (fd.st[k][p] != in[k]->strides[d] * a0->shape[d]) { ok = false; break; }
      if (ok) {
        fd.shape[p] *= a0->shape[d];
        for (int k = 0; k < n_in; ++k) fd.st[k][p] = in[k]->strides[d];
        merged = true;
      }
    }
    if (!merged) {
      if (fd.nd == HG_KDIMS) { hgpu_release(v); hgpu_release(ix); return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_extremum: more than %d merged dims", HG_KDIMS); }
      fd.shape[fd.nd] = a0->shape[d];
      for (int k = 0; k < n_in; ++k) fd.st[k][fd.nd] = in[k]->strides[d];
      fd.nd++;
    }
  }
  // ---- source: shapes and strides are constants of the kernel
  Key key;
  key.put(std::string("fused_extremum")).put(slot).put(n_reduce).put(want_max);
  put_inputs(key, n_in, in, n_instr, prog);
  const Known* hit = find_known(ctx, key);
  Src s(!hit || check_keys());
  s << kPrelude;
  s << "extern \"C\" __global__ void __launch_bounds__(256) fused_extremum(i64 n";
  for (int i = 0; i < n_in; ++i) s << ", const " << ctype(in[i]->dtype) << "* __restrict__ i" << i;
  s << ", " << ctype(dt[(size_t)slot]) << "* __restrict__ ov, i64* __restrict__ oi) {\n";
  s << "  const i64 step = (i64)gridDim.x * 256;\n";
  for (int i = 0; i < n_in; ++i)
    if (layout[(size_t)i] == 's') s << "  const " << ctype(in[i]->dtype) << " s" << i << " = i" << i << "[0];\n";
  s << "  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {\n";
  s << "    unsigned r = (unsigned)i;\n";
  for (int q = fd.nd - 1; q >= 0; --q) {
    if (q > 0) s << "    const unsigned c" << q << " = r % " << fd.shape[q] << "u; r /= " << fd.shape[q] << "u;\n";
    else s << "    const unsigned c0 = r;\n";
  }
  for (int i = 0; i < n_in; ++i) {
    if (layout[(size_t)i] == 's') continue;
    s << "    const " << ctype(in[i]->dtype) << "* p" << i << " = i" << i;
    for (int q = 0; q < fd.nd; ++q)
      if (fd.st[i][q] != 0) s << " + (i64)c" << q << " * " << fd.st[i][q] << "ll";
    s << ";\n";
  }
  s << "    " << ctype(dt[(size_t)slot]) << " best;\n    i64 bi = 0;\n";
  for (int64_t e = 0; e < L; ++e) {
    // offsets of reduced position e
    std::string suf = "_" + std::to_string(e);
    s << "    {\n";
    for (int i = 0; i < n_in; ++i) {
      s << "      const " << ctype(in[i]->dtype) << " v" << i << suf << " = ";
      if (layout[(size_t)i] == 's') { s << "s" << i << ";\n"; continue; }
      int64_t off = 0, rr = e;
      for (int d = a0->rank - 1; d >= rank_o; --d) {
        off += (rr % a0->shape[d]) * in[i]->strides[d];
        rr /= a0->shape[d];
      }
      s << "p" << i << "[" << off << "ll];\n";
    }
    emit_program(s, n_in, n_instr, prog, dt, "      ", suf);
    if (e == 0) s << "      best = v" << slot << suf << ";\n";
    else s << "      if (v" << slot << suf << (want_max ? " > " : " < ") << "best) { best = v" << slot << suf << "; bi = " << e << "; }\n";
    s << "    }\n";
  }
  s << "    ov[i] = best;\n    oi[i] = bi;\n  }\n}\n";
  std::string src = s.str();

  const char* label = "fused_extremum";
  if (ctx->profiling && ctx->profile_shapes) {
    std::string sh;
    for (int d = 0; d < a0->rank; ++d) sh += (d ? "x" : "") + std::to_string(a0->shape[d]);
    char buf[160];
    snprintf(buf, sizeof buf, "fused_extremum[%s,reduce%d,in%d(%s),instr%d]", sh.c_str(), n_reduce, n_in, layout.c_str(), n_instr);
    label = intern_label(ctx, buf);
  }
  double bytes = (double)n_out * (dtype_size(dt[(size_t)slot]) + 8);
  for (int i = 0; i < n_in; ++i) {
    if (layout[(size_t)i] == 's') continue;
    int64_t distinct = 1;
    for (int d = 0; d < in[i]->rank; ++d)
      if (in[i]->strides[d] != 0) distinct *= in[i]->shape[d];
    bytes += (double)distinct * dtype_size(in[i]->dtype);
  }
  LaunchGuard lg(ctx, label, bytes, (double)n_out * L * (n_instr + 1));
  Compiled kernel;
  rc = kernel_for(ctx, key, hit, src, "fused_extremum", &kernel);
  if (rc) { hgpu_release(v); hgpu_release(ix); return rc; }
  std::vector<void*> args;
  int64_t nn = n_out;
  args.push_back(&nn);
  std::vector<const void*> ptrs((size_t)n_in);
  for (int i = 0; i < n_in; ++i) { ptrs[(size_t)i] = data_ptr(in[i]); args.push_back(&ptrs[(size_t)i]); }
  void* pv = data_ptr(v);
  void* pi = data_ptr(ix);
  args.push_back(&pv);
  args.push_back(&pi);
  unsigned grid = grid_for(n_out, 256, ctx->num_cu * 16);
  hipError_t e = launch_module(lg, kernel.fn, grid, 256, args.data());
  if (e != hipSuccess) { hgpu_release(v); hgpu_release(ix); return check_hip(ctx, e, "fused_extremum launch"); }
  *values = v;
  *indices = ix;
  return HGPU_OK;
}

// The sum of all elements of an elementwise program's result, evaluated on the
// fly (the result is never written): per-block partial sums in double / int64,
// added up in a fixed order by a second, one-block launch.  Inputs must be dense
// (16-byte aligned) or one broadcast element; anything else is left to the
// caller (HGPU_ERR_UNSUPPORTED), who writes the result out and sums that.
extern "C" int hgpu_fused_sum(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int slot,
                              hgpu_array** out) {
  if (!ctx || !in || (!prog && n_instr > 0) || !out) return HGPU_ERR_INVALID;
  if (n_in < 1 || n_in > kMaxIn || n_instr < 0 || n_instr > kMaxInstr) return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_sum: %d inputs, %d instructions", n_in, n_instr);
  const hgpu_array* a0 = in[0];
  for (int i = 0; i < n_in; ++i) {
    if (!in[i]) return HGPU_ERR_INVALID;
    if (!same_shape(in[i], a0)) return fail(ctx, HGPU_ERR_INVALID, "fused_sum: input %d has another shape", i);
  }
  std::vector<int> dt;
  if (int rc = check_program(ctx, n_in, in, n_instr, prog, &dt)) return rc;
  if (slot < 0 || slot >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "fused_sum: bad slot");
  const int odt = dt[(size_t)slot];
  if (odt == HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "fused_sum: Bool values have no sum");
  std::string layout((size_t)n_in, 'g');
  size_t widest = dtype_size(odt);
  for (int i = 0; i < n_in; ++i) {
    bool all0 = true;
    for (int d = 0; d < in[i]->rank; ++d)
      if (in[i]->shape[d] != 1 && in[i]->strides[d] != 0) all0 = false;
    if (all0) layout[(size_t)i] = 's';
    else if (is_dense(in[i]) && ((uintptr_t)data_ptr(in[i]) & 15) == 0) layout[(size_t)i] = 'd';
    else return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_sum: input %d is a strided view", i);
    widest = std::max(widest, dtype_size(in[i]->dtype));
  }
  const int vec = (int)(16 / widest);
  const int64_t n = nelem(a0);
  hgpu_array* o = nullptr;
  int rc = n == 0 ? new_zeros(ctx, odt, 0, nullptr, &o) : new_dense(ctx, odt, 0, nullptr, &o);   // the last launch writes it
  if (rc) return rc;
  if (n == 0) { *out = o; return HGPU_OK; }
  const bool fp = dtype_is_float(odt);
  const char* acc = fp ? "double" : "i64";
  // Very few elements: one block of 1024 threads sums them and writes the result.
  const bool single = (n + vec - 1) / vec <= 1024;
  const int NT = single ? 1024 : 256;
  const unsigned grid = single ? 1u : grid_for((n + vec - 1) / vec, 256, ctx->num_cu * 8);
  hgpu_buffer* part = nullptr;
  if (!single) {
    rc = buffer_alloc(ctx, (size_t)grid * 8, &part);
    if (rc) { hgpu_release(o); return rc; }
  }
  auto drop_part = [&] { if (part) buffer_release(part); };
  // Up to 131072 elements (at most a few hundred blocks) the block that finishes last adds the blocks' sums up; beyond, a second launch does
  // (handing a sum over takes a fence per block, and the thousands of blocks of a large array would each pay it).
  const bool ticketed = !single && n <= (1 << 17);
  void* ticket = nullptr;
  if (ticketed) {
    rc = ticket_block(ctx, &ticket);
    if (rc) { drop_part(); hgpu_release(o); return rc; }
  }

  Key key;
  key.put(std::string("fused_sum")).put(slot);
  put_inputs(key, n_in, in, n_instr, prog);
  const Known* hit = find_known(ctx, key);
  Src s(!hit || check_keys());
  s << kPrelude;
  s << "template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };\n";
  s << "typedef " << acc << " ACC;\n";
  s << "__device__ __forceinline__ ACC wave_sum(ACC v) {\n"
       "  for (int off = 32; off > 0; off >>= 1) {\n"
       "    unsigned long long u = *reinterpret_cast<unsigned long long*>(&v);\n"
       "    unsigned lo = __shfl_down((unsigned)(u & 0xffffffffu), off, 64), hi = __shfl_down((unsigned)(u >> 32), off, 64);\n"
       "    unsigned long long w = ((unsigned long long)hi << 32) | lo;\n"
       "    v += *reinterpret_cast<ACC*>(&w);\n"
       "  }\n  return v;\n}\n";
  s << "extern \"C\" __global__ void __launch_bounds__(" << NT << ") fused_sum(i64 n";
  for (int i = 0; i < n_in; ++i) s << ", const " << ctype(in[i]->dtype) << "* __restrict__ i" << i;
  if (single) s << ", " << ctype(odt) << "* __restrict__ out) {\n";
  else if (ticketed) s << ", unsigned long long* part, unsigned int* ticket, " << ctype(odt) << "* __restrict__ out) {\n";
  else s << ", ACC* __restrict__ part) {\n";
  s << "  __shared__ ACC red[" << NT / 64 << "];\n";
  s << "  const i64 step = (i64)gridDim.x * " << NT << ";\n";
  for (int i = 0; i < n_in; ++i)
    if (layout[(size_t)i] == 's') s << "  const " << ctype(in[i]->dtype) << " s" << i << " = i" << i << "[0];\n";
  s << "  ACC acc = 0;\n";
  s << "  const i64 nv = n / " << vec << ";\n";
  s << "  for (i64 i = (i64)blockIdx.x * " << NT << " + threadIdx.x; i < nv; i += step) {\n";
  for (int i = 0; i < n_in; ++i)
    if (layout[(size_t)i] == 'd') s << "    const Vec<" << ctype(in[i]->dtype) << ", " << vec << "> l" << i << " = reinterpret_cast<const Vec<" << ctype(in[i]->dtype) << ", " << vec << ">*>(i" << i << ")[i];\n";
  for (int e = 0; e < vec; ++e) {
    std::string suf = "_" + std::to_string(e);
    s << "    {\n";
    for (int i = 0; i < n_in; ++i) {
      s << "      const " << ctype(in[i]->dtype) << " v" << i << suf << " = ";
      if (layout[(size_t)i] == 's') s << "s" << i; else s << "l" << i << ".v[" << e << "]";
      s << ";\n";
    }
    emit_program(s, n_in, n_instr, prog, dt, "      ", suf);
    s << "      acc += (ACC)v" << slot << suf << ";\n    }\n";
  }
  s << "  }\n";
  s << "  const i64 t = nv * " << vec << " + (i64)blockIdx.x * " << NT << " + threadIdx.x;\n";
  s << "  if (t < n) {\n";
  for (int i = 0; i < n_in; ++i) {
    s << "    const " << ctype(in[i]->dtype) << " v" << i << "_t = ";
    if (layout[(size_t)i] == 's') s << "s" << i; else s << "i" << i << "[t]";
    s << ";\n";
  }
  emit_program(s, n_in, n_instr, prog, dt, "    ", "_t");
  s << "    acc += (ACC)v" << slot << "_t;\n  }\n";
  s << "  acc = wave_sum(acc);\n";
  s << "  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;\n";
  s << "  __syncthreads();\n";
  if (single) s << "  if (threadIdx.x == 0) {\n    ACC tot = 0;\n    for (int k = 0; k < " << NT / 64 << "; ++k) tot += red[k];\n    out[0] = (" << ctype(odt) << ")tot;\n  }\n";
  else if (!ticketed) s << "  if (threadIdx.x == 0) part[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);\n";
  else {
    // The block that finishes last adds the blocks' sums up, always in the same order, and writes the result:
    // every block hands its sum over (store, fence, ticket), the last one to draw a ticket sees them all.
    s << "  __shared__ int last;\n";
    s << "  if (threadIdx.x == 0) {\n    ACC tot = (red[0] + red[1]) + (red[2] + red[3]);\n";
    s << "    __hip_atomic_store(part + blockIdx.x, *reinterpret_cast<unsigned long long*>(&tot), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
    s << "    __threadfence();\n    last = atomicAdd(ticket, 1u) == gridDim.x - 1;\n  }\n";
    s << "  __syncthreads();\n  if (!last) return;\n  __threadfence();\n";
    s << "  acc = 0;\n";
    s << "  for (int i = threadIdx.x; i < (int)gridDim.x; i += 256) {\n";
    s << "    unsigned long long u = __hip_atomic_load(part + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n    acc += *reinterpret_cast<ACC*>(&u);\n  }\n";
    s << "  acc = wave_sum(acc);\n";
    s << "  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;\n";
    s << "  __syncthreads();\n";
    s << "  if (threadIdx.x == 0) {\n    out[0] = (" << ctype(odt) << ")((red[0] + red[1]) + (red[2] + red[3]));\n";
    s << "    __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch\n  }\n";
  }
  s << "}\n";
  if (!single && !ticketed) {
    // second launch: one block adds the partial sums up, in the same order
    s << "extern \"C\" __global__ void __launch_bounds__(256) fused_sum_final(int g, const ACC* __restrict__ part, " << ctype(odt) << "* __restrict__ out) {\n";
    s << "  __shared__ ACC red[4];\n";
    s << "  ACC acc = 0;\n";
    s << "  for (int i = threadIdx.x; i < g; i += 256) acc += part[i];\n";
    s << "  acc = wave_sum(acc);\n";
    s << "  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;\n";
    s << "  __syncthreads();\n";
    s << "  if (threadIdx.x == 0) out[0] = (" << ctype(odt) << ")((red[0] + red[1]) + (red[2] + red[3]));\n";
    s << "}\n";
  }
  std::string src = s.str();

  const char* label = "fused_sum";
  if (ctx->profiling && ctx->profile_shapes) {
    std::string sh;
    for (int d = 0; d < a0->rank; ++d) sh += (d ? "x" : "") + std::to_string(a0->shape[d]);
    char buf[160];
    snprintf(buf, sizeof buf, "fused_sum[%s,in%d(%s),instr%d,vec%d]", sh.c_str(), n_in, layout.c_str(), n_instr, vec);
    label = intern_label(ctx, buf);
  }
  double bytes = 0;
  for (int i = 0; i < n_in; ++i) {
    if (layout[(size_t)i] == 's') continue;
    bool dup = false;
    for (int j = 0; j < i; ++j)
      if (data_ptr(in[j]) == data_ptr(in[i]) && layout[(size_t)j] != 's') dup = true;
    if (!dup) bytes += (double)n * dtype_size(in[i]->dtype);
  }
  LaunchGuard lg(ctx, label, bytes, (double)n * (n_instr + 1));
  Compiled kernel;
  rc = kernel_for(ctx, key, hit, src, "fused_sum", &kernel);
  if (rc) { drop_part(); hgpu_release(o); return rc; }
  std::vector<void*> args;
  int64_t nn = n;
  args.push_back(&nn);
  std::vector<const void*> ptrs((size_t)n_in);
  for (int i = 0; i < n_in; ++i) { ptrs[(size_t)i] = data_ptr(in[i]); args.push_back(&ptrs[(size_t)i]); }
  void* po = data_ptr(o);
  void* pp = single ? nullptr : part->ptr;
  if (!single) args.push_back(&pp);
  if (ticketed) args.push_back(&ticket);
  if (single || ticketed) args.push_back(&po);
  hipFunction_t fin = nullptr;
  hipError_t e = hipSuccess;
  if (!single && !ticketed) e = hipModuleGetFunction(&fin, kernel.mod, "fused_sum_final");
  if (e == hipSuccess) e = launch_module(lg, kernel.fn, grid, (unsigned)NT, args.data(), true, fin == nullptr);
  if (e == hipSuccess && fin) {
    int g = (int)grid;
    void* fargs[] = {&g, &pp, &po};
    e = launch_module(lg, fin, 1, 256, fargs, false, true);
  }
  drop_part();
  if (e != hipSuccess) { hgpu_release(o); return check_hip(ctx, e, "fused_sum launch"); }
  *out = o;
  return HGPU_OK;
}

// hgpu_fused_map with sums: the map's outputs and the sums of some slots from
// one pass over dense inputs.  Per-block partial sums (double / int64), added
// up in a fixed order by the block that finishes last (by a second, one-block launch for large arrays).
extern "C" int hgpu_fused_map_sums(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int n_out,
                                   const int* out_slots, hgpu_array** outs, int n_sum, const int* sum_slots, hgpu_array** sums) {
  if (!ctx || !in || !prog || (n_out > 0 && (!out_slots || !outs)) || (n_sum > 0 && (!sum_slots || !sums))) return HGPU_ERR_INVALID;
  if (n_in < 1 || n_in > kMaxIn || n_out < 0 || n_out > kMaxOut || n_sum < 1 || n_sum > 4 || n_instr < 1 || n_instr > kMaxInstr)
    return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_map_sums: %d inputs, %d instructions, %d outputs, %d sums", n_in, n_instr, n_out, n_sum);
  const hgpu_array* a0 = in[0];
  for (int i = 0; i < n_in; ++i) {
    if (!in[i]) return HGPU_ERR_INVALID;
    if (!same_shape(in[i], a0)) return fail(ctx, HGPU_ERR_INVALID, "fused_map_sums: input %d has another shape", i);
  }
  std::vector<int> dt;
  if (int rc = check_program(ctx, n_in, in, n_instr, prog, &dt)) return rc;
  for (int o = 0; o < n_out; ++o)
    if (out_slots[o] < 0 || out_slots[o] >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "fused_map_sums: bad output slot");
  for (int j = 0; j < n_sum; ++j) {
    if (sum_slots[j] < 0 || sum_slots[j] >= n_in + n_instr) return fail(ctx, HGPU_ERR_INVALID, "fused_map_sums: bad sum slot");
    if (dt[(size_t)sum_slots[j]] == HGPU_BOOL) return fail(ctx, HGPU_ERR_INVALID, "fused_map_sums: Bool values have no sum");
  }
  const int64_t n = nelem(a0);
  if (n == 0) return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_map_sums: empty arrays");
  std::string layout((size_t)n_in, 'g');
  size_t widest = 1;
  for (int i = 0; i < n_in; ++i) {
    bool all0 = true;
    for (int d = 0; d < in[i]->rank; ++d)
      if (in[i]->shape[d] != 1 && in[i]->strides[d] != 0) all0 = false;
    if (all0) layout[(size_t)i] = 's';
    else if (is_dense(in[i]) && ((uintptr_t)data_ptr(in[i]) & 15) == 0) layout[(size_t)i] = 'd';
    else return fail(ctx, HGPU_ERR_UNSUPPORTED, "fused_map_sums: input %d is a strided view", i);
    widest = std::max(widest, dtype_size(in[i]->dtype));
  }
  std::vector<hgpu_array*> res((size_t)n_out, nullptr), sres((size_t)n_sum, nullptr);
  auto release_all = [&] { for (auto* r : res) if (r) hgpu_release(r); for (auto* r : sres) if (r) hgpu_release(r); };
  for (int o = 0; o < n_out; ++o) {
    int rc = new_dense(ctx, dt[(size_t)out_slots[o]], a0->rank, a0->shape, &res[(size_t)o]);
    if (rc) { release_all(); return rc; }
    widest = std::max(widest, dtype_size(res[(size_t)o]->dtype));
  }
  for (int j = 0; j < n_sum; ++j) {
    int rc = new_dense(ctx, dt[(size_t)sum_slots[j]], 0, nullptr, &sres[(size_t)j]);
    if (rc) { release_all(); return rc; }
    widest = std::max(widest, dtype_size(dt[(size_t)sum_slots[j]]));
  }
  const int vec = (int)(16 / widest);
  // Very few elements: one block of 1024 threads writes the outputs and the finished sums.
  const bool single = (n + vec - 1) / vec <= 1024;
  const int NT = single ? 1024 : 256;
  const unsigned grid = single ? 1u : grid_for((n + vec - 1) / vec, 256, ctx->num_cu * 16);
  hgpu_buffer* part = nullptr;
  int rc = HGPU_OK;
  if (!single) {
    rc = buffer_alloc(ctx, (size_t)grid * 8 * (size_t)n_sum, &part);
    if (rc) { release_all(); return rc; }
  }
  auto drop_part = [&] { if (part) buffer_release(part); };
  // Up to 131072 elements (at most a few hundred blocks) the block that finishes last adds the blocks' sums up; beyond, a second launch
  // does (handing the sums over takes a fence per block, which also waits for the block's share of the outputs
  // to leave the cache: 16.8 M elements with three outputs take 0.42 ms that way, 0.18 ms with two launches).
  const bool ticketed = !single && n <= (1 << 17);
  void* ticket = nullptr;
  if (ticketed) {
    rc = ticket_block(ctx, &ticket);
    if (rc) { drop_part(); release_all(); return rc; }
  }

  Key key;
  key.put(std::string("fused_map_sums")).put(n_out).put(n_sum);
  for (int o = 0; o < n_out; ++o) key.put(out_slots[o]);
  for (int j = 0; j < n_sum; ++j) key.put(sum_slots[j]);
  put_inputs(key, n_in, in, n_instr, prog);
  const Known* hit = find_known(ctx, key);
  Src s(!hit || check_keys());
  s << kPrelude;
  s << "template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };\n";
  s << "template <typename A> __device__ __forceinline__ A wave_sum(A v) {\n"
       "  for (int off = 32; off > 0; off >>= 1) {\n"
       "    unsigned long long u = *reinterpret_cast<unsigned long long*>(&v);\n"
       "    unsigned lo = __shfl_down((unsigned)(u & 0xffffffffu), off, 64), hi = __shfl_down((unsigned)(u >> 32), off, 64);\n"
       "    unsigned long long w = ((unsigned long long)hi << 32) | lo;\n"
       "    v += *reinterpret_cast<A*>(&w);\n"
       "  }\n  return v;\n}\n";
  auto acc_t = [&](int j) { return dtype_is_float(dt[(size_t)sum_slots[j]]) ? "double" : "i64"; };
  s << "extern \"C\" __global__ void __launch_bounds__(" << NT << ") fused_map_sums(i64 n";
  for (int i = 0; i < n_in; ++i) s << ", const " << ctype(in[i]->dtype) << "* __restrict__ i" << i;
  for (int o = 0; o < n_out; ++o) s << ", " << ctype(res[(size_t)o]->dtype) << "* __restrict__ o" << o;
  if (ticketed) s << ", unsigned long long* part, unsigned int* ticket";
  else if (!single) s << ", unsigned long long* __restrict__ part";
  if (single || ticketed) for (int j = 0; j < n_sum; ++j) s << ", " << ctype(dt[(size_t)sum_slots[j]]) << "* __restrict__ sum" << j;
  s << ") {\n";
  s << "  __shared__ unsigned long long red[" << NT / 64 << "];\n";
  s << "  const i64 step = (i64)gridDim.x * " << NT << ";\n";
  for (int i = 0; i < n_in; ++i)
    if (layout[(size_t)i] == 's') s << "  const " << ctype(in[i]->dtype) << " s" << i << " = i" << i << "[0];\n";
  for (int j = 0; j < n_sum; ++j) s << "  " << acc_t(j) << " acc" << j << " = 0;\n";
  s << "  const i64 nv = n / " << vec << ";\n";
  s << "  for (i64 i = (i64)blockIdx.x * " << NT << " + threadIdx.x; i < nv; i += step) {\n";
  for (int i = 0; i < n_in; ++i)
    if (layout[(size_t)i] == 'd') s << "    const Vec<" << ctype(in[i]->dtype) << ", " << vec << "> l" << i << " = reinterpret_cast<const Vec<" << ctype(in[i]->dtype) << ", " << vec << ">*>(i" << i << ")[i];\n";
  for (int o = 0; o < n_out; ++o) s << "    Vec<" << ctype(res[(size_t)o]->dtype) << ", " << vec << "> r" << o << ";\n";
  for (int e = 0; e < vec; ++e) {
    std::string suf = "_" + std::to_string(e);
    s << "    {\n";
    for (int i = 0; i < n_in; ++i) {
      s << "      const " << ctype(in[i]->dtype) << " v" << i << suf << " = ";
      if (layout[(size_t)i] == 's') s << "s" << i; else s << "l" << i << ".v[" << e << "]";
      s << ";\n";
    }
    emit_program(s, n_in, n_instr, prog, dt, "      ", suf);
    for (int o = 0; o < n_out; ++o) s << "      r" << o << ".v[" << e << "] = v" << out_slots[o] << suf << ";\n";
    for (int j = 0; j < n_sum; ++j) s << "      acc" << j << " += (" << acc_t(j) << ")v" << sum_slots[j] << suf << ";\n";
    s << "    }\n";
  }
  for (int o = 0; o < n_out; ++o) s << "    reinterpret_cast<Vec<" << ctype(res[(size_t)o]->dtype) << ", " << vec << ">*>(o" << o << ")[i] = r" << o << ";\n";
  s << "  }\n";
  s << "  const i64 t = nv * " << vec << " + (i64)blockIdx.x * " << NT << " + threadIdx.x;\n";
  s << "  if (t < n) {\n";
  for (int i = 0; i < n_in; ++i) {
    s << "    const " << ctype(in[i]->dtype) << " v" << i << "_t = ";
    if (layout[(size_t)i] == 's') s << "s" << i; else s << "i" << i << "[t]";
    s << ";\n";
  }
  emit_program(s, n_in, n_instr, prog, dt, "    ", "_t");
  for (int o = 0; o < n_out; ++o) s << "    o" << o << "[t] = v" << out_slots[o] << "_t;\n";
  for (int j = 0; j < n_sum; ++j) s << "    acc" << j << " += (" << acc_t(j) << ")v" << sum_slots[j] << "_t;\n";
  s << "  }\n";
  for (int j = 0; j < n_sum; ++j) {
    s << "  acc" << j << " = wave_sum(acc" << j << ");\n";
    s << "  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = *reinterpret_cast<unsigned long long*>(&acc" << j << ");\n";
    s << "  __syncthreads();\n";
    if (single) {
      s << "  if (threadIdx.x == 0) {\n    " << acc_t(j) << " tot = 0;\n    for (int k = 0; k < " << NT / 64 << "; ++k) tot += *reinterpret_cast<" << acc_t(j) << "*>(&red[k]);\n";
      s << "    sum" << j << "[0] = (" << ctype(dt[(size_t)sum_slots[j]]) << ")tot;\n  }\n";
    } else {
      s << "  if (threadIdx.x == 0) {\n    " << acc_t(j) << " t4[4];\n    for (int k = 0; k < 4; ++k) t4[k] = *reinterpret_cast<" << acc_t(j) << "*>(&red[k]);\n";
      s << "    " << acc_t(j) << " tot = (t4[0] + t4[1]) + (t4[2] + t4[3]);\n";
      if (ticketed) s << "    __hip_atomic_store(part + ((i64)" << j << " * gridDim.x + blockIdx.x), *reinterpret_cast<unsigned long long*>(&tot), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n  }\n";
      else s << "    part[(i64)" << j << " * gridDim.x + blockIdx.x] = *reinterpret_cast<unsigned long long*>(&tot);\n  }\n";
    }
    s << "  __syncthreads();\n";
  }
  if (ticketed) {
    // The block that finishes last adds the blocks' sums up, always in the same order, and writes the results:
    // every block hands its sums over (stores, fence, ticket), the last one to draw a ticket sees them all.
    s << "  __shared__ int last;\n";
    s << "  if (threadIdx.x == 0) {\n    __threadfence();\n    last = atomicAdd(ticket, 1u) == gridDim.x - 1;\n  }\n";
    s << "  __syncthreads();\n  if (!last) return;\n  __threadfence();\n  const int g = (int)gridDim.x;\n";
    for (int j = 0; j < n_sum; ++j) {
      s << "  {\n    " << acc_t(j) << " acc = 0;\n";
      s << "    for (int i = threadIdx.x; i < g; i += 256) {\n";
      s << "      unsigned long long u = __hip_atomic_load(part + ((i64)" << j << " * g + i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n      acc += *reinterpret_cast<" << acc_t(j) << "*>(&u);\n    }\n";
      s << "    acc = wave_sum(acc);\n    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = *reinterpret_cast<unsigned long long*>(&acc);\n    __syncthreads();\n";
      s << "    if (threadIdx.x == 0) {\n      " << acc_t(j) << " t4[4];\n      for (int k = 0; k < 4; ++k) t4[k] = *reinterpret_cast<" << acc_t(j) << "*>(&red[k]);\n";
      s << "      sum" << j << "[0] = (" << ctype(dt[(size_t)sum_slots[j]]) << ")((t4[0] + t4[1]) + (t4[2] + t4[3]));\n    }\n    __syncthreads();\n  }\n";
    }
    s << "  if (threadIdx.x == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch\n";
  }
  s << "}\n";
  if (!single && !ticketed) {
    // second launch: block j adds the partial sums of sum j, in the same order
    s << "extern \"C\" __global__ void __launch_bounds__(256) fused_map_sums_final(int g, const unsigned long long* __restrict__ part";
    for (int j = 0; j < n_sum; ++j) s << ", " << ctype(dt[(size_t)sum_slots[j]]) << "* __restrict__ out" << j;
    s << ") {\n  __shared__ unsigned long long red[4];\n";
    for (int j = 0; j < n_sum; ++j) {
      s << "  if (blockIdx.x == " << j << ") {\n    " << acc_t(j) << " acc = 0;\n";
      s << "    for (int i = threadIdx.x; i < g; i += 256) acc += *reinterpret_cast<const " << acc_t(j) << "*>(&part[(i64)" << j << " * g + i]);\n";
      s << "    acc = wave_sum(acc);\n    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = *reinterpret_cast<unsigned long long*>(&acc);\n    __syncthreads();\n";
      s << "    if (threadIdx.x == 0) {\n      " << acc_t(j) << " t4[4];\n      for (int k = 0; k < 4; ++k) t4[k] = *reinterpret_cast<" << acc_t(j) << "*>(&red[k]);\n";
      s << "      out" << j << "[0] = (" << ctype(dt[(size_t)sum_slots[j]]) << ")((t4[0] + t4[1]) + (t4[2] + t4[3]));\n    }\n  }\n";
    }
    s << "}\n";
  }
  std::string src = s.str();

  const char* label = "fused_map_sums";
  if (ctx->profiling && ctx->profile_shapes) {
    std::string sh;
    for (int d = 0; d < a0->rank; ++d) sh += (d ? "x" : "") + std::to_string(a0->shape[d]);
    char buf[160];
    snprintf(buf, sizeof buf, "fused_map_sums[%s,in%d(%s),instr%d,out%d,sums%d,vec%d]", sh.c_str(), n_in, layout.c_str(), n_instr, n_out, n_sum, vec);
    label = intern_label(ctx, buf);
  }
  double bytes = 0;
  for (int i = 0; i < n_in; ++i) {
    if (layout[(size_t)i] == 's') continue;
    bool dup = false;
    for (int k = 0; k < i; ++k)
      if (data_ptr(in[k]) == data_ptr(in[i]) && layout[(size_t)k] != 's') dup = true;
    if (!dup) bytes += (double)n * dtype_size(in[i]->dtype);
  }
  for (int o = 0; o < n_out; ++o) bytes += (double)n * dtype_size(res[(size_t)o]->dtype);
  LaunchGuard lg(ctx, label, bytes, (double)n * n_instr);
  Compiled kernel;
  rc = kernel_for(ctx, key, hit, src, "fused_map_sums", &kernel);
  if (rc) { drop_part(); release_all(); return rc; }
  std::vector<void*> args;
  int64_t nn = n;
  args.push_back(&nn);
  std::vector<const void*> ptrs((size_t)n_in);
  std::vector<void*> optrs((size_t)n_out), sptrs((size_t)n_sum);
  for (int i = 0; i < n_in; ++i) { ptrs[(size_t)i] = data_ptr(in[i]); args.push_back(&ptrs[(size_t)i]); }
  for (int o = 0; o < n_out; ++o) { optrs[(size_t)o] = data_ptr(res[(size_t)o]); args.push_back(&optrs[(size_t)o]); }
  for (int j = 0; j < n_sum; ++j) sptrs[(size_t)j] = data_ptr(sres[(size_t)j]);
  void* pp = part ? part->ptr : nullptr;
  if (!single) args.push_back(&pp);
  if (ticketed) args.push_back(&ticket);
  if (single || ticketed) for (int j = 0; j < n_sum; ++j) args.push_back(&sptrs[(size_t)j]);
  hipFunction_t fin = nullptr;
  hipError_t e = hipSuccess;
  if (!single && !ticketed) e = hipModuleGetFunction(&fin, kernel.mod, "fused_map_sums_final");
  if (e == hipSuccess) e = launch_module(lg, kernel.fn, grid, (unsigned)NT, args.data(), true, fin == nullptr);
  if (e == hipSuccess && fin) {
    int g = (int)grid;
    std::vector<void*> fargs = {&g, &pp};
    for (int j = 0; j < n_sum; ++j) fargs.push_back(&sptrs[(size_t)j]);
    e = launch_module(lg, fin, (unsigned)n_sum, 256, fargs.data(), false, true);
  }
  drop_part();
  if (e != hipSuccess) { release_all(); return check_hip(ctx, e, "fused_map_sums launch"); }
  for (int o = 0; o < n_out; ++o) outs[o] = res[(size_t)o];
  for (int j = 0; j < n_sum; ++j) sums[j] = sres[(size_t)j];
  return HGPU_OK;
}
