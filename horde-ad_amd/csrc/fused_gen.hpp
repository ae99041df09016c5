// Pieces of the run-time code generators that turn elementwise programs
// (hgpu_fused_instr) into HIP source: the C type of a dtype, the device-side
// meaning of the opcodes, the type check of a program and the emitter of its
// straight-line code.  Shared by the fused maps and by the matrix-product
// kernels that run a program over their result or their operands.
#pragma once
#include <charconv>
#include <cstdlib>
#include <string>
#include <type_traits>
#include <vector>

#include "common.hpp"

namespace hg {
namespace fusedgen {

// The text of a generated kernel, appended to piece by piece: the interface of
// an output stream for text and integers, without a stream's locale and virtual
// calls.  A compiled kernel is kept under its text; calls find it under a Key
// (below) without writing the text again.
struct Src {
  std::string text;
  bool on = true;   // false: the kernel is known already, nothing is written (the generator still runs: it also works out how to launch)
  Src() { text.reserve(16384); }
  explicit Src(bool write) : on(write) { if (on) text.reserve(16384); }
  Src& operator<<(const char* t) { if (on) text.append(t); return *this; }
  Src& operator<<(const std::string& t) { if (on) text.append(t); return *this; }
  Src& operator<<(char c) { if (on) text.push_back(c); return *this; }
  template <typename I, typename std::enable_if<std::is_integral<I>::value && !std::is_same<I, char>::value && !std::is_same<I, bool>::value &&
                                                    !std::is_same<I, signed char>::value && !std::is_same<I, unsigned char>::value, int>::type = 0>
  Src& operator<<(I v) {
    if (!on) return *this;
    char buf[24];
    auto r = std::to_chars(buf, buf + sizeof buf, v);
    text.append(buf, (size_t)(r.ptr - buf));
    return *this;
  }
  Src& operator<<(bool v) { if (on) text.push_back(v ? '1' : '0'); return *this; }
  const std::string& str() const { return text; }
};

// What a generator's text depends on, as bytes: the key under which a call
// finds the kernel that the same call generated before, without writing the
// text again.  With HORDEAD_GPU_CHECK_KEYS set, every such find writes the text
// anyway and compares it with the one kept (a key that leaves out something the
// text depends on then shows as an error instead of a wrong kernel).
struct Key {
  std::string bytes;
  template <typename X, typename std::enable_if<std::is_arithmetic<X>::value, int>::type = 0>
  Key& put(X x) { bytes.append(reinterpret_cast<const char*>(&x), sizeof x); return *this; }
  template <typename X> Key& put(const std::vector<X>& v) { put(v.size()); for (const X& x : v) put(x); return *this; }
  Key& put(int n, const int64_t* v) { put(n); for (int i = 0; i < n; ++i) put(v[i]); return *this; }
  Key& put(const std::string& t) { put(t.size()); bytes.append(t); return *this; }
  Key& put(int n, const hgpu_fused_instr* prog) {
    put(n);
    for (int k = 0; k < n; ++k) put(prog[k].kind).put(prog[k].op).put(prog[k].dtype).put(prog[k].a).put(prog[k].b).put(prog[k].c);
    return *this;
  }
};
// The arrays and the program of a fused call, as far as a kernel's text can depend on them.
inline void put_inputs(Key& k, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog) {
  k.put(n_in);
  for (int i = 0; i < n_in; ++i) k.put(in[i]->dtype).put(in[i]->rank, in[i]->shape).put(in[i]->rank, in[i]->strides).put((int)((uintptr_t)data_ptr(in[i]) & 63));
  k.put(n_instr, prog);
}
inline bool check_keys() {
  static const bool on = getenv("HORDEAD_GPU_CHECK_KEYS") != nullptr;
  return on;
}

inline const char* ctype(int dt) {
  switch (dt) {
    case HGPU_F64: return "double";
    case HGPU_F32: return "float";
    case HGPU_I64: return "long long";
    case HGPU_I32: return "int";
    case HGPU_I16: return "short";
    case HGPU_I8: return "signed char";
    case HGPU_BOOL: return "unsigned char";
  }
  return "void";
}

// The device-side semantics of the opcodes: the same rules as the eager
// kernels (signum of floats keeps zeros, quotH / remH divisor-0 rules, floor).
static const char* const kPrelude = R"HG(
typedef long long i64;
template <typename T> struct is_fp { static constexpr bool value = false; };
template <> struct is_fp<double> { static constexpr bool value = true; };
template <> struct is_fp<float> { static constexpr bool value = true; };
template <int OP, typename T> __device__ __forceinline__ T op1(T x) {
  if constexpr (is_fp<T>::value) {
    if constexpr (OP == 0) return -x;
    else if constexpr (OP == 1) return fabs(x);
    else if constexpr (OP == 2) return x > T(0) ? T(1) : (x < T(0) ? T(-1) : x);
    else if constexpr (OP == 3) return T(1) / x;
    else if constexpr (OP == 4) return exp(x);
    else if constexpr (OP == 5) return log(x);
    else if constexpr (OP == 6) return sqrt(x);
    else if constexpr (OP == 7) return sin(x);
    else if constexpr (OP == 8) return cos(x);
    else if constexpr (OP == 9) return tan(x);
    else if constexpr (OP == 10) return asin(x);
    else if constexpr (OP == 11) return acos(x);
    else if constexpr (OP == 12) return atan(x);
    else if constexpr (OP == 13) return sinh(x);
    else if constexpr (OP == 14) return cosh(x);
    else if constexpr (OP == 15) return tanh(x);
    else if constexpr (OP == 16) return asinh(x);
    else if constexpr (OP == 17) return acosh(x);
    else if constexpr (OP == 18) return atanh(x);
    else return x;
  } else {
    if constexpr (OP == 0) return (T)(-x);
    else if constexpr (OP == 1) return x < 0 ? (T)(-x) : x;
    else if constexpr (OP == 2) return x > 0 ? T(1) : (x < 0 ? T(-1) : T(0));
    else if constexpr (OP == 19) return (T)(x == 0 ? 1 : 0);
    else return x;
  }
}
template <int OP, typename T> __device__ __forceinline__ T op2(T x, T y) {
  if constexpr (is_fp<T>::value) {
    if constexpr (OP == 0) return x + y;
    else if constexpr (OP == 1) return x * y;
    else if constexpr (OP == 2) return x - y;
    else if constexpr (OP == 3) return x / y;
    else if constexpr (OP == 4) return pow(x, y);
    else if constexpr (OP == 5) return log(y) / log(x);
    else if constexpr (OP == 6) return atan2(x, y);
    else if constexpr (OP == 10) return x <= y ? x : y;
    else if constexpr (OP == 11) return x >= y ? x : y;
    else return x;
  } else {
    if constexpr (OP == 0) return (T)(x + y);
    else if constexpr (OP == 1) return (T)(x * y);
    else if constexpr (OP == 2) return (T)(x - y);
    else if constexpr (OP == 7) return y == 0 ? x : (T)(x / y);
    else if constexpr (OP == 8) return y == 0 ? T(0) : (T)(x % y);
    else if constexpr (OP == 9) return y == 0 ? x : (T)(x % y);
    else if constexpr (OP == 10) return x <= y ? x : y;
    else if constexpr (OP == 11) return x >= y ? x : y;
    else if constexpr (OP == 12) return (T)((x != 0 && y != 0) ? 1 : 0);
    else return x;
  }
}
template <int OP, typename T> __device__ __forceinline__ unsigned char cmp2(T x, T y) {
  if constexpr (OP == 0) return x <= y;
  else if constexpr (OP == 1) return x == y;
  else return x < y;
}
template <int CM, typename D, typename S> __device__ __forceinline__ D conv(S x) {
  if constexpr (is_fp<S>::value && !is_fp<D>::value) {
    if constexpr (CM == 1) return (D)(i64)floor((double)x);
    else return (D)(i64)x;
  } else {
    return (D)x;
  }
}
)HG";

// Slot types of a program, with the same checks the eager entry points make.
inline int check_program(hgpu_ctx* ctx, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, std::vector<int>* dtp) {
  std::vector<int>& dt = *dtp;
  dt.assign((size_t)(n_in + n_instr), 0);
  for (int i = 0; i < n_in; ++i) dt[(size_t)i] = in[i]->dtype;
  for (int k = 0; k < n_instr; ++k) {
    const hgpu_fused_instr& q = prog[k];
    int self = n_in + k;
    auto ok = [&](int s) { return s >= 0 && s < self; };
    switch (q.kind) {
      case HGPU_FUSED_OP1:
        if (!ok(q.a) || q.op < 0 || q.op >= HGPU_OP1_COUNT) return fail(ctx, HGPU_ERR_INVALID, "fused_map: bad unary instruction %d", k);
        if (q.op >= HGPU_RECIP && q.op <= HGPU_ATANH && !dtype_is_float(dt[(size_t)q.a])) return fail(ctx, HGPU_ERR_INVALID, "fused_map: floating opcode on a non-floating operand");
        if ((q.op == HGPU_NOT) != (dt[(size_t)q.a] == HGPU_BOOL)) return fail(ctx, HGPU_ERR_INVALID, "fused_map: Bool mismatch");
        dt[(size_t)self] = dt[(size_t)q.a];
        break;
      case HGPU_FUSED_OP2:
        if (!ok(q.a) || !ok(q.b) || q.op < 0 || q.op >= HGPU_OP2_COUNT || dt[(size_t)q.a] != dt[(size_t)q.b]) return fail(ctx, HGPU_ERR_INVALID, "fused_map: bad binary instruction %d", k);
        if (q.op >= HGPU_DIV && q.op <= HGPU_ATAN2 && !dtype_is_float(dt[(size_t)q.a])) return fail(ctx, HGPU_ERR_INVALID, "fused_map: floating opcode on a non-floating operand");
        if (q.op >= HGPU_QUOT && q.op <= HGPU_REM_SCALAR && !dtype_is_int(dt[(size_t)q.a])) return fail(ctx, HGPU_ERR_INVALID, "fused_map: integral opcode on a non-integral operand");
        if ((q.op == HGPU_AND) != (dt[(size_t)q.a] == HGPU_BOOL)) return fail(ctx, HGPU_ERR_INVALID, "fused_map: Bool mismatch");
        dt[(size_t)self] = dt[(size_t)q.a];
        break;
      case HGPU_FUSED_CMP:
        if (!ok(q.a) || !ok(q.b) || q.op < HGPU_LEQ || q.op > HGPU_LT || dt[(size_t)q.a] != dt[(size_t)q.b]) return fail(ctx, HGPU_ERR_INVALID, "fused_map: bad comparison %d", k);
        dt[(size_t)self] = HGPU_BOOL;
        break;
      case HGPU_FUSED_SELECT:
        if (!ok(q.a) || !ok(q.b) || !ok(q.c) || dt[(size_t)q.a] != HGPU_BOOL || dt[(size_t)q.b] != dt[(size_t)q.c]) return fail(ctx, HGPU_ERR_INVALID, "fused_map: bad select %d", k);
        dt[(size_t)self] = dt[(size_t)q.b];
        break;
      case HGPU_FUSED_CONVERT:
        if (!ok(q.a) || dtype_size(q.dtype) == 0) return fail(ctx, HGPU_ERR_INVALID, "fused_map: bad conversion %d", k);
        if (q.op == HGPU_CONV_FLOOR && !(dtype_is_float(dt[(size_t)q.a]) && dtype_is_int(q.dtype))) return fail(ctx, HGPU_ERR_INVALID, "fused_map: floor needs float -> int");
        dt[(size_t)self] = q.dtype;
        break;
      default:
        return fail(ctx, HGPU_ERR_INVALID, "fused_map: unknown instruction kind %d", q.kind);
    }
  }
  return HGPU_OK;
}

// One instruction per line: `const T v<slot><suffix> = ...;`
inline void emit_program(Src& s, int n_in, int n_instr, const hgpu_fused_instr* prog, const std::vector<int>& dt, const char* ind, const std::string& lane_suffix) {
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
}


}  // namespace fusedgen
}  // namespace hg
