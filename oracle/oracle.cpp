// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// CPU restatement of the array semantics of horde-ad's `Concrete` backend
// (reference: src/HordeAd/Core/OpsConcrete.hs, CarriersConcrete.hs, Types.hs,
// over the ox-arrays package, `ox-arrays >= 0.2 && < 0.3`, horde-ad.cabal:207-208,
// which is not vendored in the reference tree).  It exports the SAME C ABI as
// include/hordead_gpu.h under the prefix `horc_` so that one host program can
// be run against either provider.  Only tests, the smoke check and the
// benchmark's CPU-baseline leg load this library; the product never does.
//
// Deliberately simple and independent of the GPU library's code:
//   * every array is DENSE row-major; every "view" operation copies;
//   * single thread, plain loops, one full pass per operation (which is also
//     how the reference executes: one ox-arrays kernel call per AST node);
//   * gather / scatter / index follow the reference's per-position loops:
//       ixInBoundsS / ixsToLinearMaybe   OpsConcrete.hs:923-950
//       tindexZSScalar / tindex0SImpl    OpsConcrete.hs:1477-1506 (OOB => zeros)
//       toneHotS / manyHotNS             OpsConcrete.hs:1430-1446,1516-1525
//       tscatterZSScalar                 OpsConcrete.hs:1581-1619 (ascending
//                                        row-major enumeration of positions,
//                                        accumulation with (+) in that order)
//       tgatherZSScalar                  OpsConcrete.hs:1654-1665
//       targMinS / targMaxS              OpsConcrete.hs:1712-1746 (first extremal
//                                        element of the last dim; tie-break of
//                                        ox-arrays' minIndex assumed "first")
//   * quotH / remH with the divisor-0 rules of Types.hs:394-419 (scalars) and
//     CarriersConcrete.hs:40-56,140-144 (arrays: divisor 0 replaced by 1);
//   * whole-array EqH / OrdH are lexicographic on the row-major sequence
//     (CarriersConcrete.hs:310-331, Ord of storable vectors);
//   * floating-point sums and dot products accumulate in double and round
//     once (ox-arrays' own blocking is not known here; the parity tolerance
//     covers the difference).
//
// What pins each function: numpy and brute force in tests/test_oracle_numpy.py,
// the reference's own known answers in tests/test_reference_kats.py,
// tests/test_highrank_kats.py and tests/test_fold_kats.py (vectors under
// tests/golden/).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../include/hordead_gpu.h"

struct hgpu_ctx {
  std::string err;
};

struct hgpu_array {
  hgpu_ctx* ctx;
  int refs;
  int dtype;
  std::vector<int64_t> shape;
  std::vector<char> data;
};

namespace {

size_t dsize(int dt) {
  switch (dt) {
    case HGPU_F64: case HGPU_I64: return 8;
    case HGPU_F32: case HGPU_I32: return 4;
    case HGPU_I16: return 2;
    case HGPU_I8: case HGPU_BOOL: return 1;
  }
  return 0;
}
bool is_float(int dt) { return dt == HGPU_F64 || dt == HGPU_F32; }
bool is_int(int dt) { return dt >= HGPU_I64 && dt <= HGPU_I8; }

int64_t prod(const std::vector<int64_t>& s, size_t from = 0, size_t to = (size_t)-1) {
  int64_t n = 1;
  if (to > s.size()) to = s.size();
  for (size_t i = from; i < to; ++i) n *= s[i];
  return n;
}

int fail(hgpu_ctx* c, int code, const std::string& msg) {
  if (c) c->err = msg;
  return code;
}

hgpu_array* make(hgpu_ctx* c, int dt, const std::vector<int64_t>& sh) {
  hgpu_array* a = new hgpu_array;
  a->ctx = c;
  a->refs = 1;
  a->dtype = dt;
  a->shape = sh;
  a->data.assign((size_t)prod(sh) * dsize(dt), 0);
  return a;
}

std::vector<int64_t> dense_strides(const std::vector<int64_t>& sh) {
  std::vector<int64_t> st(sh.size());
  int64_t s = 1;
  for (int i = (int)sh.size() - 1; i >= 0; --i) { st[i] = s; s *= sh[i]; }
  return st;
}

// Calls f(linear_out, multi_index) for every index of `sh` in row-major order.
template <typename F>
void for_each_index(const std::vector<int64_t>& sh, F f) {
  int64_t n = prod(sh);
  std::vector<int64_t> ix(sh.size(), 0);
  for (int64_t lin = 0; lin < n; ++lin) {
    f(lin, ix);
    for (int i = (int)sh.size() - 1; i >= 0; --i) {
      if (++ix[i] < sh[i]) break;
      ix[i] = 0;
    }
  }
}

#define DISPATCH(dt, T, ...)                                        \
  switch (dt) {                                                     \
    case HGPU_F64: { using T = double; __VA_ARGS__; break; }        \
    case HGPU_F32: { using T = float; __VA_ARGS__; break; }         \
    case HGPU_I64: { using T = int64_t; __VA_ARGS__; break; }       \
    case HGPU_I32: { using T = int32_t; __VA_ARGS__; break; }       \
    case HGPU_I16: { using T = int16_t; __VA_ARGS__; break; }       \
    case HGPU_I8: { using T = int8_t; __VA_ARGS__; break; }         \
    case HGPU_BOOL: { using T = uint8_t; __VA_ARGS__; break; }      \
    default: break;                                                 \
  }

template <typename T> T* ptr(hgpu_array* a) { return reinterpret_cast<T*>(a->data.data()); }
template <typename T> const T* ptr(const hgpu_array* a) { return reinterpret_cast<const T*>(a->data.data()); }

template <typename T> constexpr bool fp() { return std::is_floating_point<T>::value; }

// interpretAstN1 / interpretAstR1 (AstInterpret.hs:394-421)
template <typename T>
T op1(int op, T x) {
  if constexpr (fp<T>()) {
    switch (op) {
      case HGPU_NEG: return -x;
      case HGPU_ABS: return std::fabs(x);
      case HGPU_SIGNUM: return x > 0 ? T(1) : (x < 0 ? T(-1) : x);
      case HGPU_RECIP: return T(1) / x;
      case HGPU_EXP: return std::exp(x);
      case HGPU_LOG: return std::log(x);
      case HGPU_SQRT: return std::sqrt(x);
      case HGPU_SIN: return std::sin(x);
      case HGPU_COS: return std::cos(x);
      case HGPU_TAN: return std::tan(x);
      case HGPU_ASIN: return std::asin(x);
      case HGPU_ACOS: return std::acos(x);
      case HGPU_ATAN: return std::atan(x);
      case HGPU_SINH: return std::sinh(x);
      case HGPU_COSH: return std::cosh(x);
      case HGPU_TANH: return std::tanh(x);
      case HGPU_ASINH: return std::asinh(x);
      case HGPU_ACOSH: return std::acosh(x);
      case HGPU_ATANH: return std::atanh(x);
    }
  } else {
    switch (op) {
      case HGPU_NEG: return (T)(0 - x);
      case HGPU_ABS: return x < 0 ? (T)(0 - x) : x;
      case HGPU_SIGNUM: return x > 0 ? T(1) : (x < 0 ? T(-1) : T(0));
      case HGPU_NOT: return (T)(x == 0 ? 1 : 0);
    }
  }
  return x;
}

// + * (AstInterpret.hs:187-188), interpretAstR2 (:423-429), interpretAstI2 (:431-435)
template <typename T>
T op2(int op, T x, T y) {
  if constexpr (fp<T>()) {
    switch (op) {
      case HGPU_ADD: return x + y;
      case HGPU_MUL: return x * y;
      case HGPU_SUB: return x - y;
      case HGPU_DIV: return x / y;
      case HGPU_POW: return std::pow(x, y);
      case HGPU_LOGBASE: return std::log(y) / std::log(x);
      case HGPU_ATAN2: return std::atan2(x, y);
      case HGPU_MIN: return x <= y ? x : y;
      case HGPU_MAX: return x >= y ? x : y;
    }
  } else {
    switch (op) {
      case HGPU_ADD: return (T)(x + y);
      case HGPU_MUL: return (T)(x * y);
      case HGPU_SUB: return (T)(x - y);
      case HGPU_QUOT: return y == 0 ? x : (T)(x / y);          // Types.hs:402-419; arrays: quot a 1
      case HGPU_REM: return y == 0 ? T(0) : (T)(x % y);        // arrays: rem a 1 (CarriersConcrete.hs:40-56)
      case HGPU_REM_SCALAR: return y == 0 ? x : (T)(x % y);    // scalars: Types.hs:402-419
      case HGPU_MIN: return x <= y ? x : y;
      case HGPU_MAX: return x >= y ? x : y;
      case HGPU_AND: return (T)((x != 0 && y != 0) ? 1 : 0);
    }
  }
  return x;
}

bool same_shape(const hgpu_array* a, const hgpu_array* b) { return a->shape == b->shape; }

// General helper: out[ix] = a[map(ix)] where map gives a linear source index or -1 for zero.
template <typename F>
static hgpu_array* remap(hgpu_ctx* c, const hgpu_array* a, const std::vector<int64_t>& osh, F map) {
  hgpu_array* o = make(c, a->dtype, osh);
  size_t es = dsize(a->dtype);
  for_each_index(osh, [&](int64_t lin, const std::vector<int64_t>& ix) {
    int64_t src = map(ix);
    if (src >= 0) std::memcpy(o->data.data() + (size_t)lin * es, a->data.data() + (size_t)src * es, es);
  });
  return o;
}


}  // namespace

extern "C" {

int horc_init(int, hgpu_ctx** out) { *out = new hgpu_ctx; return HGPU_OK; }
int horc_shutdown(hgpu_ctx*) { return HGPU_OK; }
int horc_sync(hgpu_ctx*) { return HGPU_OK; }
const char* horc_last_error(hgpu_ctx* c) { return c ? c->err.c_str() : "no context"; }

int horc_upload(hgpu_ctx* c, int dt, int rank, const int64_t* shape, const void* host, hgpu_array** out) {
  if (dsize(dt) == 0 || rank < 0 || rank > HGPU_MAX_RANK) return fail(c, HGPU_ERR_INVALID, "upload: bad dtype or rank");
  std::vector<int64_t> sh(shape, shape + rank);
  for (auto s : sh) if (s < 0) return fail(c, HGPU_ERR_INVALID, "upload: negative extent");
  hgpu_array* a = make(c, dt, sh);
  if (!a->data.empty()) {
    if (!host) { delete a; return fail(c, HGPU_ERR_INVALID, "upload: null host pointer"); }
    std::memcpy(a->data.data(), host, a->data.size());
  }
  *out = a;
  return HGPU_OK;
}
int horc_download(hgpu_ctx*, const hgpu_array* a, void* host) {
  if (!a->data.empty()) std::memcpy(host, a->data.data(), a->data.size());
  return HGPU_OK;
}
int horc_read_scalar(hgpu_ctx* c, const hgpu_array* a, void* host) {
  if (prod(a->shape) != 1) return fail(c, HGPU_ERR_INVALID, "read_scalar: not one element");
  std::memcpy(host, a->data.data(), dsize(a->dtype));
  return HGPU_OK;
}
int horc_retain(hgpu_array* a) { a->refs++; return HGPU_OK; }
int horc_release(hgpu_array* a) { if (a && --a->refs == 0) delete a; return HGPU_OK; }
int horc_rank(const hgpu_array* a) { return (int)a->shape.size(); }
int horc_dtype_of(const hgpu_array* a) { return a->dtype; }
int64_t horc_size(const hgpu_array* a) { return prod(a->shape); }
int horc_shape(const hgpu_array* a, int64_t* s) { std::copy(a->shape.begin(), a->shape.end(), s); return HGPU_OK; }
int horc_strides(const hgpu_array* a, int64_t* s) { auto st = dense_strides(a->shape); std::copy(st.begin(), st.end(), s); return HGPU_OK; }
int horc_is_dense(const hgpu_array*) { return 1; }

// Nested.stranspose: result dim i = source dim perm[i] (OpsConcrete.hs:647-649).
int horc_transpose(hgpu_ctx* c, const hgpu_array* a, int np, const int* perm, hgpu_array** out) {
  int rank = (int)a->shape.size();
  if (np > rank) return fail(c, HGPU_ERR_INVALID, "transpose: permutation longer than rank");
  std::vector<int> p(rank);
  std::vector<bool> seen(rank, false);
  for (int i = 0; i < rank; ++i) {
    p[i] = i < np ? perm[i] : i;
    if (i < np && (p[i] < 0 || p[i] >= np || seen[p[i]])) return fail(c, HGPU_ERR_INVALID, "transpose: not a permutation");
    if (i < np) seen[p[i]] = true;
  }
  std::vector<int64_t> osh(rank);
  for (int i = 0; i < rank; ++i) osh[i] = a->shape[p[i]];
  auto st = dense_strides(a->shape);
  *out = remap(c, a, osh, [&](const std::vector<int64_t>& ix) {
    int64_t s = 0;
    for (int i = 0; i < rank; ++i) s += ix[i] * st[p[i]];
    return s;
  });
  return HGPU_OK;
}

int horc_reshape(hgpu_ctx* c, const hgpu_array* a, int rank, const int64_t* shape, hgpu_array** out) {
  std::vector<int64_t> sh(shape, shape + rank);
  if (prod(sh) != prod(a->shape)) return fail(c, HGPU_ERR_INVALID, "reshape: element counts differ");
  hgpu_array* o = make(c, a->dtype, sh);
  o->data = a->data;
  *out = o;
  return HGPU_OK;
}

int horc_slice(hgpu_ctx* c, const hgpu_array* a, int dim, int64_t start, int64_t len, hgpu_array** out) {
  int rank = (int)a->shape.size();
  if (dim < 0 || dim >= rank || start < 0 || len < 0 || start + len > a->shape[dim]) return fail(c, HGPU_ERR_INVALID, "slice: out of range");
  auto osh = a->shape;
  osh[dim] = len;
  auto st = dense_strides(a->shape);
  *out = remap(c, a, osh, [&](const std::vector<int64_t>& ix) {
    int64_t s = start * st[dim];
    for (int i = 0; i < rank; ++i) s += ix[i] * st[i];
    return s;
  });
  return HGPU_OK;
}

int horc_reverse(hgpu_ctx* c, const hgpu_array* a, int dim, hgpu_array** out) {
  int rank = (int)a->shape.size();
  if (dim < 0 || dim >= rank) return fail(c, HGPU_ERR_INVALID, "reverse: bad dim");
  auto st = dense_strides(a->shape);
  *out = remap(c, a, a->shape, [&](const std::vector<int64_t>& ix) {
    int64_t s = 0;
    for (int i = 0; i < rank; ++i) s += (i == dim ? a->shape[i] - 1 - ix[i] : ix[i]) * st[i];
    return s;
  });
  return HGPU_OK;
}

int horc_replicate(hgpu_ctx* c, const hgpu_array* a, int np, const int64_t* pre, hgpu_array** out) {
  if (np < 0 || np + (int)a->shape.size() > HGPU_MAX_RANK) return fail(c, HGPU_ERR_INVALID, "replicate: rank too large");
  std::vector<int64_t> osh(pre, pre + np);
  for (auto s : osh) if (s < 0) return fail(c, HGPU_ERR_INVALID, "replicate: negative extent");
  osh.insert(osh.end(), a->shape.begin(), a->shape.end());
  hgpu_array* o = make(c, a->dtype, osh);
  int64_t reps = prod(osh, 0, np);
  for (int64_t r = 0; r < reps; ++r)
    if (!a->data.empty()) std::memcpy(o->data.data() + (size_t)r * a->data.size(), a->data.data(), a->data.size());
  *out = o;
  return HGPU_OK;
}

// tindexZSScalar (OpsConcrete.hs:1477-1490): OOB => zeros.
int horc_index_prefix(hgpu_ctx* c, const hgpu_array* a, int n, const int64_t* ix, hgpu_array** out) {
  int rank = (int)a->shape.size();
  if (n < 0 || n > rank) return fail(c, HGPU_ERR_INVALID, "index: too many indices");
  std::vector<int64_t> osh(a->shape.begin() + n, a->shape.end());
  hgpu_array* o = make(c, a->dtype, osh);
  bool ok = true;  // ixInBoundsS
  int64_t lin = 0;
  for (int i = 0; i < n; ++i) {
    if (!(0 <= ix[i] && ix[i] < a->shape[i])) ok = false;
    lin = lin * a->shape[i] + ix[i];
  }
  if (ok && !o->data.empty()) std::memcpy(o->data.data(), a->data.data() + (size_t)lin * o->data.size(), o->data.size());
  *out = o;
  return HGPU_OK;
}

int horc_as_strided(hgpu_ctx* c, const hgpu_array* a, int rank, const int64_t* shape, const int64_t* strides, int64_t offset, hgpu_array** out) {
  std::vector<int64_t> osh(shape, shape + rank);
  int64_t n = prod(a->shape);
  int64_t lo = offset, hi = offset;
  bool empty = false;
  for (int i = 0; i < rank; ++i) {
    if (shape[i] == 0) { empty = true; continue; }
    int64_t span = (shape[i] - 1) * strides[i];
    if (span > 0) hi += span; else lo += span;
  }
  if (!empty && (lo < 0 || hi >= n)) return fail(c, HGPU_ERR_INVALID, "as_strided: outside the source");
  *out = remap(c, a, osh, [&](const std::vector<int64_t>& ix) {
    int64_t s = offset;
    for (int i = 0; i < rank; ++i) s += ix[i] * strides[i];
    return s;
  });
  return HGPU_OK;
}

int horc_materialize(hgpu_ctx* c, const hgpu_array* a, hgpu_array** out) {
  hgpu_array* o = make(c, a->dtype, a->shape);
  o->data = a->data;
  *out = o;
  return HGPU_OK;
}

int horc_pad(hgpu_ctx* c, const hgpu_array* a, const int64_t* lo, const int64_t* hi, hgpu_array** out) {
  int rank = (int)a->shape.size();
  std::vector<int64_t> osh(rank);
  for (int i = 0; i < rank; ++i) {
    if (lo[i] < 0 || hi[i] < 0) return fail(c, HGPU_ERR_INVALID, "pad: negative padding");
    osh[i] = a->shape[i] + lo[i] + hi[i];
  }
  auto st = dense_strides(a->shape);
  *out = remap(c, a, osh, [&](const std::vector<int64_t>& ix) -> int64_t {
    int64_t s = 0;
    for (int i = 0; i < rank; ++i) {
      int64_t j = ix[i] - lo[i];
      if (j < 0 || j >= a->shape[i]) return -1;
      s += j * st[i];
    }
    return s;
  });
  return HGPU_OK;
}

int horc_ewise1(hgpu_ctx* c, int op, const hgpu_array* a, hgpu_array** out) {
  if (op < 0 || op >= HGPU_OP1_COUNT) return fail(c, HGPU_ERR_INVALID, "ewise1: unknown opcode");
  if (op >= HGPU_RECIP && op <= HGPU_ATANH && !is_float(a->dtype)) return fail(c, HGPU_ERR_INVALID, "ewise1: floating opcode on a non-floating array");
  if ((op == HGPU_NOT) != (a->dtype == HGPU_BOOL)) return fail(c, HGPU_ERR_INVALID, "ewise1: Bool mismatch");
  hgpu_array* o = make(c, a->dtype, a->shape);
  int64_t n = prod(a->shape);
  DISPATCH(a->dtype, T, { for (int64_t i = 0; i < n; ++i) ptr<T>(o)[i] = op1<T>(op, ptr<T>(a)[i]); });
  *out = o;
  return HGPU_OK;
}

int horc_ewise2(hgpu_ctx* c, int op, const hgpu_array* a, const hgpu_array* b, hgpu_array** out) {
  if (op < 0 || op >= HGPU_OP2_COUNT) return fail(c, HGPU_ERR_INVALID, "ewise2: unknown opcode");
  if (a->dtype != b->dtype || !same_shape(a, b)) return fail(c, HGPU_ERR_INVALID, "ewise2: operands differ in dtype or shape");
  if (op >= HGPU_DIV && op <= HGPU_ATAN2 && !is_float(a->dtype)) return fail(c, HGPU_ERR_INVALID, "ewise2: floating opcode on a non-floating array");
  if (op >= HGPU_QUOT && op <= HGPU_REM_SCALAR && !is_int(a->dtype)) return fail(c, HGPU_ERR_INVALID, "ewise2: integral opcode on a non-integral array");
  if ((op == HGPU_AND) != (a->dtype == HGPU_BOOL)) return fail(c, HGPU_ERR_INVALID, "ewise2: Bool mismatch");
  hgpu_array* o = make(c, a->dtype, a->shape);
  int64_t n = prod(a->shape);
  DISPATCH(a->dtype, T, { for (int64_t i = 0; i < n; ++i) ptr<T>(o)[i] = op2<T>(op, ptr<T>(a)[i], ptr<T>(b)[i]); });
  *out = o;
  return HGPU_OK;
}

int horc_compare(hgpu_ctx* c, int cmp, const hgpu_array* a, const hgpu_array* b, hgpu_array** out) {
  if (cmp < HGPU_LEQ || cmp > HGPU_LT) return fail(c, HGPU_ERR_INVALID, "compare: unknown opcode");
  if (a->dtype != b->dtype || !same_shape(a, b)) return fail(c, HGPU_ERR_INVALID, "compare: operands differ in dtype or shape");
  hgpu_array* o = make(c, HGPU_BOOL, a->shape);
  int64_t n = prod(a->shape);
  DISPATCH(a->dtype, T, {
    for (int64_t i = 0; i < n; ++i) {
      T x = ptr<T>(a)[i], y = ptr<T>(b)[i];
      ptr<uint8_t>(o)[i] = cmp == HGPU_LEQ ? x <= y : (cmp == HGPU_EQ ? x == y : x < y);
    }
  });
  *out = o;
  return HGPU_OK;
}

// Ord on the row-major element vectors (CarriersConcrete.hs:310-331).
int horc_compare_all(hgpu_ctx* c, int cmp, const hgpu_array* a, const hgpu_array* b, int* result) {
  if (cmp < HGPU_LEQ || cmp > HGPU_LT) return fail(c, HGPU_ERR_INVALID, "compare_all: unknown opcode");
  if (a->dtype != b->dtype || !same_shape(a, b)) return fail(c, HGPU_ERR_INVALID, "compare_all: operands differ in dtype or shape");
  int64_t n = prod(a->shape);
  int ord = 0;  // -1: a < b, 0: equal, 1: a > b, 2: unordered at first difference
  DISPATCH(a->dtype, T, {
    for (int64_t i = 0; i < n && ord == 0; ++i) {
      T x = ptr<T>(a)[i], y = ptr<T>(b)[i];
      if (!(x == y)) ord = x < y ? -1 : (x > y ? 1 : 2);
    }
  });
  *result = cmp == HGPU_EQ ? ord == 0 : (cmp == HGPU_LEQ ? (ord == 0 || ord == -1) : ord == -1);
  return HGPU_OK;
}

int horc_select(hgpu_ctx* c, const hgpu_array* cond, const hgpu_array* a, const hgpu_array* b, hgpu_array** out) {
  if (cond->dtype != HGPU_BOOL || a->dtype != b->dtype || !same_shape(a, b) || !same_shape(cond, a))
    return fail(c, HGPU_ERR_INVALID, "select: operands differ in dtype or shape");
  hgpu_array* o = make(c, a->dtype, a->shape);
  int64_t n = prod(a->shape);
  size_t es = dsize(a->dtype);
  for (int64_t i = 0; i < n; ++i)
    std::memcpy(o->data.data() + i * es, (ptr<uint8_t>(cond)[i] ? a : b)->data.data() + i * es, es);
  *out = o;
  return HGPU_OK;
}

// tsfloor / tsfromIntegral / tscast (OpsConcrete.hs:455-532)
int horc_convert(hgpu_ctx* c, const hgpu_array* a, int dt, int mode, hgpu_array** out) {
  if (dsize(dt) == 0) return fail(c, HGPU_ERR_INVALID, "convert: unknown dtype");
  if (mode == HGPU_CONV_FLOOR && !(is_float(a->dtype) && is_int(dt))) return fail(c, HGPU_ERR_INVALID, "convert: floor needs float -> int");
  hgpu_array* o = make(c, dt, a->shape);
  int64_t n = prod(a->shape);
  DISPATCH(a->dtype, S, {
    DISPATCH(dt, D, {
      for (int64_t i = 0; i < n; ++i) {
        S x = ptr<S>(a)[i];
        if constexpr (fp<S>() && !fp<D>()) ptr<D>(o)[i] = (D)(int64_t)(mode == HGPU_CONV_FLOOR ? std::floor((double)x) : (double)x);
        else ptr<D>(o)[i] = (D)x;
      }
    });
  });
  *out = o;
  return HGPU_OK;
}

// ssumOuter1Prim / ssumAllPrim / sdot / sdot1Inner (OpsConcrete.hs:215-242):
// out[o] = sum_r a[o,r] * b[o,r].
int horc_contract(hgpu_ctx* c, const hgpu_array* a, const hgpu_array* b, int n_keep, hgpu_array** out) {
  int rank = (int)a->shape.size();
  if (n_keep < 0 || n_keep > rank) return fail(c, HGPU_ERR_INVALID, "contract: bad n_keep");
  if (b && (b->dtype != a->dtype || !same_shape(a, b))) return fail(c, HGPU_ERR_INVALID, "contract: operands differ in dtype or shape");
  if (a->dtype == HGPU_BOOL) return fail(c, HGPU_ERR_INVALID, "contract: Bool arrays have no sum");
  std::vector<int64_t> osh(a->shape.begin(), a->shape.begin() + n_keep);
  hgpu_array* o = make(c, a->dtype, osh);
  int64_t no = prod(osh), R = prod(a->shape, n_keep);
  DISPATCH(a->dtype, T, {
    for (int64_t i = 0; i < no; ++i) {
      if constexpr (fp<T>()) {
        double acc = 0;
        for (int64_t r = 0; r < R; ++r) acc += (double)ptr<T>(a)[i * R + r] * (b ? (double)ptr<T>(b)[i * R + r] : 1.0);
        ptr<T>(o)[i] = (T)acc;
      } else {
        T acc = 0;
        for (int64_t r = 0; r < R; ++r) acc = (T)(acc + (T)(ptr<T>(a)[i * R + r] * (b ? ptr<T>(b)[i * R + r] : T(1))));
        ptr<T>(o)[i] = acc;
      }
    }
  });
  *out = o;
  return HGPU_OK;
}

// targMinS / targMaxS (OpsConcrete.hs:1712-1746)
int horc_argminmax_last(hgpu_ctx* c, const hgpu_array* a, int want_max, hgpu_array** out) {
  int rank = (int)a->shape.size();
  if (rank < 1 || a->shape[rank - 1] < 1) return fail(c, HGPU_ERR_INVALID, "argminmax: empty last dim");
  std::vector<int64_t> osh(a->shape.begin(), a->shape.end() - 1);
  hgpu_array* o = make(c, HGPU_I64, osh);
  int64_t no = prod(osh), L = a->shape[rank - 1];
  DISPATCH(a->dtype, T, {
    for (int64_t i = 0; i < no; ++i) {
      const T* p = ptr<T>(a) + i * L;
      int64_t bi = 0;
      for (int64_t j = 1; j < L; ++j)
        if (want_max ? p[j] > p[bi] : p[j] < p[bi]) bi = j;
      ptr<int64_t>(o)[i] = bi;
    }
  });
  *out = o;
  return HGPU_OK;
}

int horc_iota(hgpu_ctx* c, int64_t n, int dt, hgpu_array** out) {
  if (n < 0 || dsize(dt) == 0 || dt == HGPU_BOOL) return fail(c, HGPU_ERR_INVALID, "iota: bad arguments");
  hgpu_array* o = make(c, dt, {n});
  DISPATCH(dt, T, { for (int64_t i = 0; i < n; ++i) ptr<T>(o)[i] = (T)i; });
  *out = o;
  return HGPU_OK;
}

int horc_concat(hgpu_ctx* c, int n, const hgpu_array* const* parts, hgpu_array** out) {
  if (n < 1 || parts[0]->shape.empty()) return fail(c, HGPU_ERR_INVALID, "concat: bad arguments");
  auto osh = parts[0]->shape;
  osh[0] = 0;
  for (int k = 0; k < n; ++k) {
    const hgpu_array* p = parts[k];
    if (p->dtype != parts[0]->dtype || p->shape.size() != osh.size()) return fail(c, HGPU_ERR_INVALID, "concat: parts differ");
    for (size_t i = 1; i < osh.size(); ++i) if (p->shape[i] != osh[i]) return fail(c, HGPU_ERR_INVALID, "concat: parts differ");
    osh[0] += p->shape[0];
  }
  hgpu_array* o = make(c, parts[0]->dtype, osh);
  size_t off = 0;
  for (int k = 0; k < n; ++k) {
    if (!parts[k]->data.empty()) std::memcpy(o->data.data() + off, parts[k]->data.data(), parts[k]->data.size());
    off += parts[k]->data.size();
  }
  *out = o;
  return HGPU_OK;
}

static int check_ix(hgpu_ctx* c, int n_ix, const hgpu_array* const* ix, const std::vector<int64_t>& shm) {
  for (int k = 0; k < n_ix; ++k)
    if (!ix[k] || ix[k]->dtype != HGPU_I64 || ix[k]->shape != shm) return fail(c, HGPU_ERR_INVALID, "index array is not I64 of shape shm");
  return HGPU_OK;
}

// tgatherZSScalar (OpsConcrete.hs:1654-1665) = tbuildS shm shn (tindexZSScalar shn t . f)
int horc_gather(hgpu_ctx* c, const hgpu_array* src, int n_ix, const hgpu_array* const* ix, int rank_m, const int64_t* shm_, hgpu_array** out) {
  int rank = (int)src->shape.size();
  if (n_ix < 0 || n_ix > rank) return fail(c, HGPU_ERR_INVALID, "gather: too many indices");
  std::vector<int64_t> shm(shm_, shm_ + rank_m);
  int rc = check_ix(c, n_ix, ix, shm);
  if (rc) return rc;
  std::vector<int64_t> osh = shm;
  osh.insert(osh.end(), src->shape.begin() + n_ix, src->shape.end());
  if ((int)osh.size() > HGPU_MAX_RANK) return fail(c, HGPU_ERR_INVALID, "gather: result rank too large");
  hgpu_array* o = make(c, src->dtype, osh);
  int64_t M = prod(shm), N = prod(src->shape, n_ix);
  size_t slice = (size_t)N * dsize(src->dtype);
  for (int64_t m = 0; m < M; ++m) {        // tbuildS: every position of shm
    bool ok = true;                        // ixInBoundsS
    int64_t lin = 0;
    for (int k = 0; k < n_ix; ++k) {
      int64_t i = ptr<int64_t>(ix[k])[m];
      if (!(0 <= i && i < src->shape[k])) ok = false;
      lin = lin * src->shape[k] + i;
    }
    if (ok && slice) std::memcpy(o->data.data() + (size_t)m * slice, src->data.data() + (size_t)lin * slice, slice);
  }
  *out = o;
  return HGPU_OK;
}

// tscatterZSScalar (OpsConcrete.hs:1581-1619)
int horc_scatter_add(hgpu_ctx* c, const hgpu_array* src, int n_ix, const hgpu_array* const* ix, int rank_m, const int64_t* shp, int, hgpu_array** out) {
  int rank = (int)src->shape.size();
  if (rank_m < 0 || rank_m > rank || n_ix < 0) return fail(c, HGPU_ERR_INVALID, "scatter: bad ranks");
  if (src->dtype == HGPU_BOOL) return fail(c, HGPU_ERR_INVALID, "scatter: Bool arrays have no sum");
  std::vector<int64_t> shm(src->shape.begin(), src->shape.begin() + rank_m);
  int rc = check_ix(c, n_ix, ix, shm);
  if (rc) return rc;
  std::vector<int64_t> osh(shp, shp + n_ix);
  osh.insert(osh.end(), src->shape.begin() + rank_m, src->shape.end());
  if ((int)osh.size() > HGPU_MAX_RANK) return fail(c, HGPU_ERR_INVALID, "scatter: result rank too large");
  hgpu_array* o = make(c, src->dtype, osh);   // VSM.replicate ... 0
  int64_t M = prod(shm), N = prod(src->shape, rank_m);
  DISPATCH(src->dtype, T, {
    for (int64_t m = 0; m < M; ++m) {         // forM_ (shsEnum shm): ascending row-major
      bool ok = true;                         // ixsToLinearMaybe shp
      int64_t lin = 0;
      for (int k = 0; k < n_ix; ++k) {
        int64_t i = ptr<int64_t>(ix[k])[m];
        if (!(0 <= i && i < shp[k])) ok = false;
        lin = lin * shp[k] + i;
      }
      if (!ok) continue;                      // Nothing -> return ()
      for (int64_t n = 0; n < N; ++n) ptr<T>(o)[lin * N + n] = (T)(ptr<T>(o)[lin * N + n] + ptr<T>(src)[m * N + n]);
    }
  });
  *out = o;
  return HGPU_OK;
}

// tscatterZSScalar (OpsConcrete.hs:1581-1619) with the index function given as
// an affine form: the same loop, the index computed instead of read.
int horc_scatter_affine(hgpu_ctx* c, const hgpu_array* src, int rank_m, int n_ix, const int64_t* c0, const int64_t* coef,
                        const int64_t* shp, hgpu_array** out) {
  int rank = (int)src->shape.size();
  if (rank_m < 0 || rank_m > rank || n_ix < 0) return fail(c, HGPU_ERR_INVALID, "scatter_affine: bad ranks");
  std::vector<int64_t> shm(src->shape.begin(), src->shape.begin() + rank_m);
  std::vector<int64_t> osh(shp, shp + n_ix);
  osh.insert(osh.end(), src->shape.begin() + rank_m, src->shape.end());
  if ((int)osh.size() > HGPU_MAX_RANK) return fail(c, HGPU_ERR_INVALID, "scatter_affine: result rank too large");
  int64_t M = prod(shm), N = prod(src->shape, rank_m);
  std::vector<int64_t> lins((size_t)M);
  std::vector<int64_t> idx((size_t)rank_m, 0);
  for (int64_t m = 0; m < M; ++m) {
    int64_t lin = 0;
    for (int k = 0; k < n_ix; ++k) {
      int64_t i = c0[k];
      for (int d = 0; d < rank_m; ++d) i += coef[d * n_ix + k] * idx[(size_t)d];
      if (!(0 <= i && i < shp[k])) return fail(c, HGPU_ERR_INVALID, "scatter_affine: a position leaves the bounds");
      lin = lin * shp[k] + i;
    }
    lins[(size_t)m] = lin;
    for (int d = rank_m - 1; d >= 0; --d) {
      if (++idx[(size_t)d] < shm[(size_t)d]) break;
      idx[(size_t)d] = 0;
    }
  }
  hgpu_array* o = make(c, src->dtype, osh);
  DISPATCH(src->dtype, T, {
    for (int64_t m = 0; m < M; ++m)
      for (int64_t n = 0; n < N; ++n) ptr<T>(o)[lins[(size_t)m] * N + n] = ptr<T>(src)[m * N + n];
  });
  *out = o;
  return HGPU_OK;
}

// Sum of n contractions of one shape, term by term in order.
int horc_contract_sum(hgpu_ctx* c, int n, const hgpu_array* const* as, const hgpu_array* const* bs, int n_keep, hgpu_array** out) {
  if (n < 1) return fail(c, HGPU_ERR_INVALID, "contract_sum: no terms");
  hgpu_array* acc = nullptr;
  for (int t = 0; t < n; ++t) {
    hgpu_array* part = nullptr;
    int rc = horc_contract(c, as[t], bs[t], n_keep, &part);
    if (rc) return rc;
    if (!acc) { acc = part; continue; }
    hgpu_array* sum = nullptr;
    rc = horc_ewise2(c, HGPU_ADD, acc, part, &sum);
    horc_release(acc);
    horc_release(part);
    if (rc) return rc;
    acc = sum;
  }
  *out = acc;
  return HGPU_OK;
}

// Every array of the checker owns dense data, so assigning is copying the data.
int horc_assign(hgpu_ctx* c, hgpu_array* dst, const hgpu_array* src) {
  if (dst->dtype != src->dtype || dst->shape != src->shape) return fail(c, HGPU_ERR_INVALID, "assign: shapes or dtypes differ");
  if (dst == src) return fail(c, HGPU_ERR_INVALID, "assign: source and destination share memory");
  dst->data = src->data;
  return HGPU_OK;
}

// toneHotS (OpsConcrete.hs:1516-1525)
int horc_onehot(hgpu_ctx* c, const hgpu_array* v, int n, const int64_t* ix, const int64_t* shp, hgpu_array** out) {
  if (n < 0 || n + (int)v->shape.size() > HGPU_MAX_RANK) return fail(c, HGPU_ERR_INVALID, "onehot: rank too large");
  std::vector<int64_t> osh(shp, shp + n);
  osh.insert(osh.end(), v->shape.begin(), v->shape.end());
  hgpu_array* o = make(c, v->dtype, osh);
  bool ok = true;
  int64_t lin = 0;
  for (int i = 0; i < n; ++i) {
    if (!(0 <= ix[i] && ix[i] < shp[i])) ok = false;
    lin = lin * shp[i] + ix[i];
  }
  if (ok && !v->data.empty()) std::memcpy(o->data.data() + (size_t)lin * v->data.size(), v->data.data(), v->data.size());
  *out = o;
  return HGPU_OK;
}

// The meaning of a fused program: the single operations applied in program order.
int horc_fused_map(hgpu_ctx* c, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog,
                   int n_out, const int* out_slots, hgpu_array** outs) {
  // the limits of the device library's kernel generator are part of the entry point's contract: a host layer that
  // exceeds them is caught here, without a device
  if (n_in < 1 || n_in > 12 || n_out < 1 || n_out > 6 || n_instr < 1 || n_instr > 96)
    return fail(c, HGPU_ERR_UNSUPPORTED, "fused_map: " + std::to_string(n_in) + " inputs, " + std::to_string(n_instr) + " instructions, " + std::to_string(n_out) + " outputs");
  std::vector<hgpu_array*> slots;
  std::vector<hgpu_array*> made;
  for (int i = 0; i < n_in; ++i) slots.push_back(const_cast<hgpu_array*>(in[i]));
  int rc = HGPU_OK;
  for (int k = 0; k < n_instr && rc == HGPU_OK; ++k) {
    const hgpu_fused_instr& q = prog[k];
    int self = n_in + k;
    auto ok = [&](int s) { return s >= 0 && s < self; };
    hgpu_array* o = nullptr;
    if (!ok(q.a) || (q.kind != HGPU_FUSED_OP1 && q.kind != HGPU_FUSED_CONVERT && !ok(q.b)) || (q.kind == HGPU_FUSED_SELECT && !ok(q.c))) {
      rc = fail(c, HGPU_ERR_INVALID, "fused_map: bad operand slot");
      break;
    }
    switch (q.kind) {
      case HGPU_FUSED_OP1: rc = horc_ewise1(c, q.op, slots[q.a], &o); break;
      case HGPU_FUSED_OP2: rc = horc_ewise2(c, q.op, slots[q.a], slots[q.b], &o); break;
      case HGPU_FUSED_CMP: rc = horc_compare(c, q.op, slots[q.a], slots[q.b], &o); break;
      case HGPU_FUSED_SELECT: rc = horc_select(c, slots[q.a], slots[q.b], slots[q.c], &o); break;
      case HGPU_FUSED_CONVERT: rc = horc_convert(c, slots[q.a], q.dtype, q.op, &o); break;
      default: rc = fail(c, HGPU_ERR_INVALID, "fused_map: unknown instruction kind");
    }
    if (rc == HGPU_OK) { slots.push_back(o); made.push_back(o); }
  }
  if (rc == HGPU_OK) {
    for (int i = 0; i < n_out; ++i) {
      int s = out_slots[i];
      if (s < 0 || s >= (int)slots.size()) { rc = fail(c, HGPU_ERR_INVALID, "fused_map: bad output slot"); break; }
      if (s < n_in) rc = horc_materialize(c, slots[s], &outs[i]);
      else { outs[i] = slots[s]; horc_retain(slots[s]); }
    }
  }
  for (auto* m : made) horc_release(m);
  return rc;
}

// ---- definitions by composition of the optional fused entry points ----------
// The checker's own table (horc_get_api) leaves them out, so a host program
// run on it takes the reference's route (a gather at the arg-extremum, one pass
// per operation).  horc_get_api_fused offers them, each DEFINED as the single
// entry points applied one after another, so that the host layer's rewrites
// onto them can be exercised without a device and compared with the plain table.

int horc_extremum_last(hgpu_ctx* c, const hgpu_array* a, int want_max, hgpu_array** values, hgpu_array** indices) {
  hgpu_array* ix = nullptr;
  int rc = horc_argminmax_last(c, a, want_max, &ix);
  if (rc) return rc;
  if (values) {
    std::vector<int64_t> osh(a->shape.begin(), a->shape.end() - 1);
    hgpu_array* v = make(c, a->dtype, osh);
    int64_t no = prod(osh), L = a->shape.back();
    size_t es = dsize(a->dtype);
    for (int64_t i = 0; i < no; ++i)
      std::memcpy(v->data.data() + (size_t)i * es, a->data.data() + (size_t)(i * L + ptr<int64_t>(ix)[i]) * es, es);
    *values = v;
  }
  *indices = ix;
  return HGPU_OK;
}

// first extremum of `r` over its trailing n_reduce dims taken together
static int extremum_trailing(hgpu_ctx* c, const hgpu_array* r, int n_reduce, int want_max, hgpu_array** values, hgpu_array** indices) {
  int rank = (int)r->shape.size();
  if (n_reduce < 1 || n_reduce > rank) return fail(c, HGPU_ERR_INVALID, "extremum: bad n_reduce");
  std::vector<int64_t> sh(r->shape.begin(), r->shape.end() - n_reduce);
  sh.push_back(prod(r->shape, (size_t)(rank - n_reduce)));
  hgpu_array* flat = nullptr;
  int rc = horc_reshape(c, r, (int)sh.size(), sh.data(), &flat);
  if (rc) return rc;
  rc = horc_extremum_last(c, flat, want_max, values, indices);
  horc_release(flat);
  return rc;
}

int horc_fused_extremum(hgpu_ctx* c, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int slot, int n_reduce,
                        int want_max, hgpu_array** values, hgpu_array** indices) {
  hgpu_array* r = nullptr;
  int rc = horc_fused_map(c, n_in, in, n_instr, prog, 1, &slot, &r);
  if (rc) return rc;
  rc = extremum_trailing(c, r, n_reduce, want_max, values, indices);
  horc_release(r);
  return rc;
}

int horc_fused_sum(hgpu_ctx* c, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int slot, hgpu_array** out) {
  hgpu_array* r = nullptr;
  int rc = horc_fused_map(c, n_in, in, n_instr, prog, 1, &slot, &r);
  if (rc) return rc;
  rc = horc_contract(c, r, nullptr, 0, out);
  horc_release(r);
  return rc;
}

int horc_contract_map(hgpu_ctx* c, const hgpu_array* a, const hgpu_array* b, int n_keep, int n_in, const hgpu_array* const* in, int n_instr,
                      const hgpu_fused_instr* prog, int n_out, const int* out_slots, hgpu_array** outs, int ext_slot, int view_rank,
                      const int64_t* view_shape, const int64_t* view_strides, int n_reduce, int want_max, hgpu_array** values, hgpu_array** indices) {
  hgpu_array* cr = nullptr;
  int rc = horc_contract(c, a, b, n_keep, &cr);
  if (rc) return rc;
  std::vector<const hgpu_array*> ins(in, in + n_in);
  int n_null = 0;
  for (auto& p : ins)
    if (!p) { p = cr; ++n_null; }
  if (n_null != 1) { horc_release(cr); return fail(c, HGPU_ERR_INVALID, "contract_map: exactly one input must stand for the contraction"); }
  std::vector<int> slots(out_slots, out_slots + n_out);
  if (values) slots.push_back(ext_slot);
  std::vector<hgpu_array*> res(slots.size(), nullptr);
  if (!slots.empty()) rc = horc_fused_map(c, n_in, ins.data(), n_instr, prog, (int)slots.size(), slots.data(), res.data());
  horc_release(cr);
  if (rc) return rc;
  for (int i = 0; i < n_out; ++i) outs[i] = res[(size_t)i];
  if (values) {
    hgpu_array* v = nullptr;
    rc = horc_as_strided(c, res.back(), view_rank, view_shape, view_strides, 0, &v);
    horc_release(res.back());
    if (!rc) {
      rc = extremum_trailing(c, v, n_reduce, want_max, values, indices);
      horc_release(v);
    }
    if (rc)
      for (int i = 0; i < n_out; ++i) { horc_release(outs[i]); outs[i] = nullptr; }
  }
  return rc;
}

// an operand of horc_contract_operands written out: program, merged dims, zero-extension, view
static int operand_array(hgpu_ctx* c, const hgpu_operand* o, hgpu_array** out) {
  if (o->array) { horc_retain(const_cast<hgpu_array*>(o->array)); *out = const_cast<hgpu_array*>(o->array); return HGPU_OK; }
  hgpu_array *e = nullptr, *m = nullptr, *p = nullptr;
  int rc = o->slot < o->n_in ? horc_materialize(c, o->in[o->slot], &e) : horc_fused_map(c, o->n_in, o->in, o->n_instr, o->prog, 1, &o->slot, &e);
  if (rc) return rc;
  rc = horc_reshape(c, e, o->rank_m, o->mshape, &m);
  horc_release(e);
  if (rc) return rc;
  if (o->lo && o->hi) {
    rc = horc_pad(c, m, o->lo, o->hi, &p);
    horc_release(m);
    if (rc) return rc;
  } else {
    p = m;
  }
  rc = horc_as_strided(c, p, o->rank, o->shape, o->strides, o->offset, out);
  horc_release(p);
  return rc;
}

int horc_contract_operands(hgpu_ctx* c, const hgpu_operand* a, const hgpu_operand* b, int n_keep, int, hgpu_array** out) {
  if (getenv("HORC_TRACE")) {
    auto show = [](const char* name, const hgpu_operand* o) {
      if (!o) { fprintf(stderr, "  %s: none\n", name); return; }
      if (o->array) { fprintf(stderr, "  %s: array rank %d\n", name, (int)o->array->shape.size()); return; }
      fprintf(stderr, "  %s: program in%d instr%d, mshape", name, o->n_in, o->n_instr);
      for (int i = 0; i < o->rank_m; ++i) fprintf(stderr, " %lld", (long long)o->mshape[i]);
      if (o->lo) { fprintf(stderr, " lo"); for (int i = 0; i < o->rank_m; ++i) fprintf(stderr, " %lld", (long long)o->lo[i]); fprintf(stderr, " hi"); for (int i = 0; i < o->rank_m; ++i) fprintf(stderr, " %lld", (long long)o->hi[i]); }
      fprintf(stderr, "; view");
      for (int i = 0; i < o->rank; ++i) fprintf(stderr, " %lld:%lld", (long long)o->shape[i], (long long)o->strides[i]);
      fprintf(stderr, " +%lld\n", (long long)o->offset);
    };
    fprintf(stderr, "contract_operands n_keep %d\n", n_keep);
    show("a", a);
    show("b", b);
  }
  hgpu_array *aa = nullptr, *bb = nullptr;
  int rc = operand_array(c, a, &aa);
  if (!rc && b) rc = operand_array(c, b, &bb);
  if (!rc) rc = horc_contract(c, aa, bb, n_keep, out);
  if (aa) horc_release(aa);
  if (bb) horc_release(bb);
  return rc;
}

int horc_fused_map_sums(hgpu_ctx* c, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int n_out, const int* out_slots,
                        hgpu_array** outs, int n_sum, const int* sum_slots, hgpu_array** sums) {
  int rc = HGPU_OK;
  if (n_out > 0) rc = horc_fused_map(c, n_in, in, n_instr, prog, n_out, out_slots, outs);
  for (int j = 0; j < n_sum && !rc; ++j) rc = horc_fused_sum(c, n_in, in, n_instr, prog, sum_slots[j], &sums[j]);
  return rc;
}

// the program by horc_fused_map; the sum of one slot over all dims but keep_dim: that slot written
// out, keep_dim brought to the front (horc_transpose), every other dim summed (horc_contract)
int horc_fused_map_dimsum(hgpu_ctx* c, int n_in, const hgpu_array* const* in, int n_instr, const hgpu_fused_instr* prog, int n_out, const int* out_slots,
                          hgpu_array** outs, int sum_slot, int keep_dim, hgpu_array** sum) {
  if (!sum || sum_slot < 0 || sum_slot >= n_in + n_instr) return fail(c, HGPU_ERR_INVALID, "fused_map_dimsum: bad sum slot");
  int rc = horc_fused_map(c, n_in, in, n_instr, prog, n_out, out_slots, outs);
  if (rc) return rc;
  hgpu_array *v = nullptr, *t = nullptr;
  if (sum_slot < n_in) { v = const_cast<hgpu_array*>(in[sum_slot]); horc_retain(v); }
  else rc = horc_fused_map(c, n_in, in, n_instr, prog, 1, &sum_slot, &v);
  if (!rc) {
    const int rank = horc_rank(v);
    if (keep_dim < 0 || keep_dim >= rank) rc = fail(c, HGPU_ERR_INVALID, "fused_map_dimsum: bad dim");
    if (!rc) {
      std::vector<int> perm{keep_dim};
      for (int d = 0; d < rank; ++d)
        if (d != keep_dim) perm.push_back(d);
      rc = horc_transpose(c, v, (int)perm.size(), perm.data(), &t);
    }
    if (!rc) rc = horc_contract(c, t, nullptr, 1, sum);
  }
  if (t) horc_release(t);
  if (v) horc_release(v);
  if (rc)
    for (int o = 0; o < n_out; ++o) { horc_release(outs[o]); outs[o] = nullptr; }
  return rc;
}

// sum of contractions (terms may differ in their contracted dims), then the program: each term by
// horc_contract, the terms added in order, the program by horc_fused_map
int horc_contract_sum_map(hgpu_ctx* c, int n_terms, const hgpu_array* const* a, const hgpu_array* const* b, int n_keep, int n_in, const hgpu_array* const* in,
                          int n_instr, const hgpu_fused_instr* prog, int n_out, const int* out_slots, hgpu_array** outs) {
  if (n_terms < 1 || n_out < 1) return fail(c, HGPU_ERR_INVALID, "contract_sum_map: needs a term and an output");
  hgpu_array* acc = nullptr;
  for (int t = 0; t < n_terms; ++t) {
    hgpu_array* part = nullptr;
    int rc = horc_contract(c, a[t], b[t], n_keep, &part);
    if (!rc && acc) {
      hgpu_array* sum = nullptr;
      rc = horc_ewise2(c, HGPU_ADD, acc, part, &sum);
      horc_release(part);
      horc_release(acc);
      acc = sum;
    } else if (!rc) {
      acc = part;
    }
    if (rc) { if (acc) horc_release(acc); return rc; }
  }
  std::vector<const hgpu_array*> ins(in, in + n_in);
  int n_null = 0;
  for (auto& p : ins)
    if (!p) { p = acc; ++n_null; }
  int rc = n_null == 1 ? HGPU_OK : fail(c, HGPU_ERR_INVALID, "contract_sum_map: exactly one input must stand for the sum");
  if (!rc && n_instr == 0) {   // no program: the outputs are inputs, written out
    for (int o = 0; o < n_out && !rc; ++o) {
      if (out_slots[o] < 0 || out_slots[o] >= n_in) rc = fail(c, HGPU_ERR_INVALID, "contract_sum_map: bad output slot");
      else rc = horc_materialize(c, ins[(size_t)out_slots[o]], &outs[o]);
    }
  } else if (!rc) {
    rc = horc_fused_map(c, n_in, ins.data(), n_instr, prog, n_out, out_slots, outs);
  }
  horc_release(acc);
  return rc;
}

const hgpu_api* horc_get_api(void) {
  static const hgpu_api api = {
      sizeof(hgpu_api),
      horc_init,        horc_shutdown,  horc_sync,         horc_last_error, horc_upload,      horc_download,
      horc_read_scalar, horc_retain,    horc_release,      horc_rank,       horc_dtype_of,    horc_size,
      horc_shape,       horc_strides,   horc_is_dense,     horc_transpose,  horc_reshape,     horc_slice,
      horc_reverse,     horc_replicate, horc_index_prefix, horc_as_strided, horc_materialize, horc_pad,
      horc_ewise1,      horc_ewise2,    horc_compare,      horc_compare_all, horc_select,     horc_convert,
      horc_contract,    horc_argminmax_last, horc_iota,    horc_concat,     horc_gather,      horc_scatter_add,
      horc_onehot,      horc_fused_map, horc_scatter_affine,
      nullptr, nullptr, nullptr, nullptr, nullptr,   // no graphs: the checker executes eagerly
      horc_contract_sum, horc_assign,
      nullptr,   // no extremum_last: the checker gathers at the arg-extremum as the reference does
      nullptr,   // no fused_extremum
      nullptr,   // no fused_sum
      nullptr,   // no contract_map
      nullptr,   // no contract_operands
      nullptr,   // no fused_map_sums
      nullptr,   // no contract_sum_map
      nullptr,   // no fused_map_dimsum
  };
  return &api;
}

const hgpu_api* horc_get_api_fused(void) {
  static hgpu_api api = *horc_get_api();
  api.extremum_last = horc_extremum_last;
  api.fused_extremum = horc_fused_extremum;
  api.fused_sum = horc_fused_sum;
  api.contract_map = horc_contract_map;
  api.contract_operands = horc_contract_operands;
  api.fused_map_sums = horc_fused_map_sums;
  api.contract_sum_map = horc_contract_sum_map;
  api.fused_map_dimsum = horc_fused_map_dimsum;
  return &api;
}

}  // extern "C"
