// The `Gpu` carrier's array operations: thin wrappers over the ABI table, the
// BaseTensor-named methods built from them, and the lane-batched evaluation of
// index functions that turns gathers with affine indices into strided views.
#include <algorithm>
#include <cstddef>
#include <cstring>
#include <numeric>
#include <set>

#include "host.hpp"

namespace hordead {

void Backend::check(int rc) const {
  if (rc != HGPU_OK) throw HostError(rc, api->last_error(ctx));
}

Shape T::shape() const {
  if (pending_sum()) return {};
  if (meta_only()) return p_->vmeta.shape;
  if (pending_pieces()) return p_->pshape;
  if (pending_merged()) return p_->mv_shape;
  if (pending_expr()) return p_->eshape;
  if (contraction_like()) {   // the kept dims of the first factor
    Shape f = T(p_->fa).shape();
    return Shape(f.begin(), f.begin() + p_->keep);
  }
  Shape s((size_t)rank());
  if (!s.empty()) be()->api->shape(meta_h(), s.data());
  return s;
}
Shape T::strides() const {
  if (meta_only()) return p_->vmeta.strides;   // over the dense result of the source: what its array will have
  Shape s((size_t)rank());
  if (!s.empty()) be()->api->strides(h(), s.data());
  return s;
}

static int64_t prod(const Shape& s, size_t from = 0) {
  int64_t n = 1;
  for (size_t i = from; i < s.size(); ++i) n *= s[i];
  return n;
}
static const int64_t* ptr_or_dummy(const Shape& s) {
  static const int64_t dummy = 0;
  return s.empty() ? &dummy : s.data();
}

// ---------------------------------------------------------------- primitives

T upload(Backend* be, int dtype, const Shape& shape, const void* host) {
  hgpu_array* o = nullptr;
  be->check(be->api->upload(be->ctx, dtype, (int)shape.size(), ptr_or_dummy(shape), host, &o));
  T t(be, o);
  // keep small integer tables on the host as well (see ArrHolder::host_i64)
  int64_t n = prod(shape);
  if (dtype == HGPU_I64 && n > 0 && n <= 65536) {
    auto v = std::make_shared<std::vector<int64_t>>((size_t)n);
    std::memcpy(v->data(), host, (size_t)n * 8);
    t.set_host_i64(v);
  }
  return t;
}

static T upload_scalar(Backend* be, int dtype, double v, int64_t vi, bool integral) {
  union { double d; float f; int64_t i64; int32_t i32; int16_t i16; int8_t i8; uint8_t b; } u;
  std::memset(&u, 0, sizeof u);
  switch (dtype) {
    case HGPU_F64: u.d = integral ? (double)vi : v; break;
    case HGPU_F32: u.f = integral ? (float)vi : (float)v; break;
    case HGPU_I64: u.i64 = integral ? vi : (int64_t)v; break;
    case HGPU_I32: u.i32 = (int32_t)(integral ? vi : (int64_t)v); break;
    case HGPU_I16: u.i16 = (int16_t)(integral ? vi : (int64_t)v); break;
    case HGPU_I8: u.i8 = (int8_t)(integral ? vi : (int64_t)v); break;
    case HGPU_BOOL: u.b = (integral ? vi : (int64_t)v) != 0; break;
    default: throw HostError(HGPU_ERR_INVALID, "unknown dtype");
  }
  return upload(be, dtype, {}, &u);
}

T constant(Backend* be, int dtype, double value) {
  uint64_t bits;
  std::memcpy(&bits, &value, 8);
  auto key = std::make_pair(dtype, bits);
  auto it = be->const_cache.find(key);
  if (it != be->const_cache.end()) return T(it->second);
  T t = upload_scalar(be, dtype, value, 0, false);
  be->const_cache[key] = t.holder();
  return t;
}

T constant_i(Backend* be, int dtype, int64_t value) {
  if (dtype == HGPU_F64 || dtype == HGPU_F32) return constant(be, dtype, (double)value);
  auto key = std::make_pair(dtype + 100, (uint64_t)value);
  auto it = be->const_cache.find(key);
  if (it != be->const_cache.end()) return T(it->second);
  T t = upload_scalar(be, dtype, 0, value, true);
  be->const_cache[key] = t.holder();
  return t;
}

T iota(Backend* be, int64_t n, int dtype) {
  auto key = std::make_pair(dtype, n);
  auto it = be->iota_cache.find(key);
  if (it != be->iota_cache.end()) return T(it->second);
  // Made inside a recording, the array would only be filled when the graph is
  // launched, yet the cache would hand it to eager code before (or after an
  // aborted recording, never filled): refused, as an upload is -- run the
  // program once before recording it.
  if (be->capturing) throw HostError(HGPU_ERR_UNSUPPORTED, "iota of a length first asked for during a recording: run the program once before recording it");
  hgpu_array* o = nullptr;
  be->check(be->api->iota(be->ctx, n, dtype, &o));
  T t(be, o);
  be->iota_cache[key] = t.holder();
  return t;
}

// ---- views known on the host only: probes and pending views -----------------

namespace {
struct ProbeFail {};   // a view operation that cannot be expressed by strides alone was tried on a probe

Meta dense_meta(const Shape& sh) {
  Meta m;
  m.shape = sh;
  m.strides.assign(sh.size(), 0);
  int64_t s = 1;
  for (size_t i = sh.size(); i-- > 0;) { m.strides[i] = s; s *= sh[i]; }
  return m;
}

bool meta_transpose(const Meta& a, const std::vector<int>& perm, Meta* o) {
  const size_t rank = a.shape.size();
  if (perm.size() > rank) return false;
  std::vector<bool> seen(perm.size(), false);
  *o = a;
  for (size_t i = 0; i < perm.size(); ++i) {
    int sdim = perm[i];
    if (sdim < 0 || sdim >= (int)perm.size() || seen[(size_t)sdim]) return false;
    seen[(size_t)sdim] = true;
    o->shape[i] = a.shape[(size_t)sdim];
    o->strides[i] = a.strides[(size_t)sdim];
  }
  return true;
}

// `shape` as a view of a (the rule of hgpu_reshape: runs of dims that are contiguous among themselves may be split and merged)
bool meta_reshape(const Meta& a, const Shape& shape, Meta* o) {
  int64_t na = 1, nn = 1;
  for (auto e : a.shape) na *= e;
  for (auto e : shape) nn *= e;
  if (na != nn || na == 0) return false;
  Shape rsh, rst;
  for (size_t i = 0; i < a.shape.size(); ++i) {
    if (a.shape[i] == 1) continue;
    if (!rsh.empty() && rst.back() == a.strides[i] * a.shape[i]) { rsh.back() *= a.shape[i]; rst.back() = a.strides[i]; }
    else { rsh.push_back(a.shape[i]); rst.push_back(a.strides[i]); }
  }
  o->shape = shape;
  o->strides.assign(shape.size(), 0);
  o->offset = a.offset;
  size_t r = 0;
  int64_t rem = rsh.empty() ? 1 : rsh[0];
  for (size_t i = 0; i < shape.size(); ++i) {
    int64_t e = shape[i];
    if (e == 1) continue;
    if (r >= rsh.size() || rem % e != 0) return false;
    rem /= e;
    o->strides[i] = rst[r] * rem;
    if (rem == 1) { ++r; rem = r < rsh.size() ? rsh[r] : 1; }
  }
  return r == rsh.size();
}

bool meta_slice(const Meta& a, int dim, int64_t start, int64_t len, Meta* o) {
  if (dim < 0 || dim >= (int)a.shape.size() || start < 0 || len < 0 || start + len > a.shape[(size_t)dim]) return false;
  *o = a;
  o->shape[(size_t)dim] = len;
  o->offset += start * a.strides[(size_t)dim];
  return true;
}

bool meta_reverse(const Meta& a, int dim, Meta* o) {
  if (dim < 0 || dim >= (int)a.shape.size()) return false;
  *o = a;
  if (a.shape[(size_t)dim] > 0) o->offset += (a.shape[(size_t)dim] - 1) * a.strides[(size_t)dim];
  o->strides[(size_t)dim] = -a.strides[(size_t)dim];
  return true;
}

bool meta_replicate(const Meta& a, const Shape& pre, Meta* o) {
  for (auto e : pre)
    if (e <= 0) return false;
  o->shape = pre;
  o->shape.insert(o->shape.end(), a.shape.begin(), a.shape.end());
  o->strides.assign(pre.size(), 0);
  o->strides.insert(o->strides.end(), a.strides.begin(), a.strides.end());
  o->offset = a.offset;
  return true;
}

bool meta_index_prefix(const Meta& a, const Shape& ix, Meta* o) {
  if (ix.size() > a.shape.size()) return false;
  o->offset = a.offset;
  for (size_t i = 0; i < ix.size(); ++i) {
    if (ix[i] < 0 || ix[i] >= a.shape[i]) return false;   // out of bounds means zeros: not a view
    o->offset += ix[i] * a.strides[i];
  }
  o->shape.assign(a.shape.begin() + (long)ix.size(), a.shape.end());
  o->strides.assign(a.strides.begin() + (long)ix.size(), a.strides.end());
  return true;
}

// the elements a view addresses, relative to the start of its source's layout
void meta_range(const Meta& a, int64_t* lo, int64_t* hi, bool* empty) {
  *lo = *hi = a.offset;
  *empty = false;
  for (size_t i = 0; i < a.shape.size(); ++i) {
    if (a.shape[i] == 0) { *empty = true; continue; }
    int64_t span = (a.shape[i] - 1) * a.strides[i];
    if (span > 0) *hi += span; else *lo += span;
  }
}

bool meta_as_strided(const Meta& a, const Shape& shape, const Shape& strides, int64_t offset, Meta* o) {
  if (shape.size() != strides.size()) return false;
  o->shape = shape;
  o->strides = strides;
  o->offset = a.offset + offset;
  int64_t lo, hi, alo, ahi;
  bool e1, e2;
  meta_range(*o, &lo, &hi, &e1);
  meta_range(a, &alo, &ahi, &e2);
  return !e1 && !e2 && lo >= alo && hi <= ahi;   // as hgpu_as_strided: inside what the source view addresses
}
}  // namespace

static T make_probe(Backend* be, const Meta& m, int dtype) {
  auto p = new_holder(be, nullptr);
  p->probe = true;
  p->probe_dtype = dtype;
  p->vmeta = m;
  return T(p);
}
// The view m over the dense result of the pending value src.
static T make_view(const std::shared_ptr<ArrHolder>& src, const Meta& m) {
  auto p = new_holder(src->be, nullptr);
  p->vsrc = src;
  p->vmeta = m;
  return T(p);
}
// a with the strides of m: a probe stays a probe, a pending view stays one of the same source
static T with_meta(const T& a, const Meta& m) {
  if (a.is_probe()) return make_probe(a.be(), m, a.dtype());
  T v = make_view(a.holder()->vsrc, m);
  v.holder()->vlo = a.holder()->vlo;
  v.holder()->vhi = a.holder()->vhi;
  return v;
}
// an elementwise expression (also one over a refined index space) that is not yet written out
static bool expression_like(const T& t) {
  return t.valid() && (t.pending_expr() || (t.pending_merged() && T(t.holder()->mv_inner).pending_expr()));
}
// The zero-extension of a pending view, when the view merely permutes and
// replicates the dims of its source's (zero-extended) result: the extension is
// then one of the source's dims, and the view one of the larger layout.
static bool pad_view(const T& a, const Shape& lo, const Shape& hi, T* out) {
  const ArrHolder* h = a.holder().get();
  T src(h->vsrc);
  Shape M = src.shape();
  Shape slo = h->vlo.empty() ? Shape(M.size(), 0) : h->vlo, shi = h->vhi.empty() ? Shape(M.size(), 0) : h->vhi;
  Shape P(M.size());
  for (size_t k = 0; k < M.size(); ++k) P[k] = M[k] + slo[k] + shi[k];
  const Meta pd = dense_meta(P);
  const Meta& vm = h->vmeta;
  if (vm.offset != 0 || lo.size() != vm.shape.size() || hi.size() != vm.shape.size()) return false;
  std::vector<int> dim_of(vm.shape.size(), -1);
  std::vector<bool> used(M.size(), false);
  for (size_t d = 0; d < vm.shape.size(); ++d) {
    if (vm.shape[d] == 1 || vm.strides[d] == 0) {
      if (lo[d] != 0 || hi[d] != 0) return false;   // a replicated dim cannot be extended by zeros here
      continue;
    }
    for (size_t k = 0; k < M.size(); ++k)
      if (!used[k] && P[k] == vm.shape[d] && pd.strides[k] == vm.strides[d] && P[k] > 1) { dim_of[d] = (int)k; break; }
    if (dim_of[d] < 0) return false;
    used[(size_t)dim_of[d]] = true;
  }
  for (size_t d = 0; d < vm.shape.size(); ++d) {
    if (lo[d] < 0 || hi[d] < 0) return false;
    if (dim_of[d] >= 0) { slo[(size_t)dim_of[d]] += lo[d]; shi[(size_t)dim_of[d]] += hi[d]; }
  }
  Shape P2(M.size());
  for (size_t k = 0; k < M.size(); ++k) P2[k] = M[k] + slo[k] + shi[k];
  const Meta pd2 = dense_meta(P2);
  Meta m2;
  m2.shape = vm.shape;
  m2.strides.assign(vm.shape.size(), 0);
  for (size_t d = 0; d < vm.shape.size(); ++d)
    if (dim_of[d] >= 0) { m2.shape[d] = P2[(size_t)dim_of[d]]; m2.strides[d] = pd2.strides[(size_t)dim_of[d]]; }
  T v = make_view(h->vsrc, m2);
  v.holder()->vlo = slo;
  v.holder()->vhi = shi;
  *out = v;
  return true;
}
// Tries a view operation on strides alone.  A probe that cannot take it gives
// up (ProbeFail); a pending view falls through to the array path, which
// computes its source first.
#define HD_META_VIEW(call)                          \
  if (a.meta_only()) {                              \
    Meta m__;                                       \
    if (call) return with_meta(a, m__);             \
    if (a.is_probe()) throw ProbeFail{};            \
  }

#define HD_OUT(call)                      \
  hgpu_array* o__ = nullptr;              \
  Backend* be__ = a.be();                 \
  be__->check(be__->api->call);           \
  return T(be__, o__)

static T contract_now(const T& a, const T* b, int n_keep);
static bool holds_pending_contraction(const ArrHolder* root);
static void pieces_of(const T& t, std::vector<ArrHolder::Piece>* out);
static T make_merged(const T& inner, const Shape& shape, const std::vector<int>& groups);
static T split_view(const T& y, const Shape& fine);
static T lift_merged(const std::vector<const T*>& ops, const std::function<T(const std::vector<T>&)>& apply);
static T from_pieces(Backend* be, std::vector<ArrHolder::Piece> pcs, const Shape& shape, int dtype);
static T slice_pieces(const T& a, int64_t start, int64_t len);
static T ewise1_now(int op, const T& a);
static T ewise2_now(int op, const T& a, const T& b);
static T compare_now(int cmp, const T& a, const T& b);
static T select_now(const T& c, const T& a, const T& b);
static T convert_now(const T& a, int dtype, int mode);

// ------------------------------------------- pending elementwise expressions

static bool fuses(Backend* be) {
  return be->fuse && be->api->struct_size >= offsetof(hgpu_api, fused_map) + sizeof(be->api->fused_map) && be->api->fused_map != nullptr;
}
static int pending_size(const std::shared_ptr<ArrHolder>& p) { return (p && !p->h && p->ekind >= 0) ? p->esize : 0; }

static T make_expr(int kind, int op, int dtype, const T& a, const T* b, const T* c);

// f (view A) (view B) = view (f A B): when every operand of a new elementwise
// node is the SAME view of some expression's dense result (or one broadcast
// element), the node is that view of the node over the sources.  The note
// (vsrc, vmeta -- as map_leaves leaves it) lets a consumer that knows how to
// evaluate the source expression inside another kernel (a window extremum in a
// convolution's epilogue) recognise `mask (windows t) * windows t`, the way the
// reference's derived programs write relu under pooling, as windows of
// `mask t * t`.
static bool one_element(const T& t) { return (bool)t.holder()->scalar_src; }
static void note_common_view(ArrHolder* p, int kind, int op, int dtype, const T& a, const T* b, const T* c) {
  const T* ops[3] = {&a, b, c};
  const ArrHolder* first = nullptr;
  for (auto* o : ops) {
    if (!o) continue;
    const ArrHolder* h = o->holder().get();
    const bool noted = !h->h && h->vsrc && h->vlo.empty() && !h->probe && (h->ekind >= 0 || o->pending_view());
    if (noted) {
      if (first && (h->vmeta.shape != first->vmeta.shape || h->vmeta.strides != first->vmeta.strides || h->vmeta.offset != first->vmeta.offset ||
                    T(h->vsrc).shape() != T(first->vsrc).shape())) {
        return;
      }
      if (!first) first = h;
    } else if (!one_element(*o)) {
      return;
    }
  }
  if (!first) return;
  const Shape src_shape = T(first->vsrc).shape();
  T src[3];
  for (int i = 0; i < 3; ++i) {
    if (!ops[i]) continue;
    const ArrHolder* h = ops[i]->holder().get();
    if (!h->h && h->vsrc) src[i] = T(h->vsrc);
    else src[i] = broadcast_scalar(T(h->scalar_src), src_shape);
  }
  T whole = make_expr(kind, op, dtype, src[0], b ? &src[1] : nullptr, c ? &src[2] : nullptr);
  p->vsrc = whole.holder();
  p->vmeta = first->vmeta;
}

static T make_expr(int kind, int op, int dtype, const T& a, const T* b, const T* c) {
  auto p = new_holder(a.be(), nullptr);
  p->ekind = kind;
  p->eop = op;
  p->edtype = dtype;
  p->eshape = a.shape();
  p->fa = a.holder();
  if (b) p->fb = b->holder();
  if (c) p->fc = c->holder();
  // keep programs small: a large operand is written out first
  int sz = 1 + pending_size(p->fa) + pending_size(p->fb) + pending_size(p->fc);
  if (sz > 40) {
    std::shared_ptr<ArrHolder>* big = &p->fa;
    if (pending_size(p->fb) > pending_size(*big)) big = &p->fb;
    if (pending_size(p->fc) > pending_size(*big)) big = &p->fc;
    (*big)->force();
    sz = 1 + pending_size(p->fa) + pending_size(p->fb) + pending_size(p->fc);
  }
  p->esize = sz;
  note_common_view(p.get(), kind, op, dtype, a, b, c);
  return T(p);
}

namespace {
struct Program {
  std::vector<const ArrHolder*> inputs;
  std::vector<std::pair<ArrHolder*, hgpu_fused_instr>> instrs;   // operands hold holder slots until numbered
  std::map<const ArrHolder*, int> in_slot, instr_slot;
  // keep_contraction: one pending contraction of two arrays among the leaves
  // stays as it is (an input without an array), for a kernel that computes it
  // and runs the program over its result in one pass
  bool keep_contraction = false;
  bool keep_sums = false;     // ... or one pending SUM of contractions (for a kernel that adds the products too)
  ArrHolder* kept = nullptr;
};

bool single_contraction(const ArrHolder* p) {
  return !p->h && p->ekind < 0 && p->fa && p->fb && p->keep >= 1 && p->more.empty() && !p->origin && !p->vsrc && p->pieces.empty() && !p->mv_inner && !p->ones_b;
}

// Post-order walk: materialised values (and pending contractions, which are
// forced here) become inputs, pending elementwise nodes become instructions.
// a pending contraction of two arrays, or a pending sum of such
bool contraction_or_sum(const ArrHolder* p) {
  return !p->h && p->ekind < 0 && p->fa && p->fb && p->keep >= 1 && !p->origin && !p->vsrc && p->pieces.empty() && !p->mv_inner && !p->ssrc && !p->probe && !p->ones_b;
}

int visit(Program& pg, ArrHolder* p) {
  if (pg.keep_contraction && (pg.keep_sums ? contraction_or_sum(p) : single_contraction(p)) && (!pg.kept || pg.kept == p)) {
    pg.kept = p;
    auto it = pg.in_slot.find(p);
    if (it != pg.in_slot.end()) return -1 - it->second;
    int k = (int)pg.inputs.size();
    pg.inputs.push_back(p);
    pg.in_slot[p] = k;
    return -1 - k;
  }
  if (!p->h && p->ekind < 0) p->force();   // a pending contraction, concatenation or refined expression
  if (!p->h && p->vsrc && p->vsrc->h) p->view_of_written_source();
  if (p->h) {
    auto it = pg.in_slot.find(p);
    if (it != pg.in_slot.end()) return -1 - it->second;
    int k = (int)pg.inputs.size();
    pg.inputs.push_back(p);
    pg.in_slot[p] = k;
    return -1 - k;          // inputs are numbered after the walk: encode as negative
  }
  auto it = pg.instr_slot.find(p);
  if (it != pg.instr_slot.end()) return it->second;
  hgpu_fused_instr q;
  q.kind = p->ekind;
  q.op = p->eop;
  q.dtype = p->edtype;
  q.a = visit(pg, p->fa.get());
  q.b = p->fb ? visit(pg, p->fb.get()) : 0;
  q.c = p->fc ? visit(pg, p->fc.get()) : 0;
  int k = (int)pg.instrs.size();
  pg.instrs.push_back({p, q});
  pg.instr_slot[p] = k;
  return k;
}
}  // namespace

// The roots' expressions as one numbered program: inputs, instructions, and the slot of every root.
// With `kept`: one pending contraction among the leaves stays pending (*kept; its
// entry of ins is null), and nodes receives the holder of every instruction.
// Computing a leaf can run other programs, and those may write out (and take
// apart) nodes of the very expression that is being numbered.  So everything
// that has to be computed is computed first, one leaf at a time with a fresh
// look at the expression after each; the numbering walk that follows computes
// nothing and its raw pointers stay good.  In numbering order: the pending
// contraction that stays pending (with keep_contraction) has its operands
// written out, every other pending leaf is written out itself.
namespace {
// One look at the expression: the first thing that has to be computed, in numbering order.
struct SettleWalk {
  bool keep_contraction, keep_sums;
  uint64_t gen;                          // nodes seen in this walk carry it (no allocation per walk)
  const std::set<const ArrHolder*>* tried_view;
  const ArrHolder* kept = nullptr;
  std::shared_ptr<ArrHolder> todo;       // shared: what it is computed from may let go of it meanwhile
  ArrHolder* todo_root = nullptr;
  bool todo_is_view = false;
  bool take(ArrHolder* p, const std::shared_ptr<ArrHolder>* owner, bool view) {
    if (owner) todo = *owner; else todo_root = p;
    todo_is_view = view;
    return true;
  }
  bool walk(ArrHolder* p, const std::shared_ptr<ArrHolder>* owner) {
    if (p->walk_mark == gen) return false;
    p->walk_mark = gen;
    if (keep_contraction && (keep_sums ? contraction_or_sum(p) : single_contraction(p)) && (!kept || kept == p)) {
      kept = p;
      for (auto* f : {&p->fa, &p->fb})
        if (*f && !(*f)->h) { todo = *f; return true; }
      for (auto& m : p->more)
        for (auto* f : {&m.first, &m.second})
          if (*f && !(*f)->h) { todo = *f; return true; }
      return false;
    }
    if (!p->h && p->ekind < 0) return take(p, owner, false);
    if (!p->h && p->vsrc && p->vsrc->h && !tried_view->count(p)) return take(p, owner, true);
    if (p->h) return false;
    for (auto* f : {&p->fa, &p->fb, &p->fc})
      if (*f && walk(f->get(), f)) return true;
    return false;
  }
};
}  // namespace

static void settle_leaves(const std::vector<ArrHolder*>& roots, bool keep_contraction, bool keep_sums) {
  if (roots.empty()) return;
  Backend* be = roots[0]->be;
  std::set<const ArrHolder*> tried_view;
  for (int round = 0; round < 100000; ++round) {
    SettleWalk w{keep_contraction, keep_sums, ++be->walk_gen, &tried_view};
    bool found = false;
    for (auto* r : roots)
      if (w.walk(r, nullptr)) { found = true; break; }
    if (!found) return;
    ArrHolder* q = w.todo ? w.todo.get() : w.todo_root;
    if (w.todo_is_view) {
      tried_view.insert(q);
      q->view_of_written_source();
    } else {
      q->force();
    }
  }
}

static void number_program(const std::vector<ArrHolder*>& roots, std::vector<const hgpu_array*>* ins, std::vector<hgpu_fused_instr>* prog,
                           std::vector<int>* outs_slot, ArrHolder** kept = nullptr, std::vector<ArrHolder*>* nodes = nullptr, bool keep_sums = false) {
  settle_leaves(roots, kept != nullptr, keep_sums);
  Program pg;
  pg.keep_contraction = kept != nullptr;
  pg.keep_sums = keep_sums;
  std::vector<int> root_slot;
  for (auto* r : roots) root_slot.push_back(visit(pg, r));
  int n_in = (int)pg.inputs.size();
  auto slot = [&](int v) { return v < 0 ? -1 - v : n_in + v; };
  for (auto& pi : pg.instrs) {
    hgpu_fused_instr q = pi.second;
    q.a = slot(q.a);
    q.b = pi.first->fb ? slot(q.b) : 0;
    q.c = pi.first->fc ? slot(q.c) : 0;
    prog->push_back(q);
  }
  for (auto* p : pg.inputs) ins->push_back(p->h);
  for (int v : root_slot) outs_slot->push_back(slot(v));
  if (kept) *kept = pg.kept;
  if (nodes)
    for (auto& pi : pg.instrs) nodes->push_back(pi.first);
}

static void measure(const std::vector<ArrHolder*>& roots, int* n_in, int* n_instr);

// `tanh (W x + V s + b)`: when one leaf of the roots' expressions is a pending
// contraction (or sum of contractions) and the provider has
// hgpu_contract_sum_map, the products, their sum and the program go out as one
// call and the sum is never written -- unless someone outside the program still
// holds it, in which case it is one more result of the same call.
static bool products_then_program(Backend* be, const std::vector<ArrHolder*>& roots, std::vector<hgpu_array*>* outs) {
  const hgpu_api* api = be->api;
  if (!be->fuse || !(api->struct_size >= offsetof(hgpu_api, contract_sum_map) + sizeof(api->contract_sum_map) && api->contract_sum_map)) return false;
  if (roots.size() > 5) return false;
  // is there such a leaf at all?  (walk without forcing anything)
  {
    std::map<const ArrHolder*, int> seen;
    std::vector<const ArrHolder*> stack(roots.begin(), roots.end());
    bool found = false;
    while (!stack.empty() && !found) {
      const ArrHolder* p = stack.back();
      stack.pop_back();
      if (seen.count(p)) continue;
      seen[p] = 1;
      if (contraction_or_sum(p)) { found = true; break; }
      if (p->h || p->ekind < 0) continue;
      if (p->fa) stack.push_back(p->fa.get());
      if (p->fb) stack.push_back(p->fb.get());
      if (p->fc) stack.push_back(p->fc.get());
    }
    if (!found) return false;
  }
  std::vector<const hgpu_array*> ins;
  std::vector<hgpu_fused_instr> prog;
  std::vector<int> slots;
  std::vector<ArrHolder*> nodes;
  ArrHolder* kept = nullptr;
  number_program(roots, &ins, &prog, &slots, &kept, &nodes, true);
  if (!kept) return false;
  // Computed during the walk after all (a view of it among the later leaves needed it as an array): nothing is left to fuse.
  if (kept->h || !kept->fa) return false;
  if (T(kept->fa).dtype() != HGPU_F64 && T(kept->fa).dtype() != HGPU_F32) { kept->force(); return false; }
  int c_slot = -1;
  for (size_t i = 0; i < ins.size(); ++i)
    if (!ins[i]) c_slot = (int)i;
  // who else holds the sum?
  std::shared_ptr<ArrHolder> ks;
  long inside = 0;
  for (auto* nd : nodes)
    for (auto* f : {&nd->fa, &nd->fb, &nd->fc})
      if (f->get() == kept) { ks = *f; ++inside; }
  for (auto* r : roots)
    if (r == kept) return false;   // cannot be: roots are expressions
  const bool shared = !ks || ks.use_count() - 1 > inside;
  if (c_slot < 0 || (int)ins.size() > 12 || (int)prog.size() > 96) { kept->force(); return false; }
  std::vector<T> fas{T(kept->fa)}, fbs{T(kept->fb)};
  for (auto& m : kept->more) { fas.push_back(T(m.first)); fbs.push_back(T(m.second)); }
  std::vector<const hgpu_array*> ah, bh;
  for (size_t t = 0; t < fas.size(); ++t) { ah.push_back(fas[t].h()); bh.push_back(fbs[t].h()); }
  // An inner node of the program that contains the products and that someone
  // outside still holds (the condition of a select, kept for the reverse pass)
  // would later be computed again, products and all: it is one more result of
  // the same call.  (Inner nodes without the products are cheap to redo.)
  std::vector<std::pair<ArrHolder*, int>> promoted;   // node, its slot
  {
    std::map<const ArrHolder*, bool> has_products;     // instructions come children first
    has_products[kept] = true;
    for (size_t i = 0; i < nodes.size(); ++i) {
      ArrHolder* nd = nodes[i];
      bool hp = false;
      for (auto* f : {&nd->fa, &nd->fb, &nd->fc})
        if (*f) { auto it = has_products.find(f->get()); hp = hp || (it != has_products.end() && it->second); }
      has_products[nd] = hp;
      if (!hp || std::find(roots.begin(), roots.end(), nd) != roots.end()) continue;
      std::shared_ptr<ArrHolder> sp;
      long in = 0;
      for (auto* q : nodes)
        for (auto* f : {&q->fa, &q->fb, &q->fc})
          if (f->get() == nd) { sp = *f; ++in; }
      if (sp && sp.use_count() - 1 > in && roots.size() + promoted.size() < 6) {
        // `ifH c 0 1` between constants: its condition says as much in a byte per element
        ArrHolder* w = nd;
        size_t wi = i;
        if (nd->ekind == HGPU_FUSED_SELECT && nd->fa && !nd->fa->h && nd->fa->ekind >= 0 && has_products[nd->fa.get()] && !has_products[nd->fb.get()] &&
            !has_products[nd->fc.get()] && std::find(roots.begin(), roots.end(), nd->fa.get()) == roots.end()) {
          auto at = std::find(nodes.begin(), nodes.end(), nd->fa.get());
          if (at != nodes.end() && T(nd->fa).dtype() == HGPU_BOOL) { w = *at; wi = (size_t)(at - nodes.begin()); }
        }
        bool have = false;
        for (auto& pr : promoted) have = have || pr.first == w;
        if (!have) promoted.push_back({w, (int)ins.size() + (int)wi});
        has_products[w] = false;      // written: what is built on it can be redone from the array
        has_products[nd] = false;
      }
    }
  }
  std::vector<int> out_slots(slots);
  for (auto& pr : promoted) out_slots.push_back(pr.second);
  if (shared) out_slots.push_back(c_slot);
  std::vector<hgpu_array*> res(out_slots.size(), nullptr);
  int rc = api->contract_sum_map(be->ctx, (int)ah.size(), ah.data(), bh.data(), kept->keep, (int)ins.size(), ins.data(), (int)prog.size(), prog.data(), (int)out_slots.size(),
                                 out_slots.data(), res.data());
  if (rc == HGPU_ERR_UNSUPPORTED) { kept->force(); return false; }
  be->check(rc);
  be->counters["contract_sum_map"]++;
  for (size_t i = 0; i < roots.size(); ++i) (*outs)[i] = res[i];
  for (size_t j = 0; j < promoted.size(); ++j) {
    ArrHolder* nd = promoted[j].first;
    nd->h = res[roots.size() + j];
    nd->fa.reset();
    nd->fb.reset();
    nd->fc.reset();
    nd->vsrc.reset();
    nd->ekind = -1;
    be->counters["contract_sum_map_kept_nodes"]++;
  }
  if (shared) {
    kept->h = res.back();
    kept->fa.reset();
    kept->fb.reset();
    kept->more.clear();
    kept->keep = -1;
  }
  return true;
}

// A view that brings ONE dim of its source to the front and leaves the others
// in order (offset 0, nothing repeated or left out): that dim, counted in the
// dims of the expression that computes the source; else -1.
static int front_dim_of_view(const ArrHolder* v) {
  if (!v || v->h || !v->vsrc || !v->vlo.empty() || v->vmeta.offset != 0 || v->probe) return -1;   // (an expression over viewed leaves carries the view as a note)
  T src(v->vsrc);
  const Shape M = src.shape();
  const Shape& vs = v->vmeta.shape;
  const Shape& vt = v->vmeta.strides;
  if (M.empty() || vs.size() != M.size()) return -1;
  Shape ds(M.size());
  int64_t acc = 1;
  for (size_t i = M.size(); i-- > 0;) { ds[i] = acc; acc *= M[i]; }
  int d = -1;
  for (size_t i = 0; i < M.size(); ++i)
    if (vs[0] == M[i] && vt[0] == ds[i] && M[i] > 1) { d = (int)i; break; }
  if (d < 0) return -1;
  size_t k = 1;
  for (size_t i = 0; i < M.size(); ++i) {
    if ((int)i == d) continue;
    if (vs[k] != M[i] || (M[i] > 1 && vt[k] != ds[i])) return -1;
    ++k;
  }
  if (!src.pending_merged()) return d;
  // the source is an expression over a refined index space: its dim d must be one dim there too
  const auto& g = src.holder()->mv_groups;
  if ((size_t)d >= g.size() || g[(size_t)d] != 1) return -1;
  int rd = 0;
  for (int i = 0; i < d; ++i) rd += g[(size_t)i];
  return rd;
}

static void run_program(Backend* be, const std::vector<ArrHolder*>& all_roots) {
  // computing the leaves may write a root out on the way (as a view of a source written meanwhile): those are done
  settle_leaves(all_roots, true, true);
  std::vector<ArrHolder*> roots;
  for (auto* r : all_roots)
    if (!r->h && r->ekind >= 0) roots.push_back(r);
  if (roots.empty()) return;
  std::vector<const hgpu_array*> ins;
  std::vector<hgpu_fused_instr> prog;
  std::vector<int> outs_slot;
  std::vector<hgpu_array*> outs(roots.size(), nullptr);
  // Pending sums over expressions of this shape ride along: one pass for the
  // values written out and the sums.
  std::vector<std::shared_ptr<ArrHolder>> sums;
  const hgpu_api* api = be->api;
  if (api->struct_size >= offsetof(hgpu_api, fused_map_sums) + sizeof(api->fused_map_sums) && api->fused_map_sums) {
    for (auto& w : be->pending_sums) {
      auto q = w.lock();
      if (!q || q->h || !q->ssrc || sums.size() >= 4) continue;
      T e(q->ssrc);
      if (e.pending_expr() && e.shape() == roots[0]->eshape && e.be() == be) sums.push_back(q);
    }
  }
  if (!sums.empty()) {
    std::vector<ArrHolder*> all(roots);
    for (auto& q : sums) all.push_back(q->ssrc.get());
    int n_in_all, n_instr_all;
    measure(all, &n_in_all, &n_instr_all);
    if (n_in_all <= 12 && n_instr_all <= 96 && roots.size() <= 6) {
      std::vector<int> slots;
      number_program(all, &ins, &prog, &slots);
      std::vector<int> sum_slots(slots.begin() + (long)roots.size(), slots.end());
      std::vector<hgpu_array*> souts(sums.size(), nullptr);
      int rc = api->fused_map_sums(be->ctx, (int)ins.size(), ins.data(), (int)prog.size(), prog.data(), (int)roots.size(), slots.data(), outs.data(),
                                   (int)sums.size(), sum_slots.data(), souts.data());
      if (rc == HGPU_OK) {
        be->counters["fused_map_sums"]++;
        for (size_t j = 0; j < sums.size(); ++j) { sums[j]->h = souts[j]; sums[j]->ssrc.reset(); }
        outs_slot.assign(slots.begin(), slots.begin() + (long)roots.size());
      } else {
        if (rc != HGPU_ERR_UNSUPPORTED) be->check(rc);
        ins.clear();
        prog.clear();
        sums.clear();
      }
    } else {
      sums.clear();
    }
  }
  if (sums.empty() && products_then_program(be, roots, &outs)) {
    // done by one kernel: products, their sum and the program
  } else if (sums.empty()) {
    number_program(roots, &ins, &prog, &outs_slot);
    {
      // the attempt above may have written the source a root is a view of: that root is done (the walk has made it the view)
      std::vector<ArrHolder*> rest;
      for (auto* r : roots)
        if (!r->h && r->ekind >= 0) rest.push_back(r);
      if (rest.size() != roots.size()) {
        if (!rest.empty()) run_program(be, rest);
        return;
      }
    }
    int n_in = (int)ins.size(), n_instr = (int)prog.size();
    // A pending sum over all dims but one of what is being written out (a
    // bias's cotangent) is taken in the same pass.
    bool done = false;
    if (api->struct_size >= offsetof(hgpu_api, fused_map_dimsum) + sizeof(api->fused_map_dimsum) && api->fused_map_dimsum && n_instr >= 1) {
      auto& pd = be->pending_dimsums;
      pd.erase(std::remove_if(pd.begin(), pd.end(), [](const std::weak_ptr<ArrHolder>& w) { auto q = w.lock(); return !q || q->h || !q->ones_b; }), pd.end());
      for (auto& w : pd) {
        auto q = w.lock();
        if (!q || !q->fa || !q->more.empty() || q->keep != 1) continue;
        const ArrHolder* v = q->fa.get();
        if (v->h || !v->vsrc) continue;
        const ArrHolder* src = v->vsrc.get();
        const ArrHolder* e = src->mv_inner ? src->mv_inner.get() : src;
        size_t ri = 0;
        while (ri < roots.size() && roots[ri] != e) ++ri;
        if (ri == roots.size()) continue;
        const int d = front_dim_of_view(v);
        if (d < 0) continue;
        hgpu_array* so = nullptr;
        int rc = api->fused_map_dimsum(be->ctx, n_in, ins.data(), n_instr, prog.data(), (int)roots.size(), outs_slot.data(), outs.data(), outs_slot[ri], d, &so);
        if (rc == HGPU_OK) {
          be->counters["fused_map_dimsum"]++;
          q->h = so;
          q->fa.reset();
          q->fb.reset();
          q->keep = -1;
          q->ones_b = false;
          done = true;
        } else if (rc != HGPU_ERR_UNSUPPORTED) {
          be->check(rc);
        }
        break;
      }
    }
    if (!done) be->check(be->api->fused_map(be->ctx, n_in, ins.data(), n_instr, prog.data(), (int)roots.size(), outs_slot.data(), outs.data()));
  }
  for (size_t i = 0; i < roots.size(); ++i) {
    ArrHolder* r = roots[i];
    r->h = outs[i];
    r->fa.reset();
    r->fb.reset();
    r->fc.reset();
    r->vsrc.reset();
    r->ekind = -1;
  }
}

// Counts the inputs and instructions a set of roots would need.
static void measure(const std::vector<ArrHolder*>& roots, int* n_in, int* n_instr) {
  std::map<const ArrHolder*, int> seen;
  std::vector<const ArrHolder*> stack(roots.begin(), roots.end());
  *n_in = *n_instr = 0;
  while (!stack.empty()) {
    const ArrHolder* p = stack.back();
    stack.pop_back();
    if (seen.count(p)) continue;
    seen[p] = 1;
    if (p->h || p->ekind < 0) { ++*n_in; continue; }
    ++*n_instr;
    if (p->fa) stack.push_back(p->fa.get());
    if (p->fb) stack.push_back(p->fb.get());
    if (p->fc) stack.push_back(p->fc.get());
  }
}

static void force_roots(Backend* be, std::vector<ArrHolder*> roots) {
  // drop roots that are already arrays, or that appear twice
  std::vector<ArrHolder*> rs;
  for (auto* r : roots)
    if (!r->h && r->ekind >= 0 && std::find(rs.begin(), rs.end(), r) == rs.end()) rs.push_back(r);
  if (rs.empty()) return;
  // the leaves first: what they turn into decides how many inputs and instructions there are to count
  settle_leaves(rs, true, true);
  rs.erase(std::remove_if(rs.begin(), rs.end(), [](ArrHolder* r) { return r->h || r->ekind < 0; }), rs.end());
  if (rs.empty()) return;
  int n_in, n_instr;
  measure(rs, &n_in, &n_instr);
  const int kIn = 12, kInstr = 96, kOut = 6;
  if (rs.size() > 1 && ((int)rs.size() > kOut || n_in > kIn || n_instr > kInstr)) {
    // too much for one pass: halve the set
    std::vector<ArrHolder*> lo(rs.begin(), rs.begin() + (long)rs.size() / 2), hi(rs.begin() + (long)rs.size() / 2, rs.end());
    force_roots(be, lo);
    force_roots(be, hi);
    return;
  }
  if (n_in > kIn || n_instr > kInstr) {
    // one root with too many leaves: write its largest pending operand out first
    ArrHolder* r = rs[0];
    std::shared_ptr<ArrHolder> big = r->fa;
    if (pending_size(r->fb) > pending_size(big)) big = r->fb;
    if (pending_size(r->fc) > pending_size(big)) big = r->fc;
    if (pending_size(big) == 0) {   // only arrays beneath: cannot shrink further
      run_program(be, rs);
      return;
    }
    force_roots(be, {big.get()});
    force_roots(be, rs);
    return;
  }
  run_program(be, rs);
}

void force_many(const std::vector<T>& ts) {
  std::map<std::pair<Backend*, Shape>, std::vector<ArrHolder*>> groups;
  for (auto& t : ts)
    if (t.valid() && t.pending_expr()) groups[{t.be(), t.shape()}].push_back(t.holder().get());
  for (auto& g : groups) force_roots(g.first.first, g.second);
  // Small pending contractions (the bias and readout gradients at the end of a reverse pass) are asked for last,
  // one after another: a provider that holds such launches back then sends them out as one kernel.
  auto small_reduction = [](const T& t) {
    const ArrHolder* p = t.holder().get();
    return !p->h && p->ekind < 0 && p->fa && p->fb && p->keep >= 0 && p->more.empty() && !p->origin && t.size() <= 16384;
  };
  for (auto& t : ts)
    if (t.valid() && !small_reduction(t)) (void)t.h();
  for (auto& t : ts)
    if (t.valid()) (void)t.h();
}

// An expression noted to be a view of another expression's dense result, when
// that result has been written out in the meantime (as a side result of the
// kernel that consumed it): the view of that array, nothing to compute.
bool ArrHolder::view_of_written_source() {
  if (h || ekind < 0 || !vsrc || !vsrc->h || !vlo.empty()) return false;
  hgpu_array* base = vsrc->h;
  if (!be->api->is_dense(base)) return false;
  hgpu_array* o = nullptr;
  if (be->api->as_strided(be->ctx, base, (int)vmeta.shape.size(), vmeta.shape.empty() ? nullptr : vmeta.shape.data(),
                          vmeta.strides.empty() ? nullptr : vmeta.strides.data(), vmeta.offset, &o) != HGPU_OK)
    return false;
  h = o;
  fa.reset();
  fb.reset();
  fc.reset();
  vsrc.reset();
  ekind = -1;
  return true;
}

void ArrHolder::force() {
  if (h) return;
  if (probe) throw ProbeFail{};
  if (ssrc) {   // a sum nobody's pass has taken along: a pass of its own
      T e(ssrc);
    ssrc.reset();
    T r;
    const hgpu_api* api = be->api;
    if (e.pending_expr() && api->struct_size >= offsetof(hgpu_api, fused_sum) + sizeof(api->fused_sum) && api->fused_sum) {
      std::vector<const hgpu_array*> ins;
      std::vector<hgpu_fused_instr> prog;
      std::vector<int> slots;
      number_program({e.holder().get()}, &ins, &prog, &slots);
      if ((int)ins.size() <= 12 && (int)prog.size() <= 96) {
        hgpu_array* o = nullptr;
        int rc = api->fused_sum(be->ctx, (int)ins.size(), ins.data(), (int)prog.size(), prog.data(), slots[0], &o);
        if (rc == HGPU_OK) r = T(be, o);
        else if (rc != HGPU_ERR_UNSUPPORTED) be->check(rc);
      }
    }
    if (!r.valid()) r = contract_now(e, nullptr, 0);
    be->check(be->api->retain(r.h()));
    h = r.h();
    return;
  }
  if (vsrc && ekind < 0) {   // a pending view: its source once, for every view of it, then the strides
    T s(vsrc);
    hgpu_array* base = s.h();
    be->check(be->api->retain(base));
    if (!be->api->is_dense(base)) {   // vmeta counts in the dense row-major layout of the source
      hgpu_array* d = nullptr;
      int rc = be->api->materialize(be->ctx, base, &d);
      be->api->release(base);
      be->check(rc);
      base = d;
    }
    if (!vlo.empty()) {
      hgpu_array* d = nullptr;
      int rc = be->api->pad(be->ctx, base, ptr_or_dummy(vlo), ptr_or_dummy(vhi), &d);
      be->api->release(base);
      be->check(rc);
      base = d;
    }
    hgpu_array* o = nullptr;
    int rc = be->api->as_strided(be->ctx, base, (int)vmeta.shape.size(), ptr_or_dummy(vmeta.shape), ptr_or_dummy(vmeta.strides), vmeta.offset, &o);
    be->api->release(base);
    be->check(rc);
    h = o;
    vsrc.reset();
    return;
  }
  if (mv_inner) {   // the refined expression written out densely, its dims merged (a view)
    T in(mv_inner);
    hgpu_array* o = nullptr;
    be->check(be->api->reshape(be->ctx, in.h(), (int)mv_shape.size(), ptr_or_dummy(mv_shape), &o));
    h = o;
    mv_inner.reset();
    return;
  }
  if (!pieces.empty()) {   // write the concatenation out: one allocation, one copy (or fill) per piece
    std::vector<T> parts;
    for (auto& pc : pieces) {
      Shape sh = pshape;
      sh[0] = pc.len;
      parts.push_back(pc.v ? T(pc.v) : zeros(be, pdtype, sh));
    }
    std::vector<const hgpu_array*> hs;
    for (auto& t : parts) hs.push_back(t.h());
    hgpu_array* o = nullptr;
    be->check(be->api->concat(be->ctx, (int)hs.size(), hs.data(), &o));
    h = o;
    pieces.clear();
    return;
  }
  if (ekind >= 0) {
    if (view_of_written_source()) return;
    force_roots(be, {this});
    return;
  }
  if (!fa) return;
  if (!more.empty()) {   // a sum of contractions: one grouped call when the provider has it
    std::vector<T> as{T(fa)}, bs{T(fb)};
    for (auto& m : more) { as.push_back(T(m.first)); bs.push_back(T(m.second)); }
    const hgpu_api* api = be->api;
    hgpu_array* o = nullptr;
    bool one_shape = true;
    for (size_t i = 1; i < as.size(); ++i) one_shape = one_shape && as[i].shape() == as[0].shape();
    if (!one_shape && api->struct_size >= offsetof(hgpu_api, contract_sum_map) + sizeof(api->contract_sum_map) && api->contract_sum_map) {
      // products over contracted dims of different lengths (W x + V s): the sum alone, by the kernel that would also run a program over it
      std::vector<const hgpu_array*> ah, bh;
      for (size_t i = 0; i < as.size(); ++i) { ah.push_back(as[i].h()); bh.push_back(bs[i].h()); }
      const hgpu_array* none = nullptr;
      const int slot = 0;
      be->check(api->contract_sum_map(be->ctx, (int)ah.size(), ah.data(), bh.data(), keep, 1, &none, 0, nullptr, 1, &slot, &o));
    } else if (one_shape && api->struct_size >= offsetof(hgpu_api, contract_sum) + sizeof(api->contract_sum) && api->contract_sum) {
      std::vector<const hgpu_array*> ah, bh;
      for (size_t i = 0; i < as.size(); ++i) { ah.push_back(as[i].h()); bh.push_back(bs[i].h()); }
      be->check(api->contract_sum(be->ctx, (int)ah.size(), ah.data(), bh.data(), keep, &o));
    } else {
      T acc = contract_now(as[0], &bs[0], keep);
      for (size_t i = 1; i < as.size(); ++i) acc = ewise2_now(HGPU_ADD, acc, contract_now(as[i], &bs[i], keep));
      be->check(api->retain(acc.h()));
      o = acc.h();
    }
    h = o;
    fa.reset();
    fb.reset();
    more.clear();
    origin.reset();
    keep = -1;
    return;
  }
  T p;
  if (origin && (origin->h || origin.use_count() > 1)) {
    origin->force();   // once for all its users
    p = transpose(T(origin), origin_perm);
  } else {
    if (whole && !whole->h && whole->vsrc && whole->vsrc->h) whole->view_of_written_source();
    T fbt(fb);
    if (whole && whole->h && !ones_b) p = contract_now(T(whole), nullptr, keep);   // the product has been written out meanwhile
    else p = ones_b ? contract_now(T(fa), nullptr, keep) : contract_now(T(fa), &fbt, keep);   // a sum nobody's pass has taken along
  }
  be->check(be->api->retain(p.h()));
  h = p.h();
  fa.reset();
  fb.reset();
  whole.reset();
  origin.reset();
  keep = -1;
  ones_b = false;
}

// Two pending contractions can wait as one pending sum when their factors have
// one shape, or -- with a provider that sums products of different contracted
// lengths in one kernel (hgpu_contract_sum_map) -- when they keep the same dims.
static bool sums_with(const T& a, const T& b) {
  if (T(a.holder()->fa).shape() == T(b.holder()->fa).shape()) return true;
  const hgpu_api* api = a.be()->api;
  if (!(api->struct_size >= offsetof(hgpu_api, contract_sum_map) + sizeof(api->contract_sum_map) && api->contract_sum_map)) return false;
  return a.holder()->keep >= 1 && a.shape() == b.shape();
}

T add_cotangents(const T& a, const T& b) {
  if (a.contraction_like() && b.contraction_like() && a.be() == b.be() && a.holder()->keep == b.holder()->keep &&
      a.dtype() == b.dtype() && sums_with(a, b)) {
    auto p = new_holder(a.be(), nullptr);
    const ArrHolder* x = a.holder().get();
    const ArrHolder* y = b.holder().get();
    p->fa = x->fa;
    p->fb = x->fb;
    p->keep = x->keep;
    p->more = x->more;
    p->more.push_back({y->fa, y->fb});
    p->more.insert(p->more.end(), y->more.begin(), y->more.end());
    return T(p);
  }
  if ((a.pending_pieces() || b.pending_pieces()) && a.be() == b.be() && a.dtype() == b.dtype() && a.shape() == b.shape()) {
    // piece by piece over the common segmentation: data is added only where both have some
    std::vector<ArrHolder::Piece> pa, pb, out;
    pieces_of(a, &pa);
    pieces_of(b, &pb);
    size_t i = 0, j = 0;
    int64_t ua = 0, ub = 0;   // rows of pa[i] / pb[j] already consumed
    while (i < pa.size() && j < pb.size()) {
      int64_t n = std::min(pa[i].len - ua, pb[j].len - ub);
      auto part = [&](const ArrHolder::Piece& pc, int64_t used) -> T {
        if (!pc.v) return T();
        return (used == 0 && n == pc.len) ? T(pc.v) : slice(T(pc.v), 0, used, n);
      };
      T x = part(pa[i], ua), y = part(pb[j], ub);
      if (x.valid() && y.valid()) out.push_back({n, add_cotangents(x, y).holder()});
      else if (x.valid()) out.push_back({n, x.holder()});
      else if (y.valid()) out.push_back({n, y.holder()});
      else out.push_back({n, nullptr});
      ua += n;
      ub += n;
      if (ua == pa[i].len) { ++i; ua = 0; }
      if (ub == pb[j].len) { ++j; ub = 0; }
    }
    return from_pieces(a.be(), std::move(out), a.shape(), a.dtype());
  }
  return ewise2(HGPU_ADD, a, b);
}

T lazy_mul(const T& a, const T& b) { return ewise2(HGPU_MUL, a, b); }

T lazy_contract(const T& a, const T& b, int n_keep) {
  auto p = new_holder(a.be(), nullptr);
  p->fa = a.holder();
  p->fb = b.holder();
  p->keep = n_keep;
  return T(p);
}

// A view of a pending elementwise expression is the expression of the views
// of its leaves (every operand of an expression has the expression's shape), so
// transposes, slices and windows between two elementwise stages cost no pass
// over memory.  Shared sub-expressions stay shared.
static T map_leaves(const T& a, const std::function<T(const T&)>& view) {
  std::map<const ArrHolder*, std::shared_ptr<ArrHolder>> memo;
  std::function<std::shared_ptr<ArrHolder>(const std::shared_ptr<ArrHolder>&)> go =
      [&](const std::shared_ptr<ArrHolder>& p) -> std::shared_ptr<ArrHolder> {
    auto it = memo.find(p.get());
    if (it != memo.end()) return it->second;
    std::shared_ptr<ArrHolder> r;
    if (!p->h && p->ekind >= 0 && p->vsrc && p->vsrc->h) p->view_of_written_source();   // its source has been written since: a leaf
    if (p->h || p->ekind < 0) {
      // A pending contraction among the leaves is computed once, for every view
      // of it -- but not yet: the view stays pending (strides over its dense
      // result), so that whoever consumes the viewed expression may still take
      // the contraction in with it.
      T leaf(p);
      if (!p->h && p->ekind < 0 && p->fa && p->keep >= 0 && T(p).size() > 0) leaf = make_view(p, dense_meta(T(p).shape()));
      else if (!p->h && !leaf.pending_view()) p->force();
      r = view(leaf).holder();
    } else {
      r = new_holder(p->be, nullptr);
      r->ekind = p->ekind;
      r->eop = p->eop;
      r->edtype = p->edtype;
      r->esize = p->esize;
      r->fa = go(p->fa);
      if (p->fb) r->fb = go(p->fb);
      if (p->fc) r->fc = go(p->fc);
      r->eshape = T(r->fa).shape();
    }
    memo[p.get()] = r;
    return r;
  };
  T res(go(a.holder()));
  // the note: res equals this view of the dense result of the expression it was made from
  if (res.pending_expr() && !a.is_probe()) {
    const ArrHolder* ah = a.holder().get();
    try {
      T pr = view(make_probe(a.be(), ah->vsrc ? ah->vmeta : dense_meta(a.shape()), a.dtype()));
      if (pr.is_probe() && pr.shape() == res.shape()) {
        res.holder()->vsrc = ah->vsrc ? ah->vsrc : a.holder();
        res.holder()->vmeta = pr.holder()->vmeta;
      }
    } catch (ProbeFail&) {
    }
  }
  return res;
}
#define HD_VIEW_OF_EXPR(call) \
  if (a.pending_expr()) return map_leaves(a, [&](const T& x) { return call; });

// ---- pending expressions over a refined index space (ArrHolder::mv_inner) ----

// fine splits dims of coarse: groups[d] adjacent dims of fine multiply to coarse[d].
static bool refines(const Shape& fine, const Shape& coarse, std::vector<int>* groups) {
  groups->clear();
  size_t f = 0;
  for (size_t d = 0; d < coarse.size(); ++d) {
    int64_t n = 1;
    int cnt = 0;
    if (coarse[d] == 1 && (f >= fine.size() || fine[f] != 1)) { groups->push_back(0); continue; }
    while (f < fine.size() && (cnt == 0 || n < coarse[d])) { n *= fine[f++]; ++cnt; }
    if (n != coarse[d]) return false;
    groups->push_back(cnt);
  }
  return f == fine.size();
}

static T make_merged(const T& inner, const Shape& shape, const std::vector<int>& groups) {
  if (!inner.pending_expr()) return reshape(inner, shape);   // already an array: merge its dims now
  auto p = new_holder(inner.be(), nullptr);
  p->mv_inner = inner.holder();
  p->mv_shape = shape;
  p->mv_groups = groups;
  return T(p);
}

// y, whose shape `fine` refines, seen over the refined space (a view for arrays
// and for the leaves of a pending expression: splitting a dim never copies).
static T split_view(const T& y, const Shape& fine) {
  if (y.pending_merged()) {
    T in(y.holder()->mv_inner);
    if (in.shape() == fine) return in;
    return reshape(y, fine);     // writes y out first
  }
  if (y.shape() == fine) return y;
  if (y.pending_expr()) return map_leaves(y, [&](const T& x) { return reshape(x, fine); });
  return reshape(y, fine);
}

// An elementwise operation with a refined operand is applied over the refined
// space; the result is again a refined expression of the same logical shape.
static T lift_merged(const std::vector<const T*>& ops, const std::function<T(const std::vector<T>&)>& apply) {
  const T* m = nullptr;
  for (const T* o : ops)
    if (o->pending_merged()) { m = o; break; }
  const Shape fine = T(m->holder()->mv_inner).shape();
  std::vector<T> split;
  for (const T* o : ops) split.push_back(split_view(*o, fine));
  return make_merged(apply(split), m->holder()->mv_shape, m->holder()->mv_groups);
}
static bool any_merged_same_shape(const std::vector<const T*>& ops) {
  bool any = false;
  for (const T* o : ops) any = any || o->pending_merged();
  if (!any) return false;
  for (const T* o : ops)
    if (o->shape() != ops[0]->shape()) return false;
  return true;
}

T transpose(const T& a, const std::vector<int>& perm) {
  // A refined expression that others hold too (a cotangent fanning out to several
  // consumers) is written out once, below, and viewed; one of our own is permuted
  // group by group and stays pending.
  if (a.pending_merged() && a.holder().use_count() <= 1) {
    const ArrHolder* h = a.holder().get();
    const int rank = (int)h->mv_shape.size();
    std::vector<int> full(perm);
    for (int d = (int)perm.size(); d < rank; ++d) full.push_back(d);
    std::vector<int> first((size_t)rank, 0);
    for (int d = 1; d < rank; ++d) first[(size_t)d] = first[(size_t)d - 1] + h->mv_groups[(size_t)d - 1];
    std::vector<int> fine_perm, groups;
    Shape shape;
    for (int d : full) {
      if (d < 0 || d >= rank) throw HostError(HGPU_ERR_INVALID, "transpose: bad permutation");
      for (int k = 0; k < h->mv_groups[(size_t)d]; ++k) fine_perm.push_back(first[(size_t)d] + k);
      groups.push_back(h->mv_groups[(size_t)d]);
      shape.push_back(h->mv_shape[(size_t)d]);
    }
    return make_merged(transpose(T(h->mv_inner), fine_perm), shape, groups);
  }
  HD_META_VIEW(meta_transpose(a.holder()->vmeta, perm, &m__))
  if (a.pending_merged() && expression_like(a) && a.size() > 0) return transpose(make_view(a.holder(), dense_meta(a.shape())), perm);
  // A product that others hold too and that has an uncomputed contraction beneath
  // it (a cotangent `(W^T dz) * (1 - h * h)` on its way to the bias and to the
  // next products): one kernel will write it out for all of them; this is a view of that.
  if (a.pending_product() && a.holder().use_count() > 1 && a.size() > 0 && holds_pending_contraction(a.holder().get()))
    return transpose(make_view(a.holder(), dense_meta(a.shape())), perm);
  HD_VIEW_OF_EXPR(transpose(x, perm))
  if (a.pending_contraction() && (int)perm.size() <= a.pending_keep())   // permutes kept dims only
  {
    T r = lazy_contract(transpose(a.factor_a(), perm), transpose(a.factor_b(), perm), a.pending_keep());
    r.holder()->origin = a.holder();
    r.holder()->origin_perm = perm;
    return r;
  }
  static const int dummy = 0;
  HD_OUT(transpose(be__->ctx, a.h(), (int)perm.size(), perm.empty() ? &dummy : perm.data(), &o__));
}
T reshape(const T& a, const Shape& s) {
  HD_META_VIEW(meta_reshape(a.holder()->vmeta, s, &m__))
  if (a.pending_expr() && s != a.shape()) {   // only splits dims: a view of every leaf
    std::vector<int> g;
    if (refines(s, a.shape(), &g)) return map_leaves(a, [&](const T& x) { return reshape(x, s); });
    // only merges dims: the expression stays pending over its own, finer space
    if (refines(a.shape(), s, &g)) return make_merged(a, s, g);
  }
  HD_OUT(reshape(be__->ctx, a.h(), (int)s.size(), ptr_or_dummy(s), &o__));
}
T slice(const T& a, int dim, int64_t start, int64_t len) {
  if (dim == 0 && a.pending_pieces() && start >= 0 && len >= 0 && start + len <= a.shape().at(0)) return slice_pieces(a, start, len);
  HD_META_VIEW(meta_slice(a.holder()->vmeta, dim, start, len, &m__))
  HD_VIEW_OF_EXPR(slice(x, dim, start, len))
  HD_OUT(slice(be__->ctx, a.h(), dim, start, len, &o__));
}
T reverse(const T& a, int dim) {
  HD_META_VIEW(meta_reverse(a.holder()->vmeta, dim, &m__))
  HD_VIEW_OF_EXPR(reverse(x, dim))
  HD_OUT(reverse(be__->ctx, a.h(), dim, &o__));
}
T replicate(const T& a, const Shape& pre) {
  if (pre.empty()) return a;
  HD_META_VIEW(meta_replicate(a.holder()->vmeta, pre, &m__))
  // a one-element expression: evaluated by whoever consumes the copies (see broadcast_scalar)
  if (a.pending_expr() && a.size() == 1 && fuses(a.be()) && pending_size(a.holder()) <= 8) {
    Shape sh(pre);
    for (auto e : a.shape()) sh.push_back(e);
    if (prod(sh) > 1) return broadcast_scalar(a, sh);
  }
  // An expression that is replicated stays unevaluated behind a pending view:
  // a contraction may take it in as it is, anything else computes it once, for
  // every view of it.
  if (expression_like(a) && a.size() > 0 && a.be()->fuse) {
    bool pos = true;
    for (auto e : pre) pos = pos && e > 0;
    if (pos) return replicate(make_view(a.holder(), dense_meta(a.shape())), pre);
  }
  // a pending expression is written out before it is replicated: only shrinking
  // or permuting views of it are worth keeping pending
  HD_OUT(replicate(be__->ctx, a.h(), (int)pre.size(), pre.data(), &o__));
}
T index_prefix(const T& a, const Shape& ix) {
  HD_META_VIEW(meta_index_prefix(a.holder()->vmeta, ix, &m__))
  HD_VIEW_OF_EXPR(index_prefix(x, ix))
  HD_OUT(index_prefix(be__->ctx, a.h(), (int)ix.size(), ptr_or_dummy(ix), &o__));
}
T as_strided(const T& a, const Shape& shape, const Shape& strides, int64_t offset) {
  HD_META_VIEW(meta_as_strided(a.holder()->vmeta, shape, strides, offset, &m__))
  HD_OUT(as_strided(be__->ctx, a.h(), (int)shape.size(), ptr_or_dummy(shape), ptr_or_dummy(strides), offset, &o__));
}
T materialize(const T& a) {
  if (a.is_probe()) throw ProbeFail{};
  HD_OUT(materialize(be__->ctx, a.h(), &o__));
}
T pad(const T& a, const Shape& lo, const Shape& hi) {
  if (a.is_probe()) throw ProbeFail{};
  if (a.pending_view() && expression_like(T(a.holder()->vsrc))) {
    T v;
    if (pad_view(a, lo, hi, &v)) return v;
  }
  // zeros before and after along the first dim only: a pending concatenation
  bool first_only = a.be()->fuse && a.rank() >= 1 && (int)lo.size() == a.rank() && (int)hi.size() == a.rank() && lo[0] >= 0 && hi[0] >= 0 && lo[0] + hi[0] > 0;
  for (size_t i = 1; i < lo.size() && first_only; ++i) first_only = lo[i] == 0 && hi[i] == 0;
  if (first_only) {
    std::vector<ArrHolder::Piece> pcs;
    pcs.push_back({lo[0], nullptr});
    pieces_of(a, &pcs);
    pcs.push_back({hi[0], nullptr});
    Shape sh = a.shape();
    sh[0] += lo[0] + hi[0];
    return from_pieces(a.be(), std::move(pcs), sh, a.dtype());
  }
  HD_OUT(pad(be__->ctx, a.h(), ptr_or_dummy(lo), ptr_or_dummy(hi), &o__));
}
static T ewise1_now(int op, const T& a) { HD_OUT(ewise1(be__->ctx, op, a.h(), &o__)); }
static T ewise2_now(int op, const T& a, const T& b) { HD_OUT(ewise2(be__->ctx, op, a.h(), b.h(), &o__)); }
static T compare_now(int cmp, const T& a, const T& b) { HD_OUT(compare(be__->ctx, cmp, a.h(), b.h(), &o__)); }

// The elementwise methods defer when the provider can run fused programs and
// the operands agree (a mismatch goes to the eager entry point, which reports it).
static bool agree(const T& a, const T& b) { return a.dtype() == b.dtype() && a.shape() == b.shape(); }
static bool is_fp_dt(int dt) { return dt == HGPU_F64 || dt == HGPU_F32; }
static bool is_int_dt(int dt) { return dt >= HGPU_I64 && dt <= HGPU_I8; }
static bool op1_ok(int op, int dt) {
  if (op < 0 || op >= HGPU_OP1_COUNT) return false;
  if (op >= HGPU_RECIP && op <= HGPU_ATANH) return is_fp_dt(dt);
  return (op == HGPU_NOT) == (dt == HGPU_BOOL);
}
static bool op2_ok(int op, int dt) {
  if (op < 0 || op >= HGPU_OP2_COUNT) return false;
  if (op >= HGPU_DIV && op <= HGPU_ATAN2) return is_fp_dt(dt);
  if (op >= HGPU_QUOT && op <= HGPU_REM_SCALAR) return is_int_dt(dt);
  return (op == HGPU_AND) == (dt == HGPU_BOOL);
}
T ewise1(int op, const T& a) {
  if (a.pending_merged()) return lift_merged({&a}, [&](const std::vector<T>& v) { return ewise1(op, v[0]); });
  if (!fuses(a.be()) || !op1_ok(op, a.dtype()) || a.size() == 0) return ewise1_now(op, a);
  return make_expr(HGPU_FUSED_OP1, op, a.dtype(), a, nullptr, nullptr);
}
T ewise2(int op, const T& a, const T& b) {
  if (any_merged_same_shape({&a, &b})) return lift_merged({&a, &b}, [&](const std::vector<T>& v) { return ewise2(op, v[0], v[1]); });
  // W x + V s, both products still pending and of one shape: a pending sum of contractions
  if (op == HGPU_ADD && a.contraction_like() && b.contraction_like() && a.be() == b.be() && a.be()->fuse && a.holder()->keep == b.holder()->keep &&
      a.dtype() == b.dtype() && sums_with(a, b))
    return add_cotangents(a, b);
  if (!fuses(a.be()) || !agree(a, b) || !op2_ok(op, a.dtype()) || a.size() == 0) return ewise2_now(op, a, b);
  return make_expr(HGPU_FUSED_OP2, op, a.dtype(), a, &b, nullptr);
}
T compare(int cmp, const T& a, const T& b) {
  if (any_merged_same_shape({&a, &b})) return lift_merged({&a, &b}, [&](const std::vector<T>& v) { return compare(cmp, v[0], v[1]); });
  if (!fuses(a.be()) || !agree(a, b) || cmp < HGPU_LEQ || cmp > HGPU_LT || a.size() == 0) return compare_now(cmp, a, b);
  return make_expr(HGPU_FUSED_CMP, cmp, HGPU_BOOL, a, &b, nullptr);
}
bool compare_all(int cmp, const T& a, const T& b) {
  int r = 0;
  a.be()->check(a.be()->api->compare_all(a.be()->ctx, cmp, a.h(), b.h(), &r));
  return r != 0;
}
static T select_now(const T& c, const T& a, const T& b) { HD_OUT(select(be__->ctx, c.h(), a.h(), b.h(), &o__)); }
static T convert_now(const T& a, int dtype, int mode) { HD_OUT(convert(be__->ctx, a.h(), dtype, mode, &o__)); }
T select(const T& c, const T& a, const T& b) {
  if (any_merged_same_shape({&c, &a, &b})) return lift_merged({&c, &a, &b}, [&](const std::vector<T>& v) { return select(v[0], v[1], v[2]); });
  if (!fuses(a.be()) || !agree(a, b) || c.dtype() != HGPU_BOOL || c.shape() != a.shape() || a.size() == 0) return select_now(c, a, b);
  return make_expr(HGPU_FUSED_SELECT, 0, a.dtype(), c, &a, &b);
}
T convert(const T& a, int dtype, int mode) {
  if (a.dtype() == dtype && mode == HGPU_CONV_CAST) return a;
  if (a.pending_merged()) return lift_merged({&a}, [&](const std::vector<T>& v) { return convert(v[0], dtype, mode); });
  bool ok = dtype >= HGPU_F64 && dtype <= HGPU_BOOL && (mode == HGPU_CONV_CAST || (mode == HGPU_CONV_FLOOR && is_fp_dt(a.dtype()) && is_int_dt(dtype)));
  if (!fuses(a.be()) || !ok || a.size() == 0) return convert_now(a, dtype, mode);
  return make_expr(HGPU_FUSED_CONVERT, mode, dtype, a, nullptr, nullptr);
}
// Does the expression beneath p have a leaf that is a contraction (or a sum of contractions) not yet computed?
// The pending contraction (or sum of contractions) among the leaves of an expression, if there is one.
static const ArrHolder* pending_contraction_in(const ArrHolder* root) {
  std::map<const ArrHolder*, int> seen;
  std::vector<const ArrHolder*> stack{root};
  while (!stack.empty()) {
    const ArrHolder* p = stack.back();
    stack.pop_back();
    if (seen.count(p)) continue;
    seen[p] = 1;
    if (contraction_or_sum(p)) return p;
    if (!p->h && p->vsrc) { stack.push_back(p->vsrc.get()); continue; }
    if (p->h || p->ekind < 0) continue;
    if (p->fa) stack.push_back(p->fa.get());
    if (p->fb) stack.push_back(p->fb.get());
    if (p->fc) stack.push_back(p->fc.get());
  }
  return nullptr;
}

// A matrix product with a short contracted dim (two kept dims that are not 1,
// at most 1024 contracted elements over all terms): what the provider's
// hgpu_contract_sum_map computes together with a program over it.
static bool short_matrix_product(const ArrHolder* c) {
  if (!c || c->keep < 1) return false;
  const Shape kept = T(std::const_pointer_cast<ArrHolder>(c->fa)).shape();
  int wide = 0;
  for (int d = 0; d < c->keep; ++d) wide += kept[(size_t)d] != 1;
  if (wide != 2) return false;
  int64_t k = 0;
  auto contracted = [&](const std::shared_ptr<ArrHolder>& f) {
    const Shape sh = T(f).shape();
    int64_t n = 1;
    for (size_t d = (size_t)c->keep; d < sh.size(); ++d) n *= sh[d];
    return n;
  };
  k += contracted(c->fa);
  for (auto& m : c->more) k += contracted(m.first);
  return k <= 1024;
}

static bool holds_pending_contraction(const ArrHolder* root) {
  std::map<const ArrHolder*, int> seen;
  std::vector<const ArrHolder*> stack{root};
  while (!stack.empty()) {
    const ArrHolder* p = stack.back();
    stack.pop_back();
    if (seen.count(p)) continue;
    seen[p] = 1;
    if (contraction_or_sum(p)) return true;
    if (!p->h && p->vsrc) { stack.push_back(p->vsrc.get()); continue; }
    if (p->h || p->ekind < 0) continue;
    if (p->fa) stack.push_back(p->fa.get());
    if (p->fb) stack.push_back(p->fb.get());
    if (p->fc) stack.push_back(p->fc.get());
  }
  return false;
}

T contract(const T& a, const T* b, int n_keep) {
  if (!b && a.pending_product()) {   // sum (u * v) = the contraction of u and v; stays pending
    // ... unless a factor still holds an uncomputed contraction (the cotangent
    // W^T dz under `* (1 - h * h)`): taken apart, the factors would be written
    // out one by one; whole, the product is one kernel's result, which the
    // other consumers of the product need anyway.  Its sum is then its
    // contraction with ones.
    if (n_keep >= 1 && fuses(a.be()) && holds_pending_contraction(a.holder().get()))
      return lazy_contract(a, broadcast_scalar(constant(a.be(), a.dtype(), 1.0), a.shape()), n_keep);
    T r = lazy_contract(a.factor_a(), a.factor_b(), n_keep);
    r.holder()->whole = a.holder();
    return r;
  }
  // the sum of a view of such a product likewise waits (sums of one shape then go out together)
  if (!b && n_keep >= 1 && n_keep < a.rank() && a.pending_view() && fuses(a.be()) && a.holder()->vlo.empty() && T(a.holder()->vsrc).pending_product() &&
      (a.dtype() == HGPU_F64 || a.dtype() == HGPU_F32) && holds_pending_contraction(a.holder()->vsrc.get()))
    return lazy_contract(a, broadcast_scalar(constant(a.be(), a.dtype(), 1.0), a.shape()), n_keep);
  // The sum over all dims but one of an expression seen through a transpose (the
  // cotangent of a bias that was replicated and transposed into a layer's
  // shape): when somebody writes the expression out, the sum is taken in that
  // pass; it waits for that (forced on its own it is what it would be now).
  if (!b && n_keep == 1 && (a.pending_view() || (a.pending_expr() && a.holder()->vsrc)) && fuses(a.be()) && (a.dtype() == HGPU_F64 || a.dtype() == HGPU_F32) && a.size() > 0 &&
      expression_like(T(a.holder()->vsrc)) && front_dim_of_view(a.holder().get()) >= 0) {
    const hgpu_api* api = a.be()->api;
    if (api->struct_size >= offsetof(hgpu_api, fused_map_dimsum) + sizeof(api->fused_map_dimsum) && api->fused_map_dimsum) {
      T r = lazy_contract(a, broadcast_scalar(constant(a.be(), a.dtype(), 1.0), a.shape()), 1);
      r.holder()->ones_b = true;
      a.be()->pending_dimsums.push_back(r.holder());
      return r;
    }
  }
  // ssum0 of a pending expression: summed while it is evaluated, never written
  if (!b && n_keep == 0 && a.pending_expr() && a.size() > 0 && (a.dtype() == HGPU_F64 || a.dtype() == HGPU_F32)) {
    Backend* be = a.be();
    const hgpu_api* api = be->api;
    // ... and when the provider can sum in the pass that writes other expressions
    // of this shape, the sum waits for such a pass (the gradient's)
    if (be->fuse && api->struct_size >= offsetof(hgpu_api, fused_map_sums) + sizeof(api->fused_map_sums) && api->fused_map_sums && pending_size(a.holder()) <= 40 &&
        a.size() >= 4096) {
      auto p = new_holder(be, nullptr);
      p->ssrc = a.holder();
      auto& ps = be->pending_sums;
      ps.erase(std::remove_if(ps.begin(), ps.end(), [](const std::weak_ptr<ArrHolder>& w) { auto q = w.lock(); return !q || q->h || !q->ssrc; }), ps.end());
      ps.push_back(p);
      return T(p);
    }
    if (api->struct_size >= offsetof(hgpu_api, fused_sum) + sizeof(api->fused_sum) && api->fused_sum && pending_size(a.holder()) <= 96) {
      std::vector<const hgpu_array*> ins;
      std::vector<hgpu_fused_instr> prog;
      std::vector<int> slots;
      number_program({a.holder().get()}, &ins, &prog, &slots);
      if ((int)ins.size() <= 12 && (int)prog.size() <= 96) {
        hgpu_array* o = nullptr;
        int rc = api->fused_sum(be->ctx, (int)ins.size(), ins.data(), (int)prog.size(), prog.data(), slots[0], &o);
        if (rc == HGPU_OK) return T(be, o);
        if (rc != HGPU_ERR_UNSUPPORTED) be->check(rc);
      }
    }
  }
  // sdot0 with an expression for an operand (`sdot0 (log soft) expected`, an objective's value): the sum
  // of the product expression, which waits for a pass over arrays of this shape like any other such sum
  if (b && n_keep == 0 && (a.pending_expr() || b->pending_expr()) && a.dtype() == b->dtype() && a.shape() == b->shape() && a.size() >= 4096 &&
      (a.dtype() == HGPU_F64 || a.dtype() == HGPU_F32) && fuses(a.be()) && pending_size(a.holder()) + pending_size(b->holder()) < 40) {
    const hgpu_api* api = a.be()->api;
    if (api->struct_size >= offsetof(hgpu_api, fused_map_sums) + sizeof(api->fused_map_sums) && api->fused_map_sums) {
      Backend* be = a.be();
      auto p = new_holder(be, nullptr);
      p->ssrc = make_expr(HGPU_FUSED_OP2, HGPU_MUL, a.dtype(), a, b, nullptr).holder();
      auto& ps = be->pending_sums;
      ps.erase(std::remove_if(ps.begin(), ps.end(), [](const std::weak_ptr<ArrHolder>& w) { auto q = w.lock(); return !q || q->h || !q->ssrc; }), ps.end());
      ps.push_back(p);
      return T(p);
    }
  }
  // a contraction of two arrays of one shape and dtype stays pending too: sums of
  // such (add_cotangents) are then written out by one grouped launch
  if (b && a.be()->fuse && a.dtype() == b->dtype() && a.shape() == b->shape() && n_keep >= 0 && n_keep <= a.rank() && a.size() > 0 &&
      (a.dtype() == HGPU_F64 || a.dtype() == HGPU_F32))
    return lazy_contract(a, *b, n_keep);
  return contract_now(a, b, n_keep);
}
namespace {
// One operand of hgpu_contract_operands and the storage its pointers point into.
struct OperandBuf {
  hgpu_operand op;
  std::vector<const hgpu_array*> ins;
  std::vector<hgpu_fused_instr> prog;
  std::vector<int> slots;
  Shape mshape, lo, hi, shape, strides;
};
bool virtual_operand(const T& t) { return t.valid() && t.pending_view() && expression_like(T(t.holder()->vsrc)); }
void fill_operand(const T& t, OperandBuf* ob) {
  std::memset(&ob->op, 0, sizeof ob->op);
  if (!virtual_operand(t)) { ob->op.array = t.h(); return; }
  const ArrHolder* h = t.holder().get();
  T src(h->vsrc);
  T e = src.pending_merged() ? T(src.holder()->mv_inner) : src;
  number_program({e.holder().get()}, &ob->ins, &ob->prog, &ob->slots);
  ob->mshape = src.shape();
  ob->lo = h->vlo;
  ob->hi = h->vhi;
  ob->shape = h->vmeta.shape;
  ob->strides = h->vmeta.strides;
  ob->op.n_in = (int)ob->ins.size();
  ob->op.in = ob->ins.data();
  ob->op.n_instr = (int)ob->prog.size();
  ob->op.prog = ob->prog.data();
  ob->op.slot = ob->slots[0];
  ob->op.rank_m = (int)ob->mshape.size();
  ob->op.mshape = ptr_or_dummy(ob->mshape);
  ob->op.lo = ob->lo.empty() ? nullptr : ob->lo.data();
  ob->op.hi = ob->hi.empty() ? nullptr : ob->hi.data();
  ob->op.rank = (int)ob->shape.size();
  ob->op.shape = ptr_or_dummy(ob->shape);
  ob->op.strides = ptr_or_dummy(ob->strides);
  ob->op.offset = h->vmeta.offset;
}
}  // namespace

static T contract_now(const T& a, const T* b, int n_keep) {
  // An operand that is a view of an unevaluated expression goes to the provider
  // as the expression: a kernel that evaluates it while staging never writes it
  // out.  Where there is no such kernel the expression is computed once (for
  // all its views) and the plain contraction runs on the views.
  Backend* be = a.be();
  const hgpu_api* api = be->api;
  // ... unless the expression stands on a short matrix product that is still
  // pending (the cotangent `W^T dz` under `* (1 - h * h)`): product and program
  // are one kernel of their own, and numbering the expression as an operand
  // would write the product out alone first.
  if (api->struct_size >= offsetof(hgpu_api, contract_sum_map) + sizeof(api->contract_sum_map) && api->contract_sum_map && be->fuse) {
    for (const T* t : {&a, b}) {
      if (!t || !virtual_operand(*t)) continue;
      const ArrHolder* src = t->holder()->vsrc.get();
      if (short_matrix_product(pending_contraction_in(src->mv_inner ? src->mv_inner.get() : src))) (void)T(t->holder()->vsrc).h();
    }
  }
  if ((virtual_operand(a) || (b && virtual_operand(*b))) && api->struct_size >= offsetof(hgpu_api, contract_operands) + sizeof(api->contract_operands) &&
      api->contract_operands && a.size() > 0) {
    OperandBuf oa, ob;
    fill_operand(a, &oa);
    if (b) fill_operand(*b, &ob);
    if ((int)oa.ins.size() <= 12 && (int)oa.prog.size() <= 96 && (int)ob.ins.size() <= 12 && (int)ob.prog.size() <= 96) {
      hgpu_array* o = nullptr;
      int rc = api->contract_operands(be->ctx, &oa.op, b ? &ob.op : nullptr, n_keep, 1, &o);
      if (rc == HGPU_OK) {
        be->counters["contract_operands"]++;
        return T(be, o);
      }
      if (rc != HGPU_ERR_UNSUPPORTED) be->check(rc);
    }
  }
  HD_OUT(contract(be__->ctx, a.h(), b ? b->h() : nullptr, n_keep, &o__));
}
T argminmax_last(const T& a, bool want_max) { HD_OUT(argminmax_last(be__->ctx, a.h(), want_max ? 1 : 0, &o__)); }
// The pieces of t along its first dim (t itself when it is not a pending concatenation).
static void pieces_of(const T& t, std::vector<ArrHolder::Piece>* out) {
  if (t.pending_pieces()) {
    for (auto& pc : t.holder()->pieces) out->push_back(pc);
  } else {
    out->push_back({t.shape().at(0), t.holder()});
  }
}
static T from_pieces(Backend* be, std::vector<ArrHolder::Piece> pcs, const Shape& shape, int dtype) {
  // neighbours without data merge; a single piece with data is that array
  std::vector<ArrHolder::Piece> m;
  for (auto& pc : pcs) {
    if (pc.len == 0) continue;
    if (!pc.v && !m.empty() && !m.back().v) m.back().len += pc.len;
    else m.push_back(pc);
  }
  if (m.size() == 1 && m[0].v) return T(m[0].v);
  if (m.empty()) return zeros(be, dtype, shape);
  auto p = new_holder(be, nullptr);
  p->pieces = std::move(m);
  p->pshape = shape;
  p->pdtype = dtype;
  return T(p);
}
// rows [start, start + len) of a pending concatenation: the pieces that overlap them
static T slice_pieces(const T& a, int64_t start, int64_t len) {
  std::vector<ArrHolder::Piece> out;
  int64_t at = 0;
  for (auto& pc : a.holder()->pieces) {
    int64_t lo = std::max(start, at), hi = std::min(start + len, at + pc.len);
    if (lo < hi) {
      if (!pc.v) out.push_back({hi - lo, nullptr});
      else if (lo == at && hi == at + pc.len) out.push_back(pc);
      else out.push_back({hi - lo, slice(T(pc.v), 0, lo - at, hi - lo).holder()});
    }
    at += pc.len;
  }
  Shape sh = a.shape();
  sh[0] = len;
  return from_pieces(a.be(), std::move(out), sh, a.dtype());
}

T concat(const std::vector<T>& parts) {
  if (parts.empty()) throw HostError(HGPU_ERR_INVALID, "concat of nothing");
  {
    const T& a0 = parts[0];
    bool lazy = a0.be()->fuse && a0.rank() >= 1;
    Shape sh = a0.shape();
    int64_t total = 0;
    for (auto& p : parts) {
      Shape s = p.shape();
      lazy = lazy && p.dtype() == a0.dtype() && s.size() == sh.size() && std::equal(s.begin() + 1, s.end(), sh.begin() + 1);
      if (lazy) total += s[0];
    }
    if (lazy) {   // shapes agree: stays a list of pieces until someone needs the whole
      std::vector<ArrHolder::Piece> pcs;
      for (auto& p : parts) pieces_of(p, &pcs);
      sh[0] = total;
      return from_pieces(a0.be(), std::move(pcs), sh, a0.dtype());
    }
  }
  std::vector<const hgpu_array*> hs;
  for (auto& p : parts) hs.push_back(p.h());
  const T& a = parts[0];
  HD_OUT(concat(be__->ctx, (int)hs.size(), hs.data(), &o__));
}
T gather_raw(const T& a, const std::vector<T>& ix, const Shape& shm) {
  std::vector<const hgpu_array*> hs;
  for (auto& p : ix) hs.push_back(p.h());
  const hgpu_array* dummy = nullptr;
  HD_OUT(gather(be__->ctx, a.h(), (int)hs.size(), hs.empty() ? &dummy : hs.data(), (int)shm.size(), ptr_or_dummy(shm), &o__));
}
T scatter_raw(const T& a, const std::vector<T>& ix, int rank_m, const Shape& shp, int flags) {
  std::vector<const hgpu_array*> hs;
  for (auto& p : ix) hs.push_back(p.h());
  const hgpu_array* dummy = nullptr;
  HD_OUT(scatter_add(be__->ctx, a.h(), (int)hs.size(), hs.empty() ? &dummy : hs.data(), rank_m, ptr_or_dummy(shp), flags, &o__));
}
T onehot(const T& a, const Shape& ix, const Shape& shp) {
  HD_OUT(onehot(be__->ctx, a.h(), (int)ix.size(), ptr_or_dummy(ix), ptr_or_dummy(shp), &o__));
}

T broadcast_scalar(const T& s, const Shape& shape) {
  if (s.size() != 1) throw HostError(HGPU_ERR_INVALID, "broadcast_scalar: not a scalar");
  Shape st(shape.size(), 0);
  for (auto e : shape)
    if (e == 0) return replicate(reshape(s, {}), shape);
  // A one-element EXPRESSION that is repeated stays an expression, over its leaves repeated: the
  // consumer's pass evaluates it (`recip (ssum0 e)` under `sreplicate0N`, the negated cotangent
  // of a negated objective), instead of a launch of its own for one element.
  if (s.pending_expr() && prod(shape) > 1 && fuses(s.be()) && pending_size(s.holder()) <= 8)
    return map_leaves(s, [&](const T& x) { return broadcast_scalar(x, shape); });
  T r = as_strided(s, shape, st, 0);
  if (r.holder() != s.holder()) r.holder()->scalar_src = s.holder();
  return r;
}

T zeros(Backend* be, int dtype, const Shape& shape) { return broadcast_scalar(constant_i(be, dtype, 0), shape); }

// ------------------------------------------------- BaseTensor-named methods

static std::vector<int> rotate_left(int rank, int k) {  // [k..rank-1, 0..k-1]
  std::vector<int> p((size_t)rank);
  for (int i = 0; i < rank; ++i) p[(size_t)i] = (i + k) % rank;
  return p;
}

// Ops.hs:511-516, OpsConcrete.hs:215-228
T tssumN(const T& t, int k) {
  int r = t.rank();
  if (k < 0 || k > r) throw HostError(HGPU_ERR_INVALID, "tssumN: more summed dims than rank");
  if (k == 0) return t;
  return contract(k == r ? t : transpose(t, rotate_left(r, k)), nullptr, r - k);
}
T tssum(const T& t) { return tssumN(t, 1); }
T tssum0(const T& t) { return contract(t, nullptr, 0); }                      // Ops.hs:517, OpsConcrete.hs:229
T tsdot0(const T& a, const T& b) { return contract(a, &b, 0); }                // Ops.hs:519, OpsConcrete.hs:231
T tsdot1In(const T& a, const T& b) {                                           // Ops.hs:522, OpsConcrete.hs:233
  if (a.rank() < 1) throw HostError(HGPU_ERR_INVALID, "tsdot1In: rank 0");
  return contract(a, &b, a.rank() - 1);
}
// ssumN @sh (sdot1In u v) in one pass: the form conv layers reach the backend in
// (test/simplified/TestMnistPP.hs:735, `t259 = ssumN @[3, 4] (sdot1In ...)`).
T tsdotNIn(const T& a, const T& b, int n) {
  if (n < 0 || n > a.rank()) throw HostError(HGPU_ERR_INVALID, "tsdotNIn: more contracted dims than rank");
  return contract(a, &b, a.rank() - n);
}
T tsmatvecmul(const T& m, const T& v) {                                        // OpsConcrete.hs:236
  return tsdot1In(m, tsreplicate(v, m.shape().at(0)));
}
T tsmatmul2(const T& m1, const T& m2) {                                        // OpsConcrete.hs:237-242
  Shape s1 = m1.shape(), s2 = m2.shape();
  if (s1.size() != 2 || s2.size() != 2 || s1[1] != s2[0]) throw HostError(HGPU_ERR_INVALID, "tsmatmul2: shapes do not agree");
  T lhs = transpose(tsreplicate(m1, s2[1]), {1, 0});       // [m, p, n]
  T rhs = transpose(tsreplicate(m2, s1[0]), {0, 2, 1});    // [m, p, n]
  return tsdot1In(lhs, rhs);
}
T tsreplicate(const T& t, int64_t k) { return replicate(t, {k}); }            // Ops.hs:548
T tsreplicateN(const T& t, const Shape& shm) { return replicate(t, shm); }     // OpsConcrete.hs:243
T tsreplicate0N(const T& s, const Shape& sh) { return broadcast_scalar(s, sh); }  // OpsConcrete.hs:245
T tsappend(const T& a, const T& b) { return concat({a, b}); }                  // OpsConcrete.hs:638
T tsslice(const T& t, int64_t i, int64_t n) { return slice(t, 0, i, n); }      // OpsConcrete.hs:641
T tsreverse(const T& t) { return reverse(t, 0); }                              // OpsConcrete.hs:644
T tstranspose(const T& t, const std::vector<int>& perm) { return transpose(t, perm); }  // OpsConcrete.hs:647
T tsreshape(const T& t, const Shape& sh) { return reshape(t, sh); }            // OpsConcrete.hs:650
T tsindex(const T& t, const Shape& ix) { return index_prefix(t, ix); }         // OpsConcrete.hs:1477
T tsoneHot(const T& v, const Shape& ix, const Shape& shp) { return onehot(v, ix, shp); }  // OpsConcrete.hs:1516
T tsfloor(const T& t, int dtype) { return convert(t, dtype, HGPU_CONV_FLOOR); }            // OpsConcrete.hs:455
T tsfromIntegral(const T& t, int dtype) { return convert(t, dtype, HGPU_CONV_CAST); }      // OpsConcrete.hs:456
T tscast(const T& t, int dtype) { return convert(t, dtype, HGPU_CONV_CAST); }              // OpsConcrete.hs:518
static T arg_with_values(const T& t, bool want_max) {
  Backend* be = t.be();
  const hgpu_api* api = be->api;
  if (be->fuse && t.rank() >= 1 && api->struct_size >= offsetof(hgpu_api, extremum_last) + sizeof(api->extremum_last) && api->extremum_last) {
    hgpu_array *vals = nullptr, *idx = nullptr;
    be->check(api->extremum_last(be->ctx, t.h(), want_max ? 1 : 0, &vals, &idx));
    T r(be, idx);
    r.holder()->arg_src = t.holder();
    r.holder()->arg_values = T(be, vals).holder();
    return r;
  }
  return argminmax_last(t, want_max);
}
T tsargMin(const T& t) { return arg_with_values(t, false); }                   // OpsConcrete.hs:533
T tsargMax(const T& t) { return arg_with_values(t, true); }                    // OpsConcrete.hs:534
T tsiota(Backend* be, int64_t n, int dtype) { return iota(be, n, dtype); }     // OpsConcrete.hs:535

// ----------------------------------------------------- lane-batched scalars

Ix ix_var(Backend*, const Shape& shm, int d) {
  if (d < 0 || d >= (int)shm.size()) throw HostError(HGPU_ERR_INVALID, "ix_var: no such position variable");
  Ix x;
  x.shm = shm;
  x.affine = true;
  x.coef.assign(shm.size(), 0);
  x.coef[(size_t)d] = 1;
  return x;
}

Ix ix_const(Backend* be, const Shape& shm, int dtype, double v) {
  Ix x;
  x.shm = shm;
  x.dtype = dtype;
  if (dtype == HGPU_I64) {
    x.affine = true;
    x.coef.assign(shm.size(), 0);
    x.c0 = (int64_t)v;
  } else {
    x.arr = broadcast_scalar(constant(be, dtype, v), shm);
  }
  return x;
}

Ix ix_lift(const Shape& shm, const T& scalar) {
  Ix x;
  x.shm = shm;
  x.dtype = scalar.dtype();
  x.arr = broadcast_scalar(scalar, shm);
  if (shm.empty() && scalar.rank() == 0 && scalar.holder()->arg_src) {   // kargMin t of a rank-1 t, used once
    x.arg_of = scalar.holder()->arg_src;
    x.arg_vals = T(scalar.holder()->arg_values);
  }
  return x;
}

static bool is_const(const Ix& x) {
  if (!x.affine) return false;
  for (size_t d = 0; d < x.coef.size(); ++d)
    if (x.coef[d] != 0 && x.shm[d] > 1) return false;
  return true;
}

T ix_array(Backend* be, const Ix& x) {
  if (!x.affine) return x.arr;
  T acc;
  bool c0_done = false;
  for (size_t d = 0; d < x.coef.size(); ++d) {
    if (x.coef[d] == 0 || x.shm[d] <= 1) continue;
    T v = iota(be, x.shm[d], HGPU_I64);
    if (x.coef[d] != 1) v = ewise2(HGPU_MUL, v, broadcast_scalar(constant_i(be, HGPU_I64, x.coef[d]), {x.shm[d]}));
    if (!c0_done && x.c0 != 0) {
      v = ewise2(HGPU_ADD, v, broadcast_scalar(constant_i(be, HGPU_I64, x.c0), {x.shm[d]}));
      c0_done = true;
    }
    Shape st(x.shm.size(), 0);
    st[d] = 1;
    T view = as_strided(v, x.shm, st, 0);
    acc = acc.valid() ? ewise2(HGPU_ADD, acc, view) : view;
  }
  if (!acc.valid()) return broadcast_scalar(constant_i(be, HGPU_I64, x.c0), x.shm);
  if (!c0_done && x.c0 != 0) acc = ewise2(HGPU_ADD, acc, broadcast_scalar(constant_i(be, HGPU_I64, x.c0), x.shm));
  return acc;
}

static Ix from_array(const Shape& shm, const T& arr) {
  Ix x;
  x.shm = shm;
  x.arr = arr;
  x.dtype = arr.dtype();
  return x;
}

static void same_space(const Ix& a, const Ix& b) {
  if (a.shm != b.shm) throw HostError(HGPU_ERR_INVALID, "index values of different position spaces");
  if (a.dtype != b.dtype) throw HostError(HGPU_ERR_INVALID, "index values of different scalar types");
}

Ix ix_op1(Backend* be, int op, const Ix& a) {
  if (a.affine && op == HGPU_NEG) {
    Ix r = a;
    r.c0 = -r.c0;
    for (auto& c : r.coef) c = -c;
    return r;
  }
  return from_array(a.shm, ewise1(op, ix_array(be, a)));
}

Ix ix_op2(Backend* be, int op, const Ix& a, const Ix& b) {
  same_space(a, b);
  if (a.affine && b.affine) {
    if (op == HGPU_ADD || op == HGPU_SUB) {
      Ix r = a;
      int64_t s = op == HGPU_ADD ? 1 : -1;
      r.c0 += s * b.c0;
      for (size_t d = 0; d < r.coef.size(); ++d) r.coef[d] += s * b.coef[d];
      return r;
    }
    if (op == HGPU_MUL && (is_const(a) || is_const(b))) {
      const Ix& k = is_const(a) ? a : b;
      Ix r = is_const(a) ? b : a;
      r.c0 *= k.c0;
      for (auto& c : r.coef) c *= k.c0;
      return r;
    }
    if (is_const(a) && is_const(b)) {  // fold the remaining integer operations (Types.hs:394-419)
      int64_t x = a.c0, y = b.c0, v = 0;
      bool folded = true;
      switch (op) {
        case HGPU_QUOT: v = y == 0 ? x : x / y; break;
        case HGPU_REM: case HGPU_REM_SCALAR: v = y == 0 ? x : x % y; break;
        case HGPU_MIN: v = std::min(x, y); break;
        case HGPU_MAX: v = std::max(x, y); break;
        default: folded = false;
      }
      if (folded) {
        Ix r = a;
        r.c0 = v;
        std::fill(r.coef.begin(), r.coef.end(), 0);
        return r;
      }
    }
  }
  return from_array(a.shm, ewise2(op, ix_array(be, a), ix_array(be, b)));
}

Ix ix_compare(Backend* be, int cmp, const Ix& a, const Ix& b) {
  same_space(a, b);
  return from_array(a.shm, compare(cmp, ix_array(be, a), ix_array(be, b)));
}

Ix ix_select(Backend* be, const Ix& c, const Ix& a, const Ix& b) {
  same_space(a, b);
  if (c.shm != a.shm || c.dtype != HGPU_BOOL) throw HostError(HGPU_ERR_INVALID, "ix_select: condition is not a Bool of the same space");
  T cond = ix_array(be, c);
  Ix r = from_array(a.shm, select(cond, ix_array(be, a), ix_array(be, b)));
  if (is_const(a) && is_const(b) && a.dtype == HGPU_I64) {
    r.sel_cond = cond;
    r.sel_a = a.c0;
    r.sel_b = b.c0;
  }
  return r;
}

Ix ix_convert(Backend* be, const Ix& a, int dtype, int mode) {
  if (a.dtype == dtype) return a;
  return from_array(a.shm, convert(ix_array(be, a), dtype, mode));
}

// Range of an affine index over its position box.
static void affine_range(const Ix& x, int64_t* lo, int64_t* hi) {
  *lo = *hi = x.c0;
  for (size_t d = 0; d < x.coef.size(); ++d) {
    int64_t span = x.coef[d] * (x.shm[d] - 1);
    if (span > 0) *hi += span; else *lo += span;
  }
}

// out[m.., n..] = src[ix(m).., n..] as a view of src (zero-extended first when
// some index leaves the bounds): tgatherZSScalar with an affine index function.
// Returns an invalid T when a view is not sensible.
static T affine_view(const T& src0, const Shape& shm, const std::vector<Ix>& ix) {
  Backend* be = src0.be();
  T src = src0;
  Shape ssh = src.shape();
  size_t n_ix = ix.size();
  Shape oshape = shm;
  oshape.insert(oshape.end(), ssh.begin() + (long)n_ix, ssh.end());
  if (prod(oshape) == 0) return zeros(be, src.dtype(), oshape);
  for (size_t j = 0; j < n_ix; ++j)
    if (ssh[j] == 0) return zeros(be, src.dtype(), oshape);
  std::vector<int64_t> c0(n_ix);
  Shape lo_pad(ssh.size(), 0), hi_pad(ssh.size(), 0);
  bool need_pad = false;
  int64_t padded = 1;
  for (size_t j = 0; j < n_ix; ++j) {
    int64_t lo, hi;
    affine_range(ix[j], &lo, &hi);
    c0[j] = ix[j].c0;
    if (lo < 0) { lo_pad[j] = -lo; need_pad = true; }
    if (hi > ssh[j] - 1) { hi_pad[j] = hi - (ssh[j] - 1); need_pad = true; }
    padded *= ssh[j] + lo_pad[j] + hi_pad[j];
  }
  if (need_pad) {
    int64_t plain = 1;
    for (size_t j = 0; j < n_ix; ++j) plain *= ssh[j];
    if (padded > 4 * plain + 4096) return T();  // mostly out of bounds: not worth a zero-extended copy
    src = pad(src, lo_pad, hi_pad);
    for (size_t j = 0; j < n_ix; ++j) c0[j] += lo_pad[j];
  }
  Shape sst = src.strides();
  Shape ost(oshape.size(), 0);
  int64_t offset = 0;
  for (size_t j = 0; j < n_ix; ++j) {
    offset += c0[j] * sst[j];
    for (size_t d = 0; d < shm.size(); ++d) ost[d] += ix[j].coef[d] * sst[j];
  }
  for (size_t i = n_ix; i < ssh.size(); ++i) ost[shm.size() + (i - n_ix)] = sst[i];
  return as_strided(src, oshape, ost, offset);
}

static bool all_affine(const std::vector<Ix>& ix) {
  for (auto& x : ix)
    if (!x.affine) return false;
  return true;
}

static void check_ix(const Shape& shm, const std::vector<Ix>& ix) {
  for (auto& x : ix) {
    if (x.shm != shm) throw HostError(HGPU_ERR_INVALID, "index function built over another position space");
    if (x.dtype != HGPU_I64) throw HostError(HGPU_ERR_INVALID, "index component is not an Int");
  }
}

// Ops.hs:701-705; OpsConcrete.hs:1621-1665
T tsgather(const T& src, const Shape& shm, const std::vector<Ix>& ix) {
  if ((int)ix.size() > src.rank()) throw HostError(HGPU_ERR_INVALID, "tsgather: more indices than dims");
  check_ix(shm, ix);
  Backend* be = src.be();
  // src at [m_0, .., kargMax (src !$ [m_0, ..])]: the values the arg pass produced
  if (!ix.empty() && (int)ix.size() == src.rank() && ix.back().arg_of && ix.back().arg_of == src.holder() && shm.size() + 1 == ix.size()) {
    bool identity = true;
    Shape ssh = src.shape();
    for (size_t d = 0; d + 1 < ix.size() && identity; ++d) {
      const Ix& x = ix[d];
      identity = x.affine && x.c0 == 0 && shm[d] == ssh[d];
      for (size_t e = 0; e < x.coef.size() && identity; ++e) identity = x.coef[e] == (e == d ? 1 : 0);
    }
    if (identity) return ix.back().arg_vals;
  }
  // A rank-1 table at `ifH c a b` with constant a, b: c ? table[a] : table[b],
  // an elementwise choice (positions outside the table read zero, as any gather).
  if (ix.size() == 1 && src.rank() == 1 && ix[0].sel_cond.valid() && prod(shm) > 0) {
    const int64_t n = src.shape()[0];
    auto element = [&](int64_t k) {
      if (k < 0 || k >= n) return zeros(be, src.dtype(), shm);
      return broadcast_scalar(index_prefix(src, {k}), shm);
    };
    return select(ix[0].sel_cond, element(ix[0].sel_a), element(ix[0].sel_b));
  }
  if (all_affine(ix)) {
    // windows of a pending expression that stay in bounds and do not multiply
    // its elements are taken of its leaves instead
    if (src.pending_expr()) {
      Shape ssh = src.shape();
      int64_t n_out = prod(shm) * prod(ssh, ix.size());
      bool inside = n_out <= src.size();
      for (size_t j = 0; j < ix.size() && inside; ++j) {
        int64_t lo, hi;
        affine_range(ix[j], &lo, &hi);
        inside = lo >= 0 && hi <= ssh[j] - 1;
      }
      if (inside && n_out > 0) return map_leaves(src, [&](const T& x) { return affine_view(x, shm, ix); });
    }
    T v = affine_view(src, shm, ix);
    if (v.valid()) return v;
  }
  std::vector<T> arrs;
  for (auto& x : ix) arrs.push_back(ix_array(be, x));
  return gather_raw(src, arrs, shm);
}

// True when distinct positions provably go to distinct destinations: every
// component, read as a mixed-radix number in the variables it uses, determines
// those variables, and together the components use every variable.
static bool provably_injective(const Shape& shm, const std::vector<Ix>& ix) {
  std::vector<bool> covered(shm.size(), false);
  for (auto& x : ix) {
    if (!x.affine) continue;   // the affine components alone may already separate all positions
    std::vector<std::pair<int64_t, size_t>> terms;
    for (size_t d = 0; d < shm.size(); ++d)
      if (x.coef[d] != 0 && shm[d] > 1) terms.push_back({std::llabs(x.coef[d]), d});
    std::sort(terms.begin(), terms.end());
    int64_t reach = 0;  // largest value the smaller terms can sum to
    bool ok = true;
    for (auto& t : terms) {
      if (t.first <= reach) { ok = false; break; }
      reach += t.first * (shm[t.second] - 1);
    }
    if (ok)
      for (auto& t : terms) covered[t.second] = true;
  }
  for (size_t d = 0; d < shm.size(); ++d)
    if (shm[d] > 1 && !covered[d]) return false;
  return true;
}

// A view of f with the dims listed in `dims` zero-extended by lo / hi; dims f
// is merely replicated along (stride 0) and that get no padding stay replicated.
static T pad_dims(const T& f, const Shape& lo, const Shape& hi) {
  Shape sh = f.shape(), st = f.strides();
  bool any = false;
  for (size_t d = 0; d < sh.size(); ++d) any = any || lo[d] > 0 || hi[d] > 0;
  if (!any) return f;
  Shape sh1 = sh, st1 = st;
  for (size_t d = 0; d < sh.size(); ++d)
    if (st[d] == 0 && lo[d] == 0 && hi[d] == 0) sh1[d] = 1;
  T small = as_strided(f, sh1, st1, 0);
  T padded = pad(small, lo, hi);
  Shape psh = padded.shape(), pst = padded.strides();
  for (size_t d = 0; d < sh.size(); ++d)
    if (sh1[d] == 1 && sh[d] != 1) { psh[d] = sh[d]; pst[d] = 0; }
  return as_strided(padded, psh, pst, 0);
}

// tsscatter with an affine, overlapping index function as a contraction:
//   out[P.., n..] = sum over the positions m with ix(m) = P of src[m.., n..].
// Every component P_j = c_j + m_v + sum_u a_ju m_u must have a "pivot" variable
// m_v (coefficient 1, used by no other component); substituting
// m_v = P_j - c_j - sum_u a_ju m_u turns src into a skewed view over
// (P.., n.., u..) of its zero-extended self, summed over the remaining
// variables u: col2im without atomics, in a fixed summation order.  When src is
// itself a pending contraction the skew is applied to its factors and the
// whole is ONE contraction (the transposed convolution).
static T scatter_as_contraction(const T& src, int rank_m, const Shape& shp, const std::vector<Ix>& ix) {
  Shape ssh = src.shape();
  size_t rm = (size_t)rank_m, n_ix = ix.size(), rank_n = ssh.size() - rm;
  std::vector<int> pivot(n_ix, -1);
  std::vector<bool> is_pivot(rm, false);
  for (size_t j = 0; j < n_ix; ++j) {
    for (size_t d = 0; d < rm && pivot[j] < 0; ++d) {
      if (ix[j].coef[d] != 1 || ssh[d] <= 1 || is_pivot[d]) continue;
      bool elsewhere = false;
      for (size_t j2 = 0; j2 < n_ix; ++j2)
        if (j2 != j && ix[j2].coef[d] != 0) elsewhere = true;
      if (!elsewhere) { pivot[j] = (int)d; is_pivot[d] = true; }
    }
    if (pivot[j] < 0) return T();
  }
  std::vector<size_t> summed;   // position variables that are not pivots
  for (size_t d = 0; d < rm; ++d)
    if (!is_pivot[d]) summed.push_back(d);

  std::vector<T> factors;
  int keep0;   // kept dims of the factors = rank_m + rank_n
  if (src.pending_contraction()) {
    factors = {src.factor_a(), src.factor_b()};
    keep0 = src.pending_keep();
  } else {
    factors = {src};
    keep0 = (int)ssh.size();
  }
  // every pivot must be felt by at least one factor, or out-of-range positions would not vanish
  for (size_t j = 0; j < n_ix; ++j) {
    bool felt = false;
    for (auto& f : factors)
      if (f.strides()[(size_t)pivot[j]] != 0) felt = true;
    if (!felt) return T();
  }
  std::vector<T> views;
  for (auto& f0 : factors) {
    Shape fsh = f0.shape(), fst0 = f0.strides();
    Shape lo(fsh.size(), 0), hi(fsh.size(), 0);
    for (size_t j = 0; j < n_ix; ++j) {
      size_t v = (size_t)pivot[j];
      if (fst0[v] == 0) continue;
      int64_t smin = 0, smax = 0;   // range of sum_u a_ju m_u
      for (size_t d = 0; d < rm; ++d) {
        if (d == v) continue;
        int64_t span = ix[j].coef[d] * (ssh[d] - 1);
        if (span > 0) smax += span; else smin += span;
      }
      int64_t c = ix[j].c0;
      lo[v] = std::max<int64_t>(0, c + smax);
      hi[v] = std::max<int64_t>(0, (shp[j] - 1 - c - smin) - (ssh[v] - 1));
    }
    int64_t grown = 1, plain = 1;
    for (size_t d = 0; d < fsh.size(); ++d)
      if (fst0[d] != 0) { plain *= fsh[d]; grown *= fsh[d] + lo[d] + hi[d]; }
    if (grown > 4 * plain + 4096) return T();
    T f = pad_dims(f0, lo, hi);
    Shape fst = f.strides();
    Shape nsh, nst;
    int64_t offset = 0;
    for (size_t j = 0; j < n_ix; ++j) {            // P dims
      size_t v = (size_t)pivot[j];
      nsh.push_back(shp[j]);
      nst.push_back(fst[v]);
      offset += (lo[v] - ix[j].c0) * fst[v];
    }
    for (size_t i = 0; i < rank_n; ++i) {          // n dims
      nsh.push_back(fsh[rm + i]);
      nst.push_back(fst[rm + i]);
    }
    for (size_t u : summed) {                      // summed position variables, skewed
      int64_t s = fst[u];
      for (size_t j = 0; j < n_ix; ++j) s -= ix[j].coef[u] * fst[(size_t)pivot[j]];
      nsh.push_back(ssh[u]);
      nst.push_back(s);
    }
    for (size_t i = (size_t)keep0; i < fsh.size(); ++i) {   // the factors' own reduced dims
      nsh.push_back(fsh[i]);
      nst.push_back(fst[i]);
    }
    views.push_back(as_strided(f, nsh, nst, offset));
  }
  int n_keep = (int)(n_ix + rank_n);
  // The result may be laid out in any order of its dims: take the memory order
  // of the larger factor (most distinct elements), so the contraction streams
  // it and writes the result in the same order, and hand back a transposed view.
  size_t main_f = 0;
  if (views.size() == 2) {
    auto distinct = [](const T& v) {
      Shape sh = v.shape(), st = v.strides();
      int64_t n = 1;
      for (size_t d = 0; d < sh.size(); ++d)
        if (st[d] != 0) n *= sh[d];
      return n;
    };
    if (distinct(views[1]) > distinct(views[0])) main_f = 1;
  }
  Shape mst = views[main_f].strides();
  std::vector<int> order((size_t)n_keep);
  for (int i = 0; i < n_keep; ++i) order[(size_t)i] = i;
  std::stable_sort(order.begin(), order.end(), [&](int x, int y) {
    int64_t sx = std::llabs(mst[(size_t)x]), sy = std::llabs(mst[(size_t)y]);
    if (sx == 0) sx = INT64_MAX;   // dims the main factor is replicated along go outermost
    if (sy == 0) sy = INT64_MAX;
    return sx > sy;
  });
  bool identity = true;
  for (int i = 0; i < n_keep; ++i) identity = identity && order[(size_t)i] == i;
  if (identity) {
    if (views.size() == 2) return contract_now(views[0], &views[1], n_keep);
    return contract_now(views[0], nullptr, n_keep);
  }
  std::vector<int> inv((size_t)n_keep);
  for (int i = 0; i < n_keep; ++i) inv[(size_t)order[(size_t)i]] = i;
  T va = transpose(views[0], order);
  if (views.size() == 2) {
    T vb = transpose(views[1], order);
    return transpose(contract_now(va, &vb, n_keep), inv);
  }
  return transpose(contract_now(va, nullptr, n_keep), inv);
}

// Ops.hs:689-693; OpsConcrete.hs:1581-1619
T tsscatter(const T& src, int rank_m, const Shape& shp, const std::vector<Ix>& ix) {
  if (rank_m > src.rank() || ix.size() != shp.size()) throw HostError(HGPU_ERR_INVALID, "tsscatter: ranks do not agree");
  Shape ssh = src.shape();
  Shape shm(ssh.begin(), ssh.begin() + rank_m);
  check_ix(shm, ix);
  Backend* be = src.be();
  // "Write each position's value at a data-dependent place of a new small dim"
  // (the adjoint of taking the maximum of a window): every component but the
  // last is the position variable of its own dim.  Then
  //   out[m.., e, n..] = (last(m) == e) ? src[m.., n..] : 0,
  // an elementwise expression: no zero fill, no index traffic, and it fuses
  // with whatever consumes it.  Out-of-bounds places match no e, as they must.
  if (fuses(be) && (size_t)rank_m + 1 == ix.size() && rank_m > 0 && src.size() > 0 && !ix.back().affine && shp.back() > 0) {
    bool identity = true;
    for (size_t j = 0; j + 1 < ix.size() && identity; ++j) {
      const Ix& x = ix[j];
      identity = x.affine && x.c0 == 0 && shp[j] == shm[j];
      for (size_t d = 0; d < x.coef.size() && identity; ++d) identity = x.coef[d] == (d == j ? 1 : 0);
    }
    if (identity) {
      const int64_t E = shp.back();
      const size_t rm = (size_t)rank_m, rank_n = ssh.size() - rm;
      Shape osh(shm);
      osh.push_back(E);
      osh.insert(osh.end(), ssh.begin() + rank_m, ssh.end());
      auto spread = [&](const T& a, size_t lead, bool has_e) {     // a: [lead dims of osh] (+ [E]) -> shape osh, missing dims replicated
        Shape ast = a.strides(), st(osh.size(), 0);
        for (size_t d = 0; d < lead; ++d) st[d] = ast[d];
        if (has_e) st[rm] = ast[lead];
        return as_strided(a, osh, st, 0);
      };
      T srcv;
      {
        Shape ast = src.strides(), st(osh.size(), 0);
        for (size_t d = 0; d < rm; ++d) st[d] = ast[d];
        for (size_t d = 0; d < rank_n; ++d) st[rm + 1 + d] = ast[rm + d];
        srcv = as_strided(src, osh, st, 0);
      }
      T where = spread(ix_array(be, ix.back()), rm, false);
      T which;
      {
        T io = iota(be, E, HGPU_I64);
        Shape st(osh.size(), 0);
        st[rm] = 1;
        which = as_strided(io, osh, st, 0);
      }
      return select(compare(HGPU_EQ, which, where), srcv, zeros(be, src.dtype(), osh));
    }
  }
  bool injective = provably_injective(shm, ix);
  if (!injective && all_affine(ix) && src.size() > 0) {
    T r = scatter_as_contraction(src, rank_m, shp, ix);
    if (r.valid()) return r;
  }
  // Every destination index is a mixed-radix number whose digits are position
  // variables (out[2 i + p, 2 j + q] = src[i, j, p, q], the adjoint of taking
  // pooling windows) and all of the destination is written exactly once: the
  // scatter is a transposition followed by a merge of the digits.  Of a
  // pending expression that costs nothing: it stays pending over the refined
  // space and is written out, dims merged, by whoever consumes it.
  if (injective && all_affine(ix) && src.size() > 0 && src.pending_expr()) {
    std::vector<int> perm, groups;
    std::vector<bool> used((size_t)rank_m, false);
    bool ok = true;
    for (size_t j = 0; j < ix.size() && ok; ++j) {
      std::vector<std::pair<int64_t, int>> digits;   // (coefficient, position dim)
      for (int d = 0; d < rank_m; ++d)
        if (ix[j].coef[(size_t)d] != 0) digits.push_back({ix[j].coef[(size_t)d], d});
      std::sort(digits.begin(), digits.end(), [](const std::pair<int64_t, int>& x, const std::pair<int64_t, int>& y) { return x.first > y.first; });
      ok = ix[j].c0 == 0 && !digits.empty() && digits.back().first == 1;
      for (size_t k = 0; k < digits.size() && ok; ++k) {
        int d = digits[k].second;
        ok = !used[(size_t)d];
        used[(size_t)d] = true;
        int64_t above = k == 0 ? shp[j] : digits[k - 1].first;      // the next digit up counts in units of this one's range
        ok = ok && digits[k].first * shm[(size_t)d] == above && shm[(size_t)d] > 1;
        perm.push_back(d);
      }
      groups.push_back((int)digits.size());
    }
    for (int d = 0; d < rank_m && ok; ++d) ok = used[(size_t)d];
    if (ok) {
      for (int d = rank_m; d < (int)ssh.size(); ++d) { perm.push_back(d); groups.push_back(1); }
      Shape osh(shp);
      osh.insert(osh.end(), ssh.begin() + rank_m, ssh.end());
      return make_merged(transpose(src, perm), osh, groups);
    }
  }
  if (injective && all_affine(ix) && src.size() > 0 &&
      be->api->struct_size >= offsetof(hgpu_api, scatter_affine) + sizeof(be->api->scatter_affine) && be->api->scatter_affine) {
    // no index arrays: the places are computed from the positions
    bool inside = true;
    for (size_t j = 0; j < ix.size() && inside; ++j) {
      int64_t lo, hi;
      affine_range(ix[j], &lo, &hi);
      inside = lo >= 0 && hi <= shp[j] - 1;
    }
    if (inside) {
      std::vector<int64_t> c0(ix.size() + 1, 0), coef((size_t)rank_m * ix.size() + 1, 0);
      for (size_t j = 0; j < ix.size(); ++j) {
        c0[j] = ix[j].c0;
        for (size_t d = 0; d < (size_t)rank_m; ++d) coef[d * ix.size() + j] = ix[j].coef[d];
      }
      hgpu_array* o = nullptr;
      be->check(be->api->scatter_affine(be->ctx, src.h(), rank_m, (int)ix.size(), c0.data(), coef.data(), ptr_or_dummy(shp), &o));
      return T(be, o);
    }
  }
  std::vector<T> arrs;
  for (auto& x : ix) arrs.push_back(ix_array(be, x));
  be->counters[injective ? "scatter_stores" : "scatter_general"]++;
  return scatter_raw(src, arrs, rank_m, shp, injective ? 1 : 0);
}

// tsindex0 at lane-batched indices (AstIndexK, AstInterpret.hs:181-185)
Ix ix_index0(Backend* be, const T& t, const std::vector<Ix>& ix) {
  if ((int)ix.size() != t.rank()) throw HostError(HGPU_ERR_INVALID, "ix_index0: needs one index per dim");
  if (ix.empty()) throw HostError(HGPU_ERR_INVALID, "ix_index0: rank 0");
  const Shape& shm = ix[0].shm;
  check_ix(shm, ix);
  if (all_affine(ix)) {
    // A lookup in a host-known integer table that is itself affine in its
    // indices, with all lookups in bounds, is again an affine form
    // (e.g. the window tables [0..2n-1] reshaped [n,2]: tbl[i,k] = 2i + k).
    if (t.host_i64() && t.dtype() == HGPU_I64) {
      Shape tsh = t.shape(), tst = t.strides();
      bool dense = true;
      int64_t s = 1;
      for (int i = (int)tsh.size() - 1; i >= 0; --i) { if (tsh[(size_t)i] != 1 && tst[(size_t)i] != s) dense = false; s *= tsh[(size_t)i]; }
      bool inb = true;
      for (size_t j = 0; j < ix.size(); ++j) {
        int64_t lo, hi;
        affine_range(ix[j], &lo, &hi);
        if (lo < 0 || hi >= tsh[j]) inb = false;
      }
      const std::vector<int64_t>& tab = *t.host_i64();
      if (dense && inb && (int64_t)tab.size() == prod(tsh) && !tab.empty()) {
        std::vector<int64_t> a(tsh.size(), 0);
        Shape dst(tsh.size());
        int64_t q = 1;
        for (int i = (int)tsh.size() - 1; i >= 0; --i) { dst[(size_t)i] = q; q *= tsh[(size_t)i]; }
        for (size_t j = 0; j < tsh.size(); ++j)
          if (tsh[j] > 1) a[j] = tab[(size_t)dst[j]] - tab[0];
        bool affine_tab = true;
        std::vector<int64_t> idx(tsh.size(), 0);
        for (size_t lin = 0; lin < tab.size() && affine_tab; ++lin) {
          int64_t want = tab[0];
          for (size_t j = 0; j < tsh.size(); ++j) want += a[j] * idx[j];
          if (tab[lin] != want) affine_tab = false;
          for (int j = (int)tsh.size() - 1; j >= 0; --j) {
            if (++idx[(size_t)j] < tsh[(size_t)j]) break;
            idx[(size_t)j] = 0;
          }
        }
        if (affine_tab) {
          t.holder()->host_i64_folded = true;
          Ix r;
          r.shm = shm;
          r.affine = true;
          r.c0 = tab[0];
          r.coef.assign(shm.size(), 0);
          for (size_t j = 0; j < ix.size(); ++j) {
            r.c0 += a[j] * ix[j].c0;
            for (size_t d = 0; d < shm.size(); ++d) r.coef[d] += a[j] * ix[j].coef[d];
          }
          return r;
        }
      }
    }
    // (through tsgather: windows of a pending expression are taken of its leaves, and the result remembers which view of it they are)
    if (t.pending_expr()) return from_array(shm, tsgather(t, shm, ix));
    T v = affine_view(t, shm, ix);
    if (v.valid()) return from_array(shm, v);
  }
  std::vector<T> arrs;
  for (auto& x : ix) arrs.push_back(ix_array(be, x));
  return from_array(shm, gather_raw(t, arrs, shm));
}

// `inner` (a pending expression over [lead.., reduced..]) is noted to be a view
// of an expression whose leaves are arrays and ONE pending contraction of the
// expression's own shape.  Then hgpu_contract_map computes the contraction, the
// expression over it and the first extremum over the view's trailing n_reduce
// dims as one kernel.  Returns false when the pattern or the provider does not fit.
static bool contract_map_extremum(Backend* be, const T& inner, int n_reduce, bool want_max, const Shape& shm, const Shape& lead, Ix* out) {
  const hgpu_api* api = be->api;
  if (!(api->struct_size >= offsetof(hgpu_api, contract_map) + sizeof(api->contract_map) && api->contract_map)) return false;
  const ArrHolder* ih = inner.holder().get();
  if (!ih->vsrc || ih->vmeta.offset != 0 || ih->vmeta.shape != inner.shape()) return false;
  T origin(ih->vsrc);
  if (!origin.pending_expr() || pending_size(origin.holder()) > 40) return false;
  // is there exactly one pending contraction among the leaves?  (look before anything is forced)
  {
    std::map<const ArrHolder*, int> seen;
    std::vector<const ArrHolder*> stack{origin.holder().get()};
    int n_contr = 0;
    while (!stack.empty()) {
      const ArrHolder* p = stack.back();
      stack.pop_back();
      if (seen.count(p)) continue;
      seen[p] = 1;
      if (single_contraction(p)) { ++n_contr; continue; }
      if (p->h || p->ekind < 0) continue;
      if (p->fa) stack.push_back(p->fa.get());
      if (p->fb) stack.push_back(p->fb.get());
      if (p->fc) stack.push_back(p->fc.get());
    }
    if (n_contr != 1) return false;
  }
  std::vector<const hgpu_array*> ins;
  std::vector<hgpu_fused_instr> prog;
  std::vector<int> slots;
  std::vector<ArrHolder*> nodes;
  ArrHolder* kept = nullptr;
  number_program({origin.holder().get()}, &ins, &prog, &slots, &kept, &nodes);
  if (!kept || (int)ins.size() > 12 || (int)prog.size() > 96) {
    if (kept) kept->force();
    return false;
  }
  T fa(kept->fa), fb(kept->fb);
  if (fa.shape() != fb.shape() || fa.dtype() != fb.dtype() || (fa.dtype() != HGPU_F64 && fa.dtype() != HGPU_F32)) return false;
  // Bool results that depend on the contraction are written out as well
  const int n_in = (int)ins.size();
  int c_slot = -1;
  for (int i = 0; i < n_in; ++i)
    if (!ins[(size_t)i]) c_slot = i;
  std::vector<char> dep((size_t)n_in + prog.size(), 0);
  dep[(size_t)c_slot] = 1;
  std::vector<int> out_slots;
  std::vector<ArrHolder*> out_nodes;
  for (size_t k = 0; k < prog.size(); ++k) {
    const hgpu_fused_instr& q = prog[k];
    bool d = dep[(size_t)q.a] != 0;
    if (q.kind == HGPU_FUSED_OP2 || q.kind == HGPU_FUSED_CMP) d = d || dep[(size_t)q.b];
    if (q.kind == HGPU_FUSED_SELECT) d = d || dep[(size_t)q.b] || dep[(size_t)q.c];
    dep[(size_t)n_in + k] = d;
    const bool is_bool = q.kind == HGPU_FUSED_CMP || nodes[k]->edtype == HGPU_BOOL;
    if (d && is_bool && (int)out_slots.size() < 4 && n_in + (int)k != slots[0]) { out_slots.push_back(n_in + (int)k); out_nodes.push_back(nodes[k]); }
  }
  std::vector<hgpu_array*> outs(out_slots.size() + 1, nullptr);
  hgpu_array *vals = nullptr, *idx = nullptr;
  int rc = api->contract_map(be->ctx, fa.h(), fb.h(), kept->keep, n_in, ins.data(), (int)prog.size(), prog.data(), (int)out_slots.size(), out_slots.data(),
                             outs.data(), slots[0], (int)ih->vmeta.shape.size(), ptr_or_dummy(ih->vmeta.shape), ptr_or_dummy(ih->vmeta.strides), n_reduce,
                             want_max ? 1 : 0, &vals, &idx);
  be->check(rc);
  be->counters["contract_map"]++;
  for (size_t i = 0; i < out_nodes.size(); ++i) {
    ArrHolder* r = out_nodes[i];
    r->h = outs[i];
    r->fa.reset();
    r->fb.reset();
    r->fc.reset();
    r->vsrc.reset();
    r->ekind = -1;
  }
  *out = Ix();
  out->shm = shm;
  out->arr = reshape(T(be, idx), lead);
  out->dtype = HGPU_I64;
  out->arg_vals = reshape(T(be, vals), lead);
  return true;
}

Ix ix_argminmax(Backend* be, const T& t, const std::vector<Ix>& ix, bool want_max) {
  if ((int)ix.size() + 1 != t.rank()) throw HostError(HGPU_ERR_INVALID, "ix_argminmax: the partial index must leave one dim");
  if (ix.empty()) throw HostError(HGPU_ERR_INVALID, "ix_argminmax: no position space");
  const Shape& shm = ix[0].shm;
  // the index is the position itself (kargMax (t !$ [i, j, ..]) over t's own
  // leading dims): one pass yields the arguments and the extremal values
  bool identity = shm.size() == ix.size();
  Shape tsh = t.shape();
  for (size_t d = 0; d < ix.size() && identity; ++d) {
    const Ix& x = ix[d];
    identity = x.affine && x.c0 == 0 && shm[d] == tsh[d];
    for (size_t e = 0; e < x.coef.size() && identity; ++e) identity = x.coef[e] == (e == d ? 1 : 0);
  }
  const hgpu_api* api = be->api;
  // t is a pending expression whose last dim merges trailing dims of its own
  // space (pooling windows [.., 2, 2] seen as [.., 4]): the extremum is taken
  // while the expression is evaluated, which is then never written out
  if (identity && be->fuse && t.pending_merged() && api->struct_size >= offsetof(hgpu_api, fused_extremum) + sizeof(api->fused_extremum) &&
      api->fused_extremum) {
    const ArrHolder* mh = t.holder().get();
    int n_reduce = mh->mv_groups.back();
    T inner(mh->mv_inner);
    if (n_reduce >= 1 && inner.pending_expr() && tsh.back() <= 64 && inner.size() / tsh.back() < (int64_t(1) << 31) &&
        pending_size(inner.holder()) <= 40) {
      // The expression is a view of another one that sits right on a pending
      // contraction (windows of relu (conv + bias)): the contraction, the
      // expression and the extremum in one pass.  The convolution's own result is
      // never written; the Bool values computed on the way (the relu mask) are, for
      // whoever differentiates the expression later.
      {
        Ix r;
        if (contract_map_extremum(be, inner, n_reduce, want_max, shm, Shape(tsh.begin(), tsh.end() - 1), &r)) {
          r.arg_of = t.holder();
          return r;
        }
      }
      std::vector<const hgpu_array*> ins;
      std::vector<hgpu_fused_instr> prog;
      std::vector<int> slots;
      number_program({inner.holder().get()}, &ins, &prog, &slots);
      if ((int)ins.size() <= 12 && (int)prog.size() <= 96) {
        hgpu_array *vals = nullptr, *idx = nullptr;
        be->check(api->fused_extremum(be->ctx, (int)ins.size(), ins.data(), (int)prog.size(), prog.data(), slots[0], n_reduce, want_max ? 1 : 0, &vals, &idx));
        // results have the inner space's leading dims: merge them to the logical ones
        Shape lead(tsh.begin(), tsh.end() - 1);
        Ix r = from_array(shm, reshape(T(be, idx), lead));
        r.arg_of = t.holder();
        r.arg_vals = reshape(T(be, vals), lead);
        return r;
      }
    }
  }
  if (identity && be->fuse && api->struct_size >= offsetof(hgpu_api, extremum_last) + sizeof(api->extremum_last) && api->extremum_last) {
    hgpu_array *vals = nullptr, *idx = nullptr;
    be->check(api->extremum_last(be->ctx, t.h(), want_max ? 1 : 0, &vals, &idx));
    Ix r = from_array(shm, T(be, idx));
    r.arg_of = t.holder();
    r.arg_vals = T(be, vals);
    return r;
  }
  T part = tsgather(t, shm, ix);  // shm ++ [n]
  return from_array(shm, argminmax_last(part, want_max));
}

}  // namespace hordead
