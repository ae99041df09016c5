// extern "C" surface of the host layer (include/hordead_host.h): handles in,
// status codes out; C++ exceptions stop here.
#include "hordead_host.h"

#include <execinfo.h>
#include <signal.h>
#include <unistd.h>

#include <cstddef>
#include <cstdlib>
#include <cstring>

#include "host.hpp"

using namespace hordead;

struct hh_ctx {
  Backend be;
  Tape tape;
  std::string err;
  bool owns_ctx = true;
  hh_ctx() : tape(&be) {}
};
struct hh_val { D d; };
struct hh_ix { Ix x; };

namespace {

template <typename F>
int guarded(hh_ctx* c, F f) {
  try {
    f();
    return HGPU_OK;
  } catch (const HostError& e) {
    if (c) c->err = e.what();
    return e.code;
  } catch (const std::exception& e) {
    if (c) c->err = e.what();
    return HGPU_ERR_INVALID;
  }
}

Shape mk(int n, const int64_t* p) { return n > 0 ? Shape(p, p + n) : Shape(); }
hh_val* box(const D& d) { return new hh_val{d}; }
hh_ix* boxi(const Ix& x) { return new hh_ix{x}; }
std::vector<Ix> ixs(int n, hh_ix* const* p) {
  std::vector<Ix> v;
  for (int i = 0; i < n; ++i) v.push_back(p[i]->x);
  return v;
}

}  // namespace

// With HORDEAD_SEGV_TRACE set, a crash in native code prints its call stack.
static void segv_trace(int sig) {
  void* frames[64];
  int n = backtrace(frames, 64);
  backtrace_symbols_fd(frames, n, STDERR_FILENO);
  signal(sig, SIG_DFL);
  raise(sig);
}

extern "C" {

int hh_create(const hgpu_api* api, int device, hh_ctx** out) {
  if (!api || !out) return HGPU_ERR_INVALID;
  if (getenv("HORDEAD_SEGV_TRACE")) signal(SIGSEGV, segv_trace);
  hh_ctx* c = new hh_ctx;
  c->be.api = api;
  c->be.ctx = nullptr;
  int rc = api->init(device, &c->be.ctx);
  if (rc) { delete c; return rc; }
  *out = c;
  return HGPU_OK;
}

int hh_create_gpu(int device, hh_ctx** out) { return hh_create(hgpu_get_api(), device, out); }

int hh_destroy(hh_ctx* c) {
  if (!c) return HGPU_OK;
  c->tape.recs.clear();
  c->be.iota_cache.clear();
  c->be.const_cache.clear();
  c->be.api->shutdown(c->be.ctx);
  // The context object stays: values released later still point at it.
  return HGPU_OK;
}

const char* hh_last_error(hh_ctx* c) { return c ? c->err.c_str() : "no context"; }
int hh_sync(hh_ctx* c) { return guarded(c, [&] { c->be.check(c->be.api->sync(c->be.ctx)); }); }
hgpu_ctx* hh_array_ctx(hh_ctx* c) { return c ? c->be.ctx : nullptr; }
int hh_set_fusion(hh_ctx* c, int on) { c->be.fuse = on != 0; return HGPU_OK; }
int hh_tape_reset(hh_ctx* c) { c->tape.recs.clear(); return HGPU_OK; }

int hh_upload(hh_ctx* c, int dtype, int rank, const int64_t* shape, const void* host, int rg, hh_val** out) {
  return guarded(c, [&] {
    T t = upload(&c->be, dtype, mk(rank, shape), host);
    *out = box(rg ? c->tape.input(t) : d_const(t));
  });
}

int hh_from_array(hh_ctx* c, hgpu_array* a, int rg, hh_val** out) {
  return guarded(c, [&] {
    c->be.check(c->be.api->retain(a));
    T t(&c->be, a);
    *out = box(rg ? c->tape.input(t) : d_const(t));
  });
}

int hh_constant(hh_ctx* c, int dtype, double value, int rank, const int64_t* shape, hh_val** out) {
  return guarded(c, [&] { *out = box(d_const(broadcast_scalar(constant(&c->be, dtype, value), mk(rank, shape)))); });
}

int hh_array(hh_val* v, hgpu_array** out) {
  if (!v || !out) return HGPU_ERR_INVALID;
  v->d.primal.be()->api->retain(v->d.primal.h());
  *out = v->d.primal.h();
  return HGPU_OK;
}

int hh_download(hh_ctx* c, hh_val* v, void* host) {
  return guarded(c, [&] { c->be.check(c->be.api->download(c->be.ctx, v->d.primal.h(), host)); });
}
struct hh_graph { hgpu_graph* g; };
static bool has_graphs(const hgpu_api* api) {
  return api->struct_size >= offsetof(hgpu_api, overwrite) + sizeof(api->overwrite) && api->capture_begin && api->capture_end &&
         api->graph_launch && api->graph_destroy && api->overwrite;
}
int hh_capture_begin(hh_ctx* c) {
  return guarded(c, [&] {
    if (!has_graphs(c->be.api)) throw HostError(HGPU_ERR_UNSUPPORTED, "this provider records no graphs");
    c->be.check(c->be.api->capture_begin(c->be.ctx));
    c->be.capturing = true;
  });
}
int hh_capture_end(hh_ctx* c, hh_graph** out) {
  return guarded(c, [&] {
    if (!has_graphs(c->be.api)) throw HostError(HGPU_ERR_UNSUPPORTED, "this provider records no graphs");
    hgpu_graph* g = nullptr;
    c->be.capturing = false;
    c->be.check(c->be.api->capture_end(c->be.ctx, &g));
    *out = new hh_graph{g};
  });
}
int hh_graph_launch(hh_ctx* c, hh_graph* g) {
  return guarded(c, [&] { c->be.check(c->be.api->graph_launch(g->g)); });
}
int hh_graph_free(hh_ctx* c, hh_graph* g) {
  if (!g) return HGPU_OK;
  int rc = guarded(c, [&] { c->be.check(c->be.api->graph_destroy(g->g)); });
  delete g;
  return rc;
}
int hh_force(hh_ctx* c, hh_val* v) {
  return guarded(c, [&] { (void)v->d.primal.h(); });
}
int hh_dense(hh_ctx* c, hh_val* v, hh_val** out) {
  if (!c || !v || !out) return HGPU_ERR_INVALID;
  return guarded(c, [&] {
    Backend* be = &c->be;
    hgpu_array* a = v->d.primal.h();
    if (be->api->is_dense(a)) { *out = box(d_const(v->d.primal)); return; }
    hgpu_array* o = nullptr;
    be->check(be->api->materialize(be->ctx, a, &o));
    *out = box(d_const(T(be, o)));
  });
}
int hh_overwrite(hh_ctx* c, hh_val* v, const void* host) {
  return guarded(c, [&] {
    if (!has_graphs(c->be.api)) throw HostError(HGPU_ERR_UNSUPPORTED, "this provider has no overwrite");
    const auto& holder = v->d.primal.holder();
    if (holder->host_i64) {     // a small integer table is also kept on the host (index functions look constants up in it)
      if (holder->host_i64_folded)
        throw HostError(HGPU_ERR_INVALID, "overwrite: an index function has been simplified with this table's values; it is a constant of the program now");
      std::memcpy(holder->host_i64->data(), host, holder->host_i64->size() * sizeof(int64_t));
    }
    c->be.check(c->be.api->overwrite(c->be.ctx, v->d.primal.h(), host));
  });
}
int hh_assign(hh_ctx* c, hh_val* dst, hh_val* src) {
  return guarded(c, [&] { assign(dst->d.primal, src->d.primal); });
}
static hh_val* box_plain(const T& t) {
  D d;
  d.primal = t;
  return box(d);
}
int hh_update_with_gradient(hh_ctx* c, double gamma, hh_val* p, hh_val* g, hh_val** out) {
  return guarded(c, [&] { *out = box_plain(update_with_gradient(gamma, p->d.primal, g->d.primal)); });
}
int hh_adam_step_size(hh_ctx* c, int dtype, double alpha, double beta1, double beta2, int t_new, hh_val** out) {
  return guarded(c, [&] { *out = box_plain(adam_step_size(&c->be, dtype, alpha, beta1, beta2, t_new)); });
}
int hh_adam_apply(hh_ctx* c, hh_val* alphat, double beta1, double beta2, double epsilon, hh_val* m, hh_val* v, hh_val* p, hh_val* g, hh_val** m_new,
                  hh_val** v_new, hh_val** p_new) {
  return guarded(c, [&] {
    T mn, vn, pn;
    adam_update(alphat->d.primal, beta1, beta2, epsilon, m->d.primal, v->d.primal, p->d.primal, g->d.primal, &mn, &vn, &pn);
    *m_new = box_plain(mn);
    *v_new = box_plain(vn);
    *p_new = box_plain(pn);
  });
}
int hh_update_with_gradient_adam(hh_ctx* c, double alpha, double beta1, double beta2, double epsilon, int t_new, hh_val* m, hh_val* v, hh_val* p,
                                 hh_val* g, hh_val** m_new, hh_val** v_new, hh_val** p_new) {
  return guarded(c, [&] {
    T mn, vn, pn;
    const T& pp = p->d.primal;
    T at = (pp.dtype() == HGPU_F64 || pp.dtype() == HGPU_F32) ? adam_step_size(&c->be, pp.dtype(), alpha, beta1, beta2, t_new) : T();
    if (!at.valid()) { mn = m->d.primal; vn = v->d.primal; pn = pp; }
    else adam_update(at, beta1, beta2, epsilon, m->d.primal, v->d.primal, pp, g->d.primal, &mn, &vn, &pn);
    *m_new = box_plain(mn);
    *v_new = box_plain(vn);
    *p_new = box_plain(pn);
  });
}
int hh_val_rank(hh_val* v) { return v->d.primal.rank(); }
int hh_val_dtype(hh_val* v) { return v->d.primal.dtype(); }
int hh_val_shape(hh_val* v, int64_t* s) {
  Shape sh = v->d.primal.shape();
  std::copy(sh.begin(), sh.end(), s);
  return HGPU_OK;
}
int hh_free(hh_val* v) { delete v; return HGPU_OK; }

int hh_backward(hh_ctx* c, hh_val* out, hh_val* dt, int n, hh_val* const* inputs, hh_val** grads) {
  return guarded(c, [&] {
    std::vector<D> ins;
    for (int i = 0; i < n; ++i) ins.push_back(inputs[i]->d);
    std::vector<T> g = c->tape.backward(out->d, dt->d.primal, ins);
    for (int i = 0; i < n; ++i) grads[i] = box(d_const(g[(size_t)i]));
  });
}

#define HH_OP(body) return guarded(c, [&] { *out = box(body); })

int hh_ewise1(hh_ctx* c, int op, hh_val* a, hh_val** out) { HH_OP(d_ewise1(c->tape, op, a->d)); }
int hh_ewise2(hh_ctx* c, int op, hh_val* a, hh_val* b, hh_val** out) { HH_OP(d_ewise2(c->tape, op, a->d, b->d)); }
int hh_compare(hh_ctx* c, int cmp, hh_val* a, hh_val* b, hh_val** out) { HH_OP(d_const(compare(cmp, a->d.primal, b->d.primal))); }
int hh_compare_all(hh_ctx* c, int cmp, hh_val* a, hh_val* b, int* result) {
  return guarded(c, [&] { *result = compare_all(cmp, a->d.primal, b->d.primal) ? 1 : 0; });
}
int hh_select(hh_ctx* c, hh_val* cond, hh_val* a, hh_val* b, hh_val** out) { HH_OP(d_select(c->tape, cond->d.primal, a->d, b->d)); }
int hh_convert(hh_ctx* c, hh_val* a, int dtype, int mode, hh_val** out) { HH_OP(d_convert(c->tape, a->d, dtype, mode)); }
int hh_tssumN(hh_ctx* c, hh_val* t, int k, hh_val** out) { HH_OP(d_tssumN(c->tape, t->d, k)); }
int hh_tssum0(hh_ctx* c, hh_val* t, hh_val** out) { HH_OP(d_tssum0(c->tape, t->d)); }
int hh_tsdot0(hh_ctx* c, hh_val* a, hh_val* b, hh_val** out) { HH_OP(d_tsdot0(c->tape, a->d, b->d)); }
int hh_tsdot1In(hh_ctx* c, hh_val* a, hh_val* b, hh_val** out) { HH_OP(d_tsdot1In(c->tape, a->d, b->d)); }
int hh_tsdotNIn(hh_ctx* c, hh_val* a, hh_val* b, int n, hh_val** out) { HH_OP(d_tsdotNIn(c->tape, a->d, b->d, n)); }
int hh_as_input(hh_ctx* c, hh_val* v, hh_val** out) { HH_OP(c->tape.input(v->d.primal)); }
int hh_tprimalPart(hh_ctx* c, hh_val* v, hh_val** out) { HH_OP(d_const(v->d.primal)); }
int hh_tD(hh_ctx* c, hh_val* primal, hh_val* dual, hh_val** out) { HH_OP(d_tD(primal->d, dual->d)); }
// ConvertTensor (ConvertTensor.hs:25-236, OpsConcrete.hs:777-904): on a carrier whose
// arrays hold their shape at run time every conversion is the identity on the
// data and on the dual part; what is left of it is the reference's check.
int hh_tconvert(hh_ctx* c, int conv, hh_val* v, int rank, const int64_t* shape, hh_val** out) {
  if (!c || !v || !out || rank < 0 || (rank > 0 && !shape)) return HGPU_ERR_INVALID;
  return guarded(c, [&] {
    const Shape have = v->d.primal.shape();
    const Shape want = mk(rank, shape);
    switch (conv) {
      case HH_CONV_K_FROM_S: case HH_CONV_S_FROM_K:
        if (!have.empty()) throw HostError(HGPU_ERR_INVALID, "tconvert: a scalar conversion of an array of rank " + std::to_string(have.size()));
        break;
      case HH_CONV_S_FROM_R: case HH_CONV_S_FROM_X:
        if (have != want) throw HostError(HGPU_ERR_INVALID, "tconvert: the array does not have the shape the shaped type names");
        break;
      case HH_CONV_R_FROM_S: case HH_CONV_X_FROM_S:
        break;
      case HH_CONV_NEST: case HH_CONV_UNNEST:   // rank = dims of the outer array; shape, when given, names them
        if ((size_t)rank > have.size() || (shape && !std::equal(want.begin(), want.end(), have.begin())))
          throw HostError(HGPU_ERR_INVALID, "tconvert: the outer dims do not lead the array's shape");
        break;
      default: throw HostError(HGPU_ERR_INVALID, "tconvert: unknown conversion");
    }
    *out = box(v->d);
  });
}
int hh_tsmatvecmul(hh_ctx* c, hh_val* m, hh_val* v, hh_val** out) {
  HH_OP(d_tsdot1In(c->tape, m->d, d_tsreplicateN(c->tape, v->d, {m->d.primal.shape().at(0)})));
}
int hh_tsmatmul2(hh_ctx* c, hh_val* a, hh_val* b, hh_val** out) { HH_OP(d_tsmatmul2(c->tape, a->d, b->d)); }
int hh_tsreplicateN(hh_ctx* c, hh_val* t, int n, const int64_t* shm, hh_val** out) { HH_OP(d_tsreplicateN(c->tape, t->d, mk(n, shm))); }
int hh_tsappend(hh_ctx* c, hh_val* a, hh_val* b, hh_val** out) { HH_OP(d_tsappend(c->tape, a->d, b->d)); }
int hh_tsslice(hh_ctx* c, hh_val* t, int64_t i, int64_t n, hh_val** out) { HH_OP(d_tsslice(c->tape, t->d, i, n)); }
int hh_tsreverse(hh_ctx* c, hh_val* t, hh_val** out) { HH_OP(d_tsreverse(c->tape, t->d)); }
int hh_tstranspose(hh_ctx* c, hh_val* t, int n, const int* perm, hh_val** out) {
  HH_OP(d_tstranspose(c->tape, t->d, n > 0 ? std::vector<int>(perm, perm + n) : std::vector<int>()));
}
int hh_tsreshape(hh_ctx* c, hh_val* t, int rank, const int64_t* shape, hh_val** out) { HH_OP(d_tsreshape(c->tape, t->d, mk(rank, shape))); }
int hh_tsindex(hh_ctx* c, hh_val* t, int n, const int64_t* ix, hh_val** out) { HH_OP(d_tsindex(c->tape, t->d, mk(n, ix))); }
int hh_tsargminmax(hh_ctx* c, hh_val* t, int want_max, hh_val** out) { HH_OP(d_const(want_max ? tsargMax(t->d.primal) : tsargMin(t->d.primal))); }
int hh_tsiota(hh_ctx* c, int64_t n, int dtype, hh_val** out) { HH_OP(d_const(tsiota(&c->be, n, dtype))); }

#define HH_IX(body) return guarded(c, [&] { *out = boxi(body); })

int hh_ix_var(hh_ctx* c, int rank_m, const int64_t* shm, int d, hh_ix** out) { HH_IX(ix_var(&c->be, mk(rank_m, shm), d)); }
int hh_ix_const(hh_ctx* c, int rank_m, const int64_t* shm, int dtype, double v, hh_ix** out) { HH_IX(ix_const(&c->be, mk(rank_m, shm), dtype, v)); }
int hh_ix_lift(hh_ctx* c, int rank_m, const int64_t* shm, hh_val* s, hh_ix** out) { HH_IX(ix_lift(mk(rank_m, shm), s->d.primal)); }
int hh_ix_op1(hh_ctx* c, int op, hh_ix* a, hh_ix** out) { HH_IX(ix_op1(&c->be, op, a->x)); }
int hh_ix_op2(hh_ctx* c, int op, hh_ix* a, hh_ix* b, hh_ix** out) { HH_IX(ix_op2(&c->be, op, a->x, b->x)); }
int hh_ix_compare(hh_ctx* c, int cmp, hh_ix* a, hh_ix* b, hh_ix** out) { HH_IX(ix_compare(&c->be, cmp, a->x, b->x)); }
int hh_ix_select(hh_ctx* c, hh_ix* cond, hh_ix* a, hh_ix* b, hh_ix** out) { HH_IX(ix_select(&c->be, cond->x, a->x, b->x)); }
int hh_ix_convert(hh_ctx* c, hh_ix* a, int dtype, int mode, hh_ix** out) { HH_IX(ix_convert(&c->be, a->x, dtype, mode)); }
int hh_ix_index0(hh_ctx* c, hh_val* t, int n, hh_ix* const* ix, hh_ix** out) { HH_IX(ix_index0(&c->be, t->d.primal, ixs(n, ix))); }
int hh_ix_argminmax(hh_ctx* c, hh_val* t, int n, hh_ix* const* ix, int want_max, hh_ix** out) {
  HH_IX(ix_argminmax(&c->be, t->d.primal, ixs(n, ix), want_max != 0));
}
int hh_ix_from_val(hh_ctx* c, hh_val* v, hh_ix** out) {
  if (!c || !v || !out) return HGPU_ERR_INVALID;
  return guarded(c, [&] {
    Ix x;
    x.shm = v->d.primal.shape();
    x.arr = v->d.primal;
    x.dtype = v->d.primal.dtype();
    *out = boxi(x);
  });
}
int hh_ix_to_val(hh_ctx* c, hh_ix* x, hh_val** out) {
  if (!c || !x || !out) return HGPU_ERR_INVALID;
  HH_OP(d_const(ix_array(&c->be, x->x)));
}
int hh_ix_dtype(hh_ix* x) { return x ? x->x.dtype : -1; }
int hh_ix_free(hh_ix* x) { delete x; return HGPU_OK; }
int hh_ix_is_affine(hh_ix* x) { return x && x->x.affine ? 1 : 0; }
int64_t hh_counter(hh_ctx* c, const char* name) {
  if (!c || !name) return -1;
  auto it = c->be.counters.find(name);
  return it == c->be.counters.end() ? 0 : it->second;
}

int hh_tsgather(hh_ctx* c, hh_val* src, int rank_m, const int64_t* shm, int n_ix, hh_ix* const* ix, hh_val** out) {
  HH_OP(d_tsgather(c->tape, src->d, mk(rank_m, shm), ixs(n_ix, ix)));
}
int hh_tsscatter(hh_ctx* c, hh_val* src, int rank_m, int n_ix, const int64_t* shp, hh_ix* const* ix, hh_val** out) {
  HH_OP(d_tsscatter(c->tape, src->d, rank_m, mk(n_ix, shp), ixs(n_ix, ix)));
}

}  // extern "C"
