// Dual numbers over the carrier and the reverse sweep: the operations of
// `ADVal target` (src/HordeAd/Core/OpsADVal.hs:232-330, CarriersADVal.hs:
// 330-475) paired with the transposition rules of `evalRev`
// (src/HordeAd/Core/DeltaEval.hs:391-595).  Each rule cites the delta
// constructor it transposes.
#include <algorithm>

#include "host.hpp"

namespace hordead {

static bool differentiable(const T& t) { return t.dtype() == HGPU_F64 || t.dtype() == HGPU_F32; }

D Tape::input(const T& t) {
  D d;
  d.primal = t;
  d.node = differentiable(t) ? push([](const T&, std::vector<T>&) {}) : -1;
  return d;
}

int Tape::push(std::function<void(const T&, std::vector<T>&)> f) {
  recs.push_back(Rec{std::move(f)});
  return (int)recs.size() - 1;
}

static void accum(std::vector<T>& slots, int node, const T& cot) {
  if (node < 0) return;
  T& s = slots[(size_t)node];
  s = s.valid() ? add_cotangents(s, cot) : cot;
}

std::vector<T> Tape::backward(const D& out, const T& dt, const std::vector<D>& inputs) {
  std::vector<T> slots(recs.size());
  std::vector<bool> keep(recs.size(), false);
  for (auto& i : inputs)
    if (i.node >= 0) keep[(size_t)i.node] = true;
  if (out.node >= 0) {
    if (dt.shape() != out.primal.shape()) throw HostError(HGPU_ERR_INVALID, "backward: cotangent shape differs from the result's");
    slots[(size_t)out.node] = dt;
    for (int n = out.node; n >= 0; --n) {
      if (!slots[(size_t)n].valid()) continue;
      recs[(size_t)n].back(slots[(size_t)n], slots);
      if (!keep[(size_t)n]) slots[(size_t)n] = T();
    }
  }
  std::vector<T> res;
  for (auto& i : inputs) {
    if (i.node >= 0 && slots[(size_t)i.node].valid()) res.push_back(slots[(size_t)i.node]);
    else res.push_back(zeros(be, i.primal.dtype(), i.primal.shape()));   // tdefTarget
  }
  // The gradient leaves are what the caller asked for: nothing stays pending,
  // and leaves of one shape that are still elementwise programs share a pass.
  force_many(res);
  return res;
}

D d_const(const T& t) {
  D d;
  d.primal = t;
  return d;
}

// Products made by transposition rules stay pending: most are summed at once
// by the rule of a `replicate` further up, which then is a single contraction.
static T mul(const T& a, const T& b) { return lazy_mul(a, b); }
static T add(const T& a, const T& b) { return ewise2(HGPU_ADD, a, b); }
static T neg(const T& a) { return ewise1(HGPU_NEG, a); }
static T recip(const T& a) { return ewise1(HGPU_RECIP, a); }
static T one_like(const T& a) { return broadcast_scalar(constant(a.be(), a.dtype(), 1.0), a.shape()); }

// CarriersADVal.hs:330-475 (Num, Fractional, Floating instances of ADVal)
D d_ewise1(Tape& tp, int op, const D& a) {
  D r;
  r.primal = ewise1(op, a.primal);
  if (a.node < 0 || !differentiable(r.primal) || op == HGPU_SIGNUM) return r;
  T u = a.primal, y = r.primal;
  int an = a.node;
  T scale;  // dScale scale u'
  switch (op) {
    case HGPU_NEG: scale = T(); break;
    case HGPU_ABS: scale = ewise1(HGPU_SIGNUM, u); break;
    case HGPU_RECIP: scale = neg(recip(mul(u, u))); break;
    case HGPU_EXP: scale = y; break;
    case HGPU_LOG: scale = recip(u); break;
    case HGPU_SQRT: scale = recip(add(y, y)); break;
    case HGPU_SIN: scale = ewise1(HGPU_COS, u); break;
    case HGPU_COS: scale = neg(ewise1(HGPU_SIN, u)); break;
    case HGPU_TAN: { T c = ewise1(HGPU_COS, u); scale = recip(mul(c, c)); break; }
    case HGPU_ASIN: scale = recip(ewise1(HGPU_SQRT, ewise2(HGPU_SUB, one_like(u), mul(u, u)))); break;
    case HGPU_ACOS: scale = neg(recip(ewise1(HGPU_SQRT, ewise2(HGPU_SUB, one_like(u), mul(u, u))))); break;
    case HGPU_ATAN: scale = recip(add(one_like(u), mul(u, u))); break;
    case HGPU_SINH: scale = ewise1(HGPU_COSH, u); break;
    case HGPU_COSH: scale = ewise1(HGPU_SINH, u); break;
    case HGPU_TANH: scale = ewise2(HGPU_SUB, one_like(u), mul(y, y)); break;
    case HGPU_ASINH: scale = recip(ewise1(HGPU_SQRT, add(one_like(u), mul(u, u)))); break;
    case HGPU_ACOSH: scale = recip(ewise1(HGPU_SQRT, ewise2(HGPU_SUB, mul(u, u), one_like(u)))); break;
    case HGPU_ATANH: scale = recip(ewise2(HGPU_SUB, one_like(u), mul(u, u))); break;
    default: return r;
  }
  r.node = tp.push([an, scale, op](const T& c, std::vector<T>& s) {
    accum(s, an, op == HGPU_NEG ? neg(c) : mul(scale, c));
  });
  return r;
}

D d_ewise2(Tape& tp, int op, const D& a, const D& b) {
  D r;
  r.primal = ewise2(op, a.primal, b.primal);
  if ((a.node < 0 && b.node < 0) || !differentiable(r.primal)) return r;
  T u = a.primal, v = b.primal, y = r.primal;
  int an = a.node, bn = b.node;
  switch (op) {
    case HGPU_ADD:
      r.node = tp.push([an, bn](const T& c, std::vector<T>& s) { accum(s, an, c); accum(s, bn, c); });
      break;
    case HGPU_SUB:
      r.node = tp.push([an, bn](const T& c, std::vector<T>& s) { accum(s, an, c); if (bn >= 0) accum(s, bn, neg(c)); });
      break;
    case HGPU_MUL: {
      // a factor is kept only for the other side's cotangent
      const T ku = bn >= 0 ? u : T(), kv = an >= 0 ? v : T();
      r.node = tp.push([an, bn, ku, kv](const T& c, std::vector<T>& s) {
        if (an >= 0) accum(s, an, mul(kv, c));
        if (bn >= 0) accum(s, bn, mul(ku, c));
      });
      break;
    }
    case HGPU_DIV:  // dAdd (dScale (recip v) u') (dScale ((-u) / (v*v)) v')
      r.node = tp.push([an, bn, u, v](const T& c, std::vector<T>& s) {
        if (an >= 0) accum(s, an, mul(recip(v), c));
        if (bn >= 0) accum(s, bn, mul(ewise2(HGPU_DIV, neg(u), mul(v, v)), c));
      });
      break;
    case HGPU_POW:  // dAdd (dScale (v * u**(v-1)) u') (dScale ((u**v) * log u) v')
      r.node = tp.push([an, bn, u, v, y](const T& c, std::vector<T>& s) {
        if (an >= 0) accum(s, an, mul(mul(v, ewise2(HGPU_POW, u, ewise2(HGPU_SUB, v, one_like(v)))), c));
        if (bn >= 0) accum(s, bn, mul(mul(y, ewise1(HGPU_LOG, u)), c));
      });
      break;
    case HGPU_LOGBASE:  // logBase x y = log y / log x
      r.node = tp.push([an, bn, u, v, y](const T& c, std::vector<T>& s) {
        T lx = ewise1(HGPU_LOG, u);
        if (an >= 0) accum(s, an, mul(neg(ewise2(HGPU_DIV, y, mul(u, lx))), c));
        if (bn >= 0) accum(s, bn, mul(recip(mul(v, lx)), c));
      });
      break;
    case HGPU_ATAN2:  // t = recip (u*u + v*v); dAdd (dScale ((-u)*t) v') (dScale (v*t) u')
      r.node = tp.push([an, bn, u, v](const T& c, std::vector<T>& s) {
        T t = recip(add(mul(u, u), mul(v, v)));
        if (bn >= 0) accum(s, bn, mul(mul(neg(u), t), c));
        if (an >= 0) accum(s, an, mul(mul(v, t), c));
      });
      break;
    case HGPU_MIN:
    case HGPU_MAX: {
      T pick_a = op == HGPU_MIN ? compare(HGPU_LEQ, u, v) : compare(HGPU_LEQ, v, u);
      r.node = tp.push([an, bn, pick_a](const T& c, std::vector<T>& s) {
        T z = zeros(c.be(), c.dtype(), c.shape());
        if (an >= 0) accum(s, an, select(pick_a, c, z));
        if (bn >= 0) accum(s, bn, select(pick_a, z, c));
      });
      break;
    }
    default: break;
  }
  return r;
}

D d_select(Tape& tp, const T& cond, const D& a, const D& b) {
  D r;
  r.primal = select(cond, a.primal, b.primal);
  if ((a.node < 0 && b.node < 0) || !differentiable(r.primal)) return r;
  int an = a.node, bn = b.node;
  r.node = tp.push([an, bn, cond](const T& c, std::vector<T>& s) {
    T z = zeros(c.be(), c.dtype(), c.shape());
    if (an >= 0) accum(s, an, select(cond, c, z));
    if (bn >= 0) accum(s, bn, select(cond, z, c));
  });
  return r;
}

// DeltaCastS (DeltaEval.hs:495)
D d_convert(Tape& tp, const D& a, int dtype, int mode) {
  D r;
  r.primal = convert(a.primal, dtype, mode);
  if (a.node < 0 || !differentiable(r.primal) || mode != HGPU_CONV_CAST) return r;
  int an = a.node, src = a.primal.dtype();
  r.node = tp.push([an, src](const T& c, std::vector<T>& s) { accum(s, an, convert(c, src, HGPU_CONV_CAST)); });
  return r;
}

// DeltaSumS -> tsreplicateN (DeltaEval.hs:531-535)
D d_tssumN(Tape& tp, const D& t, int k) {
  D r;
  r.primal = tssumN(t.primal, k);
  if (t.node < 0 || k == 0) { if (k == 0) r.node = t.node; return r; }
  Shape sh = t.primal.shape();
  Shape shm(sh.begin(), sh.begin() + k);
  int tn = t.node;
  r.node = tp.push([tn, shm](const T& c, std::vector<T>& s) { accum(s, tn, tsreplicateN(c, shm)); });
  return r;
}

// DeltaSum0S -> tsreplicate0N (DeltaEval.hs:528-530)
D d_tssum0(Tape& tp, const D& t) {
  D r;
  r.primal = tssum0(t.primal);
  if (t.node < 0) return r;
  Shape sh = t.primal.shape();
  int tn = t.node;
  r.node = tp.push([tn, sh](const T& c, std::vector<T>& s) { accum(s, tn, tsreplicate0N(c, sh)); });
  return r;
}

// DeltaDot0S v d -> v * tsreplicate0N sh c (DeltaEval.hs:496-501)
D d_tsdot0(Tape& tp, const D& a, const D& b) {
  D r;
  r.primal = tsdot0(a.primal, b.primal);
  if (a.node < 0 && b.node < 0) return r;
  T u = a.primal, v = b.primal;
  int an = a.node, bn = b.node;
  r.node = tp.push([an, bn, u, v](const T& c, std::vector<T>& s) {
    T cc = tsreplicate0N(c, u.shape());
    if (an >= 0) accum(s, an, mul(v, cc));
    if (bn >= 0) accum(s, bn, mul(u, cc));
  });
  return r;
}

// The cotangent of a contraction over the innermost dim, broadcast back along it.
static T expand_inner(const T& c, int64_t n) {
  int r = c.rank();
  std::vector<int> perm((size_t)r + 1);
  for (int i = 0; i < r; ++i) perm[(size_t)i] = i + 1;
  perm[(size_t)r] = 0;
  return transpose(replicate(c, {n}), perm);
}

// tsdot1In u v = tssum-over-inner (u * v) (Ops.hs:522-537): both factors get
// the broadcast cotangent times the other factor.
D d_tsdot1In(Tape& tp, const D& a, const D& b) {
  D r;
  r.primal = tsdot1In(a.primal, b.primal);
  if (a.node < 0 && b.node < 0) return r;
  T u = a.primal, v = b.primal;
  int an = a.node, bn = b.node;
  int64_t n = u.shape().back();
  r.node = tp.push([an, bn, u, v, n](const T& c, std::vector<T>& s) {
    T cc = expand_inner(c, n);
    if (an >= 0) accum(s, an, mul(v, cc));
    if (bn >= 0) accum(s, bn, mul(u, cc));
  });
  return r;
}

// The cotangent of a contraction over the n innermost dims, broadcast back.
static T expand_inner_n(const T& c, const Shape& inner) {
  int r = c.rank(), n = (int)inner.size();
  std::vector<int> perm((size_t)(r + n));
  for (int i = 0; i < r; ++i) perm[(size_t)i] = i + n;
  for (int i = 0; i < n; ++i) perm[(size_t)(r + i)] = i;
  return transpose(replicate(c, inner), perm);
}

D d_tsdotNIn(Tape& tp, const D& a, const D& b, int n) {
  D r;
  r.primal = tsdotNIn(a.primal, b.primal, n);
  if (a.node < 0 && b.node < 0) return r;
  T u = a.primal, v = b.primal;
  int an = a.node, bn = b.node;
  Shape sh = u.shape();
  Shape inner(sh.end() - n, sh.end());
  r.node = tp.push([an, bn, u, v, inner](const T& c, std::vector<T>& s) {
    T cc = expand_inner_n(c, inner);
    if (an >= 0) accum(s, an, mul(v, cc));
    if (bn >= 0) accum(s, bn, mul(u, cc));
  });
  return r;
}

// tD (Ops.hs, `tD stk primal dual`): used by lossSoftMaxCrossEntropyS
// (External/CommonShapedOps.hs:89-111) to pair a primal with a hand-made dual.
D d_tD(const D& primal, const D& dual) {
  if (primal.primal.shape() != dual.primal.shape()) throw HostError(HGPU_ERR_INVALID, "tD: primal and dual parts differ in shape");
  D r;
  r.primal = primal.primal;
  r.node = dual.node;
  return r;
}

// AstMatmul2S: d m1 = c * m2^T, d m2 = m1^T * c -- the form the reference's
// simplified artifacts hold (test/simplified/TestMnistPP.hs:735 `m284`).
D d_tsmatmul2(Tape& tp, const D& a, const D& b) {
  D r;
  r.primal = tsmatmul2(a.primal, b.primal);
  if (a.node < 0 && b.node < 0) return r;
  T u = a.primal, v = b.primal;
  int an = a.node, bn = b.node;
  r.node = tp.push([an, bn, u, v](const T& c, std::vector<T>& s) {
    if (an >= 0) accum(s, an, tsmatmul2(c, transpose(v, {1, 0})));
    if (bn >= 0) accum(s, bn, tsmatmul2(transpose(u, {1, 0}), c));
  });
  return r;
}

// DeltaReplicateS -> tssumN (DeltaEval.hs:549-555)
D d_tsreplicateN(Tape& tp, const D& t, const Shape& shm) {
  D r;
  r.primal = tsreplicateN(t.primal, shm);
  if (t.node < 0) return r;
  if (shm.empty()) { r.node = t.node; return r; }
  int tn = t.node, k = (int)shm.size();
  r.node = tp.push([tn, k](const T& c, std::vector<T>& s) { accum(s, tn, tssumN(c, k)); });
  return r;
}

// DeltaAppendS -> two slices (DeltaEval.hs:563-568)
D d_tsappend(Tape& tp, const D& a, const D& b) {
  D r;
  r.primal = tsappend(a.primal, b.primal);
  if (a.node < 0 && b.node < 0) return r;
  int an = a.node, bn = b.node;
  int64_t m = a.primal.shape().at(0), n = b.primal.shape().at(0);
  r.node = tp.push([an, bn, m, n](const T& c, std::vector<T>& s) {
    if (an >= 0) accum(s, an, tsslice(c, 0, m));
    if (bn >= 0) accum(s, bn, tsslice(c, m, n));
  });
  return r;
}

// DeltaSliceS -> zeros ++ c ++ zeros (DeltaEval.hs:569-575)
D d_tsslice(Tape& tp, const D& t, int64_t i, int64_t n) {
  D r;
  r.primal = tsslice(t.primal, i, n);
  if (t.node < 0) return r;
  int tn = t.node, rank = t.primal.rank();
  int64_t k = t.primal.shape().at(0) - i - n;
  r.node = tp.push([tn, rank, i, k](const T& c, std::vector<T>& s) {
    Shape lo((size_t)rank, 0), hi((size_t)rank, 0);
    lo[0] = i;
    hi[0] = k;
    accum(s, tn, pad(c, lo, hi));
  });
  return r;
}

// DeltaReverseS (DeltaEval.hs:576-579)
D d_tsreverse(Tape& tp, const D& t) {
  D r;
  r.primal = tsreverse(t.primal);
  if (t.node < 0) return r;
  int tn = t.node;
  r.node = tp.push([tn](const T& c, std::vector<T>& s) { accum(s, tn, tsreverse(c)); });
  return r;
}

// DeltaTransposeS -> the inverse permutation (DeltaEval.hs:580-591)
D d_tstranspose(Tape& tp, const D& t, const std::vector<int>& perm) {
  D r;
  r.primal = tstranspose(t.primal, perm);
  if (t.node < 0) return r;
  std::vector<int> inv(perm.size());
  for (size_t i = 0; i < perm.size(); ++i) inv[(size_t)perm[i]] = (int)i;
  int tn = t.node;
  r.node = tp.push([tn, inv](const T& c, std::vector<T>& s) { accum(s, tn, tstranspose(c, inv)); });
  return r;
}

// DeltaReshapeS (DeltaEval.hs:592-595)
D d_tsreshape(Tape& tp, const D& t, const Shape& sh) {
  D r;
  r.primal = tsreshape(t.primal, sh);
  if (t.node < 0) return r;
  Shape back = t.primal.shape();
  int tn = t.node;
  r.node = tp.push([tn, back](const T& c, std::vector<T>& s) { accum(s, tn, tsreshape(c, back)); });
  return r;
}

// DeltaIndexS -> tsoneHot (DeltaEval.hs:502-514)
D d_tsindex(Tape& tp, const D& t, const Shape& ix) {
  D r;
  r.primal = tsindex(t.primal, ix);
  if (t.node < 0) return r;
  Shape sh = t.primal.shape();
  Shape shp(sh.begin(), sh.begin() + (long)ix.size());
  int tn = t.node;
  r.node = tp.push([tn, ix, shp](const T& c, std::vector<T>& s) { accum(s, tn, tsoneHot(c, ix, shp)); });
  return r;
}

// DeltaGatherS -> tsscatter with the same index function (DeltaEval.hs:556-562)
D d_tsgather(Tape& tp, const D& src, const Shape& shm, const std::vector<Ix>& ix) {
  D r;
  r.primal = tsgather(src.primal, shm, ix);
  if (src.node < 0) return r;
  Shape ssh = src.primal.shape();
  Shape shp(ssh.begin(), ssh.begin() + (long)ix.size());
  int sn = src.node, rank_m = (int)shm.size();
  r.node = tp.push([sn, rank_m, shp, ix](const T& c, std::vector<T>& s) { accum(s, sn, tsscatter(c, rank_m, shp, ix)); });
  return r;
}

// DeltaScatterS -> tsgather with the same index function (DeltaEval.hs:536-542)
D d_tsscatter(Tape& tp, const D& src, int rank_m, const Shape& shp, const std::vector<Ix>& ix) {
  D r;
  r.primal = tsscatter(src.primal, rank_m, shp, ix);
  if (src.node < 0) return r;
  Shape ssh = src.primal.shape();
  Shape shm(ssh.begin(), ssh.begin() + rank_m);
  int sn = src.node;
  r.node = tp.push([sn, shm, ix](const T& c, std::vector<T>& s) { accum(s, sn, tsgather(c, shm, ix)); });
  return r;
}

}  // namespace hordead
