// Gradient-descent updates on device arrays (External/OptimizerTools.hs): the
// reference updates parameters array by array with elementwise arithmetic on
// the CPU; here each array's update is one fused pass on the device, so the
// parameters and the optimizer's state never leave it between gradients.
#include <cmath>

#include "host.hpp"

namespace hordead {

static bool differentiable(int dtype) { return dtype == HGPU_F64 || dtype == HGPU_F32; }

// A rank-0 array holding v, NOT cached: step sizes change with the iteration.
static T fresh_scalar(Backend* be, int dtype, double v) {
  if (dtype == HGPU_F32) {
    float f = (float)v;
    return upload(be, dtype, {}, &f);
  }
  return upload(be, dtype, {}, &v);
}

// updateWithGradient (OptimizerTools.hs:20-47): params - gamma * gradient;
// arrays of a type that is not differentiable come back unchanged.
T update_with_gradient(double gamma, const T& p, const T& g) {
  if (!differentiable(p.dtype())) return p;
  if (p.shape() != g.shape() || p.dtype() != g.dtype()) throw HostError(HGPU_ERR_INVALID, "updateWithGradient: parameter and gradient differ in shape or type");
  T gam = broadcast_scalar(constant(p.be(), p.dtype(), gamma), p.shape());
  T out = ewise2(HGPU_SUB, p, ewise2(HGPU_MUL, gam, g));
  (void)out.h();
  return out;
}

// updateWithGradientAdam (OptimizerTools.hs:137-225), one array:
//   m' = beta1 m + (1 - beta1) g
//   v' = beta2 v + (1 - beta2) g g
//   p' = p - alphat m' / (sqrt v' + epsilon),  alphat = alpha sqrt (1 - beta2^t) / (1 - beta1^t)
// alphat arrives as a rank-0 array so that a recorded step can change it
// between launches.  The three results are written by one pass.
void adam_update(const T& alphat, double beta1, double beta2, double epsilon, const T& m, const T& v, const T& p, const T& g, T* m_new, T* v_new,
                 T* p_new) {
  if (!differentiable(p.dtype())) {
    *m_new = m;
    *v_new = v;
    *p_new = p;
    return;
  }
  for (const T* x : {&m, &v, &g})
    if (x->shape() != p.shape() || x->dtype() != p.dtype()) throw HostError(HGPU_ERR_INVALID, "updateWithGradientAdam: arrays differ in shape or type");
  if (alphat.rank() != 0 || alphat.dtype() != p.dtype()) throw HostError(HGPU_ERR_INVALID, "updateWithGradientAdam: the step size is a rank-0 array of the parameters' type");
  Backend* be = p.be();
  const Shape sh = p.shape();
  auto k = [&](double c) { return broadcast_scalar(constant(be, p.dtype(), c), sh); };
  T mn = ewise2(HGPU_ADD, ewise2(HGPU_MUL, k(beta1), m), ewise2(HGPU_MUL, k(1 - beta1), g));
  T vn = ewise2(HGPU_ADD, ewise2(HGPU_MUL, k(beta2), v), ewise2(HGPU_MUL, k(1 - beta2), ewise2(HGPU_MUL, g, g)));
  T pn = ewise2(HGPU_SUB, p, ewise2(HGPU_DIV, ewise2(HGPU_MUL, broadcast_scalar(alphat, sh), mn), ewise2(HGPU_ADD, ewise1(HGPU_SQRT, vn), k(epsilon))));
  force_many({mn, vn, pn});
  *m_new = mn;
  *v_new = vn;
  *p_new = pn;
}

T adam_step_size(Backend* be, int dtype, double alpha, double beta1, double beta2, int t_new) {
  double alphat = alpha * std::sqrt(1 - std::pow(beta2, t_new)) / (1 - std::pow(beta1, t_new));
  return fresh_scalar(be, dtype, alphat);
}

void assign(const T& dst, const T& src) {
  Backend* be = dst.be();
  const hgpu_api* api = be->api;
  if (api->struct_size < offsetof(hgpu_api, assign) + sizeof(api->assign) || !api->assign) throw HostError(HGPU_ERR_UNSUPPORTED, "this provider has no assign");
  be->check(api->assign(be->ctx, dst.h(), src.h()));
}

}  // namespace hordead
