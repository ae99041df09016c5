"""Gradient descent with the parameters resident on the device: the interface
of the reference's `HordeAd.External.Optimizer` / `OptimizerTools`
(src/HordeAd/External/Optimizer.hs:20-88, OptimizerTools.hs:20-225) over the
host layer.  A tuple of parameter arrays stands for the reference's product
kinds (`STKProduct`); every array is updated by one fused pass on the device.
"""
import ctypes as C
from dataclasses import dataclass

from . import hostapi as H


def updateWithGradient(gamma, params, gradients):
    """OptimizerTools.hs:20-47: params - gamma * gradient, array by array."""
    out = []
    for p, g in zip(params, gradients):
        out.append(p.host._out(p.host.dll.hh_update_with_gradient, float(gamma), p.h, g.h))
    return out


@dataclass
class ArgsAdam:                       # OptimizerTools.hs:72-77
    alpha: float = 0.001
    betaOne: float = 0.9
    betaTwo: float = 0.999
    epsilon: float = 1e-7


defaultArgsAdam = ArgsAdam()          # OptimizerTools.hs:82-88


@dataclass
class StateAdam:                      # OptimizerTools.hs:120-125
    tAdam: int
    mAdam: list
    vAdam: list


def initialStateAdam(params):
    """OptimizerTools.hs:128-133: iteration 0, zero moments of the parameters' shapes."""
    zeros = lambda p: p.host.srepl(p.shape, 0.0, p.dtype)  # noqa: E731
    return StateAdam(0, [zeros(p) for p in params], [zeros(p) for p in params])


def _three(host, fn, *args):
    outs = [C.c_void_p() for _ in range(3)]
    host.check(fn(host.h, *args, *[C.byref(o) for o in outs]))
    return [H.V(host, o) for o in outs]


def updateWithGradientAdam(args, state, params, gradients):
    """OptimizerTools.hs:137-225: (new parameters, new state)."""
    t_new = state.tAdam + 1
    ms, vs, ps = [], [], []
    for m, v, p, g in zip(state.mAdam, state.vAdam, params, gradients):
        mn, vn, pn = _three(p.host, p.host.dll.hh_update_with_gradient_adam, args.alpha, args.betaOne, args.betaTwo, args.epsilon, t_new,
                            m.h, v.h, p.h, g.h)
        ms.append(mn)
        vs.append(vn)
        ps.append(pn)
    return ps, StateAdam(t_new, ms, vs)


def adamStepSize(host, dtype, args, t_new):
    """alphat of OptimizerTools.hs:152-153 as a rank-0 device array."""
    return host._out(host.dll.hh_adam_step_size, dtype, args.alpha, args.betaOne, args.betaTwo, t_new)


def adamApply(args, alphat, ms, vs, params, gradients):
    """The Adam update with the step size given as a device scalar: the form a
    recorded training step uses (the scalar is overwritten between launches)."""
    out_m, out_v, out_p = [], [], []
    for m, v, p, g in zip(ms, vs, params, gradients):
        mn, vn, pn = _three(p.host, p.host.dll.hh_adam_apply, alphat.h, args.betaOne, args.betaTwo, args.epsilon, m.h, v.h, p.h, g.h)
        out_m.append(mn)
        out_v.append(vn)
        out_p.append(pn)
    return out_m, out_v, out_p


def _as_inputs(host, values):
    """The values as fresh inputs of an emptied tape (the next step differentiates with respect to them)."""
    host.tape_reset()
    return [host._out(host.dll.hh_as_input, v.h) for v in values]


def sgd(gamma, f, training_data, params):
    """Optimizer.hs:20-49: one gradient step per datum.  f(datum, params) is the
    objective; params is a list of values made with Host.param.  Returns the
    final parameters and the last objective value."""
    host = params[0].host
    value = None
    for a in training_data:
        value = f(a, params)
        grads = host.grad(value, params)
        params = _as_inputs(host, updateWithGradient(gamma, params, grads))
    return params, value


def sgdAdam(f, training_data, params, state, args=defaultArgsAdam):
    """Optimizer.hs:54-88."""
    host = params[0].host
    for a in training_data:
        grads = host.grad(f(a, params), params)
        new, state = updateWithGradientAdam(args, state, params, grads)
        params = _as_inputs(host, new)
    return params, state
