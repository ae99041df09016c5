"""Gradient descent on device arrays against the reference's formulas
(src/HordeAd/External/OptimizerTools.hs:20-47 updateWithGradient, :137-225
updateWithGradientAdam, defaults :82-88) restated in numpy.  The CPU half runs
the host layer on the checker, the GPU half on the device, where a whole
training step -- gradient, Adam update, parameters and moments written back in
place -- is also recorded once and replayed.
"""
import numpy as np
import pytest

from conftest import capi, entry, pkg

H, OPT = pkg.hostapi, pkg.optimizer
RNG = np.random.default_rng(5)


@pytest.fixture(scope="module")
def host_cpu():
    h = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    h.set_fusion(0)      # every operation at once: nothing of the deferral under test takes part in the reference
    return h


@pytest.fixture(scope="module")
def host_gpu():
    return H.Host()


def adam_numpy(args, t, m, v, p, g):
    t = t + 1
    m = args.betaOne * m + (1 - args.betaOne) * g
    v = args.betaTwo * v + (1 - args.betaTwo) * (g * g)
    alphat = args.alpha * np.sqrt(1 - args.betaTwo ** t) / (1 - args.betaOne ** t)
    return t, m, v, p - (alphat * m) / (np.sqrt(v) + args.epsilon)


def check_updates(host, dt, rtol):
    shapes = [(7, 5), (13,), ()]
    ps = [RNG.uniform(-1, 1, s).astype(dt) for s in shapes]
    gs = [RNG.uniform(-1, 1, s).astype(dt) for s in shapes]
    dp, dg = [host.concrete(x) for x in ps], [host.concrete(x) for x in gs]
    # updateWithGradient
    for new, p, g in zip(OPT.updateWithGradient(0.1, dp, dg), ps, gs):
        assert np.allclose(new.numpy(), p - dt(0.1) * g, rtol=rtol, atol=rtol)
    # integers are not differentiable: unchanged
    ip = host.concrete(np.arange(6, dtype=np.int64))
    assert np.array_equal(OPT.updateWithGradient(0.5, [ip], [ip])[0].numpy(), np.arange(6))
    # five Adam steps with changing gradients
    args = OPT.ArgsAdam(alpha=0.01, betaOne=0.8, betaTwo=0.95, epsilon=1e-6)
    state = OPT.initialStateAdam(dp)
    t, ms, vs = 0, [np.zeros_like(p) for p in ps], [np.zeros_like(p) for p in ps]
    cur, dcur = [p.copy() for p in ps], dp
    for step in range(5):
        gs = [RNG.uniform(-1, 1, p.shape).astype(dt) for p in ps]
        dcur, state = OPT.updateWithGradientAdam(args, state, dcur, [host.concrete(g) for g in gs])
        for i in range(len(ps)):
            t_new, ms[i], vs[i], cur[i] = adam_numpy(args, t, ms[i].astype(np.float64), vs[i].astype(np.float64), cur[i].astype(np.float64), gs[i].astype(np.float64))
        t = t_new
        assert state.tAdam == t
        for d, w in zip(dcur, cur):
            assert np.allclose(d.numpy(), w, rtol=rtol, atol=rtol), step
        for d, w in zip(state.mAdam, ms):
            assert np.allclose(d.numpy(), w, rtol=rtol, atol=rtol)
        for d, w in zip(state.vAdam, vs):
            assert np.allclose(d.numpy(), w, rtol=rtol, atol=rtol)
    # default arguments are the reference's
    a = OPT.defaultArgsAdam
    assert (a.alpha, a.betaOne, a.betaTwo, a.epsilon) == (0.001, 0.9, 0.999, 1e-7)
    with pytest.raises(capi.HgpuError):
        OPT.updateWithGradient(0.1, [dp[0]], [dg[1]])


def least_squares(a, params):
    x, y = a
    (w,) = params
    host = w.host
    r = w.smatvecmul(host.concrete(x)) - host.concrete(y)
    return (r * r).ssum0()


def check_sgd_converges(host):
    """sgd / sgdAdam (Optimizer.hs:20-88) on a least-squares problem: the loss falls
    exactly as the numpy restatement's does."""
    w0 = RNG.uniform(-1, 1, (3, 4))
    data = [(RNG.uniform(-1, 1, 4), RNG.uniform(-1, 1, 3)) for _ in range(6)]
    params, last = OPT.sgd(0.05, least_squares, data, [host.param(w0)])
    w = w0.copy()
    for x, y in data:
        r = w @ x - y
        want_last = (r * r).sum()
        w = w - 0.05 * 2 * np.outer(r, x)
    assert np.allclose(params[0].numpy(), w, rtol=1e-11)
    assert np.isclose(float(last.numpy()), want_last, rtol=1e-11)
    args = OPT.ArgsAdam(alpha=0.05)
    p0 = [host.param(w0)]
    params, state = OPT.sgdAdam(least_squares, data, p0, OPT.initialStateAdam(p0), args)
    w, m, v, t = w0.copy(), np.zeros_like(w0), np.zeros_like(w0), 0
    for x, y in data:
        r = w @ x - y
        t, m, v, w = adam_numpy(args, t, m, v, w, 2 * np.outer(r, x))
    assert state.tAdam == len(data)
    assert np.allclose(params[0].numpy(), w, rtol=1e-10)


def test_updates_cpu(host_cpu):
    check_updates(host_cpu, np.float64, 1e-12)
    check_updates(host_cpu, np.float32, 2e-6)


def test_sgd_cpu(host_cpu):
    check_sgd_converges(host_cpu)


@pytest.mark.gpu
def test_updates_gpu(host_gpu):
    check_updates(host_gpu, np.float64, 1e-12)
    check_updates(host_gpu, np.float32, 2e-6)


@pytest.mark.gpu
def test_sgd_gpu(host_gpu):
    check_sgd_converges(host_gpu)


@pytest.mark.gpu
def test_recorded_training_step(host_gpu):
    """Gradient + Adam + write-back as one recorded graph: k launches equal k eager steps."""
    host = host_gpu
    W = pkg.workloads
    wl = W.CONFIGS["c1"](batch=64, widths=(20, 16, 12, 10))
    args = OPT.ArgsAdam(alpha=0.01)

    def eager_steps(k):
        ps, ds = wl.upload(host)
        state = OPT.initialStateAdam(ps)
        losses = []
        for _ in range(k):
            loss, grads = wl.gradient(host, ps, ds)
            losses.append(float(loss.numpy()))
            new, state = OPT.updateWithGradientAdam(args, state, ps, grads)
            host.tape_reset()
            ps = [host._out(host.dll.hh_as_input, p.h) for p in new]
        return losses, [p.numpy() for p in ps]

    want_losses, want_params = eager_steps(4)

    ps, ds = wl.upload(host)
    ms = [host.concrete(np.zeros(p.shape, wl.params[i].dtype)) for i, p in enumerate(ps)]
    vs = [host.concrete(np.zeros(p.shape, wl.params[i].dtype)) for i, p in enumerate(ps)]
    alphat = OPT.adamStepSize(host, ps[0].dtype, args, 1)

    def step():
        loss, grads = wl.gradient(host, ps, ds)
        mn, vn, pn = OPT.adamApply(args, alphat, ms, vs, ps, grads)
        for dst, src in zip(ms + vs + ps, mn + vn + pn):
            dst.assign(src)
        return loss

    # a plain run first (makes constants and kernels), then undo its effect
    step()
    for dst, x in zip(ps, wl.params):
        dst.overwrite(x)
    for z in ms + vs:
        z.overwrite(np.zeros(z.shape, dtype=z.numpy().dtype))
    graph, loss = host.capture(step)
    got = []
    try:
        for t in range(1, 5):
            alphat.overwrite(OPT.adamStepSize(host, ps[0].dtype, args, t).numpy())
            graph.launch()
            host.sync()
            got.append(float(loss.numpy()))
    finally:
        graph.free()
    assert np.allclose(got, want_losses, rtol=1e-12)
    for p, w in zip(ps, want_params):
        assert np.allclose(p.numpy(), w, rtol=1e-10, atol=1e-13)
