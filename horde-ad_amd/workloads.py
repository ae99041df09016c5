"""The five benchmark objectives as user programs over the carrier.

Each function mirrors a definition of the reference, written in the form the
reference's vectoriser leaves it in (builds over the batch eliminated, index
functions kept), and calls the host layer one tensor operation at a time -- the
way horde-ad's interpreter drives a `BaseTensor` instance:

  reluS, lossSoftMaxCrossEntropyS, conv2dPreservingS, maxPool2dUnpaddedS
      src/HordeAd/External/CommonShapedOps.hs:42-44, 89-111, 136-157, 241-260
  convMnistLayerS / convMnistTwoS / convMnistLossFusedS
      example/MnistCnnShaped2.hs:45-64, 67-108, 111-136
  afcnnMnist2 (batched), rnnMnistLayerR / rnnMnistTwoR / rnnMnistZeroR
      example/MnistFcnnRanked2.hs:52-66, example/MnistRnnRanked2.hs:62-110
  foo (the elementwise objective)
      test/simplified/TestAdaptorSimplified.hs:610-624

Inputs are synthetic, drawn from numpy's counter-based Philox generator with
fixed seeds, so that every provider of the array ABI sees the same numbers.
"""
import numpy as np

from . import capi

F64, F32 = capi.F64, capi.F32
NP = {F64: np.float64, F32: np.float32}


def _rng(seed):
    return np.random.Generator(np.random.Philox(seed))


def uniform(seed, shape, lo, hi, dtype):
    return _rng(seed).uniform(lo, hi, shape).astype(NP[dtype])


def pixels(seed, shape, dtype):
    """Uniform integers 0..255 scaled by 1/255."""
    return (_rng(seed).integers(0, 256, shape).astype(np.float64) / 255.0).astype(NP[dtype])


def one_hot_labels(seed, n_classes, batch, dtype):
    """[n_classes, batch] one-hot columns, classes uniform."""
    cls = _rng(seed).integers(0, n_classes, batch)
    out = np.zeros((n_classes, batch), NP[dtype])
    out[cls, np.arange(batch)] = 1
    return out


# --------------------------------------------------------------- shared pieces

def reluS(v):
    """oneIfGtZero * v with oneIfGtZero = smap0N (\\x -> ifH (x <=. 0) 0 1) (sprimalPart v),
    the closure applied once to a lane value (External/CommonShapedOps.hs:42-44)."""
    from .hostapi import ifH
    one_if = v.sprimalPart().smap0N(lambda x: ifH(x.leq(0.0), 0.0, 1.0, v.dtype))
    return one_if * v


def reluS_select(v):
    """The same with the mask written as an array comparison and an elementwise choice."""
    h = v.host
    mask = v.sprimalPart().leq(0.0)
    one_if = mask.select(h.srepl(v.shape, 0.0, v.dtype), h.srepl(v.shape, 1.0, v.dtype))
    return one_if * v


def sminimum(u):
    """sindex0 tf [kargMin tf] on the flattened tensor."""
    n = int(np.prod(u.shape))
    tf = u.sreshape([n])
    arg = tf.sargMin()
    return tf.sgather((), lambda: [arg.lift(())])


def lossSoftMaxCrossEntropyS(expected, d):
    u = d.sprimalPart()
    exp_u = (u - sminimum(u).sreplicate0N(u.shape)).op1("exp")
    recip_sum = exp_u.ssum0().op1("recip")
    soft = recip_sum.sreplicate0N(u.shape) * exp_u
    primal = -(soft.op1("log").sdot0(expected))
    dual = (soft - expected).sdot0(d)
    return primal.tD(dual)


def conv2dPreservingS(ker, arr):
    """out[img, co, h, w] = sum_{ci, p, q} arr[img, ci, h + p, w + q] * ker[co, ci, p, q],
    reading zeros beyond the image (slicezS)."""
    co, ci, kh, kw = ker.shape
    b, ci2, h, w = arr.shape
    assert ci == ci2
    win = arr.stranspose([2, 3, 0, 1]).sgather((h, kh, w, kw), lambda i, p, j, q: [i + p, j + q])
    # win: [h, kh, w, kw, b, ci]
    lhs = win.sreplicate(co).stranspose([5, 0, 1, 3, 6, 2, 4])          # [b, co, h, w, ci, kh, kw]
    rhs = ker.sreplicateN([b, h, w]).stranspose([0, 3, 1, 2])           # [b, co, h, w, ci, kh, kw]
    return lhs.sdotNIn(rhs, 3)


def maxPool2dUnpaddedS(arr):
    """ksize = stride = 2: smaximum of every 2x2 window."""
    b, c, h, w = arr.shape
    h2, w2 = h // 2, w // 2
    win = arr.stranspose([2, 3, 0, 1]).sgather((h2, 2, w2, 2), lambda i, p, j, q: [2 * i + p, 2 * j + q])
    win = win.stranspose([4, 5, 0, 2, 1, 3]).sreshape([b, c, h2, w2, 4])
    wp = win.sprimalPart()
    return win.sgather((b, c, h2, w2), lambda i, j, k, l: [i, j, k, l, wp.kargMax([i, j, k, l])])


def convMnistLayerS(ker, inp, bias):
    b, _, h, w = inp.shape
    y = conv2dPreservingS(ker, inp)
    bias_stretched = bias.sreplicateN([b, h, w]).stranspose([0, 3, 1, 2])
    return maxPool2dUnpaddedS(reluS(y + bias_stretched))


def reluMaxPoolArtifactS(t):
    """relu and 2x2 max-pooling of t [b, c, h, w] written as the reference's derived
    (simplified) programs express them (test/simplified/TestMnistPP.hs:734-735):
      w248 = sgather table (\\ix -> [ifH (0.0 <=. negate (splainPart t `sindex0` [.., m_h `sindex0` [j, p], m_w `sindex0` [k, q]])) 0 1])
      w249 = sgather t (\\[j, k, p, q] -> [m_h `sindex0` [j, p], m_w `sindex0` [k, q]])
      u    = sreshape (w248 * w249)               -- the windows, relu applied
      sgather u (\\[i, j, k, l] -> [i, j, k, l, kargMax (splainPart u !$ [i, j, k, l])])
    with table = [0.0, 1.0] and the constant index tables m = [[0, 1], [2, 3], ..]."""
    from .hostapi import IxV, ifH
    host = t.host
    b, c, h, w = t.shape
    h2, w2 = h // 2, w // 2
    table = host.sconcrete(np.array([0.0, 1.0], NP[t.dtype]))
    m_h = host.sconcrete(np.arange(2 * h2, dtype=np.int64).reshape(h2, 2))
    m_w = host.sconcrete(np.arange(2 * w2, dtype=np.int64).reshape(w2, 2))
    tp = t.sprimalPart()
    shm = (b, c, h2, w2, 2, 2)

    def mask_index(n, i, j, k, p, q):
        zero = IxV.const(host, shm, 0.0, t.dtype)
        x = tp.sindex0([n, i, m_h.sindex0([j, p]), m_w.sindex0([k, q])])
        return [ifH(zero.leq(-x, t.dtype), 0, 1)]

    w248 = table.sgather(shm, mask_index)
    w249 = t.stranspose([2, 3, 0, 1]).sgather((h2, w2, 2, 2), lambda j, k, p, q: [m_h.sindex0([j, p]), m_w.sindex0([k, q])])
    w249 = w249.stranspose([4, 5, 0, 1, 2, 3])                          # [b, c, h2, w2, 2, 2]
    u = (w248 * w249).sreshape([b, c, h2, w2, 4])
    up = u.sprimalPart()
    return u.sgather((b, c, h2, w2), lambda i, j, k, l: [i, j, k, l, up.kargMax([i, j, k, l])])


def convMnistLayerArtifactS(ker, inp, bias):
    b, _, h, w = inp.shape
    y = conv2dPreservingS(ker, inp)
    bias_stretched = bias.sreplicateN([b, h, w]).stranspose([0, 3, 1, 2])
    return reluMaxPoolArtifactS(y + bias_stretched)


def convMnistTwoS(inp, params, layer=None):
    (k1, b1), (k2, b2), (wd, bd), (wr, br) = params
    layer = layer or convMnistLayerS
    b = inp.shape[0]
    t1 = layer(k1, inp, b1)
    t2 = layer(k2, t1, b2)
    m1 = t2.sreshape([b, int(np.prod(t2.shape[1:]))])
    dense = wd.smatmul2(m1.str_()) + bd.sreplicate(b).str_()
    return wr.smatmul2(reluS(dense)) + br.sreplicate(b).str_()


# ------------------------------------------------------------------- configs

class Workload:
    """name, dtype, batch, numpy inputs (params first), and the objective."""

    def __init__(self, name, dtype, batch, params, data, objective, flops, bytes_):
        self.name, self.dtype, self.batch = name, dtype, batch
        self.params, self.data, self.objective = params, data, objective
        self.flops, self.bytes = flops, bytes_

    def upload(self, host):
        ps = [host.param(p) for p in self.params]
        ds = [host.concrete(d) for d in self.data]
        return ps, ds

    def gradient(self, host, ps, ds):
        """One forward + reverse pass: (loss, [d loss / d param])."""
        host.tape_reset()
        ps = [p.as_input() for p in ps]    # parameters are fresh tape inputs for every gradient
        loss = self.objective(ps, ds)
        return loss, host.grad(loss, ps)


def c0_elementwise(n=4096, m=4096, dtype=F64):
    """sum (atan2 z (x * sin y) + z * (x * sin y)); gradient w.r.t. x, y, z."""
    def away(a):
        return np.where(np.abs(a) < 0.1, np.where(a < 0, a - 0.1, a + 0.1), a).astype(NP[dtype])
    x, y, z = (uniform(s, (n, m), -2, 2, dtype) for s in (1, 2, 3))
    x, z = away(x), away(z)

    def objective(ps, ds):
        x, y, z = ps
        w = x * y.op1("sin")
        return (z.atan2H(w) + z * w).ssum0()

    el = n * m
    return Workload("c0_elementwise", dtype, el, [x, y, z], [], objective, flops=20.0 * el, bytes_=6.0 * el * np.dtype(NP[dtype]).itemsize)


def _dense_net(name, dtype, batch, widths, act, seeds, init):
    n_in = widths[0]
    x = pixels(seeds[0], (n_in, batch), dtype)
    labels = one_hot_labels(seeds[1], widths[-1], batch, dtype)
    rng = _rng(seeds[2])
    params = []
    for fan_in, fan_out in zip(widths[:-1], widths[1:]):
        r = init(fan_in, fan_out)
        params.append(rng.uniform(-r, r, (fan_out, fan_in)).astype(NP[dtype]))
        params.append(rng.uniform(-r, r, (fan_out,)).astype(NP[dtype]))

    def objective(ps, ds):
        xx, lab = ds
        hcur = xx
        n_layers = len(ps) // 2
        for li in range(n_layers):
            w, bias = ps[2 * li], ps[2 * li + 1]
            hcur = w.smatmul2(hcur) + bias.sreplicate(batch).str_()
            if li < n_layers - 1:
                hcur = hcur.op1("tanh") if act == "tanh" else reluS(hcur)
        loss = lossSoftMaxCrossEntropyS(lab, hcur)
        return loss.host.srepl((), 1.0 / batch, dtype) * loss

    mm = sum(a * b for a, b in zip(widths[:-1], widths[1:]))
    dx = sum(a * b for a, b in zip(widths[1:-1], widths[2:]))
    flops = 2.0 * batch * (2 * mm + dx)
    return Workload(name, dtype, batch, params, [x, labels], objective, flops=flops, bytes_=None)


def c1_fcnn(batch=5000, dtype=F64, widths=(784, 300, 100, 10)):
    return _dense_net("c1_fcnn", dtype, batch, widths, "tanh", (11, 12, 13), lambda i, o: 0.5)


def c2_wide(batch=8192, dtype=F32, widths=(784, 2048, 2048, 10)):
    return _dense_net("c2_wide", dtype, batch, widths, "relu", (11, 12, 21), lambda i, o: float(np.sqrt(6.0 / (i + o))))


def c3_cnn(batch=1000, dtype=F64, h=28, w=28, ksize=5, c_out=16, n_hidden=128, n_classes=10):
    inp = pixels(31, (batch, 1, h, w), dtype)
    labels = one_hot_labels(32, n_classes, batch, dtype)
    rng = _rng(33)
    flat = c_out * (h // 4) * (w // 4)
    shapes = [(c_out, 1, ksize, ksize), (c_out,), (c_out, c_out, ksize, ksize), (c_out,),
              (n_hidden, flat), (n_hidden,), (n_classes, n_hidden), (n_classes,)]
    params = [rng.uniform(-0.4, 0.4, s).astype(NP[dtype]) for s in shapes]

    def objective(ps, ds, layer=None):
        x, lab = ds
        result = convMnistTwoS(x, list(zip(ps[0::2], ps[1::2])), layer)
        loss = lossSoftMaxCrossEntropyS(lab, result)
        return loss.host.srepl((), 1.0 / batch, dtype) * loss

    k2 = ksize * ksize
    conv1 = 2.0 * batch * c_out * h * w * k2
    conv2 = 2.0 * batch * c_out * c_out * (h // 2) * (w // 2) * k2
    dense = 2.0 * batch * flat * n_hidden
    ro = 2.0 * batch * n_hidden * n_classes
    flops = 2 * conv1 + 3 * conv2 + 3 * dense + 3 * ro
    wl = Workload("c3_cnn", dtype, batch, params, [inp, labels], objective, flops=flops, bytes_=None)
    wl.objective_artifact = lambda ps, ds: objective(ps, ds, convMnistLayerArtifactS)
    return wl


def c3_cnn_artifact(**kw):
    """The same network with relu and pooling written as the reference's derived programs
    print them (gathers from [0.0, 1.0] by an `ifH` index, constant index tables)."""
    wl = c3_cnn(**kw)
    wl.name = "c3_cnn_artifact_form"
    wl.objective = wl.objective_artifact
    return wl


def c4_rnn(batch=5000, dtype=F32, steps=28, n_in=28, width=128, n_classes=10):
    xs = pixels(41, (steps, n_in, batch), dtype)
    labels = one_hot_labels(43, n_classes, batch, dtype)
    rng = _rng(42)
    shapes = [(width, n_in), (width, width), (width,), (width, width), (width, width), (width,),
              (n_classes, width), (n_classes,)]
    params = [rng.uniform(-0.1, 0.1, s).astype(NP[dtype]) for s in shapes]

    # the reference writes this network with the ranked methods (rmatmul2, rtr,
    # rreplicate, rslice, rappend): here they are the shaped ones by another name
    def layer(s, x, wx, ws, b):
        return (wx.rmatmul2(x) + ws.rmatmul2(s) + b.rreplicate(batch).rtr()).op1("tanh")

    def objective(ps, ds):
        xs_, lab = ds
        wx, ws, b, wx2, ws2, b2, w3, b3 = ps
        host = wx.host
        s = host.rrepl((2 * width, batch), 0.0, dtype)           # zeroStateR
        out = None
        for t in range(steps):                                    # unrollLastR: foldl' over runravelToList
            x = xs_.rindex([t])
            s1, s2 = s.rslice(0, width), s.rslice(width, width)
            v1 = layer(s1, x, wx, ws, b)
            v2 = layer(s2, v1, wx2, ws2, b2)
            s = v1.rappend(v2)
            out = s.rslice(width, width)
        result = w3.rmatmul2(out) + b3.rreplicate(batch).rtr()
        loss = lossSoftMaxCrossEntropyS(lab, result)
        return host.srepl((), 1.0 / batch, dtype) * loss

    def objective_mapaccum(ps, ds):
        """The same network as a tmapAccumL over the sequence (the fold form of
        the reference's recurrent example) instead of an unrolled loop."""
        xs_, lab = ds
        wx, ws, b, wx2, ws2, b2, w3, b3 = ps
        host = wx.host

        def step(s, x):
            v1 = layer(s.sslice(0, width), x, wx, ws, b)
            v2 = layer(s.sslice(width, width), v1, wx2, ws2, b2)
            return v1.sappend(v2), v2

        _, outs = host.smapAccumL(step, host.srepl((2 * width, batch), 0.0, dtype), xs_)
        result = w3.smatmul2(outs.sindex([steps - 1])) + b3.sreplicate(batch).str_()
        return host.srepl((), 1.0 / batch, dtype) * lossSoftMaxCrossEntropyS(lab, result)

    per_step = 2.0 * batch * (width * n_in + 3 * width * width)
    flops = 3 * steps * per_step + 3 * 2.0 * batch * width * n_classes
    wl = Workload("c4_rnn", dtype, batch, params, [xs, labels], objective, flops=flops, bytes_=None)
    wl.objective_mapaccum = objective_mapaccum
    return wl


class Micro(Workload):
    """A chain of operations timed by itself (the reference's bench/ConvVjpBench.hs groups
    gather48 / scatter48): `gradient` evaluates the chain into a dense array and hands back
    (one element of it, [the array]) in the places of the loss and the gradients."""

    def __init__(self, name, dtype, data, chain, bytes_):
        super().__init__(name, dtype, 1, [], data, None, flops=0.0, bytes_=bytes_)
        self.chain = chain

    def gradient(self, host, ps, ds):
        out = self.chain(*ds).dense()
        return out.sindex([0] * len(out.shape)), [out]


def gather48(dtype=F64):
    """twoAd of bench/ConvVjpBench.hs:429-439: the two-gather chain of a 48x48 im2col,
    [50, 3, 3, 50] -> [48, 3, 3, 48, 3, 3] (186624 elements), big position dim first."""
    x = uniform(42, (50, 3, 3, 50), -0.5, 0.5, dtype)

    def chain(src):
        g1 = src.sgather((48, 3), lambda a, b: [a + b])                                   # [48, 3, 3, 3, 50]
        return g1.stranspose([4, 2, 0, 3, 1]).sgather((48, 3), lambda c, d: [c + d])       # [48, 3, 3, 48, 3, 3]

    es = np.dtype(NP[dtype]).itemsize
    return Micro("gather48_two_gather_chain", dtype, [x], chain, bytes_=(50 * 3 * 3 * 50 + 48 * 3 * 3 * 48 * 3 * 3) * es)


def scatter48(dtype=F64):
    """The adjoint of that chain (bench/ConvVjpBench.hs:586-700, checked there by checkAdjoint):
    [48, 3, 3, 48, 3, 3] -> [50, 3, 3, 50] through two scatters with the gathers' index functions."""
    y = uniform(43, (48, 3, 3, 48, 3, 3), -0.5, 0.5, dtype)

    def chain(cot):
        s2 = cot.sscatter(2, [50], lambda c, d: [c + d])                                    # [50, 3, 48, 3, 3]
        return s2.stranspose([2, 4, 1, 3, 0]).sscatter(2, [50], lambda a, b: [a + b])       # [50, 3, 3, 50]

    es = np.dtype(NP[dtype]).itemsize
    return Micro("scatter48_two_scatter_chain", dtype, [y], chain, bytes_=(50 * 3 * 3 * 50 + 48 * 3 * 3 * 48 * 3 * 3) * es)


CONFIGS = {"c0": c0_elementwise, "c1": c1_fcnn, "c2": c2_wide, "c3": c3_cnn, "c4": c4_rnn}
# the same work written another way: timed beside the configs, never the headline
RIDERS = {"c3_artifact_form": c3_cnn_artifact, "gather48": gather48, "scatter48": scatter48}
