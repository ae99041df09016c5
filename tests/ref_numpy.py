"""Independent numpy formulations of the five objectives and their gradients.

Nothing here is shared with the host layer or with the CPU checker: forward
passes are written with einsum / slicing, gradients by hand-derived
backpropagation.  They pin the host layer's operation sequences (workloads.py
run on the checker) to textbook mathematics.
"""
import numpy as np


def softmax_ce(u, expected, batch):
    """lossSoftMaxCrossEntropyS scaled by 1/batch: softmax over the WHOLE tensor
    (shifted by its minimum); the derivative the reference attaches is
    (softmax - expected), not the derivative of the primal expression
    (src/HordeAd/External/CommonShapedOps.hs:89-111)."""
    e = np.exp(u - u.min())
    soft = e / e.sum()
    loss = -(np.log(soft) * expected).sum() / batch
    return loss, (soft - expected) / batch


def c0(x, y, z):
    w = x * np.sin(y)
    loss = (np.arctan2(z, w) + z * w).sum()
    t = 1.0 / (z * z + w * w)
    dw = -z * t + z            # d/dw atan2(z, w) = -z / (z^2 + w^2)
    dz = w * t + w
    return loss, [dw * np.sin(y), dw * x * np.cos(y), dz]


def dense_net(params, x, labels, act):
    batch = x.shape[1]
    ws, bs = params[0::2], params[1::2]
    hs, pre = [x], []
    for i, (w, b) in enumerate(zip(ws, bs)):
        a = w @ hs[-1] + b[:, None]
        pre.append(a)
        if i < len(ws) - 1:
            a = np.tanh(a) if act == "tanh" else np.where(a > 0, a, 0.0).astype(a.dtype)
        hs.append(a)
    loss, d = softmax_ce(hs[-1].astype(np.float64), labels.astype(np.float64), batch)
    d = d.astype(x.dtype)
    grads = [None] * len(params)
    for i in reversed(range(len(ws))):
        if i < len(ws) - 1:
            d = d * ((1 - hs[i + 1] ** 2) if act == "tanh" else (pre[i] > 0))
        grads[2 * i] = d @ hs[i].T
        grads[2 * i + 1] = d.sum(axis=1)
        d = ws[i].T @ d
    return loss, grads


def conv_fwd(k, a):
    co, ci, kh, kw = k.shape
    b, _, h, w = a.shape
    ap = np.pad(a, [(0, 0), (0, 0), (0, kh - 1), (0, kw - 1)])
    out = np.zeros((b, co, h, w), a.dtype)
    for p in range(kh):
        for q in range(kw):
            out += np.einsum("bchw,oc->bohw", ap[:, :, p:p + h, q:q + w], k[:, :, p, q])
    return out


def conv_bwd(k, a, dout):
    co, ci, kh, kw = k.shape
    b, _, h, w = a.shape
    ap = np.pad(a, [(0, 0), (0, 0), (0, kh - 1), (0, kw - 1)])
    dk = np.zeros_like(k)
    dap = np.zeros_like(ap)
    for p in range(kh):
        for q in range(kw):
            dk[:, :, p, q] = np.einsum("bohw,bchw->oc", dout, ap[:, :, p:p + h, q:q + w])
            dap[:, :, p:p + h, q:q + w] += np.einsum("bohw,oc->bchw", dout, k[:, :, p, q])
    return dk, dap[:, :, :h, :w]


def pool_fwd(a):
    b, c, h, w = a.shape
    win = a[:, :, :h // 2 * 2, :w // 2 * 2].reshape(b, c, h // 2, 2, w // 2, 2).transpose(0, 1, 2, 4, 3, 5).reshape(b, c, h // 2, w // 2, 4)
    arg = win.argmax(axis=-1)            # first maximal element
    return np.take_along_axis(win, arg[..., None], -1)[..., 0], arg


def pool_bwd(a_shape, arg, dout):
    b, c, h, w = a_shape
    dwin = np.zeros(arg.shape + (4,), dout.dtype)
    np.put_along_axis(dwin, arg[..., None], dout[..., None], -1)
    da = np.zeros(a_shape, dout.dtype)
    da[:, :, :h // 2 * 2, :w // 2 * 2] = dwin.reshape(b, c, h // 2, w // 2, 2, 2).transpose(0, 1, 2, 4, 3, 5).reshape(b, c, h // 2 * 2, w // 2 * 2)
    return da


def cnn(params, x, labels):
    k1, b1, k2, b2, wd, bd, wr, br = params
    batch = x.shape[0]
    y1 = conv_fwd(k1, x) + b1[None, :, None, None]
    r1 = np.where(y1 > 0, y1, 0.0)
    p1, a1 = pool_fwd(r1)
    y2 = conv_fwd(k2, p1) + b2[None, :, None, None]
    r2 = np.where(y2 > 0, y2, 0.0)
    p2, a2 = pool_fwd(r2)
    m1 = p2.reshape(batch, -1)
    dense = wd @ m1.T + bd[:, None]
    rd = np.where(dense > 0, dense, 0.0)
    out = wr @ rd + br[:, None]
    loss, d = softmax_ce(out, labels, batch)
    gwr, gbr = d @ rd.T, d.sum(axis=1)
    dd = (wr.T @ d) * (dense > 0)
    gwd, gbd = dd @ m1, dd.sum(axis=1)
    dp2 = (wd.T @ dd).T.reshape(p2.shape)
    dy2 = pool_bwd(r2.shape, a2, dp2) * (y2 > 0)
    gk2, dp1 = conv_bwd(k2, p1, dy2)
    gb2 = dy2.sum(axis=(0, 2, 3))
    dy1 = pool_bwd(r1.shape, a1, dp1) * (y1 > 0)
    gk1, _ = conv_bwd(k1, x, dy1)
    gb1 = dy1.sum(axis=(0, 2, 3))
    return loss, [gk1, gb1, gk2, gb2, gwd, gbd, gwr, gbr]


def rnn(params, xs, labels):
    wx, ws, b, wx2, ws2, b2, w3, b3 = params
    steps, _, batch = xs.shape
    width = b.shape[0]
    s1 = np.zeros((width, batch), xs.dtype)
    s2 = np.zeros((width, batch), xs.dtype)
    hist = []
    for t in range(steps):
        v1 = np.tanh(wx @ xs[t] + ws @ s1 + b[:, None])
        v2 = np.tanh(wx2 @ v1 + ws2 @ s2 + b2[:, None])
        hist.append((s1, s2, v1, v2))
        s1, s2 = v1, v2
    out = w3 @ s2 + b3[:, None]
    loss, d = softmax_ce(out.astype(np.float64), labels.astype(np.float64), batch)
    d = d.astype(xs.dtype)
    g = [np.zeros_like(p) for p in params]
    g[6], g[7] = d @ s2.T, d.sum(axis=1)
    ds2 = w3.T @ d
    ds1 = np.zeros_like(s1)
    for t in reversed(range(steps)):
        p1, p2, v1, v2 = hist[t]
        dz2 = ds2 * (1 - v2 * v2)
        g[3] += dz2 @ v1.T
        g[4] += dz2 @ p2.T
        g[5] += dz2.sum(axis=1)
        dv1 = wx2.T @ dz2 + ds1
        ds2 = ws2.T @ dz2
        dz1 = dv1 * (1 - v1 * v1)
        g[0] += dz1 @ xs[t].T
        g[1] += dz1 @ p1.T
        g[2] += dz1.sum(axis=1)
        ds1 = ws.T @ dz1
    return loss, g
