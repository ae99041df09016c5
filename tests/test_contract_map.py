"""hgpu_contract_map: a contraction, an elementwise program over its result and
the first extremum over windows of that, in one pass -- the form
`maxPool2dUnpaddedS (reluS (conv2dPreservingS ker x + bias))` takes
(example/MnistCnnShaped2.hs:45-64, External/CommonShapedOps.hs:33-44,241-260).

The device results are checked against numpy's convolution, relu and window
maximum; the host layer's rewrite onto the entry point is checked without a
device, on the CPU checker's table of fused entry points (each defined there as
the single entry points applied one after another) against its plain table."""
import numpy as np
import pytest

from conftest import capi, entry, pkg

O2, CMP = capi.OP2, capi.CMP
# slots: 0 = the convolution, 1 = bias, 2 = zeros, 3 = ones; 4 = conv + bias; 5 = (4 <= 0); 6 = 5 ? 0 : 1; 7 = 6 * 4
RELU = [(1, O2["add"], 0, 0, 1, 0), (2, CMP["leq"], 0, 4, 2, 0), (3, 0, 0, 5, 2, 3), (1, O2["mul"], 0, 6, 4, 0)]


def conv_layer(ctx, x, ker, bias, pool=True):
    """(mask, values, indices, kernel labels) of relu (conv + bias) pooled 2x2, through hgpu_contract_map."""
    B, Ci, Hp, Wp = x.shape
    Co, _, kh, kw = ker.shape
    H, Wd = Hp - kh + 1, Wp - kw + 1
    dtype = x.dtype
    gx, gk, gb = ctx.upload(x), ctx.upload(ker), ctx.upload(bias)
    sh = [B, Co, H, Wd, Ci, kh, kw]
    a = gx.as_strided(sh, [Ci * Hp * Wp, 0, Wp, 1, Hp * Wp, Wp, 1], 0)      # windows of the zero-extended input
    b = gk.as_strided(sh, [0, Ci * kh * kw, 0, 0, kh * kw, kw, 1], 0)
    kept = [B, Co, H, Wd]
    bias_v = gb.as_strided(kept, [0, 1, 0, 0], 0)
    zero = ctx.upload(np.zeros((), dtype)).as_strided(kept, [0, 0, 0, 0], 0)
    one = ctx.upload(np.ones((), dtype)).as_strided(kept, [0, 0, 0, 0], 0)
    ext = None
    if pool:
        ext = (7, [B, Co, H // 2, Wd // 2, 2, 2], [Co * H * Wd, H * Wd, 2 * Wd, 2, Wd, 1], 2, True)
    ctx.profile(2)
    outs, vals, idx = ctx.contract_map(a, b, 4, [None, bias_v, zero, one], RELU, [5] if pool else [5, 7], ext)
    labels = list(ctx.profile_report())
    ctx.profile(0)
    return outs, vals, idx, labels


def reference(x, ker, bias):
    kh, kw = ker.shape[2:]
    win = np.lib.stride_tricks.sliding_window_view(x, (kh, kw), axis=(2, 3))
    z = np.einsum("bihwpq,oipq->bohw", win.astype(np.float64), ker.astype(np.float64)).astype(x.dtype) + bias[None, :, None, None]
    r = np.where(z <= 0, 0, 1).astype(x.dtype) * z
    B, Co, H, Wd = r.shape
    wv = r.reshape(B, Co, H // 2, 2, Wd // 2, 2).transpose(0, 1, 2, 4, 3, 5).reshape(B, Co, H // 2, Wd // 2, 4)
    return z, r, wv


CASES = [  # B, Ci, Co, H, W, k, dtype, fused kernel expected
    (300, 1, 16, 28, 28, 5, np.float64, True),
    (300, 16, 16, 14, 14, 5, np.float64, True),
    (300, 1, 16, 28, 28, 5, np.float32, True),
    (130, 3, 8, 12, 20, 3, np.float64, False),     # 8 output channels, short K: composition of the single kernels
    (7, 2, 4, 8, 8, 3, np.float64, False),
]


@pytest.mark.gpu
@pytest.mark.parametrize("B,Ci,Co,H,Wd,k,dtype,fused", CASES)
def test_conv_relu_pool_in_one_pass(gpu, B, Ci, Co, H, Wd, k, dtype, fused):
    rng = np.random.default_rng(5)
    x = np.zeros((B, Ci, H + k - 1, Wd + k - 1), dtype)
    x[:, :, :H, :Wd] = rng.uniform(-1, 1, (B, Ci, H, Wd))
    x[0, :, :H, :Wd] = 0.75                      # a constant image: whole windows of equal, positive values (ties)
    ker = rng.uniform(-0.4, 0.4, (Co, Ci, k, k)).astype(dtype)
    ker[1] = np.abs(ker[1])                      # ... in channel 1
    bias = rng.uniform(-0.4, 0.4, (Co,)).astype(dtype)
    bias[0] = -100.0                             # channel 0: every window all-negative before the relu
    bias[1] = 0.25
    outs, vals, idx, labels = conv_layer(gpu, x, ker, bias)
    assert any("map(" in l for l in labels) == fused, labels
    z, r, wv = reference(x, ker, bias)
    tol = 1e-10 if dtype == np.float64 else 1e-5
    gv, gi, gm = vals.numpy(), idx.numpy(), outs[0].numpy()
    assert gi.dtype == np.int64 and gm.dtype == np.bool_ and gv.dtype == dtype
    scale = float(np.max(np.abs(wv)))
    assert np.max(np.abs(gv - wv.max(-1))) <= tol * scale
    # all-negative windows: zeros, first position
    assert np.all(gv[:, 0] == 0) and np.all(gi[:, 0] == 0) and np.all(gm[:, 0])
    # ties of positive values (the interior of the constant image, channel 1): first position, as the reference's maxIndex
    inner = slice(0, (H - k + 1) // 2)
    assert np.all(gv[0, 1, inner, : (Wd - k + 1) // 2] > 0) and np.all(gi[0, 1, inner, : (Wd - k + 1) // 2] == 0)
    # elsewhere arguments and masks may differ from numpy's only where values are within rounding of each other / of zero
    srt = np.sort(wv, -1)
    clear = (srt[..., -1] - srt[..., -2]) > 4 * tol * scale
    assert np.array_equal(gi[clear], wv.argmax(-1)[clear])
    sure = np.abs(z) > 4 * tol * float(np.max(np.abs(z)))
    assert np.array_equal(gm[sure], (z <= 0)[sure])


@pytest.mark.gpu
def test_contract_map_without_windows(gpu):
    """Only the program: relu (conv + bias) and its mask written at full size."""
    rng = np.random.default_rng(6)
    B, Ci, Co, H, Wd, k = 260, 2, 16, 12, 12, 3
    x = rng.uniform(-1, 1, (B, Ci, H + k - 1, Wd + k - 1))
    ker = rng.uniform(-0.4, 0.4, (Co, Ci, k, k))
    bias = rng.uniform(-0.4, 0.4, (Co,))
    outs, vals, idx, labels = conv_layer(gpu, x, ker, bias, pool=False)
    assert vals is None and idx is None
    z, r, _ = reference(x, ker, bias)
    assert np.max(np.abs(outs[1].numpy() - r)) <= 1e-10 * np.max(np.abs(r))
    sure = np.abs(z) > 1e-9
    assert np.array_equal(outs[0].numpy()[sure], (z <= 0)[sure])


@pytest.mark.gpu
def test_contract_map_argument_errors(gpu):
    a = gpu.upload(np.ones((4, 3, 5)))
    k = gpu.upload(np.ones((4, 3)))
    with pytest.raises(capi.HgpuError) as e:       # no input stands for the contraction
        gpu.contract_map(a, a, 2, [k], [(0, capi.OP1["neg"], 0, 0, 0, 0)], [1])
    assert e.value.code == 1
    with pytest.raises(capi.HgpuError) as e:       # a view that leaves the result
        gpu.contract_map(a, a, 2, [None], [(0, capi.OP1["neg"], 0, 0, 0, 0)], [], (1, [4, 4], [3, 1], 1, True))
    assert e.value.code == 1
    outs, v, i = gpu.contract_map(a, a, 2, [None], [(0, capi.OP1["neg"], 0, 0, 0, 0)], [1], (1, [4, 3], [3, 1], 1, False))
    assert np.array_equal(outs[0].numpy(), np.full((4, 3), -5.0)) and np.array_equal(v.numpy(), np.full(4, -5.0)) and np.array_equal(i.numpy(), np.zeros(4, np.int64))


def test_host_rewrites_pooling_layers_onto_contract_map():
    """The CNN objective on the checker's fused table takes the rewrite for both
    convolution layers and computes what the plain table computes."""
    H, W = pkg.hostapi, pkg.workloads
    plain = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    fused = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused"))
    wl = W.c3_cnn(batch=5)
    res = []
    for host in (plain, fused):
        ps, ds = wl.upload(host)
        loss, grads = wl.gradient(host, ps, ds)
        res.append((float(loss.numpy()), [g.numpy() for g in grads]))
    assert plain.counter("contract_map") == 0 and fused.counter("contract_map") == 2
    assert res[0][0] == res[1][0]
    for g0, g1 in zip(res[0][1], res[1][1]):
        assert np.array_equal(g0, g1)


# ---- hgpu_contract_operands: operands that are unevaluated expressions ------

def pooled_cotangent(ctx, rng, B, Co, H, Wd, dtype, arg_range=(0, 4)):
    """The cotangent of relu + 2x2 max-pooling as an expression over the refined space
    [B, Co, H/2, 2, W/2, 2]: (which == arg ? dpool : 0) * (mask ? 0 : 1).  Returns
    (inputs, program, slot, merged shape, the same as a numpy array)."""
    O2, CMP = capi.OP2, capi.CMP
    H2, W2 = H // 2, Wd // 2
    dpool = rng.uniform(-1, 1, (B, Co, H2, W2)).astype(dtype)
    arg = rng.integers(arg_range[0], arg_range[1], (B, Co, H2, W2)).astype(np.int64)
    mask = rng.integers(0, 2, (B, Co, H, Wd)).astype(bool)
    cz = np.zeros((B, Co, H2, 2, W2, 2), dtype)
    for p in range(2):
        for q in range(2):
            cz[:, :, :, p, :, q] = np.where(arg == 2 * p + q, dpool, 0)
    cz = cz.reshape(B, Co, H, Wd) * np.where(mask, 0, 1)
    E = [B, Co, H2, 2, W2, 2]
    small = [Co * H2 * W2, H2 * W2, W2, 0, 1, 0]
    ins = [ctx.upload(dpool).as_strided(E, small, 0), ctx.upload(arg).as_strided(E, small, 0), ctx.upload(mask).reshape(E),
           ctx.iota(4).as_strided(E, [0, 0, 0, 2, 0, 1], 0), ctx.upload(np.zeros((), dtype)).as_strided(E, [0] * 6, 0),
           ctx.upload(np.ones((), dtype)).as_strided(E, [0] * 6, 0)]
    # 6 = (which == arg); 7 = 6 ? dpool : 0; 8 = mask ? 0 : 1; 9 = 8 * 7
    prog = [(2, CMP["eq"], 0, 3, 1, 0), (3, 0, 0, 6, 0, 4), (3, 0, 0, 2, 4, 5), (1, O2["mul"], 0, 8, 7, 0)]
    return ins, prog, 9, [B, Co, H, Wd], cz


@pytest.mark.gpu
@pytest.mark.parametrize("B,Ci,Co,H,Wd,k,dtype,fused", [(300, 16, 16, 14, 14, 5, np.float64, True), (300, 16, 16, 14, 14, 5, np.float32, None),
                                                        (280, 1, 16, 28, 28, 5, np.float64, True), (5, 2, 4, 8, 8, 3, np.float64, False)])
def test_gradients_of_a_convolution_from_an_unevaluated_cotangent(gpu, B, Ci, Co, H, Wd, k, dtype, fused):
    """Bias, kernel and input gradient of a convolution layer read the pooled
    cotangent through arg-maxima and relu mask while staging (`fused`: a kernel
    takes it so; False: the call writes it out first; None: either) -- against numpy."""
    rng = np.random.default_rng(8)
    ins, prog, slot, M, cz = pooled_cotangent(gpu, rng, B, Co, H, Wd, dtype)
    x = rng.uniform(-1, 1, (B, Ci, H + k - 1, Wd + k - 1)).astype(dtype)
    ker = rng.uniform(-0.4, 0.4, (Co, Ci, k, k)).astype(dtype)
    tol = 1e-10 if dtype == np.float64 else 1e-5
    Hp, Wp, pad = H + k - 1, Wd + k - 1, k - 1

    def close(got, want):
        return np.max(np.abs(got - want)) <= tol * np.max(np.abs(want))

    def call(a, b, n_keep):
        gpu.profile(2)
        try:
            out = gpu.contract_operands(a, b, n_keep, fused_only=True).numpy()
            took = True
        except capi.HgpuError as e:
            assert e.code == 4
            out = gpu.contract_operands(a, b, n_keep).numpy()
            took = False
        labels = list(gpu.profile_report())
        gpu.profile(0)
        return out, took, labels

    # the bias gradient: a sum over image, row and column
    op = gpu.operand(ins, prog, slot, M, ([Co, B, H, Wd], [H * Wd, Co * H * Wd, Wd, 1], 0))
    got, took, labels = call(op, None, 1)
    assert close(got, cz.sum(axis=(0, 2, 3)).astype(dtype)) and took == (B * H * Wd >= 16384), labels
    # the kernel gradient: dK[co, ci, p, q] = sum_{b, h, w} cz[b, co, h, w] * x[b, ci, h + p, w + q]
    sh = [Co, Ci, k, k, B, H, Wd]
    a_op = gpu.operand(ins, prog, slot, M, (sh, [H * Wd, 0, 0, 0, Co * H * Wd, Wd, 1], 0))
    gx = gpu.upload(x).as_strided(sh, [0, Hp * Wp, Wp, 1, Ci * Hp * Wp, Wp, 1], 0)
    got, took, labels = call(a_op, gx, 4)
    win = np.lib.stride_tricks.sliding_window_view(x, (k, k), axis=(2, 3))[:, :, :H, :Wd]
    assert close(got, np.einsum("bohw,bihwpq->oipq", cz.astype(np.float64), win.astype(np.float64))) and (fused is None or took == fused), labels
    # the input gradient over the zero-extended cotangent, the kernel flipped
    sh = [B, Ci, Hp, Wp, Co, k, k]
    Pl = [B, Co, H + 2 * pad, Wd + 2 * pad]
    ps = [Co * Pl[2] * Pl[3], Pl[2] * Pl[3], Pl[3], 1]
    b_op = gpu.operand(ins, prog, slot, M, (sh, [ps[0], 0, ps[2], ps[3], ps[1], -ps[2], -ps[3]], pad * ps[2] + pad * ps[3]),
                       pad=([0, 0, pad, pad], [0, 0, pad, pad]))
    gk = gpu.upload(ker).as_strided(sh, [0, k * k, 0, 0, Ci * k * k, k, 1], 0)
    got, took, labels = call(gk, b_op, 4)
    czp = np.pad(cz, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    wz = np.lib.stride_tricks.sliding_window_view(czp, (k, k), axis=(2, 3))
    # (whether a kernel takes this one unevaluated depends on how many loads a staging pass of the extended footprint needs)
    assert close(got, np.einsum("bcyxuv,ciuv->biyx", wz.astype(np.float64), ker[:, :, ::-1, ::-1].astype(np.float64))), labels


@pytest.mark.gpu
@pytest.mark.parametrize("B,Ci,Co,H,Wd,k,dtype,arg_range", [(280, 1, 16, 28, 28, 5, np.float64, (0, 4)), (130, 1, 16, 28, 28, 5, np.float64, (-1, 6)),
                                                            (2000, 1, 10, 12, 20, 3, np.float32, (0, 4)), (3000, 2, 7, 16, 8, 3, np.float64, (-2, 4))])
def test_kernel_gradient_of_a_first_layer_from_one_term_per_window(gpu, B, Ci, Co, H, Wd, k, dtype, arg_range):
    """The cotangent of relu + max-pooling has one non-zero per 2x2 window, at the window's
    argument.  With a few rows on the other side (the kernel gradient of a layer of few input
    channels) the contraction takes one term per window: the `onehot_contract` kernel.  Against
    numpy; arguments outside 0 .. 3 (no term at all) included."""
    rng = np.random.default_rng(18)
    ins, prog, slot, M, cz = pooled_cotangent(gpu, rng, B, Co, H, Wd, dtype, arg_range)
    x = rng.uniform(-1, 1, (B, Ci, H + k - 1, Wd + k - 1)).astype(dtype)
    Hp, Wp = H + k - 1, Wd + k - 1
    sh = [Co, Ci, k, k, B, H, Wd]
    view = (sh, [H * Wd, 0, 0, 0, Co * H * Wd, Wd, 1], 0)
    xst = [0, Hp * Wp, Wp, 1, Ci * Hp * Wp, Wp, 1]
    win = np.lib.stride_tricks.sliding_window_view(x, (k, k), axis=(2, 3))[:, :, :H, :Wd]
    want = np.einsum("bohw,bihwpq->oipq", cz.astype(np.float64), win.astype(np.float64))
    tol = 1e-10 if dtype == np.float64 else 1e-5
    for expression_first in (True, False):
        a_op = gpu.operand(ins, prog, slot, M, view)
        gx = gpu.upload(x).as_strided(sh, xst, 0)
        gpu.profile(2)
        got = (gpu.contract_operands(a_op, gx, 4, fused_only=True) if expression_first else gpu.contract_operands(gx, a_op, 4, fused_only=True)).numpy()
        labels = list(gpu.profile_report())
        gpu.profile(0)
        assert any(l.startswith("onehot_contract") for l in labels), labels
        assert got.shape == want.shape and np.max(np.abs(got - want)) <= tol * np.max(np.abs(want)), (expression_first, np.max(np.abs(got - want)))


def test_host_rewrites_gradients_onto_contract_operands():
    """On the checker's fused table the cotangents of the CNN's pooled layers reach
    the contractions unevaluated, and the gradients equal the plain table's."""
    H, W = pkg.hostapi, pkg.workloads
    plain = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    fused = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused"))
    for wl in (W.c3_cnn(batch=4), W.c1_fcnn(batch=7), W.c4_rnn(batch=3, steps=4)):
        res = []
        for host in (plain, fused):
            ps, ds = wl.upload(host)
            loss, grads = wl.gradient(host, ps, ds)
            res.append((float(loss.numpy()), [g.numpy() for g in grads]))
        assert res[0][0] == res[1][0], wl.name
        for g0, g1 in zip(res[0][1], res[1][1]):
            assert np.array_equal(g0, g1), wl.name
    assert plain.counter("contract_operands") == 0 and fused.counter("contract_operands") >= 5


def test_host_takes_a_bias_cotangent_in_the_pass_that_writes_the_layer_cotangent():
    """`stranspose @'[0, 3, 1, 2] $ sreplicate $ sreplicate $ sreplicate bias`
    (example/MnistCnnShaped2.hs:57-63) has the layer's cotangent, transposed
    back and summed over batch, height and width, as the bias's cotangent.  The
    sum waits: when the cotangent expression is written out first (the kernel
    gradient needs it as an array) the sum comes from that pass
    (hgpu_fused_map_dimsum, on the checker's fused table defined as program,
    transpose, sum); asked for first, or without that entry point, it is a pass
    of its own.  All against numpy."""
    H = pkg.hostapi
    rng = np.random.default_rng(3)
    x, y = rng.standard_normal((5, 4, 6, 7)), rng.standard_normal((5, 4, 6, 7))
    want = x * y + x
    for table, order, rides in [("get_api", "expression first", 0), ("get_api_fused", "expression first", 1), ("get_api_fused", "sum first", 0)]:
        host = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table=table))
        e = host.sconcrete(x) * host.sconcrete(y) + host.sconcrete(x)
        s = e.stranspose([0, 2, 3, 1]).ssumN(3)
        assert s.shape == (4,)
        if order == "expression first":
            ev, sv = e.numpy(), s.numpy()
        else:
            sv, ev = s.numpy(), e.numpy()
        assert host.counter("fused_map_dimsum") == rides, (table, order)
        assert np.array_equal(ev, want)
        assert np.max(np.abs(sv - want.sum(axis=(0, 2, 3)))) <= 1e-12 * np.abs(want).sum(axis=(0, 2, 3)).max()
    # a dim that is not brought to the front alone (two kept dims) is summed at once, as before
    host = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused"))
    e = host.sconcrete(x) * host.sconcrete(y) + host.sconcrete(x)
    s2 = e.stranspose([0, 2, 3, 1]).ssumN(2)
    assert np.allclose(s2.numpy(), want.transpose(0, 2, 3, 1).sum(axis=(0, 1)), rtol=1e-12, atol=1e-12) and host.counter("fused_map_dimsum") == 0
