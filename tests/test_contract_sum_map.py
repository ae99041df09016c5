"""hgpu_contract_sum_map: a sum of matrix products with short contracted dims and
an elementwise program over the sum -- the layer of the reference's recurrent
network, `tanh (wX `rmatmul2` x + wS `rmatmul2` s + rtr (rreplicate batch_size b))`
(example/MnistRnnRanked2.hs:62-75), and the head of its cotangent.

Device against the checker through the C ABI; the checker DEFINES the entry
point as hgpu_contract per term, `+` in order, hgpu_fused_map.  fp64 within
1e-10, fp32 within 1e-5 normwise; Bool results of comparisons are compared
away from the ties that rounding can flip.
"""
import numpy as np
import pytest

from conftest import capi

O1, O2 = capi.OP1, capi.OP2      # instruction kinds: 0 unary, 1 binary, 2 comparison
RNG = np.random.default_rng(2024)
TOL = {np.dtype(np.float64): 1e-10, np.dtype(np.float32): 1e-5}


def matmul_views(w, x):
    """w [m, k], x [k, n] as the two factors of tsmatmul2: both of shape [m, n, k]."""
    m, n = w.shape[0], x.shape[1]
    return w.replicate([n]).transpose([1, 0]), x.replicate([m]).transpose([0, 2, 1])


def rel(got, want):
    scale = max(float(np.max(np.abs(want))), 1e-300)
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) / scale


def layer_case(ctx, dt, m, n, ks, layouts, bias=True):
    """sum_t w_t . x_t (+ bias) -> tanh; layouts[t] = 'mk' (w stored [m, k]) or 'km' (stored [k, m], used transposed)."""
    terms, want = [], np.zeros((m, n), np.float64)
    for k, lay in zip(ks, layouts):
        w = RNG.uniform(-0.3, 0.3, (m, k)).astype(dt)
        x = RNG.uniform(-1, 1, (k, n)).astype(dt)
        wa = ctx.upload(w) if lay == "mk" else ctx.upload(np.ascontiguousarray(w.T)).transpose([1, 0])
        terms.append(matmul_views(wa, ctx.upload(x)))
        want += w.astype(np.float64) @ x.astype(np.float64)
    b = RNG.uniform(-0.5, 0.5, (m,)).astype(dt)
    if bias:
        ins = [None, ctx.upload(b).replicate([n]).transpose([1, 0])]
        prog = [(1, O2["add"], 0, 0, 1, 0), (0, O1["tanh"], 0, 2, 0, 0)]
        want = np.tanh(want + b.astype(np.float64)[:, None])
        slots = [3]
    else:
        ins, prog, slots = [None], [], [0]
    return terms, ins, prog, slots, want


SHAPES = [
    # dtype, m, n, ks, layouts
    (np.float32, 128, 1000, [28, 128], ["mk", "mk"]),       # the first layer of the recurrent network
    (np.float32, 128, 1000, [128, 128], ["km", "km"]),      # the cotangent's two products (weights transposed)
    (np.float32, 128, 1000, [128], ["mk"]),
    (np.float64, 300, 1000, [100], ["km"]),                 # a dense layer's cotangent
    (np.float64, 100, 1000, [300], ["mk"]),                 # five chunks
    (np.float64, 10, 999, [30], ["mk"]),                    # odd extent: no vectors along n, k padded to 32
    (np.float32, 10, 998, [27], ["mk"]),                    # k neither a multiple of 4 nor contiguous vectors
    (np.float32, 40, 1004, [8, 12, 16, 20], ["mk", "km", "mk", "km"]),
    (np.float32, 128, 1000, [600], ["mk"]),                 # up to 1024 contracted elements when the result is small ...
    (np.float64, 128, 1000, [784], ["mk"]),                 # ... (a dense layer over a flattened image: 13 chunks)
    (np.float64, 128, 784, [1000], ["km"]),                 # its weight gradient: 16 chunks
    (np.float64, 70, 333, [900], ["mk"]),                   # few tiles, long K, ragged everywhere: K shared out between blocks, a second launch adds the partial tiles
    (np.float32, 50, 90, [1000], ["km"]),                   # the same in fp32 with the weights transposed (6 tiles of 16 chunks)
    (np.float32, 128, 1000, [1100], ["mk"]),                # too long for the kernel: the entry points one after another
    (np.float32, 300, 1000, [600], ["mk"]),                 # too long for a result of this size
    (np.float64, 300, 5000, [784], ["mk"]),                 # ... a dense layer over a flattened image at batch 5000: split in two along K, the program adds the halves
    (np.float32, 6, 20, [5], ["mk"]),                       # too small for it
]


@pytest.mark.gpu
@pytest.mark.parametrize("dt,m,n,ks,layouts", SHAPES)
def test_layer_matches_checker_and_numpy(gpu, oracle, dt, m, n, ks, layouts):
    one_kernel = sum(ks) <= (1024 if m * n <= 160000 else 512) and m * n * sum(ks) >= 1e6      # what the compiled kernel covers
    for bias in (True, False):
        gpu.check(gpu.lib.profile_enable(gpu.h, 2))
        state = RNG.bit_generator.state
        res = []
        for ctx in (gpu, oracle):
            RNG.bit_generator.state = state
            terms, ins, prog, slots, want = layer_case(ctx, dt, m, n, ks, layouts, bias)
            res.append(ctx.contract_sum_map(terms, 2, ins, prog, slots)[0].numpy())
        labels = list(gpu.profile_report())
        gpu.check(gpu.lib.profile_enable(gpu.h, 0))
        assert any("wholeK" in k for k in labels) == one_kernel, labels
        if one_kernel:
            assert len(labels) == 1, labels
        assert res[0].shape == (m, n) and res[0].dtype == np.dtype(dt)
        tol = TOL[np.dtype(dt)]
        assert rel(res[0], res[1]) <= tol, (dt, m, n, ks, rel(res[0], res[1]))
        assert rel(res[0], want) <= 4 * tol and rel(res[1], want) <= 4 * tol


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_cotangent_head_with_several_results(gpu, oracle, dt):
    """(w2^T dz2 + w1^T dz1) * (1 - h * h), the sum itself, and a comparison, from one call;
    the program reads h (dense), and the sum stands at slot 1."""
    m, n, k = 128, 1000, 128
    w2 = RNG.uniform(-0.3, 0.3, (k, m)).astype(dt)
    w1 = RNG.uniform(-0.3, 0.3, (k, m)).astype(dt)
    dz2 = RNG.uniform(-1, 1, (k, n)).astype(dt)
    dz1 = RNG.uniform(-1, 1, (k, n)).astype(dt)
    h = np.tanh(RNG.uniform(-2, 2, (m, n))).astype(dt)
    one = np.asarray(1.0, dt)
    prog = [(1, O2["mul"], 0, 0, 0, 0),        # 3: h * h
            (1, O2["sub"], 0, 2, 3, 0),        # 4: 1 - h * h
            (1, O2["mul"], 0, 1, 4, 0),        # 5: C * (1 - h * h)
            (2, capi.CMP["lt"], 0, 1, 0, 0)]   # 6: C < h
    res = []
    for ctx in (gpu, oracle):
        terms = [matmul_views(ctx.upload(w2).transpose([1, 0]), ctx.upload(dz2)), matmul_views(ctx.upload(w1).transpose([1, 0]), ctx.upload(dz1))]
        ins = [ctx.upload(h), None, ctx.upload(one).replicate([m, n])]
        res.append([a.numpy() for a in ctx.contract_sum_map(terms, 2, ins, prog, [5, 1, 6])])
    c = w2.T.astype(np.float64) @ dz2.astype(np.float64) + w1.T.astype(np.float64) @ dz1.astype(np.float64)
    want = c * (1 - h.astype(np.float64) ** 2)
    tol = TOL[np.dtype(dt)]
    assert rel(res[0][0], res[1][0]) <= tol and rel(res[0][0], want) <= 4 * tol
    assert rel(res[0][1], res[1][1]) <= tol and rel(res[0][1], c) <= 4 * tol
    assert res[0][2].dtype == np.bool_ and res[0][2].shape == (m, n)
    clear = np.abs(c - h) > 1e-3 * np.max(np.abs(c))     # away from ties
    assert np.array_equal(res[0][2][clear], (c < h)[clear]) and np.array_equal(res[1][2][clear], (c < h)[clear])


@pytest.mark.gpu
def test_plain_contractions_with_short_k_take_the_same_kernel(gpu, oracle):
    """hgpu_contract and hgpu_contract_sum of such shapes (no program) agree with the checker too."""
    for dt, m, n, k in [(np.float32, 128, 5000, 128), (np.float64, 300, 5000, 100), (np.float32, 128, 5000, 28)]:
        w = RNG.uniform(-0.3, 0.3, (m, k)).astype(dt)
        x = RNG.uniform(-1, 1, (k, n)).astype(dt)
        got = []
        for ctx in (gpu, oracle):
            a, b = matmul_views(ctx.upload(w), ctx.upload(x))
            got.append(a.contract(b, 2).numpy())
        want = w.astype(np.float64) @ x.astype(np.float64)
        assert rel(got[0], got[1]) <= TOL[np.dtype(dt)] and rel(got[0], want) <= 4 * TOL[np.dtype(dt)]


@pytest.mark.gpu
def test_argument_errors(gpu):
    w, x = gpu.upload(np.ones((8, 4), np.float32)), gpu.upload(np.ones((4, 6), np.float32))
    a, b = matmul_views(w, x)
    with pytest.raises(capi.HgpuError) as e:
        gpu.contract_sum_map([(a, b)], 2, [gpu.upload(np.ones((8, 6), np.float32))], [], [0])     # nothing stands for the sum
    assert e.value.code == 1
    with pytest.raises(capi.HgpuError):
        gpu.contract_sum_map([(a, b)], 2, [None, gpu.upload(np.ones((8, 5), np.float32))], [], [0])   # an input of another shape
    w2, x2 = gpu.upload(np.ones((7, 4), np.float32)), gpu.upload(np.ones((4, 6), np.float32))
    with pytest.raises(capi.HgpuError):
        gpu.contract_sum_map([(a, b), matmul_views(w2, x2)], 2, [None], [], [0])                  # terms of different kept shapes
    with pytest.raises(capi.HgpuError):
        gpu.contract_sum_map([(a, b)], 2, [None], [], [3])                                        # a slot that does not exist


def test_checker_definition_against_numpy(oracle):
    """The checker's composition itself, pinned by numpy on a case small enough to read."""
    w1 = np.arange(6.0).reshape(2, 3)
    x1 = np.arange(12.0).reshape(3, 4) - 5
    w2 = np.array([[1.0, -1.0], [0.5, 2.0]])
    x2 = np.arange(8.0).reshape(2, 4)
    b = np.array([0.25, -0.75])
    terms = [matmul_views(oracle.upload(w1), oracle.upload(x1)), matmul_views(oracle.upload(w2), oracle.upload(x2))]
    ins = [None, oracle.upload(b).replicate([4]).transpose([1, 0])]
    prog = [(1, O2["add"], 0, 0, 1, 0), (0, O1["tanh"], 0, 2, 0, 0)]
    got, raw = oracle.contract_sum_map(terms, 2, ins, prog, [3, 0])
    c = w1 @ x1 + w2 @ x2
    assert np.allclose(raw.numpy(), c, rtol=0, atol=1e-12)
    assert np.allclose(got.numpy(), np.tanh(c + b[:, None]), rtol=0, atol=1e-12)


def test_host_rewrites_layers_onto_contract_sum_map():
    """On a table that has the entry point, the recurrent network's layers (two
    products of different contracted lengths, `+ b`, tanh) and the heads of their
    cotangents go out as one call each, and the gradient equals the plain table's."""
    from conftest import entry, pkg
    H, W = pkg.hostapi, pkg.workloads
    plain = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    fused = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused"))
    steps = 4
    wl = W.c4_rnn(batch=3, steps=steps)
    res = []
    for host in (plain, fused):
        ps, ds = wl.upload(host)
        loss, grads = wl.gradient(host, ps, ds)
        res.append((float(loss.numpy()), [g.numpy() for g in grads]))
    assert res[0][0] == res[1][0]
    for g0, g1 in zip(res[0][1], res[1][1]):
        assert np.array_equal(g0, g1)
    # two layers per step forward; backward one call per layer and step but the very first layer's input needs no cotangent
    assert plain.counter("contract_sum_map") == 0 and fused.counter("contract_sum_map") >= 4 * steps


def test_condition_of_relu_is_a_result_of_the_layer_call():
    """relu (W x + b) keeps `0 < W x + b` for the reverse pass.  On a table with
    the entry point the condition leaves the layer's call as one more result, so
    the reverse pass does not multiply W x a second time; values and gradients
    equal the plain table's."""
    from conftest import entry, pkg
    H, W = pkg.hostapi, pkg.workloads
    plain = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    fused = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused"))
    wl = W.c2_wide(batch=7, widths=(12, 9, 8, 5))
    res = []
    for host in (plain, fused):
        ps, ds = wl.upload(host)
        loss, grads = wl.gradient(host, ps, ds)
        res.append((float(loss.numpy()), [g.numpy() for g in grads]))
    assert res[0][0] == res[1][0]
    for g0, g1 in zip(res[0][1], res[1][1]):
        assert np.array_equal(g0, g1)
    assert fused.counter("contract_sum_map_kept_nodes") == 2        # the two hidden layers
    # products per gradient: 3 forward, 2 input cotangents, 3 weight gradients; none twice
    assert fused.counter("contract_sum_map") + fused.counter("contract") + fused.counter("contract_sum") <= 8


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_two_layer_recurrence_issued_layer_by_layer(gpu, oracle, dt):
    """h1_t = tanh (wX x_t + wS h1_(t-1) + b1), h2_t = tanh (wX2 h1_t + wS2 h2_(t-1) + b2)
    (example/MnistRnnRanked2.hs:62-110), all steps of the first layer issued before the
    second layer's: on the device the launches wait until something reads a result, and
    step t + 1 of the first layer then shares a kernel with step t of the second, which
    does not depend on it.  Results against the checker (one call after another) and numpy."""
    import os
    if os.environ.get("HORDEAD_NO_GROUPED_LAUNCH"):
        pytest.skip("grouped launches are switched off in this environment")
    width, batch, k_in, steps = 128, 1000, 28, 6
    ws = [RNG.uniform(-0.3, 0.3, s).astype(dt) for s in ((width, k_in), (width, width), (width, width), (width, width))]
    bs = [RNG.uniform(-0.5, 0.5, (width,)).astype(dt) for _ in range(2)]
    xs = [RNG.uniform(-1, 1, (k_in, batch)).astype(dt) for _ in range(steps)]
    prog = [(1, O2["add"], 0, 0, 1, 0), (0, O1["tanh"], 0, 2, 0, 0)]
    want1, want2 = [], []
    s1 = s2 = np.zeros((width, batch), np.float64)
    for t in range(steps):
        s1 = np.tanh(ws[0].astype(np.float64) @ xs[t] + ws[1].astype(np.float64) @ s1 + bs[0].astype(np.float64)[:, None])
        s2 = np.tanh(ws[2].astype(np.float64) @ s1 + ws[3].astype(np.float64) @ s2 + bs[1].astype(np.float64)[:, None])
        want1.append(s1)
        want2.append(s2)

    def run(ctx):
        w = [ctx.upload(a) for a in ws]
        b = [ctx.upload(a).replicate([batch]).transpose([1, 0]) for a in bs]
        zero = ctx.upload(np.zeros((), dt)).replicate([batch]).replicate([width])     # one element for the whole state, as `rrepl sh 0`
        xa = [ctx.upload(a) for a in xs]
        h1, h2 = [], []
        for t in range(steps):
            terms = [matmul_views(w[0], xa[t]), matmul_views(w[1], h1[-1] if h1 else zero)]
            h1.append(ctx.contract_sum_map(terms, 2, [None, b[0]], prog, [3])[0])
        for t in range(steps):
            terms = [matmul_views(w[2], h1[t]), matmul_views(w[3], h2[-1] if h2 else zero)]
            h2.append(ctx.contract_sum_map(terms, 2, [None, b[1]], prog, [3])[0])
        return h1, h2

    tol = TOL[np.dtype(dt)]
    for attempt in range(2):     # a set of problems is compiled into one kernel the second time it comes up
        gpu.check(gpu.lib.profile_enable(gpu.h, 2))
        g1, g2 = run(gpu)
        got = [a.numpy() for a in g1 + g2]
        labels = gpu.profile_report()
        gpu.check(gpu.lib.profile_enable(gpu.h, 0))
        launches = sum(v[0] for k, v in labels.items() if "wholeK" in k)
        if attempt == 1:
            # 6 + 6 problems on 7 diagonals: the two ends alone, five pairs
            assert launches == steps + 1, labels
            assert sum(v[0] for k, v in labels.items() if "[group:" in k) == steps - 1, labels
    c1, c2 = run(oracle)
    chk = [a.numpy() for a in c1 + c2]
    for g, c, w in zip(got, chk, want1 + want2):
        assert g.dtype == np.dtype(dt) and rel(g, c) <= tol * steps and rel(g, w) <= 4 * tol * steps


@pytest.mark.gpu
def test_held_back_products_come_before_whatever_reads_them(gpu, oracle):
    """A held-back product followed by other work on its result (an elementwise call, a
    product too long for the compiled kernel, a download), and by a release of its inputs
    before anything has run."""
    m, n, k = 64, 1000, 64
    w = RNG.uniform(-0.3, 0.3, (m, k)).astype(np.float32)
    x = RNG.uniform(-1, 1, (k, n)).astype(np.float32)
    res = []
    for ctx in (gpu, oracle):
        wa, xa = ctx.upload(w), ctx.upload(x)
        c = ctx.contract_sum_map([matmul_views(wa, xa)], 2, [None], [], [0])[0]
        del wa, xa                                             # the queue holds what the launch reads
        e = ctx.fused_map([c], [(0, O1["tanh"], 0, 0, 0, 0)], [1])[0]
        d = ctx.contract_sum_map([matmul_views(ctx.upload(w.T.copy()), c)], 2, [None], [], [0])[0]   # reads c, still held back
        res.append((c.numpy(), e.numpy(), d.numpy()))
    want_c = w.astype(np.float64) @ x
    for g, c, want in zip(res[0], res[1], (want_c, np.tanh(want_c), w.T.astype(np.float64) @ want_c)):
        assert rel(g, c) <= 1e-5 and rel(g, want) <= 4e-5


def test_cotangent_of_a_dense_layer_is_one_call():
    """`(W^T dz) * (1 - h * h)`, the cotangent that a dense tanh layer hands down
    (the reference's dense layers: example/MnistFcnnRanked2.hs, `tanh` hidden
    activations), reaches the weight gradient below it as an operand seen through
    views.  The product under it is short (the layer above is 8 or 5 wide): it goes
    out with its program as one call, not alone and then the program.  Gradient
    against the plain table's bit for bit and numpy's within 1e-12."""
    from conftest import entry, pkg
    import ref_numpy as ref
    H, W = pkg.hostapi, pkg.workloads
    plain = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    fused = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused"))
    wl = W.c1_fcnn(batch=9, widths=(12, 8, 5, 4))
    res = []
    for host in (plain, fused):
        ps, ds = wl.upload(host)
        loss, grads = wl.gradient(host, ps, ds)
        res.append((float(loss.numpy()), [g.numpy() for g in grads]))
    assert res[0][0] == res[1][0]
    for g0, g1 in zip(res[0][1], res[1][1]):
        assert np.array_equal(g0, g1)
    # three layers forward, two cotangents handed down
    assert fused.counter("contract_sum_map") == 5
    rloss, rgrads = ref.dense_net(wl.params, *wl.data, "tanh")
    assert abs(res[1][0] - rloss) <= 1e-12 * abs(rloss)
    for g, r in zip(res[1][1], rgrads):
        assert np.max(np.abs(g - r)) <= 1e-12 * max(1.0, float(np.max(np.abs(r))))
