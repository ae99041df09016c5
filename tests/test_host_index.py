"""Index functions through the host layer: gather / scatter with lane-batched
scalars against a per-position brute force (the reference's own algorithm,
src/HordeAd/Core/OpsConcrete.hs:1581-1665: call the index function for every
position, check bounds, copy or accumulate).  CPU half runs on the checker; the
GPU half repeats the cases on the device and compares bit for bit (gather) or
to 1e-10 (scatter sums).
"""
import itertools

import numpy as np
import pytest

from conftest import capi, entry, pkg

H = pkg.hostapi
RNG = np.random.default_rng(7)


@pytest.fixture(scope="module")
def host_cpu():
    h = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    h.set_fusion(0)      # every operation at once: nothing of the deferral under test takes part in the reference
    return h


@pytest.fixture(scope="module")
def host_gpu():
    return H.Host()


def quot(a, b):
    return a if b == 0 else int(abs(a) // abs(b)) * (1 if (a >= 0) == (b >= 0) else -1)


def rem(a, b):
    return a if b == 0 else a - quot(a, b) * b


# (source shape, position space shm, index function on IxV, the same on ints, affine?)
CASES = [
    ((9, 3), (5, 4), lambda i, k: [i + k], lambda i, k: [i + k], True),                       # conv window, runs out of bounds
    ((9, 3), (5, 4), lambda i, k: [i + k, k], lambda i, k: [i + k, k], True),
    ((8, 6, 2), (4, 2, 3, 2), lambda i, p, j, q: [2 * i + p, 2 * j + q], lambda i, p, j, q: [2 * i + p, 2 * j + q], True),  # pooling windows
    ((7, 5), (3, 6), lambda i, k: [6 - 2 * i, k - 1], lambda i, k: [6 - 2 * i, k - 1], True),  # negative coefficient, offset
    ((7,), (4, 3), lambda i, k: [i * k], lambda i, k: [i * k], False),
    ((7, 4), (5, 2), lambda i, k: [(i + 1).quotH(k), (2 * i).remH(3)], lambda i, k: [quot(i + 1, k), rem(2 * i, 3)], False),
    ((6, 4), (6,), lambda i: [i.minH(3), (5 - i).maxH(1)], lambda i: [min(i, 3), max(5 - i, 1)], False),
    ((5, 3), (), lambda: [2], lambda: [2], True),
    ((5, 3), (4,), lambda i: [7, i], lambda i: [7, i], True),                                  # always out of bounds
]


def brute_gather(src, shm, f):
    probe = f(*[0] * len(shm))
    n_ix = len(probe)
    out = np.zeros(tuple(shm) + src.shape[n_ix:], src.dtype)
    for m in itertools.product(*[range(s) for s in shm]):
        p = tuple(f(*m))
        if all(0 <= p[k] < src.shape[k] for k in range(n_ix)):
            out[m] = src[p]
    return out


def brute_scatter(src, rank_m, shp, f):
    out = np.zeros(tuple(shp) + src.shape[rank_m:], src.dtype)
    for m in itertools.product(*[range(s) for s in src.shape[:rank_m]]):
        p = tuple(f(*m))
        if all(0 <= p[k] < shp[k] for k in range(len(shp))):
            out[p] += src[m]
    return out


def run_cases(host, exact_scatter):
    for ssh, shm, f, fi, affine in CASES:
        src = RNG.uniform(-1, 1, ssh)
        v = host.concrete(src)
        g = v.sgather(shm, f)
        want = brute_gather(src, shm, fi)
        assert np.array_equal(g.numpy(), want), (ssh, shm)
        n_ix = len(fi(*[0] * len(shm)))
        data = RNG.uniform(-1, 1, tuple(shm) + ssh[n_ix:])
        s = host.concrete(data).sscatter(len(shm), ssh[:n_ix], f)
        wants = brute_scatter(data, len(shm), ssh[:n_ix], fi)
        assert s.shape == wants.shape
        assert np.allclose(s.numpy(), wants, rtol=1e-12, atol=1e-13), (ssh, shm)
        ix = f(*host.ix_space(shm)) if shm else f()
        assert all((not isinstance(x, H.IxV)) or x.is_affine == affine or x.is_affine for x in ix)
        # integer data: scatter sums are exact
        idata = RNG.integers(-9, 9, tuple(shm) + ssh[n_ix:])
        si = host.concrete(idata).sscatter(len(shm), ssh[:n_ix], f)
        assert np.array_equal(si.numpy(), brute_scatter(idata, len(shm), ssh[:n_ix], fi))


def test_gather_scatter_index_functions_cpu(host_cpu):
    run_cases(host_cpu, True)


def test_affine_gather_is_a_view(host_cpu):
    """A gather with an affine, in-bounds index function moves no data: the
    result is a strided view of the source (here checked through its values and
    through the index function's classification)."""
    src = np.arange(60.0).reshape(10, 6)
    v = host_cpu.concrete(src)
    i, k = host_cpu.ix_space((6, 4))
    assert (i + k).is_affine and (2 * i + 3).is_affine and not (i * k).is_affine
    g = v.sgather((6, 4), lambda i, k: [i + k])
    assert np.array_equal(g.numpy(), np.lib.stride_tricks.sliding_window_view(src, 4, axis=0)[:6].transpose(0, 2, 1))
    # a lookup in a constant table that is affine in its indices folds to an affine form
    tbl = host_cpu.concrete(np.arange(14, dtype=np.int64).reshape(7, 2))
    i, k = host_cpu.ix_space((7, 2))
    assert tbl.sindex0([i, k]).is_affine
    other = host_cpu.concrete(np.array([[0, 1], [2, 3], [4, 6]], np.int64))
    i, k = host_cpu.ix_space((3, 2))
    assert not other.sindex0([i, k]).is_affine


def data_dependent_indices(host):
    """relu mask and max-pool as the reference's simplified programs express them
    (test/simplified/TestMnistPP.hs:735): gather from [0, 1] by
    ifH (0 <=. negate x) 0 1, and gather at kargMax of a partial index."""
    x = RNG.uniform(-1, 1, (4, 5))
    x[1, 2] = 0.0                                            # 0 <=. negate 0: the mask is 0 at zero
    t = host.concrete(x)
    table = host.concrete(np.array([0.0, 1.0]))
    zero = lambda: H.IxV.const(host, (4, 5), 0.0, capi.F64)  # noqa: E731
    mask = table.sgather((4, 5), lambda i, j: [H.ifH(zero().leq(-t.sindex0([i, j]), capi.F64), 0, 1)])
    assert np.array_equal(mask.numpy(), np.where(0.0 <= -x, 0.0, 1.0))
    u = RNG.uniform(-1, 1, (3, 4, 6))
    u[2, 1, 3] = u[2, 1, 5] = 2.0                            # a tie: the first of the equal maxima is taken
    tu = host.concrete(u)
    mx = tu.sgather((3, 4), lambda i, j: [i, j, tu.kargMax([i, j])])
    assert np.array_equal(mx.numpy(), u.max(axis=-1))
    mn = tu.sgather((3, 4), lambda i, j: [i, j, tu.kargMin([i, j])])
    assert np.array_equal(mn.numpy(), u.min(axis=-1))
    # the VJP of the mask gather is a scatter with the same index function (DeltaEval.hs:556-562)
    cot = RNG.uniform(-1, 1, (4, 5))
    back = host.concrete(cot).sscatter(2, [2], lambda i, j: [H.ifH(zero().leq(-t.sindex0([i, j]), capi.F64), 0, 1)])
    want = np.array([cot[0.0 <= -x].sum(), cot[~(0.0 <= -x)].sum()])
    assert np.allclose(back.numpy(), want, rtol=1e-12, atol=1e-13)


def test_data_dependent_indices_cpu(host_cpu):
    data_dependent_indices(host_cpu)


@pytest.mark.gpu
def test_data_dependent_indices_gpu(host_gpu):
    data_dependent_indices(host_gpu)


def convert_tensor_is_a_checked_identity(host_cpu):
    """ConvertTensor on this carrier (ConvertTensor.hs:25-236, OpsConcrete.hs:777-904):
    arrays carry their shape at run time, so kfromS / sfromK / sfromR / rfromS / sfromX /
    xfromS / nest / unnest hand back the same data and the same dual part; the shape
    the shaped type names is checked as the reference checks it."""
    x = RNG.uniform(-1, 1, (3, 4, 5))
    p = host_cpu.param(x)
    r = p.tconvert("rfromS")                                 # forget the static shape ...
    s = r.tconvert("sfromR", (3, 4, 5))                      # ... and name it again
    assert np.array_equal(s.numpy(), x) and s.shape == (3, 4, 5)
    with pytest.raises(capi.HgpuError) as e:
        r.tconvert("sfromR", (3, 5, 4))
    assert e.value.code == 1
    assert np.array_equal(p.tconvert("xfromS").tconvert("sfromX", (3, 4, 5)).numpy(), x)
    # scalars: a rank-0 array either way
    k = (s * s).ssum0().tconvert("kfromS")
    assert k.shape == () and abs(float(k.numpy()) - float((x * x).sum())) <= 1e-12
    with pytest.raises(capi.HgpuError):
        s.tconvert("kfromS")
    # nest / unnest: the outer dims lead the shape; the data does not move
    n = s.tconvert("nest", (3, 4))
    assert np.array_equal(n.tconvert("unnest", (3,)).numpy(), x)
    with pytest.raises(capi.HgpuError):
        s.tconvert("nest", (4,))
    # the dual part flows through: d/dx sum (sfromR (rfromS x))^2 = 2 x
    host_cpu.tape_reset()
    q = host_cpu.param(x).as_input()
    y = q.tconvert("rfromS").tconvert("sfromR", (3, 4, 5))
    loss = (y * y).ssum0().tconvert("kfromS").tconvert("sfromK")
    (g,) = host_cpu.grad(loss, [q])
    assert np.allclose(g.numpy(), 2 * x, rtol=1e-13, atol=0)


def test_convert_tensor_is_a_checked_identity(host_cpu):
    convert_tensor_is_a_checked_identity(host_cpu)


@pytest.mark.gpu
def test_convert_tensor_is_a_checked_identity_gpu(host_gpu):
    convert_tensor_is_a_checked_identity(host_gpu)


def test_adjoint_law_cpu(host_cpu):
    """sdot0 (sgather x f) y == sdot0 x (sscatter y f) (bench/ConvVjpBench.hs:564-584)."""
    x = host_cpu.concrete(RNG.uniform(-1, 1, (12, 12, 3)))
    f = lambda i, p, j, q: [i + p, j + q]  # noqa: E731
    g = x.sgather((12, 3, 12, 3), f)
    y = host_cpu.concrete(RNG.uniform(-1, 1, g.shape))
    s = y.sscatter(4, (12, 12), f)
    assert np.isclose(float(g.sdot0(y).numpy()), float(x.sdot0(s).numpy()), rtol=1e-12)


def test_gradient_through_gather_matches_reference_kat(host_cpu):
    """gatherNested1-style known answer: the gradient of a sum of gathered rows
    counts how often each source element is read (cf. the expected arrays of
    test/simplified/TestGatherSimplified.hs:154-159, which are such counts)."""
    t = host_cpu.param(RNG.uniform(-1, 1, (7, 2)))
    g = t.sgather((4, 2), lambda i, k: [i + k])          # rows 0..4, overlapping
    grad = host_cpu.grad(g.ssum0(), [t])[0].numpy()
    want = np.zeros((7, 2))
    for i in range(4):
        for k in range(2):
            want[i + k] += 1
    assert np.array_equal(grad, want)


@pytest.mark.gpu
def test_gather_scatter_index_functions_gpu(host_gpu):
    run_cases(host_gpu, False)


@pytest.mark.gpu
def test_conv_vjp_chain_gpu_matches_cpu(host_gpu, host_cpu):
    """Window gather -> contraction -> gradient: on the device the input gradient
    is ONE contraction over skewed views (no patch gradient in memory, no
    atomics); it must agree with the checker's literal scatter."""
    a = RNG.uniform(-1, 1, (3, 2, 9, 8))
    k = RNG.uniform(-1, 1, (4, 2, 3, 3))
    res = []
    for host in (host_gpu, host_cpu):
        W = pkg.workloads
        arr, ker = host.param(a), host.param(k)
        out = W.conv2dPreservingS(ker, arr)
        loss = (out * out).ssum0()
        ga, gk = host.grad(loss, [arr, ker])
        res.append((out.numpy(), ga.numpy(), gk.numpy()))
    for g, c in zip(*res):
        assert np.allclose(g, c, rtol=1e-10, atol=1e-12)


def append_slice_program(host, a, b, c):
    """Stacked state of an unrolled recurrence in miniature: appends, slices that
    hit piece boundaries and slices that straddle them, a slice used twice."""
    pa, pb, pc = host.param(a), host.param(b), host.param(c)
    s = pa.sappend(pb).sappend(pc)                     # [3+4+2, 5]
    top, mid, low = s.sslice(0, 3), s.sslice(3, 4), s.sslice(7, 2)
    straddle = s.sslice(2, 4)                          # rows of a and b
    inner = s.sslice(4, 2)                             # inside b
    t = top.op1("sin").sappend(mid * mid)              # [7, 5]
    loss = (t.sslice(1, 5) * straddle.sappend(inner).sslice(0, 5)).ssum0() + (low * low).ssum0() + (s * s).ssum0() * host.srepl((), 0.5, pa.dtype)
    grads = host.grad(loss, [pa, pb, pc])
    return s.numpy(), loss.numpy(), [g.numpy() for g in grads]


def append_slice_numpy(a, b, c):
    s = np.concatenate([a, b, c])
    t = np.concatenate([np.sin(a), b * b])
    u = np.concatenate([s[2:6], s[4:6]])[0:5]
    loss = (t[1:6] * u).sum() + (c * c).sum() + 0.5 * (s * s).sum()
    # gradient by hand
    gs = s.copy()                                      # from 0.5 * sum s^2
    gt = np.zeros_like(t)
    gt[1:6] = u
    gu = np.zeros((6, 5))
    gu[0:5] = t[1:6]
    gs[2:6] += gu[0:4]
    gs[4:6] += gu[4:6]
    ga = gs[0:3] + gt[0:3] * np.cos(a)
    gb = gs[3:7] + gt[3:7] * 2 * b
    gc = gs[7:9] + 2 * c
    return s, loss, [ga, gb, gc]


def check_append_slice(host):
    a, b, c = RNG.uniform(-1, 1, (3, 5)), RNG.uniform(-1, 1, (4, 5)), RNG.uniform(-1, 1, (2, 5))
    s, loss, grads = append_slice_program(host, a, b, c)
    ws, wl, wg = append_slice_numpy(a, b, c)
    assert np.array_equal(s, ws)
    assert np.isclose(float(loss), wl, rtol=1e-12)
    for g, w in zip(grads, wg):
        assert np.allclose(g, w, rtol=1e-12, atol=1e-14)
    # the same with deferred evaluation off: every append and zero-extension is written out
    host.set_fusion(False)
    try:
        s2, loss2, grads2 = append_slice_program(host, a, b, c)
    finally:
        host.set_fusion(True)
    assert np.array_equal(s2, s)
    assert np.isclose(float(loss2), float(loss), rtol=1e-12)
    for g, w in zip(grads2, grads):
        assert np.allclose(g, w, rtol=1e-12, atol=1e-14)


def test_append_slice_pieces_cpu(host_cpu):
    check_append_slice(host_cpu)


@pytest.mark.gpu
def test_append_slice_pieces_gpu(host_gpu):
    check_append_slice(host_gpu)


@pytest.mark.gpu
def test_pooling_adjoint_stays_pending_gpu(host_gpu, host_cpu):
    """relu -> 2x2 max pooling -> a cotangent that fans out: on the device the
    adjoint of taking the windows (out[2i+p, 2j+q] = src[i, j, p, q]) is no pass
    of its own, the expression stays pending over the refined index space and is
    written out once; the checker scatters literally.  Shapes with odd channel
    counts and a second use of the pooled cotangent."""
    W = pkg.workloads
    x = RNG.uniform(-1, 1, (5, 3, 8, 12))
    b = RNG.uniform(-0.5, 0.5, (3,))
    w = RNG.uniform(-1, 1, (5, 3, 4, 6))
    res = []
    for host in (host_gpu, host_cpu):
        px, pb = host.param(x), host.param(b)
        y = px + pb.sreplicateN([5, 8, 12]).stranspose([0, 3, 1, 2])
        r = W.reluS(y)
        pooled = W.maxPool2dUnpaddedS(r)                          # [5, 3, 4, 6]
        loss = (pooled * host.concrete(w)).ssum0() + (pooled * pooled).ssum0() + (r.stranspose([1, 0, 2, 3]) * r.stranspose([1, 0, 2, 3])).ssum0()
        gx, gb = host.grad(loss, [px, pb])
        res.append((loss.numpy(), gx.numpy(), gb.numpy()))
        host.tape_reset()
    for got, want in zip(res[0], res[1]):
        assert np.allclose(got, want, rtol=1e-12, atol=1e-13)


def value_at_own_extremum(host):
    """`sindex0 t [kargMin t]` on a flat tensor (sminimum of the reference's soft-max loss,
    CommonShapedOps.hs:33-44) equals the minimum, with ties and with the index reused on
    another tensor (where it has to be a real gather)."""
    for dt in (np.float64, np.float32):
        v = RNG.uniform(-3, 3, 1000).astype(dt)
        v[[17, 400]] = v.min() - 1          # a tie: the first position counts
        w = RNG.uniform(-3, 3, 1000).astype(dt)
        t, o = host.concrete(v), host.concrete(w)
        for arg_of, pick in ((lambda x: x.sargMin(), np.argmin), (lambda x: x.sargMax(), np.argmax)):
            arg = arg_of(t)
            assert int(arg.numpy()) == int(pick(v))
            assert t.sgather((), lambda: [arg.lift(())]).numpy() == v[pick(v)]
            assert o.sgather((), lambda: [arg.lift(())]).numpy() == w[pick(v)]


def test_value_at_own_extremum_cpu(host_cpu):
    value_at_own_extremum(host_cpu)


@pytest.mark.gpu
def test_value_at_own_extremum_gpu(host_gpu):
    value_at_own_extremum(host_gpu)


def ranked_and_mixed_methods_are_the_shaped_ones(host):
    """Ops.hs:297-1255 gives every operation a ranked (tr*), a shaped (ts*) and a
    mixed (tx*) method; the ABI takes shapes at run time, so all three bind to
    one entry point.  The twins give the same arrays, through a gather with an
    index function and a scatter too."""
    rng = np.random.default_rng(5)
    a, b = rng.standard_normal((4, 6)), rng.standard_normal((6, 3))
    A, B = host.concrete(a), host.concrete(b)
    want = a @ b
    for pre in ("s", "r", "x"):
        mm = getattr(A, pre + "matmul2")(B)
        assert np.allclose(mm.numpy(), want, rtol=0, atol=1e-12)
        assert np.array_equal(getattr(A, pre + "slice")(1, 2).numpy(), a[1:3])
        assert np.array_equal(getattr(getattr(A, pre + "replicate")(2), pre + "sum")().numpy(), 2 * a)
        assert np.array_equal(getattr(A, pre + "reshape")([6, 4]).numpy(), a.reshape(6, 4))
        g = getattr(A, pre + "gather")((3,), lambda i: [i + 1, i * 2])
        assert np.array_equal(g.numpy(), np.array([a[1, 0], a[2, 2], a[3, 4]]))
        sc = getattr(g, pre + "scatter")(1, (5,), lambda i: [i * 2])
        assert np.array_equal(sc.numpy(), np.array([a[1, 0], 0, a[2, 2], 0, a[3, 4]]))
    assert np.array_equal(A.rtr().numpy(), a.T) and np.array_equal(A.rmaxIndex().numpy(), a.argmax(-1))
    assert np.array_equal(host.rrepl((2, 2), 1.5).numpy(), np.full((2, 2), 1.5))


def test_ranked_and_mixed_methods_are_the_shaped_ones(host_cpu):
    ranked_and_mixed_methods_are_the_shaped_ones(host_cpu)


@pytest.mark.gpu
def test_ranked_and_mixed_methods_are_the_shaped_ones_gpu(host_gpu):
    ranked_and_mixed_methods_are_the_shaped_ones(host_gpu)
