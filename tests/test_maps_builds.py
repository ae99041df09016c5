"""tkbuild / tsmap0N / tszipWith0N with scalar closures (Ops.hs:863-880, 929-941;
Concrete: one vector map, OpsConcrete.hs:671-714, 1081-1087, 1748-1759).

The closure runs ONCE, on lane values (`hh_ix_from_val` -> arithmetic ->
`hh_ix_to_val`), and its arithmetic is ordinary deferred array arithmetic.
Every case is held against numpy applying the same scalar function elementwise
(the reference's semantics: `f` at every element), on the CPU checker here and
on the device under `-m gpu`; integer results bit for bit.
"""
import numpy as np
import pytest

from conftest import capi, entry, pkg

H = pkg.hostapi
W = pkg.workloads
ifH = H.ifH
F64, F32, I64, I32 = capi.F64, capi.F32, capi.I64, capi.I32


def cpu_host(fuse):
    h = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    h.set_fusion(fuse)
    return h


@pytest.fixture(scope="module", params=[0, 1], ids=["undeferred", "deferred"])
def host_cpu(request):
    return cpu_host(request.param)


@pytest.fixture(scope="module")
def host_gpu():
    return H.Host()


def np_quot(a, b):
    """quotH of scalars: truncating, a zero divisor gives the dividend (Types.hs:394-419)."""
    q = np.where(b == 0, 0, np.abs(a) // np.where(b == 0, 1, np.abs(b))) * np.sign(a) * np.sign(b)
    return np.where(b == 0, a, q).astype(a.dtype)


def np_rem(a, b):
    return np.where(b == 0, a, a - np_quot(a, b) * b).astype(a.dtype)


def run_cases(host, rtol):
    rng = np.random.default_rng(5)
    # relu's mask, the closure of reluS (External/CommonShapedOps.hs:42-44)
    for dt, npdt in ((F64, np.float64), (F32, np.float32)):
        x = rng.uniform(-1, 1, (7, 5, 3)).astype(npdt)
        x[0, 0, 0] = 0.0
        v = host.concrete(x)
        got = v.smap0N(lambda s: ifH(s.leq(0), 0.0, 1.0, dt)).numpy()
        assert got.dtype == npdt and np.array_equal(got, np.where(x <= 0, 0, 1).astype(npdt))
        # a float closure with several operations and a transposed (strided) operand
        vt = host.concrete(x).stranspose([2, 0, 1])
        got = vt.smap0N(lambda s: (s * s + 1.5).op1("sqrt") / (2.0 - s)).numpy()
        want = np.sqrt(x * x + npdt(1.5)) / (npdt(2.0) - x)
        np.testing.assert_allclose(got, want.transpose(2, 0, 1), rtol=rtol[dt])
    # integer zipWith with quotH / remH: exact, zero divisors included
    for dt, npdt in ((I64, np.int64), (I32, np.int32)):
        a = rng.integers(-50, 50, (6, 9)).astype(npdt)
        b = rng.integers(-4, 5, (6, 9)).astype(npdt)
        va, vb = host.concrete(a), host.concrete(b)
        got = va.szipWith0N(lambda p, q: p.quotH(q) * 3 + p.remH(q), vb).numpy()
        assert got.dtype == npdt and np.array_equal(got, np_quot(a, b) * 3 + np_rem(a, b))
        got = va.szipWith0N(lambda p, q: ifH(p.lt(q), p.maxH(q), p.minH(q) - 1), vb).numpy()
        assert np.array_equal(got, np.where(a < b, np.maximum(a, b), np.minimum(a, b) - 1))
    # zipWith of two element types into a third: Bool conditions combined
    xa = rng.uniform(-1, 1, (4, 4))
    got = host.concrete(xa).szipWith0N(lambda p, q: ifH(p.leq(0.0).andB(q.lt(3).notB()), p, -p), host.concrete(a[:4, :4].astype(np.int64))).numpy()
    assert np.array_equal(got, np.where((xa <= 0) & ~(a[:4, :4] < 3), xa, -xa))
    # builds from the index alone, affine and not
    got = host.kbuild((4, 6), lambda i, j: 3 * i - j + 2).numpy()
    ii, jj = np.meshgrid(np.arange(4), np.arange(6), indexing="ij")
    assert got.dtype == np.int64 and np.array_equal(got, 3 * ii - jj + 2)
    got = host.kbuild((4, 6), lambda i, j: (i * j).remH(4).convert(F64) * 0.5).numpy()
    assert np.array_equal(got, ((ii * jj) % 4) * 0.5)
    got = host.kbuild1(5, lambda i: ifH(i.leq(2), i, 10 - i)).numpy()
    assert np.array_equal(got, np.where(np.arange(5) <= 2, np.arange(5), 10 - np.arange(5)))
    got = host.kbuild((2, 3), lambda i, j: 7.5, F64).numpy()
    assert np.array_equal(got, np.full((2, 3), 7.5))
    # a build that reads data: kbuild (\[i, j] -> t `sindex0` [j, i] * 2) is the doubled transpose
    t = host.concrete(xa)
    got = host.kbuild((4, 4), lambda i, j: t.sindex0([j, i]) * 2.0).numpy()
    assert np.array_equal(got, 2.0 * xa.T)
    # the host loop that remains for array-valued closures (tbuildS, OpsConcrete.hs:1776-1789)
    got = host.sbuild((2, 3), lambda i, j: t.sindex([i]) * float(j)).numpy()
    assert np.array_equal(got, np.stack([np.stack([xa[i] * j for j in range(3)]) for i in range(2)]))


def test_maps_and_builds_on_the_checker(host_cpu):
    run_cases(host_cpu, {F64: 1e-14, F32: 1e-6})


def relu_both_ways(host, x):
    """reluS through smap0N and through compare + select: values and gradients."""
    outs = []
    for relu in (W.reluS, W.reluS_select):
        host.tape_reset()
        v = host.param(x)
        y = relu(v * v - 0.3)
        loss = (y * y).ssum0()
        outs.append((y.numpy(), host.grad(loss, [v])[0].numpy()))
    return outs


def test_relu_by_map_is_relu_by_select_on_the_checker(host_cpu):
    x = np.random.default_rng(3).uniform(-1, 1, (6, 11))
    (y0, g0), (y1, g1) = relu_both_ways(host_cpu, x)
    assert np.array_equal(y0, y1) and np.array_equal(g0, g1)
    t = x * x - 0.3
    np.testing.assert_allclose(y0, np.where(t > 0, t, 0), rtol=1e-14)
    np.testing.assert_allclose(g0, 2 * np.where(t > 0, t, 0) * 2 * x, rtol=1e-13)


@pytest.mark.gpu
def test_maps_and_builds_on_the_device(host_gpu):
    run_cases(host_gpu, {F64: 1e-13, F32: 2e-6})


@pytest.mark.gpu
def test_relu_by_map_is_relu_by_select_on_the_device(host_gpu):
    for dt in (np.float64, np.float32):
        x = np.random.default_rng(3).uniform(-1, 1, (96, 301)).astype(dt)
        (y0, g0), (y1, g1) = relu_both_ways(host_gpu, x)
        assert np.array_equal(y0, y1) and np.array_equal(g0, g1)


@pytest.mark.gpu
@pytest.mark.parametrize("name,size", [("c2", dict(batch=96)), ("c2", dict(batch=1024)), ("c3", dict(batch=8)), ("c3", dict(batch=64))])
def test_workload_gradients_do_not_depend_on_how_relu_is_written(host_gpu, name, size, monkeypatch):
    """reluS with the reference's smap0N closure against the compare + select form: bit for bit."""
    res = []
    for relu in (W.reluS, W.reluS_select):
        monkeypatch.setattr(W, "reluS", relu)
        wl = W.CONFIGS[name](**size)
        ps, ds = wl.upload(host_gpu)
        loss, grads = wl.gradient(host_gpu, ps, ds)
        res.append([loss.numpy()] + [g.numpy() for g in grads])
    for a, b in zip(*res):
        assert np.array_equal(a, b)


@pytest.mark.gpu
def test_a_large_map_is_one_launch(host_gpu):
    """16.8 M elements through a three-operation closure: one fused pass, nothing per element."""
    import bench
    n = 4096
    x = np.random.default_rng(9).uniform(-2, 2, (n, n))
    v = host_gpu.concrete(x)
    actx = bench.array_ctx(capi, host_gpu)
    host_gpu.sync()
    actx.profile(1)
    y = v.smap0N(lambda s: ifH(s.leq(0.0), s * 0.01, s.op1("exp") - 1.0))
    host_gpu.check(host_gpu.dll.hh_force(host_gpu.h, y.h))
    host_gpu.sync()
    rep = actx.profile_report()
    actx.profile(0)
    launches = {k: v[0] for k, v in rep.items() if v[0]}
    assert sum(launches.values()) == 1 and list(launches)[0].startswith("fused_map"), launches
    got = y.numpy()
    np.testing.assert_allclose(got, np.where(x <= 0, x * 0.01, np.exp(x) - 1.0), rtol=1e-14, atol=1e-15)   # exp x - 1 cancels near 0
