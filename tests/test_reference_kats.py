"""Known answers held by the reference's own tests, for gather / scatter and
their transposes (test/simplified/TestGatherSimplified.hs).  The programs below
restate that file's definitions one to one; the expected gradients live in
tests/golden/gather_scatter_kats.json with the line ranges they were copied
from.  CPU: host layer on the checker.  GPU: the same on the device.
"""
import json
import os

import numpy as np
import pytest

from conftest import capi, entry, pkg

H = pkg.hostapi
KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "gather_scatter_kats.json")))


# --- the reference's definitions (rgather shm t f: out[m] = t[f m]) ---------

def gatherNested1(t):
    inner = t.sgather((4,), lambda k3: [k3])
    return inner.sgather((2,), lambda i2: [i2 + i2, i2])


def gather1(t):
    return t.sslice(0, 4).sgather((2,), lambda i2: [i2 + i2, i2])


def gatherNested02(t):
    inner = t.sgather((2,), lambda k3: [k3 + k3])
    return inner.sgather((1,), lambda i1: [i1 + i1 + i1])


def gatherNested2(t):
    inner = t.sgather((2, 3, 4), lambda k1, k2, k3: [k1 + k2 + k3])
    return inner.sgather((2, 3), lambda i1, i2: [i1, i2, i1 + i2, i1])


def gather2(t):
    return t.sgather((2, 3), lambda i1, i2: [i1 + i2 + i1 + i2, i1])


def gatherNested12(t):
    inner = t.sgather((2, 3, 4), lambda k1, k2, k3: [k1 + k2 + k3, k1])
    return inner.sgather((2,), lambda i1: [i1, i1 + i1])


def gather12(t):
    return t.sgather((2, 4), lambda i1, k3: [i1 + i1 + i1 + k3, i1])


def gatherReshape22(t):
    return t.sreshape([2, 2, 3]).sreshape([3, 1, 1, 4]).sreshape([1, 12, 1]).sreshape([3, 1, 2, 1, 1, 2]).sreshape([2, 6])


def scatterNested1(t):
    inner = t.sscatter(1, (7,), lambda k3: [k3])
    return inner.sscatter(2, (2,), lambda i1, i2: [i2.quotH(1 + i1)])


def scatter1(t):
    return t.sscatter(2, (2,), lambda i1, i2: [(i2 + 2 * i1).minH(1)])


def scatterNested2(t):
    inner = t.sscatter(1, (2, 3, 4), lambda k1: [k1.minH(1), k1.minH(2), k1.minH(3)])
    return inner.sscatter(4, (2, 3), lambda i1, i2, _i3, i4: [(i1 + i2).minH(1), (i4 + i1).minH(2)])


def scatter2(t):
    return t.sscatter(2, (2, 3), lambda i1, i2: [(i1 + i2 + i1 + i2).minH(1), i1.minH(2)])


def scatterNested12(t):
    inner = t.sscatter(2, (2, 3, 4), lambda k1, k2: [k1.minH(1), (k2 + k1).minH(2), k1.minH(3)])
    return inner.sscatter(2, (2,), lambda i1, _i2: [(i1 + i1).minH(1)])


def scatter12(t):
    return t.sscatter(2, (2, 4), lambda i1, k3: [(i1 + i1 + i1 + k3).minH(1), i1.minH(3)])


def build_if(host, f, k=5):
    """rbuild1 k (\\i -> ifH (i >. 2) (f t) (t ! [i]))"""
    return lambda t: host.sbuild1(k, lambda i: f(t) if i > 2 else t.sindex([i]))


def build_scaled(host, f, shape, k=4):
    """rbuild1 k (\\i -> f (t * rreplicate0N shape (fromIndex i)))"""
    return lambda t: host.sbuild1(k, lambda i: f(t * host.srepl(shape, float(i))))


def build12(host, f):
    """rindex (rbuild1 5 (\\i -> ifH (i >. 2) (f t) (rtranspose [1,0] $ rreplicate 4 $ t ! [i]))) [1]"""
    return lambda t: host.sbuild1(5, lambda i: f(t) if i > 2 else t.sindex([i]).sreplicate(4).str_()).sindex([1])


def programs(host):
    return {
        "gatherNested1": gatherNested1, "gather1": gather1, "gatherNested02": gatherNested02,
        "gatherNested2": gatherNested2, "gather2": gather2, "gatherNested12": gatherNested12, "gather12": gather12,
        "gatherReshape22": gatherReshape22, "scatterNested1": scatterNested1, "scatter1": scatter1,
        "gatherNestedBuild1": build_if(host, gatherNested1), "gatherBuild1": build_if(host, gather1),
        "scatterNestedBuild1": build_if(host, scatterNested1), "scatterBuild1": build_if(host, scatter1),
        "gatherNestedBuild2": build_scaled(host, gatherNested2, [7, 2]),
        "gatherReshapeBuild22": build_scaled(host, gatherReshape22, [6, 2]),
        "gatherBuild12": build12(host, gather12),
        "scatterNested2": scatterNested2, "scatter2": scatter2, "scatterNested12": scatterNested12, "scatter12": scatter12,
        "scatterNestedBuild2": build_scaled(host, scatterNested2, [7, 2]), "scatterBuild2": build_scaled(host, scatter2, [7, 2]),
        "scatterNestedBuild12": build12(host, scatterNested12), "scatterBuild12": build12(host, scatter12),
    }


def check_all(host):
    progs = programs(host)
    for name, f in progs.items():
        kat = KATS[name]
        x = np.array(kat["input"], dtype=np.float64)
        t = host.param(x)
        host.tape_reset()
        t = t.as_input()
        grad = host.grad(f(t).ssum0(), [t])[0].numpy()
        want = np.array(kat["expected"]).reshape(x.shape)
        assert np.allclose(grad, want, rtol=0, atol=1e-10), (name, grad.ravel().tolist())
    # value equalities of testGatherSimp1/2/12 on the explicit input
    vals = np.array(KATS["value_chain_input"], dtype=np.float64).reshape(7, 2)
    v = host.concrete(vals)
    assert np.array_equal(gatherNested1(v).numpy(), gather1(v).numpy())
    assert np.array_equal(gatherNested2(v).numpy(), gather2(v).numpy())
    assert np.array_equal(gatherNested12(v).numpy(), gather12(v).numpy())
    assert np.array_equal(gatherNested1(v).numpy(), np.array([vals[0, 0], vals[2, 1]]))


def overleaf_and_piecewise(host):
    """test/simplified/TestAdaptorSimplified.hs: overleaf v = rsum (rbuild [50] (\\[i] -> v ! [i `remH` width v]))
    (:503-517: positions 0..21 are read twice, 22..27 once; one position read 50 times) and the
    piecewise linear functions through ifH on the argument (:462-468, :482-488)."""
    def overleaf(v):
        return v.sgather((50,), lambda i: [i.remH(v.shape[0])]).ssum0()
    for x, want in [(np.arange(28.0), [2.0] * 22 + [1.0] * 6), (np.array([27.0]), [50.0])]:
        host.tape_reset()
        t = host.param(x).as_input()
        g = host.grad(overleaf(t), [t])[0].numpy()
        assert np.allclose(g, want, rtol=0, atol=1e-10)
    two, five = host.srepl([], 2.0), host.srepl([], 5.0)
    for x0, f, want in [(42.0, lambda x: (x * 0.0).lt(x).select(two * x, five * x), 2.0),
                        (-42.0, lambda x: (x * 0.0).lt(x).select(two, five) * x, 5.0)]:
        host.tape_reset()
        t = host.param(np.array(x0)).as_input()
        g = host.grad(f(t), [t])[0].numpy()
        assert abs(float(g) - want) <= 1e-10


def test_reference_kats_on_checker():
    host = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    check_all(host)
    overleaf_and_piecewise(host)


@pytest.mark.gpu
def test_reference_kats_on_device():
    host = H.Host()
    check_all(host)
    overleaf_and_piecewise(host)


def conv_vjp_constants(host):
    """test_conv2dPreservingVjp_dInp / _dKrn (test/simplified/TestConvQuickCheck.hs:351-387):
    constant arrays A = 1.1 [5,2,4,8], K = -2.2 / 2.2 [7,2,1,3], cotangent B = -3.3
    [5,7,4,8]; the reference compares against its handwritten derivatives
    (ibid. :290-349), which on constants are counts of in-bounds window
    positions: the window extends FORWARD from each output position, so the
    input's cotangent at column w collects min(w + 1, 3) kernel taps and the
    kernel's cotangent at tap q collects 8 - q columns."""
    W = pkg.workloads
    A = np.full((5, 2, 4, 8), 1.1)
    B = host.concrete(np.full((5, 7, 4, 8), -3.3))
    for kval in (-2.2, 2.2):
        K = np.full((7, 2, 1, 3), kval)
        host.tape_reset()
        a, k = host.param(A).as_input(), host.param(K).as_input()
        y = W.conv2dPreservingS(k, a)
        assert np.allclose(y.numpy()[0, 0, 0], 2 * 1.1 * kval * np.minimum(8 - np.arange(8), 3), atol=1e-12)
        d_inp, d_krn = [g.numpy() for g in host.grad(y.sdot0(B), [a, k])]
        want_inp = np.broadcast_to(-3.3 * kval * 7 * np.minimum(np.arange(8) + 1, 3), (5, 2, 4, 8))
        want_krn = np.broadcast_to(-3.3 * 1.1 * 5 * 4 * (8 - np.arange(3)), (7, 2, 1, 3))
        assert np.allclose(d_inp, want_inp, rtol=0, atol=1e-7)
        assert np.allclose(d_krn, want_krn, rtol=0, atol=1e-7)


def test_conv_vjp_constants_on_checker():
    conv_vjp_constants(H.Host(capi.Lib(entry.ORACLE_LIB, "horc_")))


@pytest.mark.gpu
def test_conv_vjp_constants_on_device():
    conv_vjp_constants(H.Host())
