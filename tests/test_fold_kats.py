"""Known answers the reference's tests hold for folds and scans over the serial
map-accumulate (test/simplified/TestRevFwdFold.hs): gradients at 1.1 with a
cotangent of ones.  rfold f x0 as threads x through the outermost dim of as
(tmapAccumL, OpsConcrete.hs:990-1019, via the overrides at :66-90); rscan also
keeps every intermediate x, the initial one first.  CPU: host layer on the
checker.  GPU: the same programs on the device.
"""
import numpy as np
import pytest

from conftest import capi, entry, pkg

H = pkg.hostapi


def fold(f, x0, xs):
    x = x0
    for t in range(xs.shape[0]):
        x = f(x, xs.sindex([t]))
    return x


def scan(host, f, x0, xs):
    out, x = [x0], x0
    for t in range(xs.shape[0]):
        x = f(x, xs.sindex([t]))
        out.append(x)
    return host.sfromVector(out)


def sin(t):
    return t.op1("sin")


def cases(host):
    """name -> (reference lines, shape of the input holding 1.1, program, expected gradient entry)"""
    r = lambda t, k: t.sreplicate(k)
    c42 = lambda n: host.srepl([n], 42.0)

    def f5(x, a):      # rsum (atan2H (sin (rreplicate 5 x)) (rsum (sin (rsum (rtr (rreplicate 7 a))))))
        return sin(r(x, 5)).atan2H(sin(r(a, 7).str_().ssum()).ssum()).ssum()

    def f6(x, a):      # rtr (rtr x + rreplicate 1 (rreplicate 2 a))
        return (x.str_() + r(r(a, 2), 1)).str_()

    def f7(x, _a):     # rtr (rreplicate 5 (rsum (rtr x)))
        return r(x.str_().ssum(), 5).str_()

    def f8(x, a):      # rtr (rreplicate 5 (atan2H (rsum (rtr (sin x))) (rreplicate 2 (sin (rsum (rreplicate 7 a))))))
        return r(sin(x).str_().ssum().atan2H(r(sin(r(a, 7).ssum()), 2)), 5).str_()

    s0 = []            # rank 0
    s5 = [1, 1, 1, 1, 1]
    return {
        "Fold1": ("491-496", s0, lambda a0: fold(lambda x, _a: sin(x), a0, c42(1)), 0.4535961214255773),
        "FoldB1": ("498-505", s0, lambda a0: fold(lambda _x, _a: host.srepl([], 7.0), host.srepl([], 5.0), r(a0, 1)), 0.0),
        "Fold2": ("545-550", s0, lambda a0: fold(lambda x, _a: sin(x), a0, c42(5)), 0.12389721944941383),
        "Fold3": ("558-563", s0, lambda a0: fold(lambda _x, a: sin(a), host.srepl([], 84.0), r(a0, 3)), 0.4535961214255773),
        "Fold4": ("565-570", s0, lambda a0: fold(lambda x, a: sin(x).atan2H(sin(a)), a0 * 2.0, r(a0, 3)), -0.7053476446727861),
        "Fold5": ("572-582", s0, lambda a0: fold(f5, a0 * 2.0, r(r(r(a0, 5), 2), 3)), 1.2992412552109085),
        "Fold6": ("584-592", s0, lambda a0: fold(f6, r(r(a0, 1), 2), r(a0, 2)), 6.0),
        "Fold7": ("594-601", s0, lambda a0: fold(f7, r(r(a0, 5), 2), r(a0, 2)), 250.0),
        "Fold8": ("603-613", s0, lambda a0: fold(f8, r(r(a0 * 2.0, 5), 2), r(a0, 3)), -2.200311410593445),
        "Scan1": ("934-940", s5, lambda x0: scan(host, lambda x, _a: sin(x), x0, c42(1)), 1.4535961214255773),
        "Scan2": ("949-955", s5, lambda x0: scan(host, lambda x, _a: sin(x), x0, c42(5)), 2.2207726343670955),
        "Scan3": ("957-963", s5, lambda a0: scan(host, lambda _x, a: sin(a), host.srepl(s5, 84.0), r(a0, 3)), 1.360788364276732),
        "Scan4": ("965-971", s5, lambda a0: scan(host, lambda x, a: sin(x).atan2H(sin(a)), a0 * 2.0, r(a0, 3)), -0.4458209450295252),
        "Scan6": ("985-993", s0, lambda a0: scan(host, f6, r(r(a0, 1), 2), r(a0, 2)), 12.0),
    }


def check_all(host):
    for name, (_lines, shape, prog, want) in cases(host).items():
        x = np.full(shape, 1.1)
        host.tape_reset()
        t = host.param(x).as_input()
        g = host.grad(prog(t).ssum0(), [t])[0].numpy()
        assert g.shape == tuple(shape), (name, g.shape)
        assert np.allclose(g, want, rtol=0, atol=1e-10), (name, g.ravel().tolist(), want)


def test_fold_scan_kats_on_checker():
    check_all(H.Host(capi.Lib(entry.ORACLE_LIB, "horc_")))


@pytest.mark.gpu
def test_fold_scan_kats_on_device():
    check_all(H.Host())
