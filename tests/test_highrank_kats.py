"""Known answers of the reference's high-rank tests
(test/simplified/TestHighRankSimplified.hs) on its fixed inputs t16 / t128
(test/tool/CrossTesting.hs:457-467): the elementwise objective
foo (x, y, z) = atan2H z w + z * w, w = x * sin y in fp32 (testFoo, epsilon 1e-3)
and fp64 (testFooD, 1e-10), two build1 programs (testFooBuild0,
testFooBuildOut), and the gradients of conv2dPreserving with one argument
fixed to t16b / t128b / t128c (test/simplified/TestConvSimplified.hs:287-455:
conv2dB* fixes the kernel, conv2dC* the image; kernels larger than the image
included).  The literals live in tests/golden/highrank_kats.json
(written by tests/golden/make_highrank_kats.py).  CPU: host layer on the
checker.  GPU: the same on the device.
"""
import json
import os

import numpy as np
import pytest

from conftest import capi, entry, pkg

H = pkg.hostapi
KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "highrank_kats.json")))


def fixed(name, dtype):
    t = KATS[name]
    return np.array(t["values"], dtype=dtype).reshape(t["shape"])


def foo(x, y, z):
    w = x * y.op1("sin")
    return z.atan2H(w) + z * w


def foo_gradients(host, kat):
    dt = np.float32 if kat["dtype"] == "f32" else np.float64
    shape = KATS[[i for i in kat["inputs"] if isinstance(i, str)][0]]["shape"]
    arrays = [fixed(i, dt) if isinstance(i, str) else np.full(shape, i, dtype=dt) for i in kat["inputs"]]
    host.tape_reset()
    ins = [host.param(a).as_input() for a in arrays]
    grads = [g.numpy() for g in host.grad(foo(*ins).ssum0(), ins)]
    for g, want in zip(grads, kat["expected"]):
        want = np.array(want).reshape(shape)
        assert g.dtype == dt and g.shape == want.shape
        assert np.all(np.abs(g - want) <= kat["epsilon"] * np.maximum(1.0, np.abs(want))), float(np.max(np.abs(g - want)))


def check_all(host):
    foo_gradients(host, KATS["testFoo"])
    foo_gradients(host, KATS["testFooD"])
    t16 = fixed("t16", np.float64)
    # fooBuild0 v = rbuild1 2 (const (rsum v))                               (:133-143)
    host.tape_reset()
    v = host.param(t16).as_input()
    g = host.grad(host.sbuild1(2, lambda _i: v.ssum()).ssum0(), [v])[0].numpy()
    assert np.allclose(g.ravel(), KATS["testFooBuild0"]["expected"], rtol=0, atol=1e-10)
    # fooBuildOut v = rbuild1 2 (\ix -> ifH (ix ==. 0) (rindex v [ix + 1]) (rsum v))   (:145-158)
    host.tape_reset()
    v = host.param(t16).as_input()
    out = host.sbuild1(2, lambda i: v.sindex([i + 1]) if i == 0 else v.ssum())
    g = host.grad(out.ssum0(), [v])[0].numpy()
    assert np.allclose(g.ravel(), KATS["testFooBuildOut"]["expected"], rtol=0, atol=1e-10)


RELU_INPUT = [1.1, -2.2, 0, 4.4, 5.5, 6.6, 7.7, 8.8, -9.9, -10, 11, 12]          # [3, 4]
RELU_MASK = [1.0, 0.0, 0.0, 1.0, 1.0, 1.0, 1.0, 1.0, 0.0, 0.0, 1.0, 1.0]


def relu_kats(host):
    """test/simplified/TestAdaptorSimplified.hs: testReluSimpler (:1247-1251), testReluMax
    (:1408-1412) -- the derivative at 0 is 0 for both forms -- and testReluSimpler3 /
    testReluMax3 (:1300-1308, :1451-1459): relu (t * replicate r) at r = 7."""
    W = pkg.workloads
    x = np.array(RELU_INPUT).reshape(3, 4)
    relu_max = lambda v: host.srepl(v.shape, 0.0).op2("max", v)         # rmap0N (maxH 0)
    for relu in (W.reluS, relu_max):
        host.tape_reset()
        t = host.param(x).as_input()
        g = host.grad(relu(t).ssum0(), [t])[0].numpy()
        assert np.allclose(g.ravel(), RELU_MASK, rtol=0, atol=1e-10)
        host.tape_reset()
        t, r = host.param(x).as_input(), host.param(np.array(7.0)).as_input()
        gt, gr = [a.numpy() for a in host.grad(relu(t * r.sreplicate(4).sreplicate(3)).ssum0(), [t, r])]
        assert np.allclose(gt.ravel(), 7.0 * np.array(RELU_MASK), rtol=0, atol=1e-10)
        assert abs(float(gr) - 57.1) <= 1e-10


def conv_kats(host):
    W = pkg.workloads
    t128 = np.array(KATS["t128"]["values"])
    data = {"": fixed("t16b", np.float64), "128b": t128.reshape(4, 2, 4, 4), "128c": t128.reshape(2, 2, 8, 4)}
    for name, kat in KATS["conv"].items():
        fn = kat["function"]                       # conv2dB<data>: kernel fixed; conv2dC<data>: image fixed
        held = host.concrete(data[fn[len("conv2dB"):]])
        arg = kat["argument"]
        if "fill" in arg:
            x = np.full(arg["shape"], arg["fill"])
        else:
            a, b, c = arg["enum_from_then_to"]
            x = np.arange(a, c + (b - a), b - a, dtype=np.float64).reshape(arg["shape"])
        host.tape_reset()
        v = host.param(x).as_input()
        y = W.conv2dPreservingS(held, v) if fn.startswith("conv2dB") else W.conv2dPreservingS(v, held)
        g = host.grad(y.ssum0(), [v])[0].numpy()
        want = np.array(kat["expected"]).reshape(kat["expected_shape"])
        assert g.shape == want.shape, name
        assert np.all(np.abs(g - want) <= kat["epsilon"] * np.maximum(1.0, np.abs(want))), (name, float(np.max(np.abs(g - want))))


def test_highrank_kats_on_checker():
    host = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    check_all(host)
    conv_kats(host)
    relu_kats(host)


@pytest.mark.gpu
def test_highrank_kats_on_device():
    host = H.Host()
    check_all(host)
    conv_kats(host)
    relu_kats(host)
