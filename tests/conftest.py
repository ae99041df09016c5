import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

pkg = entry.load_package()
capi = pkg.capi


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X")


@pytest.fixture(scope="session")
def oracle():
    """Context of the CPU checker (oracle/_build/liboracle.so)."""
    if not os.path.exists(entry.ORACLE_LIB):
        entry._make(os.path.join(ROOT, "oracle"))
    return capi.Lib(entry.ORACLE_LIB, "horc_").context(0)


@pytest.fixture(scope="session")
def gpu():
    """Context of the gfx950 library on device 0; fails loudly when it is missing."""
    return capi.Lib().context(0)


class Pair:
    """The same array held by two providers; every method call goes to both."""

    def __init__(self, arrays):
        self.arrays = arrays

    def __getattr__(self, name):
        def call(*args, **kw):
            outs = []
            for i, a in enumerate(self.arrays):
                aa = [x.arrays[i] if isinstance(x, Pair) else x for x in args]
                outs.append(getattr(a, name)(*aa, **kw))
            if isinstance(outs[0], capi.Array):
                return Pair(outs)
            return outs
        return call

    @property
    def shape(self):
        return self.arrays[0].shape

    def numpy(self):
        return [a.numpy() for a in self.arrays]


class Both:
    """Two contexts driven in lockstep."""

    def __init__(self, ctxs):
        self.ctxs = ctxs

    def upload(self, x):
        return Pair([c.upload(x) for c in self.ctxs])

    def iota(self, n, dtype=capi.I64):
        return Pair([c.iota(n, dtype) for c in self.ctxs])

    def concat(self, parts):
        return Pair([c.concat([p.arrays[i] for p in parts]) for i, c in enumerate(self.ctxs)])

    def gather(self, src, ix, shm):
        return Pair([c.gather(src.arrays[i], [p.arrays[i] for p in ix], shm) for i, c in enumerate(self.ctxs)])

    def scatter_add(self, src, ix, rank_m, shp, flags=0):
        return Pair([c.scatter_add(src.arrays[i], [p.arrays[i] for p in ix], rank_m, shp, flags) for i, c in enumerate(self.ctxs)])

    def contract_sum(self, pairs, n_keep):
        return Pair([c.contract_sum([(a.arrays[i], b.arrays[i]) for a, b in pairs], n_keep) for i, c in enumerate(self.ctxs)])

    def scatter_affine(self, src, rank_m, c0, coef, shp):
        return Pair([c.scatter_affine(src.arrays[i], rank_m, c0, coef, shp) for i, c in enumerate(self.ctxs)])


def assert_same(pair, rtol=0.0, what=""):
    """Device result against the checker: bit-exact, or normwise relative `rtol`."""
    g, o = pair.numpy()
    assert g.shape == o.shape and g.dtype == o.dtype, (what, g.shape, o.shape, g.dtype, o.dtype)
    if rtol == 0.0 or g.dtype.kind in "iub":
        assert np.array_equal(g, o, equal_nan=True), what
    else:
        scale = max(float(np.max(np.abs(o))) if o.size else 0.0, 1e-300)
        err = float(np.max(np.abs(g - o))) if o.size else 0.0
        record_error(what, err / scale, rtol)
        assert err <= rtol * scale, (what, err / scale)


def record_error(what, err, tol):
    """With HORDEAD_TEST_ERRORS=<file>, every floating-point comparison appends the error it
    measured and the bound it was held to (how the tolerances written in the tests were set)."""
    path = os.environ.get("HORDEAD_TEST_ERRORS")
    if path:
        import inspect
        fr = inspect.stack()[2]
        with open(path, "a") as f:
            f.write("%s:%d\t%s\t%.3e\t%.1e\n" % (os.path.basename(fr.filename), fr.lineno, str(what)[:60], err, tol))


@pytest.fixture(scope="session")
def both(gpu, oracle):
    return Both([gpu, oracle])
