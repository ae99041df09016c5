"""A gradient program recorded once and launched many times (GPU only).

Every replay must reproduce the eager result bit for bit: it launches the very
same kernels on the very same arrays.  Eager work runs between the replays, so
a block of memory that leaked out of the recording's pool would show up as a
changed result.
"""
import numpy as np
import pytest

from conftest import capi, pkg
from test_workloads import MEDIUM, SMALL

H, W = pkg.hostapi, pkg.workloads

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def host():
    return H.Host()


def eager(host, wl, ps, ds):
    loss, grads = wl.gradient(host, ps, ds)
    return loss.numpy(), [g.numpy() for g in grads]


@pytest.mark.parametrize("name,table", [("c0", SMALL), ("c1", MEDIUM), ("c3", SMALL), ("c3", MEDIUM), ("c4", SMALL), ("c4", MEDIUM), ("c2", MEDIUM)])
def test_replays_match_eager(host, name, table):
    mk, kw = table[name]
    wl = mk(**kw)
    ps, ds = wl.upload(host)
    want_loss, want_grads = eager(host, wl, ps, ds)          # also the warm-up run
    graph, (loss, grads) = host.capture(lambda: wl.gradient(host, ps, ds))
    other = mk(**kw)
    ops, ods = other.upload(host)
    try:
        for replay in range(3):
            graph.launch()
            host.sync()
            assert np.array_equal(loss.numpy(), want_loss), (name, replay)
            for g, w in zip(grads, want_grads):
                assert np.array_equal(g.numpy(), w), (name, replay)
            eager(host, other, ops, ods)                      # unrelated eager work between replays
        # new contents for the inputs: the replay follows them
        new_params = [np.ascontiguousarray(p * 0.5) for p in wl.params]
        for p, x in zip(ps, new_params):
            p.overwrite(x)
        graph.launch()
        host.sync()
        got_loss, got_grads = loss.numpy(), [g.numpy() for g in grads]
        fresh = [host.param(x) for x in new_params]
        ref_loss, ref_grads = eager(host, wl, fresh, ds)
        assert np.array_equal(got_loss, ref_loss)
        for g, w in zip(got_grads, ref_grads):
            assert np.array_equal(g, w)
    finally:
        graph.free()


def test_sorted_scatter_inside_a_recording(host):
    """The general scatter-add (positions sorted by destination, runs added in order) recorded
    into a graph: its sort is a library routine, so every replay is checked against the eager
    result, with eager scatters of other sizes (which reuse the sort's workspace blocks) between
    the replays, and again after the inputs changed."""
    rng = np.random.default_rng(21)
    m, cells_n = 50000, 301
    cells = host.concrete(rng.integers(-3, cells_n + 3, m).astype(np.int64))
    src = host.concrete(rng.standard_normal((m, 3)))
    other_cells = host.concrete(rng.integers(0, 9, 7777).astype(np.int64))
    other_src = host.concrete(rng.standard_normal(7777))

    def program():
        return src.sscatter(1, [cells_n], lambda i: [cells.sindex0([i])])

    def numpy_scatter(c, x):
        out = np.zeros((cells_n,) + x.shape[1:])
        ok = (c >= 0) & (c < cells_n)
        np.add.at(out, c[ok], x[ok])
        return out

    want = program().numpy()
    np.testing.assert_allclose(want, numpy_scatter(cells.numpy(), src.numpy()), rtol=1e-10, atol=1e-12)
    assert host.counter("scatter_general") > 0
    graph, res = host.capture(program)
    try:
        for replay in range(3):
            graph.launch()
            host.sync()
            assert np.array_equal(res.numpy(), want), replay
            other_src.sscatter(1, [9], lambda i: [other_cells.sindex0([i])]).numpy()
        new_cells = rng.integers(0, cells_n, m).astype(np.int64)
        new_src = rng.standard_normal((m, 3))
        cells.overwrite(new_cells)
        src.overwrite(new_src)
        graph.launch()
        host.sync()
        np.testing.assert_allclose(res.numpy(), numpy_scatter(new_cells, new_src), rtol=1e-10, atol=1e-12)
        fresh = host.concrete(new_src).sscatter(1, [cells_n], lambda i: [host.concrete(new_cells).sindex0([i])])
        assert np.array_equal(res.numpy(), fresh.numpy())
    finally:
        graph.free()


def test_sums_finished_by_the_last_block_inside_a_recording(host):
    """An objective's value and its cotangent from one pass over [10, 5000] (the sums of that pass are added up
    by the block that draws the last ticket, and the counter goes back to zero in the same kernel): every replay
    against the eager result, with eager sums of other sizes between the replays."""
    rng = np.random.default_rng(33)
    u = host.concrete(rng.uniform(-2, 2, (10, 5000)))
    t = host.concrete(rng.uniform(0, 1, (10, 5000)))
    other = host.concrete(rng.uniform(-1, 1, (300, 77)))

    def program():
        e = (u - 0.5).op1("exp")
        r = e.ssum0().op1("recip")
        soft = r.sreplicate0N(u.shape) * e
        return (soft - t) * 2.0, -(soft.op1("log").sdot0(t))     # the cotangent first: its pass takes the value's sum along

    def eager():
        cot, loss = program()
        c = cot.numpy()
        return loss.numpy(), c

    want = eager()
    graph, (cot, loss) = host.capture(program)
    try:
        for replay in range(3):
            graph.launch()
            host.sync()
            assert np.array_equal(cot.numpy(), want[1]) and np.array_equal(loss.numpy(), want[0]), replay
            (other * other).ssum0().numpy()
            (other.op1("sin")).ssum0().numpy()
    finally:
        graph.free()


def test_host_calls_refused_while_recording(host):
    x = host.concrete(np.arange(6.0).reshape(2, 3))
    y = (x * x).ssum0()
    y.numpy()

    def program():
        z = (x * x).ssum0()
        with pytest.raises(capi.HgpuError) as e:
            z.numpy()                     # a read-back needs the host
        assert e.value.code == 4
        with pytest.raises(capi.HgpuError):
            host.concrete(np.ones(3))     # so does an upload
        return z

    graph, z = host.capture(program)
    graph.launch()
    host.sync()
    assert float(z.numpy()) == 55.0
    graph.free()
    # the context works as before
    assert float((x * x).ssum0().numpy()) == 55.0


def test_first_iota_of_a_length_is_refused_while_recording(host):
    """An index vector is written once and kept for later calls.  Written only
    by a recorded launch it would be read unwritten by eager code, so a length
    never asked for before is refused during a recording; after one eager run
    the recording just reads the kept vector."""
    n = 1237                                   # a length no other test asks for
    x = host.concrete(np.arange(float(n)))

    def program():
        return (x * host.siota(n, capi.F64)).ssum0()

    with pytest.raises(capi.HgpuError) as e:
        host.capture(program)
    assert e.value.code == 4
    want = program().numpy()                   # eager: the vector now exists
    graph, z = host.capture(program)
    try:
        for _ in range(2):
            graph.launch()
            host.sync()
            assert np.array_equal(z.numpy(), want)
            assert np.array_equal(host.siota(n, capi.F64).numpy(), np.arange(float(n)))
    finally:
        graph.free()
