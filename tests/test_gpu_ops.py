"""Parity of the gfx950 library with the CPU checker, primitive by primitive,
through the C ABI.  Data movement, integers, indices and Bool results must be
bit-exact; floating point is held to the stated normwise relative tolerance
(fp64 1e-10, fp32 1e-5 -- reductions are associated differently on the device).
"""
import numpy as np
import pytest

from conftest import Pair, assert_same, capi

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(99)
TOL = {np.dtype(np.float64): 1e-10, np.dtype(np.float32): 1e-5}
ALL = [np.float64, np.float32, np.int64, np.int32, np.int16, np.int8]


def rnd(shape, dtype):
    k = np.dtype(dtype).kind
    if k == "f":
        return RNG.uniform(-2, 2, shape).astype(dtype)
    if k == "b":
        return RNG.integers(0, 2, shape).astype(bool)
    return RNG.integers(-50, 50, shape).astype(dtype)


def random_view(both, dtype, rank=None, max_extent=7, steps=4):
    """Uploads a random dense array to both providers and derives the same random
    chain of views (transpose / slice / reverse / replicate) on each."""
    rank = rank or int(RNG.integers(1, 5))
    shape = [int(RNG.integers(1, max_extent)) for _ in range(rank)]
    p = both.upload(rnd(shape, dtype))
    for _ in range(steps):
        shape = list(p.shape)
        kind = int(RNG.integers(0, 4))
        if kind == 0 and len(shape) >= 2:
            n = int(RNG.integers(2, len(shape) + 1))
            p = p.transpose([int(i) for i in RNG.permutation(n)])
        elif kind == 1 and shape:
            d = int(RNG.integers(0, len(shape)))
            if shape[d] > 1:
                s = int(RNG.integers(0, shape[d] - 1))
                ln = int(RNG.integers(1, shape[d] - s + 1))
                p = p.slice(d, s, ln)
        elif kind == 2 and shape:
            p = p.reverse(int(RNG.integers(0, len(shape))))
        elif kind == 3 and len(shape) < 5:
            p = p.replicate([int(RNG.integers(1, 4))])
    return p


def like(both, p, dtype, view=True):
    """Another operand of p's shape: a fresh dense array, or a stride-0 broadcast."""
    shape = p.shape
    if view and len(shape) >= 1 and RNG.integers(0, 3) == 0:
        return both.upload(rnd(shape[1:], dtype)).replicate([shape[0]])
    return both.upload(rnd(shape, dtype))


def test_upload_download_views(both):
    for dt in ALL + [np.bool_]:
        for _ in range(6):
            p = random_view(both, dt)
            assert_same(p, what="view download")
            assert_same(p.materialize())
    p = both.upload(rnd((3, 0, 4), np.float64))
    assert_same(p.transpose([2, 0, 1]))
    assert_same(both.upload(np.float32(2.5)).replicate([3, 2]))


def test_reshape_view_or_copy(both, gpu):
    x = rnd((4, 6, 5), np.float64)
    p = both.upload(x)
    for shp in ([24, 5], [4, 30], [2, 2, 3, 2, 5], [120], [4, 6, 5, 1]):
        assert_same(p.reshape(shp))
    t = p.transpose([1, 0])
    for shp in ([6, 20], [24, 5], [6, 2, 2, 5]):
        assert_same(t.reshape(shp))
    # a reshape that the strides allow costs no allocation
    a = gpu.upload(x)
    n0 = gpu.mem_stats()[2]
    v = a.transpose([1, 0]).reshape([6, 2, 2, 5])
    assert gpu.mem_stats()[2] == n0 and not v.is_dense
    r = both.upload(rnd((3,), np.float64)).replicate([4])
    assert_same(r.reshape([12]))
    assert_same(r.reshape([2, 6]))
    assert_same(p.reverse(2).reshape([24, 5]))
    assert_same(p.reverse(2).reshape([4, 30]))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [np.float64, np.float32, np.int64, np.int32, np.int16, np.int8, np.bool_])
def test_pad_against_numpy(gpu, dt):
    """Zero padding (the out-of-bounds rows of an affine gather, OpsConcrete.hs:1654-1665)
    of dense, transposed, reversed, replicated, sliced and empty sources: bit-exact."""
    x = rnd((5, 4, 6, 7), dt)
    a = gpu.upload(x)
    cases = [
        (a, x, [0, 0, 2, 2], [0, 0, 2, 2]),
        (a, x, [1, 0, 0, 3], [0, 2, 1, 0]),
        (a, x, [0, 0, 0, 0], [0, 0, 0, 0]),
        (a.transpose([2, 0, 3, 1]), np.transpose(x, (2, 0, 3, 1)), [1, 0, 2, 0], [0, 1, 0, 2]),
        (a.reverse(2), x[:, :, ::-1], [0, 1, 1, 0], [2, 0, 0, 1]),
        (a.slice(3, 2, 4), x[..., 2:6], [0, 0, 0, 1], [0, 0, 0, 1]),
        (a.slice(0, 1, 0), x[1:1], [2, 0, 0, 0], [1, 0, 1, 0]),
    ]
    v = rnd((6,), dt)
    cases.append((gpu.upload(v).replicate([3]), np.broadcast_to(v, (3, 6)), [1, 2], [0, 1]))
    cases.append((gpu.upload(v).reshape([6, 1]), v.reshape(6, 1), [0, 1], [1, 1]))
    for arr, ref, lo, hi in cases:
        got = arr.pad(lo, hi).numpy()
        want = np.pad(ref, list(zip(lo, hi)))
        assert got.dtype == want.dtype and got.shape == want.shape
        assert np.array_equal(got, want), (lo, hi)
    big = rnd((300, 16, 14, 14), dt)   # the second convolution's input at a size that fills the device
    got = gpu.upload(big).pad([0, 0, 2, 2], [0, 0, 2, 2]).numpy()
    assert np.array_equal(got, np.pad(big, [(0, 0), (0, 0), (2, 2), (2, 2)]))


def test_index_pad_onehot_as_strided(both):
    p = random_view(both, np.float64, rank=4, steps=3)
    sh = p.shape
    assert_same(p.index_prefix([sh[0] - 1, 0]))
    assert_same(p.index_prefix([sh[0], 0]))       # out of bounds: zeros
    assert_same(p.index_prefix([0, -1]))
    assert_same(p.index_prefix([]))
    r = len(sh)
    assert_same(p.pad([1, 0, 2, 0, 1][:r], [0, 3, 0, 1, 2][:r]))
    assert_same(p.onehot([1, 2], [3, 4]))
    assert_same(p.onehot([3, 2], [3, 4]))          # out of bounds: all zeros
    v = both.upload(rnd((11,), np.float32))
    assert_same(v.as_strided([8, 4], [1, 1], 0))
    assert_same(v.as_strided([4, 3], [2, -1], 2))
    for a in v.arrays:
        with pytest.raises(capi.HgpuError):
            a.as_strided([9, 4], [1, 1], 0)
        with pytest.raises(capi.HgpuError):
            a.as_strided([2], [1], -1)


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_unary_float(both, dt):
    ops = ["neg", "abs", "signum", "recip", "exp", "sin", "cos", "tan", "atan", "sinh", "cosh", "tanh", "asinh"]
    for op in ops:
        p = random_view(both, dt)
        assert_same(p.ewise1(op), TOL[np.dtype(dt)], op)
    x = rnd((5, 33), dt)
    pos = both.upload(np.abs(x) + dt(0.25))
    unit = both.upload((x / dt(2.5)).astype(dt))
    for op in ("sqrt", "log"):
        assert_same(pos.ewise1(op), TOL[np.dtype(dt)], op)
    for op in ("asin", "acos", "atanh"):
        assert_same(unit.ewise1(op), TOL[np.dtype(dt)], op)
    assert_same(both.upload(np.abs(x) + dt(1.25)).ewise1("acosh"), TOL[np.dtype(dt)], "acosh")
    # dense fast path incl. a tail that is not a multiple of the vector width
    d = both.upload(rnd((1031,), dt))
    assert_same(d.ewise1("sin"), TOL[np.dtype(dt)])


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_binary_float(both, dt):
    tol = TOL[np.dtype(dt)]
    for op in ("add", "mul", "sub", "div", "atan2", "min", "max"):
        for _ in range(3):
            p = random_view(both, dt)
            q = like(both, p, dt)
            assert_same(p.ewise2(op, q), tol, op)
    x = rnd((4, 9), dt)
    px, py = both.upload(np.abs(x) + dt(0.5)), both.upload(np.abs(x[::-1]) + dt(0.5))
    assert_same(px.ewise2("pow", both.upload(x)), tol, "pow")
    assert_same(px.ewise2("logbase", py), tol, "logbase")
    # dense paths: dense*dense, dense*broadcast scalar, odd length
    a, b = both.upload(rnd((3001,), dt)), both.upload(rnd((3001,), dt))
    s = both.upload(dt(1.5)).replicate([3001])
    assert_same(a.ewise2("mul", b), tol)
    assert_same(a.ewise2("add", s), tol)
    assert_same(s.ewise2("sub", a), tol)
    assert_same(s.ewise2("mul", s), tol)


@pytest.mark.parametrize("dt", [np.int64, np.int32, np.int16, np.int8])
def test_integer_exact(both, dt):
    for op in ("add", "mul", "sub", "quot", "rem", "rem_scalar", "min", "max"):
        p = random_view(both, dt)
        q = like(both, p, dt)       # contains zeros: the divisor-0 rules apply
        assert_same(p.ewise2(op, q), 0.0, op)
    for op in ("neg", "abs", "signum"):
        assert_same(random_view(both, dt).ewise1(op), 0.0, op)
    for a in random_view(both, dt).arrays:
        with pytest.raises(capi.HgpuError):
            a.ewise1("exp")


def test_compare_select_bool(both):
    for dt in ALL:
        p = random_view(both, dt)
        q = like(both, p, dt)
        for c in ("leq", "eq", "lt"):
            m = p.compare(c, q)
            assert_same(m)
            assert_same(m.ewise1("not"))
            assert_same(m.ewise2("and", p.compare("leq", p)))
            assert_same(m.select(p, q))
        assert p.compare_all("eq", p) == [True, True]
        assert p.compare_all("lt", p) == [False, False]
        r = p.compare_all("leq", q)
        assert r[0] == r[1]
        r = p.compare_all("lt", q)
        assert r[0] == r[1]
    a = both.upload(np.array([1, 2, 3, 4], np.int64))
    b = both.upload(np.array([1, 2, 4, 0], np.int64))
    assert a.compare_all("leq", b) == [True, True] and b.compare_all("leq", a) == [False, False]


def test_convert(both):
    f = both.upload(np.array([-2.5, -0.5, 0.0, 0.5, 2.5, 7.99, 1e6 + 0.75]))
    for dt in (capi.I64, capi.I32):
        assert_same(f.convert(dt, 1))
    assert_same(f.convert(capi.F32, 0))
    for src in ALL:
        p = random_view(both, src)
        for dst in (capi.F64, capi.F32, capi.I64, capi.I32, capi.I16, capi.I8):
            if np.dtype(src).kind == "f" and dst >= capi.I64:
                continue  # float -> int goes through floor
            assert_same(p.convert(dst, 0), 0.0, (src, dst))


@pytest.mark.parametrize("dt", ALL)
def test_contract_random_views(both, dt):
    tol = TOL.get(np.dtype(dt), 0.0)
    for _ in range(12):
        p = random_view(both, dt)
        k = int(RNG.integers(0, len(p.shape) + 1))
        assert_same(p.contract(None, k), tol, ("sum", p.shape, k))
        q = like(both, p, dt)
        assert_same(p.contract(q, k), tol, ("dot", p.shape, k))


@pytest.mark.parametrize("dt", [np.float64, np.float32, np.int32])
def test_contract_shapes_of_the_workloads(both, dt):
    tol = TOL.get(np.dtype(dt), 0.0)
    # long flat reductions (split into chunks + second pass)
    x = both.upload(rnd((300007,), dt))
    assert_same(x.contract(None, 0), tol)
    assert_same(x.contract(x, 0), tol)
    # sum over the outer dim of a matrix (lane-per-output) and over the inner dim (wave-per-output)
    m = both.upload(rnd((513, 130), dt))
    assert_same(m.transpose([1, 0]).contract(None, 1), tol)
    assert_same(m.contract(None, 1), tol)
    # few outputs, long rows
    w = both.upload(rnd((3, 70001), dt))
    assert_same(w.contract(w, 1), tol)
    # tsmatmul2 as the reference defines it: dot1In over replicated + transposed views
    m1, m2 = both.upload(rnd((37, 65), dt)), both.upload(rnd((65, 29), dt))
    lhs = m1.replicate([29]).transpose([1, 0])
    rhs = m2.replicate([37]).transpose([0, 2, 1])
    assert_same(lhs.contract(rhs, 2), tol)
    # tssumN over two leading dims after transposition
    t = both.upload(rnd((6, 7, 40, 9), dt))
    assert_same(t.transpose([2, 3, 0, 1]).contract(None, 2), tol)
    # empty reductions give zeros
    assert_same(both.upload(rnd((4, 0), dt)).contract(None, 1))
    assert_same(both.upload(rnd((0, 4), dt)).contract(None, 1))


def test_argminmax_iota_concat(both):
    for dt in ALL:
        p = random_view(both, dt, rank=3)
        assert_same(p.argminmax_last(True))
        assert_same(p.argminmax_last(False))
    t = both.upload(np.array([[3, 1, 1, 3], [0, 0, 5, 5]], np.int32))   # ties: first occurrence
    assert_same(t.argminmax_last(True))
    assert_same(t.argminmax_last(False))
    for dt in (capi.F64, capi.F32, capi.I64, capi.I32):
        assert_same(both.iota(1000, dt))
    assert_same(both.iota(0, capi.I64))
    parts = [random_view(both, np.float32, rank=1, steps=0)]
    base = parts[0].shape
    parts = [both.upload(rnd((k,) + base[1:], np.float32)) for k in (2, 0, 5)] + [both.upload(rnd((3,) + base[1:], np.float32)).reverse(0)]
    assert_same(both.concat(parts))


@pytest.mark.parametrize("dt", [np.float64, np.float32, np.int64])
def test_fused_sum_equals_program_then_sum(gpu, dt):
    """The sum of a program's result taken on the fly against numpy on the same program."""
    O1, O2 = capi.OP1, capi.OP2
    fp = np.dtype(dt).kind == "f"
    prog = [(1, O2["mul"], 0, 0, 1, 0), (1, O2["add"], 0, 3, 2, 0)] + ([(0, O1["sin"], 0, 4, 0, 0)] if fp else [(0, O1["abs"], 0, 4, 0, 0)])
    for shape in [(1031,), (37, 29), (4096, 33), ()]:
        a, b = rnd(shape, dt), rnd(shape, dt)
        c = dt(3) if fp else dt(3)
        ins = [gpu.upload(a), gpu.upload(b), gpu.upload(c).replicate(list(shape))]
        got = gpu.fused_sum(ins, prog, 5).numpy()
        acc = np.float64 if fp else np.int64
        terms = np.sin(a.astype(acc) * b + c) if fp else np.abs(a.astype(acc) * b + c)
        want = terms.sum()
        assert got.dtype == np.dtype(dt) and got.shape == ()
        if fp:   # a sum is held to the tolerance relative to the sum of the magnitudes of its terms
            assert abs(float(got) - float(want)) <= TOL[np.dtype(dt)] * float(np.abs(terms).sum())
        else:
            assert got == want
        assert np.isclose(float(gpu.fused_sum(ins, prog, 0).numpy()), float(a.astype(acc).sum()), rtol=1e-5)
    with pytest.raises(capi.HgpuError) as e:
        gpu.fused_sum([gpu.upload(rnd((8, 6), dt)).transpose([1, 0])], [], 0)        # a strided view: left to the caller
    assert e.value.code == 4


def test_small_reductions_leave_together(gpu):
    """Single-launch reductions that do not read one another's results are held back and go out as one kernel
    (the bias and readout gradients at the end of a reverse pass); one that reads another's result runs after it.
    Results against numpy, and bit-equal to the same reductions asked for one at a time."""
    import os
    if os.environ.get("HORDEAD_NO_GROUPED_LAUNCH"):
        pytest.skip("grouped launches are switched off in this environment")
    a, b, b2, c = rnd((300, 5000), np.float64), rnd((100, 5000), np.float64), rnd((100, 5000), np.float64), rnd((10, 1000), np.float64)
    A, B, B2, Cc = gpu.upload(a), gpu.upload(b), gpu.upload(b2), gpu.upload(c)
    alone = []
    for x, y in ((A, None), (B, B2), (Cc, None)):
        r = x.contract(y, 1)
        alone.append(r.numpy())                      # the read-back sends each one out by itself
    gpu.sync()
    gpu.profile(2)
    ra, rb, rc = A.contract(None, 1), B.contract(B2, 1), Cc.contract(None, 1)
    rd = ra.contract(None, 0)                        # reads ra: the next level
    got = [r.numpy() for r in (ra, rb, rc)]
    total = float(rd.numpy())
    rep = gpu.profile_report()
    gpu.profile(0)
    groups = {k: v for k, v in rep.items() if k.startswith("contract_group[") and v[0]}
    assert len(groups) == 1 and list(groups.values())[0][0] == 1 and list(groups)[0].count("|") == 2, rep
    for g, w, al in zip(got, (a.sum(1), (b * b2).sum(1), c.sum(1)), alone):
        np.testing.assert_allclose(g, w, rtol=1e-10, atol=1e-9)
        assert np.array_equal(g, al)
    assert abs(total - float(a.sum())) <= 1e-10 * float(np.abs(a).sum())


def test_fused_sum_is_finished_three_ways(gpu):
    """Up to 1024 vectors one block writes the sum; up to 131072 elements the block that draws the last
    ticket adds the blocks' sums; beyond, a second launch does.  Every size is summed twice in a row and
    again after the others (the ticket counter must be back at zero): the same bits each time, and the
    exact integer sum."""
    O2 = capi.OP2
    prog = [(1, O2["mul"], 0, 0, 1, 0)]
    sizes = [2048, 2049, 60000, 131072, 131073, 600000]
    data = {n: (rnd((n,), np.float64), rnd((n,), np.float64)) for n in sizes}
    first = {}
    for rnd_no in range(3):
        for n in sizes if rnd_no != 1 else reversed(sizes):
            a, b = data[n]
            ins = [gpu.upload(a), gpu.upload(b)]
            got = float(gpu.fused_sum(ins, prog, 2).numpy())
            assert abs(got - float((a * b).sum())) <= 1e-10 * float(np.abs(a * b).sum())
            assert first.setdefault(n, got) == got, (n, rnd_no)
            ia, ib = (a * 1000).astype(np.int64), (b * 1000).astype(np.int64)
            assert int(gpu.fused_sum([gpu.upload(ia), gpu.upload(ib)], prog, 2).numpy()) == int((ia * ib).sum())


@pytest.mark.parametrize("dt", [np.float64, np.float32, np.int32])
def test_fused_extremum_equals_program_then_extremum(gpu, dt):
    """The extremum of a program's result over its trailing dims, taken on the
    fly, against the program written out (fused_map) and reduced (extremum_last)."""
    O2 = capi.OP2
    prog = [(1, O2["mul"], 0, 0, 1, 0), (1, O2["add"], 0, 3, 2, 0), (1, O2["max"], 0, 4, 0, 0)]   # max (a * b + c) a
    for shape, n_reduce in [((6, 5, 2, 2), 2), ((4, 3, 7), 1), ((9, 64), 1), ((3, 2, 2, 2, 2), 3), ((5,), 1)]:
        a = gpu.upload(rnd(shape, dt))
        b = gpu.upload(rnd(shape[-1:], dt)).replicate(list(shape[:-1]))                # broadcast view
        c = gpu.upload(np.ascontiguousarray(np.moveaxis(rnd(shape, dt), -1, 0))).transpose(list(range(1, len(shape))) + [0]) if len(shape) > 1 else gpu.upload(rnd(shape, dt))
        ins = [a, b, c]
        for slot in (5, 3, 0):
            full = gpu.fused_map(ins, prog, [slot])[0] if slot >= 3 else a
            lead = list(shape[:len(shape) - n_reduce])
            flat = full.reshape(lead + [int(np.prod(shape[len(shape) - n_reduce:]))])
            for want_max in (True, False):
                wv, wi = flat.extremum_last(want_max)
                gv, gi = gpu.fused_extremum(ins, prog, slot, n_reduce, want_max)
                assert np.array_equal(gi.numpy(), wi.numpy()), (shape, slot, want_max)
                assert np.array_equal(gv.numpy(), wv.numpy())
    with pytest.raises(capi.HgpuError):
        gpu.fused_extremum([gpu.upload(rnd((3, 100), dt))], [], 0, 1, True)      # more than 64 reduced elements


def test_extremum_values_with_indices(gpu):
    """One pass yields the arg-extremum and the extremal value: the same indices
    as argminmax_last, and the value found there."""
    for dt in ALL:
        for shape, perm in [((6, 5, 4), None), ((3, 700), None), ((2, 9000), None), ((40, 30, 8), [1, 0, 2]), ((5, 7), [1, 0])]:
            x = rnd(shape, dt)
            a = gpu.upload(x)
            if perm:
                a, x = a.transpose(perm), x.transpose(perm)
            for want_max in (True, False):
                vals, idx = a.extremum_last(want_max)
                want_idx = (np.argmax if want_max else np.argmin)(x, axis=-1)
                assert np.array_equal(idx.numpy(), want_idx)
                assert np.array_equal(idx.numpy(), a.argminmax_last(want_max).numpy())
                assert np.array_equal(vals.numpy(), np.take_along_axis(x, want_idx[..., None], axis=-1)[..., 0])


def test_extremum_of_very_long_rows(gpu):
    """A few rows of tens of thousands of elements (the minimum of a whole tensor)
    are scanned in pieces by many blocks: first occurrence wins also when the tie
    lies in another piece, rows may be strided, and the last piece may be ragged."""
    for dt in (np.float64, np.float32, np.int32):
        for shape in [(50000,), (3, 81920), (2, 16385)]:
            x = rnd(shape, dt)
            flat = x.reshape(-1, shape[-1])
            for r in range(flat.shape[0]):                       # the extremes several times, far apart
                hi, lo = flat[r].max() + 1, flat[r].min() - 1
                flat[r, [shape[-1] - 7, 9000, 40000 % shape[-1]]] = hi
                flat[r, [shape[-1] - 1, 12001, 5]] = lo
            a = gpu.upload(x)
            for want_max in (True, False):
                vals, idx = a.extremum_last(want_max)
                want_idx = (np.argmax if want_max else np.argmin)(x, axis=-1)
                assert np.array_equal(idx.numpy(), want_idx)
                assert np.array_equal(vals.numpy(), np.take_along_axis(x, np.asarray(want_idx)[..., None], axis=-1)[..., 0])
    x = rnd((20000, 4), np.float64)                              # rows of a transposed view: stride 4
    a = gpu.upload(x).transpose([1, 0])
    assert np.array_equal(a.argminmax_last(True).numpy(), np.argmax(x.T, axis=-1))
    assert np.array_equal(a.argminmax_last(False).numpy(), np.argmin(x.T, axis=-1))


def ix_arrays(both, shm, extents, oob=True, view=False):
    out = []
    for e in extents:
        lo, hi = (-1, e + 1) if oob else (0, e)
        if view and len(shm) >= 2 and RNG.integers(0, 2) == 0:
            out.append(both.upload(RNG.integers(lo, hi, shm[1:]).astype(np.int64)).replicate([shm[0]]))
        else:
            out.append(both.upload(RNG.integers(lo, hi, shm).astype(np.int64)))
    return out


@pytest.mark.parametrize("dt", ALL + [np.bool_])
def test_gather_exact(both, dt):
    for _ in range(8):
        src = random_view(both, dt, rank=int(RNG.integers(1, 5)))
        n_ix = int(RNG.integers(0, len(src.shape) + 1))
        shm = [int(RNG.integers(1, 6)) for _ in range(int(RNG.integers(0, 4)))]
        ix = ix_arrays(both, shm, src.shape[:n_ix], view=True)
        assert_same(both.gather(src, ix, shm), 0.0, (src.shape, n_ix, shm))
    src = both.upload(rnd((4, 5), dt))
    assert_same(both.gather(src, ix_arrays(both, [0, 3], [4]), [0, 3]))


@pytest.mark.parametrize("dt", [np.float64, np.float32, np.int16, np.int8])
def test_gather_of_wide_slices(both, dt):
    """Slices that are contiguous in the table and whole 16-byte (or 8-byte) units go
    out one unit per lane; indices outside the table read zeros; tables whose rows do
    not start on a unit boundary (a sliced view, an odd row length) take the element
    kernel.  Bit-exact against the checker and numpy either way."""
    es = np.dtype(dt).itemsize
    for rows, n, m in [(300, 256 // es, 5000), (300, 1024 // es, 700), (50, 24 // es, 999), (64, 40 // es + 1, 300)]:
        t = rnd((rows, n), dt)
        idx = RNG.integers(-3, rows + 3, m).astype(np.int64)        # some outside
        got = both.gather(both.upload(t), [both.upload(idx)], [m])
        assert_same(got, 0.0, (dt, rows, n, m))
        ok = (idx >= 0) & (idx < rows)
        want = np.where(ok[:, None], t[np.clip(idx, 0, rows - 1)], 0).astype(dt)
        assert np.array_equal(got.numpy()[0], want)
    # two indexed dims, slices of the last one; and a table that is a view with an offset
    t = both.upload(rnd((12, 9, 32), dt))
    i0, i1 = both.upload(RNG.integers(0, 12, (40, 3)).astype(np.int64)), both.upload(RNG.integers(0, 9, (40, 3)).astype(np.int64))
    assert_same(both.gather(t, [i0, i1], [40, 3]), 0.0)
    v = both.upload(rnd((20, 33), dt)).slice(1, 1, 32)                  # rows start 1 element in
    assert_same(both.gather(v, [both.upload(RNG.integers(0, 20, 77).astype(np.int64))], [77]), 0.0)
    w = both.upload(rnd((16, 30), dt)).transpose([1, 0])                # slices strided in memory
    assert_same(both.gather(w, [both.upload(RNG.integers(0, 30, 50).astype(np.int64))], [50]), 0.0)


@pytest.mark.parametrize("dt", [np.float64, np.float32, np.int64, np.int32])
def test_scatter(both, dt):
    tol = TOL.get(np.dtype(dt), 0.0)
    for _ in range(8):
        src = random_view(both, dt, rank=int(RNG.integers(1, 5)))
        rank_m = int(RNG.integers(0, len(src.shape) + 1))
        shp = [int(RNG.integers(1, 6)) for _ in range(int(RNG.integers(0, 3)))]
        ix = ix_arrays(both, list(src.shape[:rank_m]), shp, view=True)
        assert_same(both.scatter_add(src, ix, rank_m, shp), 0.0, (src.shape, rank_m, shp))
    # collisions, at most 256 positions per cell: colliding positions are added in ascending
    # order, as the reference and the checker do: bit-equal, also for floats
    src = both.upload(rnd((1200, 2), dt))
    ix = ix_arrays(both, [1200], [7])
    assert np.bincount(ix[0].numpy()[0].ravel() + 1).max() <= 256
    assert_same(both.scatter_add(src, ix, 1, [7]), 0.0)
    # heavy collisions: 20000 positions into 7 cells.  A run longer than 256 is added in
    # segments of 256 (each in ascending order) whose sums are added in ascending order:
    # exact for integers, within the tolerance for floats, and the same from run to run
    src = both.upload(rnd((20000, 2), dt))
    ix = ix_arrays(both, [20000], [7])
    first = both.scatter_add(src, ix, 1, [7])
    assert_same(first, tol)
    again = both.scatter_add(src, ix, 1, [7])
    assert np.array_equal(first.numpy()[0], again.numpy()[0])
    # single elements: runs of a few entries, runs that cross a wavefront's 64 sorted entries, runs just
    # below and above the segment length, all still in the reference's order where they fit one segment
    for m, cells in ((5000, 2000), (5000, 40), (7000, 30), (1000, 1), (300, 1), (64, 1), (65, 2)):
        src = both.upload(rnd((m,), dt))
        ix = [both.upload(RNG.integers(-1, cells + 1, m).astype(np.int64))]
        longest = np.bincount(ix[0].numpy()[0] + 1).max()
        res = both.scatter_add(src, ix, 1, [cells])
        if longest <= 256 or tol == 0.0:
            assert_same(res, 0.0, (m, cells))
        else:   # a reordered sum: held against the sum of the magnitudes that went into a cell, not against what cancellation left of them
            g, o = res.numpy()
            mass = np.zeros(cells + 2)
            np.add.at(mass, ix[0].numpy()[0] + 1, np.abs(src.numpy()[0]).astype(np.float64))
            assert np.all(np.abs(g.astype(np.float64) - o) <= tol * mass[1:cells + 1]), (m, cells)
    # many destinations with a few positions each, some out of bounds, slices of 5
    src = both.upload(rnd((3000, 5), dt))
    ix = [both.upload(RNG.integers(-2, 700, 3000).astype(np.int64))]
    assert_same(both.scatter_add(src, ix, 1, [650]), 0.0)
    # distinct destinations, caller-guaranteed: plain stores
    perm = both.upload(RNG.permutation(500).astype(np.int64))
    src = both.upload(rnd((500, 3), dt))
    assert_same(both.scatter_add(src, [perm], 1, [500], flags=1))


@pytest.mark.parametrize("dt", [np.float64, np.float32, np.int64, np.int8, np.bool_])
def test_scatter_affine(both, dt):
    # pooling windows over a transposed source: a bijection, nothing stays zero
    src = both.upload(rnd((5, 3, 4, 2, 6, 2), dt)).transpose([2, 3, 4, 5, 0, 1])
    assert_same(both.scatter_affine(src, 4, [0, 0], [[2, 0], [1, 0], [0, 2], [0, 1]], [8, 12]))
    # offsets, negative and skewed coefficients, zeros left in place
    src = random_view(both, dt, rank=3)
    s = src.shape
    c0 = [3 * (s[0] - 1) + 1, 2]
    coef = [[-3, 0], [0, s[2] + 1], [0, 1]]
    shp = [c0[0] + 2, 2 + (s[1] - 1) * (s[2] + 1) + s[2] + 1]
    assert_same(both.scatter_affine(src, 3, c0, coef, shp), 0.0, (s, c0, coef, shp))
    # trailing dims carried along, rank-0 position space
    src = both.upload(rnd((4, 7), dt))
    assert_same(both.scatter_affine(src, 1, [1], [[2]], [9]))
    assert_same(both.scatter_affine(src, 0, [2], [], [5]))


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_contract_sum(both, dt):
    """Sums of products of one shape: one launch over all terms (weight gradients
    of an unrolled recurrence), small outputs, many terms, mixed layouts."""
    tol = TOL[np.dtype(dt)]
    for m, n, k, terms in [(128, 128, 600, 5), (128, 28, 900, 7), (64, 200, 512, 40), (10, 16, 3000, 3)]:
        pairs = []
        for _ in range(terms):
            a = both.upload(rnd((m, k), dt)).replicate([n]).transpose([1, 0, 2])      # [m, n, k]
            b = both.upload(rnd((k, n), dt)).transpose([1, 0]).replicate([m])          # [m, n, k], K strided
            pairs.append((a, b))
        assert_same(both.contract_sum(pairs, 2), tol, (m, n, k, terms))
    # terms of different layouts: term by term
    a1 = both.upload(rnd((40, 30, 50), dt))
    b1 = both.upload(rnd((40, 30, 50), dt))
    a2 = both.upload(rnd((30, 40, 50), dt)).transpose([1, 0, 2])
    b2 = both.upload(rnd((40, 30, 50), dt))
    assert_same(both.contract_sum([(a1, b1), (a2, b2)], 2), tol)
    assert_same(both.contract_sum([(a1, b1)], 1), tol)
    # terms of one layout that are no matrix product (row-wise dots: bias gradients
    # of an unrolled recurrence): one grouped reduction
    for shape, keep, perm in [((128, 700), 1, None), ((128, 700), 0, None), ((300, 40), 1, [1, 0]), ((6, 5, 64), 2, None), ((3000, 8), 1, None)]:
        pairs = []
        for _ in range(7):
            a, b = both.upload(rnd(shape, dt)), both.upload(rnd(shape, dt))
            if perm:
                a, b = a.transpose(perm), b.transpose(perm)
            pairs.append((a, b))
        assert_same(both.contract_sum(pairs, keep), tol, (shape, keep, perm))
    # two layouts interleaved, one of them with a replicated (stride 0) operand:
    # each layout is one grouped launch
    pairs = []
    for t in range(9):
        a = both.upload(rnd((128, 700), dt)).replicate([96]).transpose([1, 0, 2])
        if t % 3 == 0:
            b = both.upload(rnd((700,), dt)).replicate([128, 96])
        else:
            b = both.upload(rnd((700, 96), dt)).transpose([1, 0]).replicate([128])
        pairs.append((a, b))
    assert_same(both.contract_sum(pairs, 2), tol)


def test_scatter_small_ints(both, gpu):
    perm = both.upload(RNG.permutation(64).astype(np.int64))
    for dt in (np.int16, np.int8):
        src = both.upload(rnd((64,), dt))
        assert_same(both.scatter_add(src, [perm], 1, [64], flags=1))
        assert_same(both.scatter_add(src, [perm], 1, [64]))                    # the same without the promise of distinct places
        # colliding positions accumulate in the element type, wrapping like the reference's Int16 / Int8
        many = both.upload(rnd((5000, 3), dt))
        cells = [both.upload(RNG.integers(-1, 12, 5000).astype(np.int64))]
        assert_same(both.scatter_add(many, cells, 1, [11]))


def test_scatter_into_a_handful_of_cells_is_bounded(both, gpu):
    """A million positions into eight cells (a table's cotangent): runs of 125,000 are added
    in segments of 256 by separate lanes, not by one lane front to back.  Exact for
    integers; floats within the tolerance of a reordered sum; and the call, sort included,
    takes milliseconds, not seconds.  (A sum of 125,000 terms added front to back in single precision,
    which is what the reference's order gives, is itself some 1e-5 off: both are held to the sum in double.)"""
    import time
    M = 1 << 20
    cells = RNG.integers(-1, 8, M).astype(np.int64)          # some out of bounds
    for dt, n, tol in ((np.int64, 1, 0.0), (np.float64, 1, 1e-10), (np.float64, 24, 1e-10), (np.float32, 3, 1e-5)):
        src = both.upload(rnd((M, n) if n > 1 else (M,), dt))
        ix = [both.upload(cells)]
        res = both.scatter_add(src, ix, 1, [8])
        got, seq = res.numpy()                              # the device; the checker, which adds front to back in the element type
        inb = (cells >= 0) & (cells < 8)
        x64 = src.numpy()[1].astype(np.float64)
        want = np.zeros(got.shape, np.float64)              # the independent sum, in double whatever the element type
        mass = np.zeros(got.shape, np.float64)
        np.add.at(want, cells[inb], x64[inb])
        np.add.at(mass, cells[inb], np.abs(x64[inb]))
        if tol == 0.0:
            assert np.array_equal(got, seq) and np.array_equal(got, want.astype(dt)), (dt, n)
        else:
            # 125,000 terms per cell: both orders are held to the exact sum, by the magnitudes that went into a cell
            eps = float(np.finfo(dt).eps)
            assert np.all(np.abs(got - want) <= 8 * eps * mass), (dt, n, np.max(np.abs(got - want) / mass))
            assert np.all(np.abs(seq - want) <= 600 * eps * mass), (dt, n)
        dev = src.arrays[0]
        gix = [ix[0].arrays[0]]
        gpu.sync()
        t0 = time.perf_counter()
        gpu.scatter_add(dev, gix, 1, [8])
        gpu.sync()
        assert time.perf_counter() - t0 < 0.05, (dt, n, time.perf_counter() - t0)


def test_gather_scatter_adjoint_large(both):
    """<gather x f, y> == <x, scatter y f> on a conv-sized window pattern."""
    x = both.upload(rnd((48, 48), np.float64))
    shm = [48, 5]
    i = np.add.outer(np.arange(48), np.arange(5)).astype(np.int64)   # i + k, runs out of bounds
    ix = [both.upload(i)]
    y = both.upload(rnd((48, 5, 48), np.float64))
    g = both.gather(x, ix, shm)
    s = both.scatter_add(y, ix, 2, [48])
    assert_same(g)
    assert_same(s, 1e-10)
    lhs = g.contract(y, 0).numpy()
    rhs = x.contract(s, 0).numpy()
    assert abs(lhs[0] - rhs[0]) <= 1e-10 * abs(lhs[0])
    assert abs(lhs[0] - lhs[1]) <= 1e-10 * abs(lhs[1])


def test_errors_and_allocator(gpu):
    a = gpu.upload(rnd((4, 5), np.float64))
    b = gpu.upload(rnd((4, 6), np.float64))
    with pytest.raises(capi.HgpuError) as e:
        a.ewise2("add", b)
    assert e.value.code == 1 and "shape" in str(e.value)
    with pytest.raises(capi.HgpuError):
        a.ewise2("add", gpu.upload(rnd((4, 5), np.float32)))
    with pytest.raises(capi.HgpuError):
        a.contract(b, 1)
    with pytest.raises(capi.HgpuError):
        a.transpose([0, 0])
    with pytest.raises(capi.HgpuError):
        a.slice(1, 3, 4)
    # blocks are recycled: repeating the same op needs no new device allocation
    c = a.ewise1("sin")
    del c
    n0 = gpu.mem_stats()[2]
    for _ in range(10):
        c = a.ewise1("sin")
        del c
    assert gpu.mem_stats()[2] == n0
    # a device allocation that fails surfaces as a status, not a crash
    gpu.check(gpu.lib.inject_alloc_failure(gpu.h, 0))
    with pytest.raises(capi.HgpuError) as e:
        a.ewise1("cos")
    assert e.value.code == 2
    gpu.check(gpu.lib.inject_alloc_failure(gpu.h, -1))
    assert np.allclose(a.ewise1("cos").numpy(), np.cos(a.numpy()))


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_contract_on_the_matrix_cores(both, gpu, dt):
    """Contractions whose strides make them matrix products run on the MFMA
    kernel; operands stay views (replicated, transposed, windowed)."""
    tol = TOL[np.dtype(dt)]

    def matmul_views(m1, m2):
        m, n = m1.shape
        p = m2.shape[1]
        return m1.replicate([p]).transpose([1, 0]), m2.replicate([m]).transpose([0, 2, 1])

    for (m, n, p) in [(130, 70, 129), (257, 33, 64), (16, 300, 16), (1, 520, 700), (300, 4, 300), (128, 128, 128), (10, 128, 2500)]:
        a, b = both.upload(rnd((m, n), dt)), both.upload(rnd((n, p), dt))
        lhs, rhs = matmul_views(a, b)
        assert_same(lhs.contract(rhs, 2), tol, ("matmul", m, n, p))
        # transposed operands: A^T stored, B^T stored
        at, bt = both.upload(rnd((n, m), dt)).transpose([1, 0]), both.upload(rnd((p, n), dt)).transpose([1, 0])
        lhs, rhs = matmul_views(at, bt)
        assert_same(lhs.contract(rhs, 2), tol, ("matmul^T", m, n, p))
    # long K with a small output: split along K
    a, b = both.upload(rnd((24, 40000), dt)), both.upload(rnd((40000, 20), dt))
    lhs, rhs = matmul_views(a, b)
    assert_same(lhs.contract(rhs, 2), tol, "split-K")
    # a batch dim on both operands
    x, y = both.upload(rnd((5, 40, 30), dt)), both.upload(rnd((5, 30, 50), dt))
    lhs = x.replicate([50]).transpose([1, 2, 0])            # [5, 40, 50, 30]
    rhs = y.replicate([40]).transpose([1, 0, 3, 2])          # [5, 40, 50, 30]
    assert_same(lhs.contract(rhs, 3), tol, "batched")
    # convolution as a contraction over a window view: out[b, co, h, w]
    img, ker = both.upload(rnd((3, 4, 12, 10), dt)), both.upload(rnd((6, 4, 3, 3), dt))
    padded = img.pad([0, 0, 0, 0], [0, 0, 2, 2])
    st = padded.arrays[0].strides    # dense on both providers
    win = padded.as_strided([3, 12, 10, 4, 3, 3], [st[0], st[2], st[3], st[1], st[2], st[3]], 0)
    lhs = win.replicate([6]).transpose([1, 0, 2, 3])          # [b, co, h, w, ci, kh, kw]
    rhs = ker.replicate([3, 12, 10]).transpose([0, 3, 1, 2])  # [b, co, h, w, ci, kh, kw]
    assert_same(lhs.contract(rhs, 4), tol, "conv")
    # the kernel-gradient contraction: K = (b, h, w) on both operands
    dout = both.upload(rnd((3, 6, 12, 10), dt))
    lhs = win.replicate([6]).transpose([0, 4, 5, 6, 1, 2, 3])             # [co, ci, kh, kw, b, h, w]
    rhs = dout.replicate([4, 3, 3]).transpose([4, 0, 1, 2, 3, 5, 6])      # [co, ci, kh, kw, b, h, w]
    assert_same(lhs.contract(rhs, 4), tol, "conv dK")
    rep = None
    gpu.profile(True)
    a, b = gpu.upload(rnd((256, 64), dt)), gpu.upload(rnd((64, 256), dt))
    a.replicate([256]).transpose([1, 0]).contract(b.replicate([256]).transpose([0, 2, 1]), 2)
    rep = gpu.profile_report()
    gpu.profile(False)
    assert any(k.startswith("gemm") for k in rep), rep


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_staged_products_at_the_edges_of_their_tiles(both, dt):
    """The staged kernel reads whole tiles with clamped addresses and zeroes what
    lies past the end when it stores to LDS: K and rows that are no multiples
    of the K step, of the vector width or of the tile, K tables (two K dims that
    do not merge) with lanes along K, K chunks that end inside a step."""
    tol = TOL[np.dtype(dt)]

    def nt_views(a, b):      # a [m, ...k], b [n, ...k] -> operands [m, n, ...k]
        m, n = a.shape[0], b.shape[0]
        r = len(a.shape) - 1
        lhs = a.replicate([n]).transpose([1, 0] + list(range(2, 2 + r)))
        rhs = b.replicate([m])
        return lhs, rhs

    for (m, n, k) in [(70, 50, 18), (70, 50, 20), (66, 129, 130), (64, 64, 16), (65, 35, 1030), (33, 40, 7), (200, 36, 36)]:
        a, b = both.upload(rnd((m, k), dt)), both.upload(rnd((n, k), dt))      # lanes along K on both
        lhs, rhs = nt_views(a, b)
        assert_same(lhs.contract(rhs, 2), tol, ("NT", m, n, k))
        at, bt = both.upload(rnd((k, m), dt)).transpose([1, 0]), both.upload(rnd((k, n), dt)).transpose([1, 0])   # lanes along the rows
        lhs, rhs = nt_views(at, bt)
        assert_same(lhs.contract(rhs, 2), tol, ("TN", m, n, k))
    # two K dims that do not merge (the inner one is a window of a longer row): K table, vectors along K
    for (m, n, k1, k2, k2p) in [(70, 50, 5, 8, 12), (64, 48, 3, 20, 21), (40, 130, 7, 6, 16)]:
        af, bf = both.upload(rnd((m, k1, k2p), dt)), both.upload(rnd((n, k1, k2p), dt))
        a = af.as_strided([m, k1, k2], [k1 * k2p, k2p, 1], 0)
        b = bf.as_strided([n, k1, k2], [k1 * k2p, k2p, 1], k2p - k2)     # ends with the allocation
        lhs, rhs = nt_views(a, b)
        assert_same(lhs.contract(rhs, 2), tol, ("table", m, n, k1, k2))
    # K chunks that end inside a K step, partial sums
    a, b = both.upload(rnd((64, 20008), dt)), both.upload(rnd((48, 20008), dt))
    lhs, rhs = nt_views(a, b)
    assert_same(lhs.contract(rhs, 2), tol, "split-K, ragged chunks")


def conv_views(both, dt, b, ci, h, w, co, kh, kw):
    """The window views of a 'same' convolution: input windows [b, h, w, ci, kh, kw]
    of the zero-extended image, the kernel, and a cotangent of the output."""
    img, ker = both.upload(rnd((b, ci, h, w), dt)), both.upload(rnd((co, ci, kh, kw), dt))
    padded = img.pad([0, 0, 0, 0], [0, 0, kh - 1, kw - 1])
    st = padded.arrays[0].strides
    win = padded.as_strided([b, h, w, ci, kh, kw], [st[0], st[2], st[3], st[1], st[2], st[3]], 0)
    dout = both.upload(rnd((b, co, h, w), dt))
    return win, ker, dout


@pytest.mark.parametrize("dt", [np.float64, np.float32])
@pytest.mark.parametrize("shape", [
    (160, 8, 12, 12, 16, 3, 3),     # row blocks dealt evenly and split along K
    (200, 16, 14, 14, 16, 5, 5),    # the CNN's second layer at a fifth of its batch
    (512, 3, 9, 11, 12, 3, 2),      # fewer than 16 output channels, K not a multiple of 4
    (192, 1, 20, 20, 8, 5, 5),      # one input channel
    (300, 5, 7, 9, 16, 2, 4),       # odd extents everywhere, K tails
    (600, 2, 16, 16, 4, 3, 3),      # four output channels
    (128, 32, 8, 8, 16, 3, 3),      # 18 row blocks in the kernel gradient: dealt and split
    (150, 7, 10, 10, 16, 3, 3),     # 63 rows
    (130, 1, 28, 28, 16, 5, 5),     # the CNN's first layer: the kernel gradient's footprints fit LDS once, not twice
])
def test_conv_contractions_from_lds_footprints(both, gpu, dt, shape):
    """Forward convolution, kernel gradient and input gradient as contractions
    over window views, at batch sizes where a block keeps one image's footprint
    of each operand in LDS."""
    b, ci, h, w, co, kh, kw = shape
    tol = TOL[np.dtype(dt)]
    win, ker, dout = conv_views(both, dt, b, ci, h, w, co, kh, kw)
    gpu.check(gpu.lib.profile_enable(gpu.h, 2))     # kernel names with shapes
    gpu.profile_report()
    # forward: out[b, co, h, w]
    lhs = win.replicate([co]).transpose([1, 0, 2, 3])             # [b, co, h, w, ci, kh, kw]
    rhs = ker.replicate([b, h, w]).transpose([0, 3, 1, 2])        # [b, co, h, w, ci, kh, kw]
    assert_same(lhs.contract(rhs, 4), tol, ("conv", shape))
    # kernel gradient: dK[co, ci, kh, kw], K = (b, h, w) on both operands
    lhs = win.replicate([co]).transpose([0, 4, 5, 6, 1, 2, 3])            # [co, ci, kh, kw, b, h, w]
    rhs = dout.replicate([ci, kh, kw]).transpose([4, 0, 1, 2, 3, 5, 6])   # [co, ci, kh, kw, b, h, w]
    assert_same(lhs.contract(rhs, 4), tol, ("conv dK", shape))
    # input gradient as a convolution of the zero-extended cotangent with the
    # reversed kernel: dX[b, ci, y, x] = sum dout_pad[b, co, y + p, x + q] * ker[co, ci, kh-1-p, kw-1-q]
    dpad = dout.pad([0, 0, kh - 1, kw - 1], [0, 0, 0, 0])
    st = dpad.arrays[0].strides
    dwin = dpad.as_strided([b, h, w, co, kh, kw], [st[0], st[2], st[3], st[1], st[2], st[3]], 0)
    lhs = dwin.replicate([ci]).transpose([1, 0, 2, 3])                     # [b, ci, y, x, co, kh, kw]
    rker = ker.reverse(2).reverse(3).transpose([1, 0, 2, 3])               # [ci, co, kh, kw]
    rhs = rker.replicate([b, h, w]).transpose([0, 3, 1, 2])                # [b, ci, y, x, co, kh, kw]
    assert_same(lhs.contract(rhs, 4), tol, ("conv dX", shape))
    rep = gpu.profile_report()
    gpu.profile(False)
    # at least the kernel gradient and the forward product of the larger shapes run from LDS footprints
    if ci * kh * kw >= 16:
        assert any("footprint" in k for k in rep), list(rep)


def eval_program_eagerly(ctx, inputs, prog, out_slots):
    """The meaning of a fused program: the single entry points applied in order."""
    inv1 = {v: k for k, v in capi.OP1.items()}
    inv2 = {v: k for k, v in capi.OP2.items()}
    invc = {v: k for k, v in capi.CMP.items()}
    slots = list(inputs)
    for kind, op, dtype, a, b, c in prog:
        if kind == 0:
            slots.append(slots[a].ewise1(inv1[op]))
        elif kind == 1:
            slots.append(slots[a].ewise2(inv2[op], slots[b]))
        elif kind == 2:
            slots.append(slots[a].compare(invc[op], slots[b]))
        elif kind == 3:
            slots.append(slots[a].select(slots[b], slots[c]))
        else:
            slots.append(slots[a].convert(dtype, op))
    return [slots[s] for s in out_slots]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_fused_map_groups_of_the_innermost_dim(gpu, dt):
    """Large strided programs take 16 bytes of the innermost dim per lane; inputs that
    run along it (aligned or not), stand still along it, or cross it are all read
    correctly: against numpy, to the tolerance of the dtype."""
    O2 = capi.OP2
    sh = (96, 81, 72)
    a = rnd(sh, dt)
    b = rnd(sh[:2], dt)
    c = rnd((sh[2], sh[0], sh[1]), dt)
    d = rnd((sh[0], sh[1], sh[2] + 2), dt)
    m = rnd(sh, np.int32)
    ins = [gpu.upload(a),
           gpu.upload(b).replicate([sh[2]]).transpose([1, 2, 0]),
           gpu.upload(c).transpose([1, 2, 0]),
           gpu.upload(d).slice(2, 1, sh[2]),
           gpu.upload(m).reverse(2)]
    prog = [(1, O2["mul"], 0, 0, 1, 0),            # 5: a * b
            (1, O2["add"], 0, 5, 2, 0),            # 6: + c
            (1, O2["sub"], 0, 6, 3, 0),            # 7: - d
            (4, 0, capi.F64 if dt == np.float64 else capi.F32, 4, 0, 0),   # 8: m as a float
            (2, capi.CMP["leq"], 0, 8, 7, 0),      # 9: m <= (..)
            (3, 0, 0, 9, 7, 1)]                    # 10: select
    got = [o.numpy() for o in gpu.fused_map(ins, prog, [7, 9, 10])]
    t = a * b[:, :, None] + np.transpose(c, (1, 2, 0)) - d[:, :, 1:-1]
    mf = m[:, :, ::-1].astype(dt)
    want = [t, mf <= t, np.where(mf <= t, t, np.broadcast_to(b[:, :, None], sh))]
    tol = TOL[np.dtype(dt)]
    assert np.max(np.abs(got[0] - want[0])) <= tol * np.max(np.abs(want[0]))
    # comparisons may differ where rounding moves the value across m
    close_call = np.abs(mf - t) <= 4 * tol * np.abs(t)
    assert np.array_equal(got[1] | close_call, want[1] | close_call)
    sel = np.where(got[1], got[0], np.broadcast_to(b[:, :, None], sh))
    assert np.array_equal(got[2], sel)


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_fused_map_equals_the_single_operations(gpu, oracle, dt):
    tol = TOL[np.dtype(dt)]
    O1, O2 = capi.OP1, capi.OP2
    # foo's gradient program: inputs x, y, z, dret (a broadcast scalar)
    prog = [
        (0, O1["sin"], 0, 1, 0, 0),      # 4: sin y
        (1, O2["mul"], 0, 0, 4, 0),      # 5: w = x * sin y
        (1, O2["mul"], 0, 2, 2, 0),      # 6: z*z
        (1, O2["mul"], 0, 5, 5, 0),      # 7: w*w
        (1, O2["add"], 0, 6, 7, 0),      # 8
        (0, O1["recip"], 0, 8, 0, 0),    # 9: t
        (0, O1["neg"], 0, 2, 0, 0),      # 10: -z
        (1, O2["mul"], 0, 10, 9, 0),     # 11: -z t
        (1, O2["add"], 0, 11, 2, 0),     # 12: dw = -z t + z
        (1, O2["mul"], 0, 12, 3, 0),     # 13: dw * dret
        (1, O2["mul"], 0, 13, 4, 0),     # 14: dx
        (0, O1["cos"], 0, 1, 0, 0),      # 15
        (1, O2["mul"], 0, 13, 0, 0),     # 16
        (1, O2["mul"], 0, 16, 15, 0),    # 17: dy
        (1, O2["mul"], 0, 5, 9, 0),      # 18: w t
        (1, O2["add"], 0, 18, 5, 0),     # 19
        (1, O2["mul"], 0, 19, 3, 0),     # 20: dz
        (2, capi.CMP["leq"], 0, 0, 1, 0),            # 21: x <= y (Bool)
        (3, 0, 0, 21, 14, 17),                        # 22: select
        (4, 1, capi.I64, 22, 0, 0),                   # 23: floor -> Int
        (4, 0, capi.F32 if dt == np.float64 else capi.F64, 20, 0, 0),   # 24: cast
    ]
    outs = [14, 17, 20, 21, 22, 23, 24][:6]
    # the last two are large enough for the kernels compiled with their shapes and strides
    for shape, views in [((1031,), False), ((37, 29), False), ((6, 5, 7), True), ((601, 701), False), ((96, 81, 72), True)]:
        data = [rnd(shape, dt) + dt(2.5) for _ in range(3)]
        res = []
        for ctx in (gpu, oracle):
            ins = [ctx.upload(d) for d in data] + [ctx.upload(dt(1.25)).replicate(list(shape))]
            if views:
                ins[0] = ctx.upload(np.ascontiguousarray(np.transpose(data[0], (2, 0, 1)))).transpose([1, 2, 0])
                ins[1] = ins[1].reverse(1).reverse(1)
            if ctx is gpu:
                res.append([o.numpy() for o in ctx.fused_map(ins, prog, outs)])
            else:
                res.append([o.numpy() for o in eval_program_eagerly(ctx, ins, prog, outs)])
        for g, o in zip(*res):
            assert g.dtype == o.dtype and g.shape == o.shape
            if g.dtype.kind == "f":
                assert np.max(np.abs(g - o)) <= tol * max(np.max(np.abs(o)), 1e-300)
            else:
                assert np.array_equal(g, o)
    # integer programs are exact, including the divisor-0 rules
    x, y = rnd((500,), np.int32), rnd((500,), np.int32)
    prog = [(1, O2["quot"], 0, 0, 1, 0), (1, O2["rem"], 0, 0, 1, 0), (1, O2["rem_scalar"], 0, 0, 1, 0), (1, O2["add"], 0, 2, 3, 0), (0, O1["signum"], 0, 5, 0, 0)]
    g = [o.numpy() for o in gpu.fused_map([gpu.upload(x), gpu.upload(y)], prog, [2, 3, 4, 6])]
    o = [o.numpy() for o in eval_program_eagerly(oracle, [oracle.upload(x), oracle.upload(y)], prog, [2, 3, 4, 6])]
    for a, b in zip(g, o):
        assert np.array_equal(a, b)
    with pytest.raises(capi.HgpuError):
        gpu.fused_map([gpu.upload(x)], [(0, O1["exp"], 0, 0, 0, 0)], [1])


@pytest.mark.parametrize("dt", [np.float64, np.float32])
def test_fused_map_dimsum_against_checker_and_numpy(gpu, oracle, dt):
    """hgpu_fused_map_dimsum: the cotangent of a convolution layer written out
    (example/MnistCnnShaped2.hs:57-63: the cotangent of the pooled, rectified
    output spread over the pooling windows under a mask) and, from the same
    pass, its sum over batch, height and width -- the bias's cotangent.  Dense
    inputs and broadcast views over a refined index space; every kept dim."""
    O2 = capi.OP2
    rng = np.random.default_rng(77)
    b, c, h, w = 24, 16, 14, 14
    pooled = rng.standard_normal((b, c, h, w)).astype(dt)
    mask = (rng.random((b, c, h, 2, w, 2)) < 0.3).astype(dt)
    scale = np.asarray(0.5, dt)
    prog = [(1, O2["mul"], 0, 0, 1, 0), (1, O2["mul"], 0, 3, 2, 0)]     # 3: pooled * mask, 4: ... * scale
    want_map = pooled[:, :, :, None, :, None].astype(np.float64) * mask * 0.5
    tol = TOL[np.dtype(dt)]
    for keep in (1, 0, 5, 2):
        res = []
        for ctx in (gpu, oracle):
            pv = ctx.upload(pooled).reshape([b, c, h, 1, w, 1]).as_strided([b, c, h, 2, w, 2], [c * h * w, h * w, w, 0, 1, 0], 0)
            ins = [pv, ctx.upload(mask), ctx.upload(scale).replicate([b, c, h, 2, w, 2])]
            outs, sm = ctx.fused_map_dimsum(ins, prog, [4], 4, keep)
            res.append((outs[0].numpy(), sm.numpy()))
        other = tuple(d for d in range(6) if d != keep)
        want_sum = want_map.sum(axis=other)
        scale_sum = np.abs(want_map).sum(axis=other).max()
        for got_map, got_sum in res:
            assert got_map.dtype == np.dtype(dt) and np.allclose(got_map, want_map, rtol=tol, atol=0)
            assert got_sum.shape == want_sum.shape and got_sum.dtype == np.dtype(dt)
            assert np.max(np.abs(got_sum - want_sum)) <= tol * scale_sum
        assert np.array_equal(res[0][0], res[1][0])
    # all inputs dense, the kept dim last (its elements are neighbours in memory: no vectors across it)
    x = rng.standard_normal((700, 500)).astype(dt)
    y = rng.standard_normal((700, 500)).astype(dt)
    for keep in (0, 1):
        outs, sm = gpu.fused_map_dimsum([gpu.upload(x), gpu.upload(y)], [(1, O2["mul"], 0, 0, 1, 0)], [2], 2, keep)
        prod = x.astype(np.float64) * y
        assert np.allclose(outs[0].numpy(), prod, rtol=tol, atol=0)
        assert np.max(np.abs(sm.numpy() - prod.sum(axis=1 - keep))) <= tol * np.abs(prod).sum(axis=1 - keep).max()
    # too small for the compiled kernel: refused, the caller runs the two steps
    with pytest.raises(capi.HgpuError):
        gpu.fused_map_dimsum([gpu.upload(x[:10]), gpu.upload(y[:10])], [(1, O2["mul"], 0, 0, 1, 0)], [2], 2, 0)
