"""Pins the CPU checker (oracle/oracle.cpp) against what the mathematics fixes:
every array primitive is compared with an independent numpy formulation
(library routines: ufuncs, einsum, take/put, np.add.at) or with a brute-force
loop on small inputs.  Runs without a GPU.
"""
import itertools

import numpy as np
import pytest

from conftest import capi

RNG = np.random.default_rng(1234)
FLOATS = [np.float64, np.float32]
INTS = [np.int64, np.int32, np.int16, np.int8]


def rnd(shape, dtype):
    if np.dtype(dtype).kind == "f":
        return RNG.uniform(-2, 2, shape).astype(dtype)
    if np.dtype(dtype).kind == "b":
        return RNG.integers(0, 2, shape).astype(bool)
    return RNG.integers(-50, 50, shape).astype(dtype)


def test_roundtrip_and_metadata(oracle):
    for dt in FLOATS + INTS + [np.bool_]:
        x = rnd((3, 0, 2), dt)
        assert oracle.upload(x).numpy().shape == (3, 0, 2)
        x = rnd((2, 3, 4), dt)
        a = oracle.upload(x)
        assert a.shape == (2, 3, 4) and a.rank == 3 and np.array_equal(a.numpy(), x)
    s = oracle.upload(np.float64(3.5))
    assert s.rank == 0 and s.item() == 3.5


def test_views(oracle):
    x = rnd((3, 4, 5, 2), np.float64)
    a = oracle.upload(x)
    # stranspose: result dim i = source dim perm[i]; a short perm acts on the leading dims
    assert np.array_equal(a.transpose([2, 0, 1]).numpy(), np.transpose(x, (2, 0, 1, 3)))
    assert np.array_equal(a.transpose([1, 0]).numpy(), np.swapaxes(x, 0, 1))
    assert np.array_equal(a.reshape([12, 10]).numpy(), x.reshape(12, 10))
    assert np.array_equal(a.slice(1, 1, 2).numpy(), x[:, 1:3])
    assert np.array_equal(a.reverse(2).numpy(), x[:, :, ::-1])
    assert np.array_equal(a.replicate([2, 3]).numpy(), np.broadcast_to(x, (2, 3) + x.shape))
    assert np.array_equal(a.index_prefix([2, 1]).numpy(), x[2, 1])
    assert np.array_equal(a.index_prefix([3, 1]).numpy(), np.zeros((5, 2)))   # OOB => zeros
    assert np.array_equal(a.index_prefix([0, -1]).numpy(), np.zeros((5, 2)))
    assert np.array_equal(a.pad([1, 0, 2, 0], [0, 3, 0, 1]).numpy(),
                          np.pad(x, [(1, 0), (0, 3), (2, 0), (0, 1)]))
    # affine window: out[i, k] = v[i + k]
    v = rnd((9,), np.float64)
    w = oracle.upload(v).as_strided([6, 4], [1, 1], 0).numpy()
    assert np.array_equal(w, np.lib.stride_tricks.sliding_window_view(v, 4))
    with pytest.raises(capi.HgpuError):
        oracle.upload(v).as_strided([7, 4], [1, 1], 0)
    with pytest.raises(capi.HgpuError):
        a.transpose([0, 0])
    with pytest.raises(capi.HgpuError):
        a.reshape([7])


UNARY = {
    "neg": np.negative, "abs": np.abs, "signum": np.sign, "recip": np.reciprocal, "exp": np.exp,
    "sqrt": None, "log": None, "sin": np.sin, "cos": np.cos, "tan": np.tan, "asin": None, "acos": None,
    "atan": np.arctan, "sinh": np.sinh, "cosh": np.cosh, "tanh": np.tanh, "asinh": np.arcsinh,
    "acosh": None, "atanh": None,
}


@pytest.mark.parametrize("dt", FLOATS)
def test_unary_float(oracle, dt):
    eps = np.finfo(dt).eps
    x = rnd((7, 5), dt)
    pos = np.abs(x) + dt(0.1)
    unit = (x / dt(2.5)).astype(dt)
    cases = dict(UNARY)
    for op, fn in cases.items():
        arg = x
        if op in ("sqrt", "log"):
            arg, fn = pos, {"sqrt": np.sqrt, "log": np.log}[op]
        elif op in ("asin", "acos", "atanh"):
            arg, fn = unit, {"asin": np.arcsin, "acos": np.arccos, "atanh": np.arctanh}[op]
        elif op == "acosh":
            arg, fn = pos + dt(1), np.arccosh
        got = oracle.upload(arg).ewise1(op).numpy()
        want = fn(arg.astype(np.float64))
        assert got.dtype == dt
        assert np.allclose(got, want, rtol=8 * eps, atol=8 * eps), op


@pytest.mark.parametrize("dt", FLOATS)
def test_binary_float(oracle, dt):
    eps = np.finfo(dt).eps
    x, y = rnd((6, 4), dt), rnd((6, 4), dt)
    px, py = np.abs(x) + dt(0.5), np.abs(y) + dt(0.5)
    a, b, pa, pb = (oracle.upload(v) for v in (x, y, px, py))
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    for op, want in [("add", x64 + y64), ("mul", x64 * y64), ("sub", x64 - y64), ("div", x64 / y64),
                     ("atan2", np.arctan2(x64, y64)), ("min", np.minimum(x, y)), ("max", np.maximum(x, y))]:
        assert np.allclose(a.ewise2(op, b).numpy(), want, rtol=4 * eps, atol=4 * eps), op
    assert np.allclose(pa.ewise2("pow", b).numpy(), px.astype(np.float64) ** y64, rtol=16 * eps)
    # logBase x y = log y / log x
    assert np.allclose(pa.ewise2("logbase", pb).numpy(), np.log(py.astype(np.float64)) / np.log(px.astype(np.float64)),
                       rtol=64 * eps, atol=64 * eps)
    with pytest.raises(capi.HgpuError):
        a.ewise2("quot", b)
    with pytest.raises(capi.HgpuError):
        a.ewise2("add", oracle.upload(x[:3]))


@pytest.mark.parametrize("dt", INTS)
def test_integer_ops(oracle, dt):
    x, y = rnd((40,), dt), rnd((40,), dt)
    y[::7] = 0
    a, b = oracle.upload(x), oracle.upload(y)
    assert np.array_equal(a.ewise2("add", b).numpy(), (x + y).astype(dt))
    assert np.array_equal(a.ewise2("mul", b).numpy(), (x * y).astype(dt))
    assert np.array_equal(a.ewise1("neg").numpy(), -x)
    assert np.array_equal(a.ewise1("abs").numpy(), np.abs(x))
    assert np.array_equal(a.ewise1("signum").numpy(), np.sign(x))
    # Haskell quot/rem truncate toward zero; arrays replace a 0 divisor by 1
    y1 = np.where(y == 0, 1, y).astype(np.int64)
    x8 = x.astype(np.int64)
    q = (np.abs(x8) // np.abs(y1)) * np.sign(x8) * np.sign(y1)
    assert np.array_equal(a.ewise2("quot", b).numpy(), q.astype(dt))
    assert np.array_equal(a.ewise2("rem", b).numpy(), (x8 - q * y1).astype(dt))
    # the scalar rule keeps the dividend: remH a 0 = a
    rs = np.where(y == 0, x, (x8 - q * y1).astype(dt))
    assert np.array_equal(a.ewise2("rem_scalar", b).numpy(), rs)
    with pytest.raises(capi.HgpuError):
        a.ewise1("exp")


def test_bool_compare_select_convert(oracle):
    x, y = rnd((5, 6), np.float64), rnd((5, 6), np.float64)
    y[2] = x[2]
    a, b = oracle.upload(x), oracle.upload(y)
    le, eq, lt = (a.compare(c, b) for c in ("leq", "eq", "lt"))
    assert np.array_equal(le.numpy(), x <= y) and np.array_equal(eq.numpy(), x == y) and np.array_equal(lt.numpy(), x < y)
    assert np.array_equal(le.ewise1("not").numpy(), ~(x <= y))
    assert np.array_equal(le.ewise2("and", eq).numpy(), (x <= y) & (x == y))
    assert np.array_equal(le.select(a, b).numpy(), np.where(x <= y, x, y))
    # whole-array comparisons are lexicographic on the row-major sequence
    assert a.compare_all("eq", a) and a.compare_all("leq", a) and not a.compare_all("lt", a)
    for u, v in [([1, 2, 3], [1, 3, 0]), ([2, 0, 0], [1, 9, 9]), ([1, 2, 3], [1, 2, 3])]:
        au, av = oracle.upload(np.array(u, np.int64)), oracle.upload(np.array(v, np.int64))
        assert au.compare_all("leq", av) == (u <= v) and au.compare_all("lt", av) == (u < v) and au.compare_all("eq", av) == (u == v)
    # conversions
    f = np.array([-2.5, -0.5, 0.0, 0.5, 2.5, 7.99])
    af = oracle.upload(f)
    assert np.array_equal(af.convert(capi.I64, 1).numpy(), np.floor(f).astype(np.int64))
    assert np.array_equal(af.convert(capi.F32, 0).numpy(), f.astype(np.float32))
    i = rnd((9,), np.int32)
    assert np.array_equal(oracle.upload(i).convert(capi.F64, 0).numpy(), i.astype(np.float64))
    assert np.array_equal(oracle.upload(i).convert(capi.I8, 0).numpy(), i.astype(np.int8))


def test_contract_against_einsum(oracle):
    x, y = rnd((3, 4, 5, 6), np.float64), rnd((3, 4, 5, 6), np.float64)
    a, b = oracle.upload(x), oracle.upload(y)
    assert np.allclose(a.contract(None, 0).numpy(), x.sum(), rtol=1e-13)
    assert np.allclose(a.contract(b, 0).numpy(), np.einsum("abcd,abcd->", x, y), rtol=1e-13)
    assert np.allclose(a.contract(b, 3).numpy(), np.einsum("abcd,abcd->abc", x, y), rtol=1e-13)   # sdot1In
    assert np.allclose(a.contract(None, 2).numpy(), x.sum(axis=(2, 3)), rtol=1e-13)
    # tssum sums the OUTER dim: transpose it behind, keep the rest
    assert np.allclose(a.transpose([1, 2, 3, 0]).contract(None, 3).numpy(), x.sum(axis=0), rtol=1e-13)
    # tsmatmul2 m1 m2 = dot1In (tr (replicate m1)) (tr (replicate m2)) (OpsConcrete.hs:237-242)
    m1, m2 = rnd((4, 7), np.float64), rnd((7, 5), np.float64)
    lhs = oracle.upload(m1).replicate([5]).transpose([1, 0])
    rhs = oracle.upload(m2).replicate([4]).transpose([0, 2, 1])
    assert np.allclose(lhs.contract(rhs, 2).numpy(), m1 @ m2, rtol=1e-13)
    # integers wrap like the element type does
    i = rnd((50, 9), np.int8)
    assert np.array_equal(oracle.upload(i).contract(None, 1).numpy(), i.sum(axis=1, dtype=np.int8))
    assert oracle.upload(rnd((0, 3), np.float64)).contract(None, 0).numpy() == 0.0
    assert np.array_equal(oracle.upload(rnd((2, 0), np.float64)).contract(None, 1).numpy(), np.zeros(2))


def test_argminmax_iota_concat_onehot(oracle):
    x = rnd((4, 5, 6), np.float64)
    x[1, 2, 3] = x[1, 2, 0]  # a tie: the first occurrence wins
    a = oracle.upload(x)
    assert np.array_equal(a.argminmax_last(False).numpy(), np.argmin(x, axis=-1))
    assert np.array_equal(a.argminmax_last(True).numpy(), np.argmax(x, axis=-1))
    t = np.array([3, 1, 1, 3, 0, 0], np.int32)
    assert oracle.upload(t).argminmax_last(True).item() == 0 and oracle.upload(t).argminmax_last(False).item() == 4
    assert np.array_equal(oracle.iota(7, capi.F32).numpy(), np.arange(7, dtype=np.float32))
    parts = [rnd((k, 3), np.float64) for k in (2, 0, 4)]
    assert np.array_equal(oracle.concat([oracle.upload(p) for p in parts]).numpy(), np.concatenate(parts))
    v = rnd((2, 3), np.float64)
    want = np.zeros((4, 5, 2, 3))
    want[3, 1] = v
    assert np.array_equal(oracle.upload(v).onehot([3, 1], [4, 5]).numpy(), want)
    assert np.array_equal(oracle.upload(v).onehot([4, 1], [4, 5]).numpy(), np.zeros((4, 5, 2, 3)))


def brute_gather(src, ix, shm):
    n_ix = len(ix)
    out = np.zeros(tuple(shm) + src.shape[n_ix:], src.dtype)
    for m in itertools.product(*[range(s) for s in shm]):
        p = tuple(int(i[m]) for i in ix)
        if all(0 <= p[k] < src.shape[k] for k in range(n_ix)):
            out[m] = src[p]
    return out


def brute_scatter(src, ix, rank_m, shp):
    out = np.zeros(tuple(shp) + src.shape[rank_m:], src.dtype)
    for m in itertools.product(*[range(s) for s in src.shape[:rank_m]]):
        p = tuple(int(i[m]) for i in ix)
        if all(0 <= p[k] < shp[k] for k in range(len(shp))):
            out[p] += src[m]
    return out


def test_gather_scatter_bruteforce(oracle):
    src = rnd((5, 4, 3), np.float64)
    shm = (6, 2)
    ix = [RNG.integers(-1, 6, shm), RNG.integers(-1, 5, shm)]   # includes out-of-bounds
    a = oracle.upload(src)
    g = oracle.gather(a, [oracle.upload(i) for i in ix], shm).numpy()
    assert np.array_equal(g, brute_gather(src, ix, shm))
    # full-rank gather (scalars) and rank-0 position space
    ix3 = ix + [RNG.integers(0, 3, shm)]
    assert np.array_equal(oracle.gather(a, [oracle.upload(i) for i in ix3], shm).numpy(), brute_gather(src, ix3, shm))
    data = rnd((6, 2, 3), np.float64)
    shp = (5, 4)
    s = oracle.scatter_add(oracle.upload(data), [oracle.upload(i) for i in ix], 2, shp).numpy()
    assert np.allclose(s, brute_scatter(data, ix, 2, shp), rtol=1e-14)
    # integers: exact, also with collisions
    idata = rnd((50,), np.int64)
    iix = [RNG.integers(-2, 5, (50,))]
    s = oracle.scatter_add(oracle.upload(idata), [oracle.upload(iix[0])], 1, (4,)).numpy()
    assert np.array_equal(s, brute_scatter(idata, iix, 1, (4,)))
    # against numpy's own ordered scatter-add
    want = np.zeros(4, np.int64)
    ok = (iix[0] >= 0) & (iix[0] < 4)
    np.add.at(want, iix[0][ok], idata[ok])
    assert np.array_equal(s, want)


def test_scatter_affine_bruteforce(oracle):
    """The affine form agrees with the brute-force scatter fed the same indices as arrays."""
    # pooling windows: (i, p, j, q, n) -> (2 i + p, 2 j + q), a bijection
    src = rnd((3, 2, 4, 2, 5), np.float64)
    c0, coef, shp = [0, 0], [[2, 0], [1, 0], [0, 2], [0, 1]], (6, 8)
    got = oracle.scatter_affine(oracle.upload(src), 4, c0, coef, shp).numpy()
    grid = np.indices(src.shape[:4])
    ix = [c0[j] + sum(coef[d][j] * grid[d] for d in range(4)) for j in range(2)]
    assert np.array_equal(got, brute_scatter(src, ix, 4, shp))
    # offsets, a negative coefficient, and places that stay zero
    src = rnd((4, 3), np.int32)
    c0, coef, shp = [9, 1], [[-2, 0], [0, 3]], (11, 9)
    got = oracle.scatter_affine(oracle.upload(src), 2, c0, coef, shp).numpy()
    grid = np.indices(src.shape)
    ix = [c0[j] + sum(coef[d][j] * grid[d] for d in range(2)) for j in range(2)]
    assert np.array_equal(got, brute_scatter(src, ix, 2, shp))
    assert np.count_nonzero(got) <= src.size
    # a position outside the bounds is an error, not a skipped position
    with pytest.raises(capi.HgpuError):
        oracle.scatter_affine(oracle.upload(src), 2, [9, 1], coef, (9, 9))


def test_gather_scatter_adjoint(oracle):
    """<gather x f, y> == <x, scatter y f> (bench/ConvVjpBench.hs:564-584)."""
    x, shm = rnd((7, 6, 2), np.float64), (5, 3)
    ix = [RNG.integers(-1, 8, shm), RNG.integers(0, 6, shm)]
    y = rnd(shm + (2,), np.float64)
    aix = [oracle.upload(i) for i in ix]
    g = oracle.gather(oracle.upload(x), aix, shm).numpy()
    s = oracle.scatter_add(oracle.upload(y), aix, 2, (7, 6)).numpy()
    assert np.isclose((g * y).sum(), (x * s).sum(), rtol=1e-12)


def test_materialize_assign_contract_sum_fused_map(oracle):
    """The entry points that are compositions of the ones above, each against its own numpy statement."""
    x = rnd((4, 6, 5), np.float64)
    a = oracle.upload(x)
    # materialize: the logical contents of a view, densely
    v = a.transpose([2, 0, 1]).slice(1, 1, 3).reverse(0)
    assert np.array_equal(v.materialize().numpy(), np.transpose(x, (2, 0, 1))[:, 1:4][::-1])
    # assign: dst's memory takes src's elements
    dst = oracle.upload(np.zeros((5, 3, 6)))
    dst.assign(v)
    assert np.array_equal(dst.numpy(), np.transpose(x, (2, 0, 1))[:, 1:4][::-1])
    with pytest.raises(capi.HgpuError):
        dst.assign(a)                                       # another shape
    # contract_sum: the sum over the pairs of the pairwise contractions
    for dt, tol in ((np.float64, 1e-12), (np.float32, 1e-5), (np.int64, 0)):
        pairs = [(rnd((3, 4, 7), dt), rnd((3, 4, 7), dt)) for _ in range(5)]
        for keep, spec in ((2, "ijk,ijk->ij"), (1, "ijk,ijk->i"), (0, "ijk,ijk->"), (3, "ijk,ijk->ijk")):
            want = sum(np.einsum(spec, p.astype(np.float64) if tol else p, q.astype(np.float64) if tol else q) for p, q in pairs)
            got = oracle.contract_sum([(oracle.upload(p), oracle.upload(q)) for p, q in pairs], keep).numpy()
            assert got.dtype == np.dtype(dt)
            if tol == 0:
                assert np.array_equal(got, want)
            else:
                assert np.max(np.abs(got - want)) <= tol * max(1.0, float(np.max(np.abs(want))))
    # fused_map: the single operations in program order; slots: 0 x, 1 y, 2 = x * y, 3 = sin 2, 4 = (3 <= x), 5 = 4 ? y : 3, 6 = floor 5 as Int
    O1, O2, CMP = capi.OP1, capi.OP2, capi.CMP
    xx, yy = rnd((6, 7), np.float64), rnd((6, 7), np.float64)
    prog = [(1, O2["mul"], 0, 0, 1, 0), (0, O1["sin"], 0, 2, 0, 0), (2, CMP["leq"], 0, 3, 0, 0), (3, 0, 0, 4, 1, 3), (4, 1, capi.I64, 5, 0, 0)]
    outs = oracle.fused_map([oracle.upload(xx), oracle.upload(yy)], prog, [3, 4, 5, 6, 0])
    s = np.sin(xx * yy)
    assert np.array_equal(outs[0].numpy(), s) and np.array_equal(outs[1].numpy(), s <= xx)
    sel = np.where(s <= xx, yy, s)
    assert np.array_equal(outs[2].numpy(), sel) and np.array_equal(outs[3].numpy(), np.floor(sel).astype(np.int64))
    assert np.array_equal(outs[4].numpy(), xx)


def test_fused_table_definitions(oracle):
    """The checker's second table defines the optional fused entry points by
    composition; each is pinned here against numpy, as the plain ones are above."""
    lib = capi.Lib(oracle.lib.path, "horc_")
    dll = lib.dll
    import ctypes as C
    O1, O2, CMP = capi.OP1, capi.OP2, capi.CMP
    P, PP, I, LP, IP = C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int)
    x = rnd((3, 4, 2, 3), np.float64)
    x[1, 2] = x[1, 2, 0, 0]                                  # a window of equal values: the first one wins
    a = oracle.upload(x)
    # extremum_last / fused_extremum: first extremum over the trailing dims taken together
    fe = dll.horc_fused_extremum
    fe.restype, fe.argtypes = I, [P, I, PP, I, P, I, I, I, PP, PP]
    ins = (C.c_void_p * 1)(a.h)
    prog = [(0, O1["neg"], 0, 0, 0, 0)]
    flat = (C.c_int32 * 6)(*[int(v) for q in prog for v in q])
    for want_max in (1, 0):
        v, i = C.c_void_p(), C.c_void_p()
        assert fe(oracle.h, 1, ins, 1, flat, 1, 2, want_max, C.byref(v), C.byref(i)) == 0
        gv, gi = capi.Array(oracle, v).numpy(), capi.Array(oracle, i).numpy()
        w = (-x).reshape(3, 4, 6)
        assert np.array_equal(gi, w.argmax(-1) if want_max else w.argmin(-1))
        assert np.array_equal(gv, w.max(-1) if want_max else w.min(-1))
    assert gi[1, 2] == 0
    # fused_sum and fused_map_sums: sums of a slot's values
    fs = dll.horc_fused_sum
    fs.restype, fs.argtypes = I, [P, I, PP, I, P, I, PP]
    o = C.c_void_p()
    assert fs(oracle.h, 1, ins, 1, flat, 1, C.byref(o)) == 0
    assert abs(capi.Array(oracle, o).numpy() - (-x).sum()) <= 1e-12
    # fused_map_dimsum: the program's results, and one slot summed over every dim but one
    fd = dll.horc_fused_map_dimsum
    fd.restype, fd.argtypes = I, [P, I, PP, I, P, I, C.POINTER(C.c_int), PP, I, I, PP]
    x3 = x.reshape(3, 4, 6)
    a3 = oracle.upload(x3)
    ins3 = (C.c_void_p * 1)(a3.h)
    for keep in range(3):
        outs, sm = (C.c_void_p * 1)(), C.c_void_p()
        assert fd(oracle.h, 1, ins3, 1, flat, 1, (C.c_int * 1)(1), outs, 1, keep, C.byref(sm)) == 0
        assert np.array_equal(capi.Array(oracle, C.c_void_p(outs[0])).numpy(), -x3)
        other = tuple(d for d in range(3) if d != keep)
        assert np.allclose(capi.Array(oracle, sm).numpy(), (-x3).sum(axis=other), rtol=1e-13, atol=1e-13)
    # contract_operands: program, merged dims, zero-extension, view, contraction
    y = rnd((2, 3, 4), np.float64)
    z = rnd((2, 3, 4), np.float64)
    op = oracle.operand([oracle.upload(y), oracle.upload(z)], [(1, O2["mul"], 0, 0, 1, 0)], 2, [2, 12], ([14, 2], [1, 14], 0), pad=([0, 1], [0, 1]))
    co = dll.horc_contract_operands
    co.restype, co.argtypes = I, [P, P, P, I, I, PP]
    o = C.c_void_p()
    assert co(oracle.h, C.byref(op), None, 1, 0, C.byref(o)) == 0
    padded = np.pad((y * z).reshape(2, 12), [(0, 0), (1, 1)])
    assert np.allclose(capi.Array(oracle, o).numpy(), padded.T.sum(axis=1), rtol=1e-13, atol=1e-13)
