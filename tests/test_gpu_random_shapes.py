"""Random shapes, layouts and programs for the two entry points whose kernels are
compiled for the shapes they are called with (hgpu_contract_sum_map,
hgpu_fused_map_dimsum), against numpy in double precision.  The cases are
drawn from fixed seeds."""
import numpy as np
import pytest

from conftest import capi

pytestmark = pytest.mark.gpu
O1, O2 = capi.OP1, capi.OP2


def matmul_views(w, x):
    m, n = w.shape[0], x.shape[1]
    return w.replicate([n]).transpose([1, 0]), x.replicate([m]).transpose([0, 2, 1])


@pytest.mark.parametrize("seed", range(32))
def test_sum_of_products_and_program_random_case(gpu, seed):
    rng = np.random.default_rng(seed)
    dt = np.float32 if rng.random() < 0.5 else np.float64
    m = int(rng.integers(4, 200)); n = int(rng.integers(16, 1500)); nt = int(rng.integers(1, 4))
    ks = [int(rng.integers(2, 200)) for _ in range(nt)]
    terms, want = [], np.zeros((m, n))
    for k in ks:
        w = rng.uniform(-0.5, 0.5, (m, k)).astype(dt); x = rng.uniform(-1, 1, (k, n)).astype(dt)
        wa = gpu.upload(w) if rng.random() < 0.5 else gpu.upload(np.ascontiguousarray(w.T)).transpose([1, 0])
        xa = gpu.upload(x) if rng.random() < 0.5 else gpu.upload(np.ascontiguousarray(x.T)).transpose([1, 0])
        terms.append(matmul_views(wa, xa))
        want += w.astype(np.float64) @ x.astype(np.float64)
    mode = int(rng.integers(0, 3))
    b = rng.uniform(-0.5, 0.5, (m,)).astype(dt); h = rng.uniform(-1, 1, (m, n)).astype(dt)
    if mode == 0:
        ins, prog, slots, wants = [None], [], [0], [want]
    elif mode == 1:
        ins = [None, gpu.upload(b).replicate([n]).transpose([1, 0])]
        prog, slots = [(1, O2["add"], 0, 0, 1, 0), (0, O1["tanh"], 0, 2, 0, 0)], [3]
        wants = [np.tanh(want + b.astype(np.float64)[:, None])]
    else:
        ins = [gpu.upload(h), None]
        prog, slots = [(1, O2["mul"], 0, 0, 0, 0), (1, O2["mul"], 0, 1, 2, 0)], [3, 1]
        wants = [want * (h.astype(np.float64) ** 2), want]
    outs = gpu.contract_sum_map(terms, 2, ins, prog, slots)
    tol = 1e-5 if dt == np.float32 else 1e-10
    for o, w_ in zip(outs, wants):
        g = o.numpy()
        assert g.shape == w_.shape and g.dtype == np.dtype(dt)
        # a sum of sum(ks) products: the bound grows with the number of terms added
        assert float(np.max(np.abs(g - w_))) <= 8 * tol * max(float(np.max(np.abs(w_))), 1e-30), (dt, m, n, ks, mode)


@pytest.mark.parametrize("seed", range(32))
def test_map_with_sum_over_all_dims_but_one_random_case(gpu, seed):
    rng = np.random.default_rng(seed)
    dt = np.float32 if rng.random() < 0.5 else np.float64
    rank = int(rng.integers(2, 6))
    top = int(round((1 << 20) ** (1.0 / rank))) * 2 + 2
    while True:
        shape = [int(rng.integers(1, top)) for _ in range(rank)]
        if (1 << 18) <= int(np.prod(shape)) <= (1 << 22):
            break
    keep = int(rng.integers(0, rank))
    x = rng.standard_normal(shape).astype(dt)
    bdims = [d for d in range(rank) if rng.random() < 0.4]            # y is replicated along these
    yshape = [1 if d in bdims else shape[d] for d in range(rank)]
    y = rng.standard_normal(yshape).astype(dt)
    dense_st = [int(np.prod(yshape[d + 1:])) for d in range(rank)]
    yv = gpu.upload(y).as_strided(shape, [0 if d in bdims else dense_st[d] for d in range(rank)], 0)
    if rng.random() < 0.5:                                             # x through a transpose
        perm = [int(p) for p in rng.permutation(rank)]
        xa = gpu.upload(np.ascontiguousarray(x.transpose(perm))).transpose([perm.index(d) for d in range(rank)])
    else:
        xa = gpu.upload(x)
    prog = [(1, O2["mul"], 0, 0, 1, 0), (0, O1["sin"], 0, 2, 0, 0)]
    slot = int(rng.integers(2, 4))
    outs, sm = gpu.fused_map_dimsum([xa, yv], prog, [3], slot, keep)
    prod = x.astype(np.float64) * y.astype(np.float64)
    want_map = np.sin(prod)
    val = prod if slot == 2 else want_map
    other = tuple(d for d in range(rank) if d != keep)
    want_sum, scale = val.sum(axis=other), np.abs(val).sum(axis=other).max()
    tol = 1e-5 if dt == np.float32 else 1e-10
    assert float(np.max(np.abs(outs[0].numpy() - want_map))) <= 8 * tol
    got = sm.numpy()
    assert got.shape == want_sum.shape and got.dtype == np.dtype(dt)
    assert float(np.max(np.abs(got - want_sum))) <= tol * max(scale, 1e-30), (dt, shape, keep, slot, bdims)
