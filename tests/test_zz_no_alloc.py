"""hgpu_contract_noalloc: the contraction for callers that cannot allocate
device memory.  Its partial sums live in one fixed array per device; every call
is checked against hgpu_contract on the same operands, twice in a row, the
second call on a smaller input (the array keeps the first call's contents).
Partial sums that would not fit the array run in fewer chunks."""
import numpy as np
import pytest

from conftest import capi


def both_ways(gpu, a, b, n_keep):
    """(hgpu_contract, hgpu_contract_noalloc) on the same operands.  The entry point under
    test runs FIRST and on a context of its own whose block cache is empty, so that any block
    it asked the allocator for would be a counted device allocation (a cached block left by an
    earlier hgpu_contract of the same size would hide it)."""
    fresh = capi.Lib().context(0)
    fa = fresh.upload(a)
    fb = fresh.upload(b) if b is not None else None
    out = fresh.upload(np.full(a.shape[:n_keep], 7, a.dtype))     # the caller's array, holding junk
    fresh.sync()
    before = fresh.mem_stats()
    fa.contract_noalloc(fb, n_keep, out)
    fresh.sync()
    assert fresh.mem_stats()[2] == before[2], "hgpu_contract_noalloc allocated device memory"
    got = out.numpy()
    del fa, fb, out
    fresh.shutdown()
    ga = gpu.upload(a)
    gb = gpu.upload(b) if b is not None else None
    want = ga.contract(gb, n_keep)
    return want.numpy(), got


@pytest.mark.gpu
def test_no_alloc_contract_matches_contract_twice_in_a_row(gpu):
    rng = np.random.default_rng(7)
    # a split reduction (few outputs, long sums): partial sums go through the fixed array
    a1 = rng.standard_normal((16, 300000))
    w1, g1 = both_ways(gpu, a1, None, 1)
    assert np.array_equal(w1, g1)
    assert np.allclose(g1, a1.sum(axis=1), rtol=1e-10, atol=1e-9)
    # the second call, smaller, right behind the first: the array still holds the first call's partial sums
    a2 = rng.standard_normal((5, 70001))
    b2 = rng.standard_normal((5, 70001))
    w2, g2 = both_ways(gpu, a2, b2, 1)
    assert np.array_equal(w2, g2)
    assert np.allclose(g2, (a2 * b2).sum(axis=1), rtol=1e-10, atol=1e-9)
    # integers are exact, and a whole-array sum (rank-0 result) works too
    a3 = rng.integers(-1000, 1000, (3, 4099, 17)).astype(np.int64)
    w3, g3 = both_ways(gpu, a3, None, 0)
    assert np.array_equal(w3, g3) and int(g3) == int(a3.sum())
    # fp32, dot over the innermost dim of strided views
    a4 = rng.standard_normal((40, 9000)).astype(np.float32)
    ga = gpu.upload(a4).transpose([1, 0]).transpose([1, 0])
    want = ga.contract(ga, 1)
    out = gpu.upload(np.zeros(40, np.float32))
    ga.contract_noalloc(ga, 1, out)
    assert np.array_equal(want.numpy(), out.numpy())
    assert np.max(np.abs(out.numpy() - (a4.astype(np.float64) ** 2).sum(axis=1))) <= 1e-5 * np.max((a4.astype(np.float64) ** 2).sum(axis=1))


@pytest.mark.gpu
def test_no_alloc_contract_with_fewer_chunks_than_it_would_like(gpu):
    # sums over the outer dim of [16384, 5000]: hgpu_contract cuts 5000 outputs into 53 chunks (2.1 MB of
    # partial sums); the fixed 1 MiB holds 26, so the call runs with 26: integers exact, floats within rounding
    a8 = np.ones((16384, 5000), np.int8)
    a = gpu.upload(a8).transpose([1, 0])
    out = gpu.upload(np.zeros(5000, np.int8))
    a.contract_noalloc(None, 1, out)
    assert np.array_equal(out.numpy(), np.full(5000, 16384 % 256, np.int64).astype(np.int8))
    assert np.array_equal(a.contract(None, 1).numpy(), out.numpy())
    x = np.random.default_rng(11).standard_normal((16384, 5000))
    gx = gpu.upload(x).transpose([1, 0])
    outx = gpu.upload(np.zeros(5000))
    gx.contract_noalloc(None, 1, outx)
    np.testing.assert_allclose(outx.numpy(), x.sum(axis=0), rtol=1e-10, atol=1e-9)
    # so many outputs that not even two chunks fit: one unsplit launch, no scratch
    y = np.random.default_rng(12).standard_normal((600, 70000))
    gy = gpu.upload(y).transpose([1, 0])
    outy = gpu.upload(np.zeros(70000))
    gy.contract_noalloc(None, 1, outy)
    np.testing.assert_allclose(outy.numpy(), y.sum(axis=0), rtol=1e-10, atol=1e-9)
    # a result array of the wrong shape is an argument error
    with pytest.raises(capi.HgpuError) as e2:
        a.contract_noalloc(None, 1, gpu.upload(np.zeros(3, np.int8)))
    assert e2.value.code == 1
