"""The random programs of test_host_random_programs.py without a device: the
host layer with deferral on, on both of the checker's tables (on the one with
the composed entry points pending work fuses as it does on the device),
against the host layer with deferral off (every operation at once)."""
import numpy as np
import pytest

from conftest import capi, entry
import test_host_random_programs as tp


def check(seed, extended, maps=False):
    shape, steps, _ = tp.random_program(seed, extended=extended, maps=maps)
    x0 = np.random.default_rng(1000 + seed).uniform(-1, 1, shape)
    want = tp.run(tp.reference_host(), x0, steps)
    for table in ("get_api", "get_api_fused"):
        got = tp.run(tp.H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table=table)), x0, steps)
        for a, b in zip(got[0], want[0]):
            assert a.shape == b.shape and np.allclose(a, b, rtol=1e-11, atol=1e-12), (table, steps)
        assert np.isclose(got[1], want[1], rtol=1e-11), (table, steps)
        assert np.allclose(got[2], want[2], rtol=1e-10, atol=1e-11), (table, steps)


# 683: a pending product under an elementwise program, and a view of that product among the later leaves of the same
# program -- the walk that numbers the program computed the product for the view, and the fused call then found it gone
@pytest.mark.parametrize("seed", [0, 7, 19, 683, 1204])
def test_random_program_matches_every_operation_at_once(seed):
    check(seed, False)


# Programs that also hold dense layers (one or two matrix products, bias, tanh) and sums over all dims but one.
# 1, 57, 251: computing a leaf ran another program that wrote out (and took apart) nodes of the program being numbered;
# results were wrong without any error, or arrays were used after their release -- leaves are now all computed before
# the numbering walk, which computes nothing (settle_leaves)
@pytest.mark.parametrize("seed", [1, 57, 251] + list(range(2, 40)))
def test_random_program_with_layers_matches_every_operation_at_once(seed):
    check(seed, True)


# Programs that also map and zip scalar closures over arrays (the closure runs once, on lane values, and its
# arithmetic joins the deferred elementwise program) and build arrays from the position variables.
@pytest.mark.parametrize("seed", range(40))
def test_random_program_with_maps_and_builds_matches_every_operation_at_once(seed):
    check(seed, True, maps=True)


@pytest.mark.parametrize("seed", range(12))
def test_random_program_with_layers_single_precision(seed):
    shape, steps, _ = tp.random_program(seed, extended=True)
    x0 = np.random.default_rng(1000 + seed).uniform(-1, 1, shape).astype(np.float32)
    want = tp.run(tp.reference_host(), x0, steps)
    got = tp.run(tp.H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused")), x0, steps)
    for a, b in zip(got[0], want[0]):
        assert a.shape == b.shape and a.dtype == b.dtype == np.float32
        assert np.allclose(a, b, rtol=2e-4, atol=2e-4 * max(1.0, float(np.max(np.abs(b))) if b.size else 1.0)), steps
    assert np.isclose(got[1], want[1], rtol=1e-3), steps
    assert np.allclose(got[2], want[2], rtol=1e-3, atol=1e-3 * max(1.0, float(np.max(np.abs(want[2]))))), steps
