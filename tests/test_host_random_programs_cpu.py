"""The random programs of test_host_random_programs.py without a device: the
host layer on the checker's table of composed entry points (where pending
work fuses as it does on the device) against its plain table (every operation
at once)."""
import numpy as np
import pytest

from conftest import capi, entry
import test_host_random_programs as tp


# 683: a pending product under an elementwise program, and a view of that product among the later leaves of the same
# program -- the walk that numbers the program computed the product for the view, and the fused call then found it gone
@pytest.mark.parametrize("seed", [0, 7, 19, 683, 1204])
def test_random_program_fused_table_matches_plain_table(seed):
    shape, steps, _ = tp.random_program(seed)
    x0 = np.random.default_rng(1000 + seed).uniform(-1, 1, shape)
    plain = tp.run(tp.H.Host(capi.Lib(entry.ORACLE_LIB, "horc_")), x0, steps)
    fused = tp.run(tp.H.Host(capi.Lib(entry.ORACLE_LIB, "horc_", api_table="get_api_fused")), x0, steps)
    for a, b in zip(fused[0], plain[0]):
        assert a.shape == b.shape and np.allclose(a, b, rtol=1e-11, atol=1e-12), steps
    assert np.isclose(fused[1], plain[1], rtol=1e-11), steps
    assert np.allclose(fused[2], plain[2], rtol=1e-10, atol=1e-11), steps
