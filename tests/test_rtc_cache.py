"""Kernels compiled at run time are kept on disk: a second context (or process)
reads the code object back instead of compiling again.  The directory comes
from HORDEAD_GPU_CACHE; `off` means no files."""
import os
import time

import numpy as np
import pytest

from conftest import capi


def run_program(ctx, x, constant):
    """x * constant + sin x as one fused program; the constant makes the source unique to this test"""
    O1, O2 = capi.OP1, capi.OP2
    c = ctx.upload(np.float64(constant)).replicate(list(x.shape))
    prog = [(1, O2["mul"], 0, 0, 1, 0), (0, O1["sin"], 0, 0, 0, 0), (1, O2["add"], 0, 2, 3, 0), (0, O1["tanh"], 0, 4, 0, 0)]
    t0 = time.perf_counter()
    out = ctx.fused_map([ctx.upload(x), c], prog, [5])[0].numpy()
    return out, time.perf_counter() - t0


@pytest.mark.gpu
def test_compiled_kernels_are_kept_on_disk(tmp_path, monkeypatch):
    x = np.linspace(-2, 2, 4097)
    want = np.tanh(x * 1.25 + np.sin(x))
    lib = capi.Lib()
    monkeypatch.setenv("HORDEAD_GPU_CACHE", str(tmp_path))
    got1, t1 = run_program(lib.context(0), x, 1.25)
    files = sorted(os.listdir(tmp_path))
    assert len(files) == 1 and files[0].endswith(".co"), files
    stamp = os.stat(tmp_path / files[0]).st_mtime_ns
    got2, t2 = run_program(lib.context(0), x, 1.25)          # a new context: nothing compiled in memory
    assert np.array_equal(got1, got2) and np.max(np.abs(got1 - want)) <= 1e-12
    assert sorted(os.listdir(tmp_path)) == files and os.stat(tmp_path / files[0]).st_mtime_ns == stamp
    # a damaged file is not trusted: compiled again and replaced
    with open(tmp_path / files[0], "wb") as f:
        f.write(b"not a code object")
    got3, _ = run_program(lib.context(0), x, 1.25)
    assert np.array_equal(got1, got3) and os.path.getsize(tmp_path / files[0]) > 1000
    # no cache on request
    monkeypatch.setenv("HORDEAD_GPU_CACHE", "off")
    for f in os.listdir(tmp_path):
        os.remove(tmp_path / f)
    got4, _ = run_program(lib.context(0), x, 1.25)
    assert np.array_equal(got1, got4) and os.listdir(tmp_path) == []


def test_run_time_compiler_has_one_option_set():
    """Every run-time compile uses the full option list (packed FP32 off): no
    second attempt under other options than the cache key names."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = open(os.path.join(root, "horde-ad_amd", "csrc", "runtime.hip")).read()
    assert src.count("hiprtcCompileProgram(") == 1
    opts = src[src.index("kRtcOpts[] = {"):]
    opts = opts[:opts.index("};")]
    assert '"-packed-fp32-ops"' in opts and '"-target-feature"' in opts
