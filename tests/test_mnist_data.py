"""IDX ingest (example/MnistData.hs:134-171): synthetic files written here in
the IDX format, decoded on the device, against the reference's host-side rule
(glyph byte / 255, one-hot label of ten)."""
import gzip
import struct

import numpy as np
import pytest

from conftest import capi, entry, pkg

H, M = pkg.hostapi, pkg.mnist_data
RNG = np.random.default_rng(3)


def write_idx(path, arr, compress):
    body = struct.pack(">HBB", 0, 0x08, arr.ndim) + struct.pack(">" + "I" * arr.ndim, *arr.shape) + arr.astype(np.uint8).tobytes()
    with open(path, "wb") as f:
        f.write(gzip.compress(body) if compress else body)


def check(host, tmp_path):
    n = 37
    glyphs = RNG.integers(0, 256, (n, 28, 28)).astype(np.uint8)
    labels = RNG.integers(0, 10, n).astype(np.uint8)
    write_idx(tmp_path / "g.gz", glyphs, True)
    write_idx(tmp_path / "l", labels, False)
    data = M.loadMnistData(host, str(tmp_path / "g.gz"), str(tmp_path / "l"))
    assert data.n == n and data.glyph_size == 784
    for dt, npdt in ((capi.F64, np.float64), (capi.F32, np.float32)):
        g, onehot = data.batch(5, 16, dt)
        want_g = (glyphs[5:21].reshape(16, 784).astype(npdt) / npdt(255)).T
        assert np.allclose(g.numpy(), want_g, rtol=1e-6 if npdt == np.float32 else 1e-15)
        want_l = np.zeros((10, 16), npdt)
        want_l[labels[5:21], np.arange(16)] = 1
        assert np.array_equal(onehot.numpy(), want_l)
        im, _ = data.batch_images(0, 4, dt)
        assert np.allclose(im.numpy(), glyphs[:4].reshape(4, 1, 28, 28).astype(npdt) / npdt(255), rtol=1e-6)
    with pytest.raises(ValueError):
        M.decodeIDX(b"\x00\x01\x08\x01\x00\x00\x00\x01\x00")
    with pytest.raises(ValueError):
        M.readMnistData(host, (tmp_path / "g.gz").read_bytes()[:10], b"")


def test_idx_ingest_cpu(tmp_path):
    check(H.Host(capi.Lib(entry.ORACLE_LIB, "horc_")), tmp_path)


@pytest.mark.gpu
def test_idx_ingest_gpu(tmp_path):
    check(H.Host(), tmp_path)
