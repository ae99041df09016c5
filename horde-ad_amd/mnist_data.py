"""MNIST in IDX form, decoded onto the device: the interface of the
reference's example/MnistData.hs (:134-171 readMnistData / loadMnistData,
:120-132 mkMnistDataS / mkMnistDataBatchS).

The reference decodes on the host: every glyph becomes a vector of
`fromIntegral byte / 255` and every label a one-hot vector of ten, one list
element per sample.  Here the raw bytes are uploaded once (as 16-bit integers)
and both conversions run on the device, a batch at a time, so the float data
set never exists on the host.
"""
import gzip
import struct

import numpy as np

from . import capi

sizeMnistLabelInt = 10          # MnistData.hs:24
sizeMnistHeightInt = 28         # MnistData.hs:27
sizeMnistWidthInt = 28          # MnistData.hs:31
sizeMnistGlyphInt = sizeMnistHeightInt * sizeMnistWidthInt


def decodeIDX(content):
    """An IDX file of unsigned bytes (magic 0x0000 08 <rank>, big-endian extents) as a numpy array."""
    if len(content) < 4:
        raise ValueError("wrong MNIST glyphs file")
    zero, dtype_code, rank = struct.unpack(">HBB", content[:4])
    if zero != 0 or dtype_code != 0x08:
        raise ValueError("wrong MNIST glyphs file")
    shape = struct.unpack(">" + "I" * rank, content[4:4 + 4 * rank])
    data = np.frombuffer(content, dtype=np.uint8, offset=4 + 4 * rank)
    if data.size != int(np.prod(shape)):
        raise ValueError("wrong MNIST glyphs file")
    return data.reshape(shape)


def decodeIDXLabels(content):
    labels = decodeIDX(content)
    if labels.ndim != 1:
        raise ValueError("wrong MNIST labels file")
    return labels


def _read(path):
    with open(path, "rb") as f:
        raw = f.read()
    return gzip.decompress(raw) if raw[:2] == b"\x1f\x8b" else raw


class MnistDevice:
    """The data set resident on the device as integers; batches are decoded there."""

    def __init__(self, host, glyphs, labels):
        if glyphs.shape[0] != labels.shape[0]:
            raise ValueError("can't decode MNIST file into integers")
        self.host = host
        self.n = int(glyphs.shape[0])
        self.glyph_size = int(np.prod(glyphs.shape[1:]))
        self.glyphs = host.concrete(glyphs.reshape(self.n, self.glyph_size).astype(np.int16))
        self.labels = host.concrete(labels.astype(np.int64))

    def batch(self, start, size, dtype=capi.F64):
        """(glyphs [glyph_size, size], one-hot labels [10, size]) of samples start .. start + size - 1,
        columns as in the fully connected examples (MnistFcnnRanked2.hs:52-77)."""
        host = self.host
        g = self.glyphs.sslice(start, size).sfromIntegral(dtype)
        g = (g * host.srepl(g.shape, 1.0 / 255.0, dtype)).str_()
        lab = self.labels.sslice(start, size).sreplicate(sizeMnistLabelInt)          # [10, size]
        cls = host.siota(sizeMnistLabelInt).sreplicate(size).str_()                  # [10, size]: the row's class
        one, zero = host.srepl(lab.shape, 1.0, dtype), host.srepl(lab.shape, 0.0, dtype)
        return g, lab.eq(cls).select(one, zero)

    def batch_images(self, start, size, dtype=capi.F64):
        """Glyphs as [size, 1, 28, 28] for the convolutional examples (MnistCnnShaped2.hs:45-136)."""
        g, onehot = self.batch(start, size, dtype)
        return g.str_().sreshape([size, 1, sizeMnistHeightInt, sizeMnistWidthInt]), onehot


def readMnistData(host, glyphs_bytes, labels_bytes):
    """MnistData.hs:134-154 on decompressed file contents."""
    return MnistDevice(host, decodeIDX(glyphs_bytes), decodeIDXLabels(labels_bytes))


def loadMnistData(host, glyphsPath, labelsPath):
    """MnistData.hs:162-171: the two (optionally gzip-compressed) IDX files."""
    return readMnistData(host, _read(glyphsPath), _read(labelsPath))
