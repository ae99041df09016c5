"""MI355X (gfx950) tensor backend for horde-ad's concrete-array hot path.

The product is the C ABI in include/hordead_gpu.h (HIP kernels, csrc/) and the
host layer above it (host/); this Python package only carries the ctypes
binding the test-suite and the benchmark driver use to reach them.
"""
from . import capi, hostapi, mnist_data, optimizer, workloads  # noqa: F401
