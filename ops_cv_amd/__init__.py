"""MI355X-native bilinear gather/interpolate path of ops-cv behind the aclnn two-phase C API.

The product is the shared library ``libopscv_amd.so`` (HIP kernels for gfx950 plus the C-ABI host layer,
sources under ``csrc/``).  This package is the thin ctypes binding used by the tests and the benchmark;
PyTorch only supplies device memory and streams.
"""
from . import aclnn  # noqa: F401
from .aclnn import (  # noqa: F401
    grid_sampler2d,
    upsample_bilinear2d,
    grid_sampler2d_taps,
    load_library,
    library_path,
)
