"""finchmoe_amd — MI355X (gfx950) kernels for FinchMoE's quantized-expert operator path.

The product is libfinchhip.so (HIP kernels behind the C ABI of include/finch_hip.h)
plus libfinchops.so (C host layer with the reference's own operator names).
This package holds the build script, a ctypes binding used by tests and bench.py,
and numpy helpers for the reference's packed formats.
"""
from .binding import FinchHip, FinchError, lib_path  # noqa: F401
from . import formats  # noqa: F401
