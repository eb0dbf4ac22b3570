"""grape_amd — MI355X (gfx950) implementation of the Grape proving hot path.

The product is the HIP shared library ``libgrape_hip.so`` (C ABI in ``include/grape_hip.h``)
and the C++ host classes in ``grape_amd/host``.  This Python package only builds and loads the
library and offers thin helpers over device memory for the tests and the benchmark.
"""
from ._capi import GrapeError, load, LIB_PATH  # noqa: F401
