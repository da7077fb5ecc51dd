"""MI355X (gfx950) implementation of arraydiff_cuda's spatially-parallel convolution path.

The product is the C-ABI shared library ``libadh.so`` (declared in ``include/adh_capi.h``)
and the C++ host classes in ``arraydiff_cuda_amd/host``.  This Python package is only the
ctypes binding used by the tests and the benchmark; torch supplies device memory and streams.
"""
from . import capi  # noqa: F401
from .capi import lib, check, ADH_F32, ADH_BF16  # noqa: F401
