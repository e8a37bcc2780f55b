"""sptmm_amd -- MI355X (gfx950) SpTMM engine; Python binding of the C ABI.

The package is a thin ctypes mirror of include/sptmm.h.  There is no CPU
fallback: without the built HIP library every call fails.
"""
from ._capi import *  # noqa: F401,F403
from ._capi import __all__  # noqa: F401
