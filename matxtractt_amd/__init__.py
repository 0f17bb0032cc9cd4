"""matxtractt_amd -- MI355X (gfx950) implementation of MatXtract's hybrid SpMV path.

The product is ``libmatxtract_hip.so`` (C ABI in ``include/matxtract_hip.h``, the reference's
C++ surface in ``include/MatXtract.h``, the ``matxtract_perftest`` CLI in ``bin/``).  This
package is a thin ctypes face over that library for tests and benchmarks.
"""
from .api import *  # noqa: F401,F403
from .api import __all__  # noqa: F401
