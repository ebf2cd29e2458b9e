"""MI355X-native convolution backend behind Avocado's C backend API.

The product is the shared library ``libavocado_hip.so`` (hand-written HIP kernels for gfx950 plus the C++ host layer that
exports the ``cuda*`` entry points of Avocado's backend interface).  This package only locates, loads and binds it for
Python callers (tests, benchmark); it contains no compute fallback: when the library is missing, loading raises.
"""
from .api import *  # noqa: F401,F403
from .api import load_library
