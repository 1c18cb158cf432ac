"""ctypes binding of libopsnn_amd.so (the C ABI declared under include/).

The host side of this library is C++; this module only exists so that the Python
test-suite and the benchmark can drive the C entry points.  It adds no compute
path of its own and refuses to work without the built shared library.
"""
from .binding import *  # noqa: F401,F403
