"""eisen_amd -- host-side Python binding of libeisen_hip.so (MI355X / gfx950).

The product is the C-ABI library (include/eisen_hip.h, include/eisen_graph.h); this package
only loads it with ctypes for the tests, the smoke check and the benchmark.  It raises if
the library has not been built -- there is no CPU fallback.
"""
from .lib import LIB_PATH, EisenHipError, load_library  # noqa: F401
