"""Loader for libeisen_hip.so and the list of symbols include/eisen_hip.h declares."""
import ctypes as C
import os
import re

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libeisen_hip.so")
HSACO_PATH = os.path.join(_PKG, "eisen_kernels.hsaco")
INCLUDE_DIR = os.path.join(os.path.dirname(_PKG), "include")


class EisenHipError(RuntimeError):
    """A C-ABI call returned non-zero; carries the code and the library's message."""

    def __init__(self, fn, code, message):
        super().__init__(f"{fn} failed with code {code}: {message}")
        self.fn, self.code, self.message = fn, code, message


_lib = None


def load_library():
    """Load the built library.  No fallback: a missing build is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C eisen_amd/csrc` (needs hipcc)")
        _lib = C.CDLL(LIB_PATH)
    return _lib


def declared_symbols(header):
    """Names of the functions a header under include/ declares (for the export check)."""
    text = open(os.path.join(INCLUDE_DIR, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(eisen_[a-z0-9_]+)\s*\(", text)))
