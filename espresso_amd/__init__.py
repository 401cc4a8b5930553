"""MI355X-native implementation of Espresso's quantized transformer decode path.

The product is the C-ABI shared library built from csrc/ (declared in include/espresso_hip.h);
this package is the thin ctypes layer that tests and bench.py drive it through.
"""
from . import _lib  # noqa: F401
from ._lib import EspressoError, load_library, library_path  # noqa: F401
