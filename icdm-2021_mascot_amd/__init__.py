"""MI355X-native MASCOT matrix-factorization training path.

The product is the C-ABI shared library libmascot_hip.so (include/mascot_hip.h) plus the
quantized_mf command line; this package only builds them and binds the library with ctypes."""
from . import capi  # noqa: F401
from .capi import MascotHip, NODE, load  # noqa: F401
