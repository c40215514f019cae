"""MI355X (gfx950) implementation of the xFasterTransformer decoder-layer hot path.

The compute lives in libxft_hip.so (hand-written HIP, C-ABI declared in include/xft_hip.h).
This package is only the ctypes binding used by the tests and the benchmark; there is no
CPU fallback: importing `capi` fails loudly when the library has not been built.
"""
__version__ = "0.1.0"
