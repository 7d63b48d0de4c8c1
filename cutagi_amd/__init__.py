"""MI355X (gfx950) backend for the TAGI Linear / Conv2d hot path.

Everything computes inside ``libtagi_hip.so`` (hand-written HIP behind the C ABI
of ``include/tagi_hip.h``); this package is the host side that calls it. There
is no CPU fallback: importing :mod:`cutagi_amd.capi` fails if the library has not
been built (``python -m cutagi_amd.build``).
"""
__version__ = "0.1.0"
