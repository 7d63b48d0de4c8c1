"""MI355X (gfx950) backend for the TAGI Linear / Conv2d hot path.

Everything computes inside ``libtagi_hip.so`` (hand-written HIP behind the C ABI
of ``include/tagi_hip.h``); this package is the host side that calls it. There
is no CPU fallback: importing :mod:`cutagi_amd.capi` fails if the library has not
been built (``python -m cutagi_amd.build``).
"""
__version__ = "0.1.0"

import importlib.util as _ilu
import os as _os
import sys as _sys

# One HIP runtime per process: PyTorch ships its own copy, and a process in which
# this package's library initialises the GPU first can no longer initialise
# torch's ("No HIP GPUs are available"). Where torch is installed it is therefore
# imported before the native library can be loaded, so that both share torch's
# runtime. Set CUTAGI_AMD_NO_TORCH=1 in a process that will never import torch to
# skip this (and its import time).
if ("torch" not in _sys.modules and _os.environ.get("CUTAGI_AMD_NO_TORCH", "") != "1"
        and _ilu.find_spec("torch") is not None):
    import torch as _torch  # noqa: F401
