"""MI355X (gfx950) implementation of ParallelReverseAutoDiff's matrix-multiply forward/backward
path and the gradient kernels around it, behind the reference's operation interface.

The compute lives in libprad_hip.so (C ABI, include/prad_hip.h).  This package is the host side
that plays the role of the reference's C# classes: same class names, same Forward/Backward
contract, same error behaviour.
"""
from . import _lib  # noqa: F401
