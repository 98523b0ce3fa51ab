"""MI355X (gfx950) implementation of CURRENNT's backward hot path.

The product is the C-ABI shared library built from csrc/ (see include/currennt_hip.h) and the C++
layer shells in host/.  This Python package only binds the C ABI with ctypes so that tests and the
benchmark can drive it with device buffers owned by PyTorch; it contains no compute of its own and
refuses to work when the library is missing.
"""
from . import capi  # noqa: F401
from . import specs  # noqa: F401
