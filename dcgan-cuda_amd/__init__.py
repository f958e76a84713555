"""MI355X (gfx950) backend for the convolution hot path of dcgan-cuda.

`hipabi`  -- ctypes binding of the C ABI in include/dcgan_hip.h (lib/libdcgan_hip.so)
`build`   -- compiles csrc/*.hip (and host/*.cc) in-tree

The directory name carries a dash, so import it through `__graft_entry__.load_package()` (or
importlib) under the module name `dcgan_cuda_amd`.
"""
from . import hipabi  # noqa: F401
from .hipabi import Buf, HipBackend, load  # noqa: F401
from . import hostabi  # noqa: F401
