"""templar_amd - templar's gradient codec (tplr.compress) on MI355X.

`templar_amd.compress` mirrors the reference module's API; the work is done by
libtplr_hip.so (hand-written gfx950 kernels behind the C ABI of include/tplr_hip.h).
"""
from . import compress  # noqa: F401
from .compress import *  # noqa: F401,F403
from .compress import __all__ as _compress_all

__version__ = "0.1.0"
__all__ = list(_compress_all) + ["compress"]
