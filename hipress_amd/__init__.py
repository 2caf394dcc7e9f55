"""hipress_amd: MI355X (gfx950) gradient-compression operators.

Hand-written HIP encode / decode kernels for onebit, TBQ, TernGrad, DGC and
GradDrop plus the decode-and-merge aggregation step, behind a C ABI
(include/hipress_amd.h, libhipress_amd.so) and an in-place PyTorch op surface
(hipress_amd.ops, also registered as torch.ops.hipress.*).
"""
from . import _lib  # noqa: F401
from . import ops  # noqa: F401
from .ops import *  # noqa: F401,F403

__version__ = "0.1.0"
