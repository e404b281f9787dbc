"""MI355X-native (gfx950) implementation of the scaling.transformer layer hot path at tensor-parallel
size 1: attention core (forward, backward, KV-cache decode), rotary, RMSNorm and SwiGLU as hand-written
HIP kernels behind a C ABI, plus drop-in layer modules that mirror the reference's module API.
"""

from . import ops  # noqa: F401
from ._lib import LIB_PATH, load as load_library  # noqa: F401

__version__ = "0.1.0"
