"""flashlight_amd: fused attention-variant forward kernels for AMD MI355X (gfx950).

`flashlight_amd.attention_variants` mirrors the reference's attention_variants/ package function for function;
each call is one hand-written HIP kernel launch through the C ABI in include/flashlight_amd.h.
"""
__version__ = "0.1.0"

from . import _ffi  # noqa: F401
from ._ffi import FlashlightError, load_library  # noqa: F401
