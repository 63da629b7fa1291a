"""MI355X-native preshuffle quantized GEMM (int8 / OCP fp8 / MXFP4) behind FlyDSL's entry points.

Python host code -> ctypes -> ``libpsgemm.so`` (hand-written gfx950 HIP kernels).  There is no CPU
fallback: without the built library every launch raises.
"""

from .layout import shuffle_scale_w4, shuffle_weight, shuffle_weight_w4  # noqa: F401
from .quant import (  # noqa: F401
    e8m0_to_f32,
    f32_to_e8m0,
    mxfp4_to_f32,
    per_1x32_f4_quant,
    pertoken_quant,
)

__version__ = "0.1.0"
