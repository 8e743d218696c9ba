"""kalosm_amd: an MI355X (gfx950) HIP backend for the quantized-inference hot path of Fusor
(floneum/kalosm).  The product is `libfusor_hip.so` (C ABI in include/fusor_hip.h); this package
holds its sources (csrc/), the build recipe and a thin host-side mirror of the reference's
operator surface."""
from ._lib import (F16, F32, MASK_ADDITIVE, MASK_CAUSAL, MASK_NONE, Q4_0, Q4_K, Q6_K, Q8_0, FusorHipError,
                   LIB_PATH, load)

__all__ = ["load", "LIB_PATH", "FusorHipError", "Q4_0", "Q8_0", "Q4_K", "Q6_K", "MASK_NONE", "MASK_CAUSAL",
           "MASK_ADDITIVE", "F32", "F16"]
