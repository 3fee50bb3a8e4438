"""MI355X (gfx950) implementation of TurboMind's W4A16 GEMM path (`GemmS4F16` + `convert_s4`).

The compute lives in `lib/libw4a16.so` (hand-written HIP, C ABI in `include/w4a16.h`).  This
package is the Python host side: `lmdeploy_amd.turbomind` mirrors the functions that the
reference exports from its `_turbomind` extension for this path and wraps the operator.
"""
from . import _lib  # noqa: F401
from .turbomind import (GemmS4F16, convert_s4_k_m8, dequantize_s4, fuse_w1_w3_s4_k_m8,  # noqa: F401
                        transpose_qk_s4_k_m8)

__all__ = ["GemmS4F16", "convert_s4_k_m8", "dequantize_s4", "fuse_w1_w3_s4_k_m8", "transpose_qk_s4_k_m8"]
