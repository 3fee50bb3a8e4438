"""MI355X (gfx950) implementation of TurboMind's W4A16 GEMM path (`GemmS4F16` + `convert_s4`).

The compute lives in `lib/libw4a16.so` (hand-written HIP, C ABI in `include/w4a16.h`).  This
package is the Python host side: `lmdeploy_amd.turbomind` mirrors the functions that the
reference exports from its `_turbomind` extension for this path and wraps the operator.
"""
__all__ = ["GemmS4F16", "convert_s4_k_m8", "dequantize_s4", "fuse_w1_w3_s4_k_m8", "transpose_qk_s4_k_m8"]


def __getattr__(name):
    # The library is loaded on first use, not on `import lmdeploy_amd`, so that
    # `python -m lmdeploy_amd.build` can run in a tree where it has not been built yet.  Using any
    # of the names below without the library raises ImportError (there is no CPU fallback).
    if name in __all__:
        from . import turbomind
        return getattr(turbomind, name)
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
