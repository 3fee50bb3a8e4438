"""ctypes binding of libw4a16.so.  There is no fallback: if the library is missing or lacks a
symbol, importing fails loudly."""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_double, c_float, c_int, c_longlong, c_size_t, c_ulonglong,
                    c_void_p)

# The callers hand over torch tensors, so torch is in the process anyway - and it must come first:
# torch ships its own libamdhip64 and libw4a16.so has to bind to that same HIP runtime.  Loaded the
# other way round, the system runtime gets in first, two runtimes share the process, and the first
# kernel launch reports "no ROCm-capable device is detected".
import torch  # noqa: F401  (imported for its side effect on the dynamic loader)

_HERE = os.path.dirname(os.path.abspath(__file__))
# W4A16_LIB overrides the in-tree library (e.g. to try a differently tuned build)
LIB_PATH = os.environ.get("W4A16_LIB") or os.path.join(_HERE, "lib", "libw4a16.so")

OK, EGROUP, ESHAPE, EHIP, EARG, EALGO, ESCRATCH, ETIMEOUT, ETUNING = 0, -1, -2, -3, -4, -5, -6, -7, -8
GEMM, FUSED_SILU_FFN, FUSED_ADD = 0, 1, 2
SEQ_PERSISTENT = 1


class Metric(Structure):
    """struct w4a16_metric of include/w4a16.h."""
    _fields_ = [("id", c_int), ("feasible", c_int), ("best", c_int), ("kind", c_int), ("tile_n", c_int),
                ("tile_t", c_int), ("slices", c_int), ("grid", c_int), ("ms", c_float), ("count", c_int)]


class GemmDesc(Structure):
    """struct w4a16_gemm_desc of include/w4a16.h."""
    _fields_ = [("C", c_void_p), ("A", c_void_p), ("X", c_void_p), ("Q", c_void_p), ("R", c_void_p),
                ("n_out", c_int), ("k", c_int), ("epilogue", c_int), ("depends", c_int)]


class W4A16Error(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


# every symbol that include/w4a16.h declares: (restype, argtypes)
SIGNATURES = {
    "w4a16_create": (c_int, [POINTER(c_void_p)]),
    "w4a16_destroy": (None, [c_void_p]),
    "w4a16_gemm": (c_int, [c_void_p] * 6 + [c_int] * 6 + [c_void_p]),
    "w4a16_gemm_static": (c_int, [c_void_p] * 5 + [c_int] * 6 + [c_void_p]),
    "w4a16_gemm_sequence": (c_int, [c_void_p, POINTER(GemmDesc), c_int, c_int, c_int, c_int, c_void_p]),
    "w4a16_sequence_status": (c_int, [c_void_p, c_void_p]),
    "w4a16_set_barrier_timeout": (c_int, [c_void_p, c_double]),
    "w4a16_ffn": (c_int, [c_void_p] * 9 + [c_int] * 4 + [c_void_p]),
    "w4a16_measure": (c_int, [c_void_p] * 6 + [c_int] * 5 + [POINTER(Metric), c_int, c_void_p]),
    "w4a16_algo_count": (c_int, []),
    "w4a16_pick": (c_int, [c_void_p, c_int, c_int, c_int]),
    "w4a16_clear_tuning": (c_int, [c_void_p]),
    "w4a16_save_tuning": (c_int, [c_void_p, c_char_p]),
    "w4a16_load_tuning": (c_int, [c_void_p, c_char_p]),
    "w4a16_convert_s4_k_m8": (c_int, [c_void_p] * 6 + [c_int] * 3 + [c_void_p]),
    "w4a16_deploy_qkv": (c_int, [c_void_p, c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p)] + [c_int] * 5
                         + [c_void_p]),
    "w4a16_deploy_w13": (c_int, [c_void_p] * 8 + [c_int] * 3 + [c_void_p]),
    "w4a16_reformat_s4_k_m8": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "w4a16_fuse_w1_w3_s4_k_m8": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "w4a16_transpose_qk_s4_k_m8_hf": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "w4a16_dequantize_s4": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "w4a16_unpack_repacked": (c_int, [c_void_p] * 5 + [c_int] * 3 + [c_void_p]),
    "w4a16_dequantize_repacked": (c_int, [c_void_p] * 3 + [c_int] * 3 + [c_void_p]),
    "w4a16_from_reference_layout": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "w4a16_probe_read": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "w4a16_probe_stream": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_int, c_int, c_void_p]),
    "w4a16_probe_barrier": (c_int, [c_void_p, c_int, c_int, c_void_p]),
    "w4a16_probe_mfma": (c_int, [c_void_p, c_int, c_int, c_void_p]),
    "w4a16_probe_clock_begin": (c_int, [c_void_p, c_void_p]),
    "w4a16_probe_clock_end": (c_int, [c_void_p, POINTER(c_ulonglong), POINTER(c_ulonglong), POINTER(c_ulonglong),
                                      POINTER(c_longlong), c_void_p]),
    "w4a16_last_error": (c_char_p, []),
    "w4a16_version": (c_char_p, []),
}


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s not found: build it with `python -m lmdeploy_amd.build` (needs hipcc); "
            "there is no CPU fallback" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(code: int) -> int:
    if code < 0:
        raise W4A16Error(code, lib.w4a16_last_error().decode())
    return code
