"""Host-side mirror of the reference's interface to the W4A16 path.

* the four repack functions that `src/turbomind/python/bind.cpp:414-465` exports from
  `_turbomind` and `lmdeploy/serve/turbomind/deploy.py:631-665` calls, with the same names
  and argument order, taking torch tensors on the GPU;
* `GemmS4F16`, the operator of `src/turbomind/kernels/gemm_s_f16/gemm_s4_f16.h:17-56`.

Sizes follow the reference: `m` = output features, `k` = input features, `n` = tokens.
All work is queued on torch's current stream.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional

import torch

from . import _lib
from ._lib import GemmDesc, Metric, W4A16Error, check, lib  # noqa: F401


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("tensor must live on the GPU")
    if not t.is_contiguous():
        raise ValueError("tensor must be contiguous")
    return t.data_ptr()


def convert_s4_k_m8(A_dst, Q_dst, ws, A_src, scales, qzeros, m: int, k: int, group_size: int) -> None:
    """bind.cpp:431-456.  A_src int32 [k, m/8], scales fp16 [k/g, m], qzeros int32 [k/g, m/8] ->
    A_dst (same bytes as A_src, gfx950 tiled layout), Q_dst int32 [k/g, m] = half2(64 + zero, scale)."""
    if A_src.numel() * 8 != m * k or A_dst.numel() != A_src.numel():
        raise ValueError("qweight shape does not match m, k")
    g = k // group_size if group_size > 0 else 0
    if scales.numel() != g * m or qzeros.numel() * 8 != g * m or Q_dst.numel() * Q_dst.element_size() != g * m * 4:
        raise ValueError("scales / qzeros / Q shape does not match m, k, group_size")
    check(lib.w4a16_convert_s4_k_m8(_ptr(A_dst), _ptr(Q_dst), _ptr(ws), _ptr(A_src), _ptr(scales), _ptr(qzeros),
                                    m, k, group_size, _stream()))


def fuse_w1_w3_s4_k_m8(src, dst, m: int, k: int) -> None:
    """bind.cpp:424-429.  src = cat(w1, w3) int32 [2k, m/8] -> dst [k, 2m/8], columns interleaved."""
    if src.numel() * 8 != 2 * m * k or dst.numel() != src.numel():
        raise ValueError("shape does not match m, k")
    check(lib.w4a16_fuse_w1_w3_s4_k_m8(_ptr(dst), _ptr(src), m, k, _stream()))


def transpose_qk_s4_k_m8(src, dst, m: int, k: int, size_per_head: int) -> None:
    """bind.cpp:414-422.  Rotary re-ordering of the q/k columns of an AWQ-packed [k, m/8] tensor."""
    if src.numel() * 8 != m * k or dst.numel() != src.numel():
        raise ValueError("shape does not match m, k")
    check(lib.w4a16_transpose_qk_s4_k_m8_hf(_ptr(dst), _ptr(src), m, k, size_per_head, _stream()))


def deploy_qkv(q, k, v, size_per_head: int = 128, group_size: int = 128):
    """The deployable fused q|k|v matrix from the checkpoint's AWQ tensors: q, k, v are
    (qweight int32 [K, n/8], qzeros int32 [K/g, n/8], scales fp16 [K/g, n]) triples.  Does what
    deploy_awq does with transpose_qk_s4 / permute, merge_qkv and convert_s4
    (lmdeploy/serve/turbomind/deploy.py:251-260,371-383,633-639,660-670) in one pass; returns (A, Q)."""
    K = q[0].size(0)
    n_q, n_kv = q[0].size(-1) * 8, k[0].size(-1) * 8
    if v[0].size(-1) * 8 != n_kv or any(t[0].size(0) != K for t in (k, v)):
        raise ValueError("q, k, v shapes do not fit together")
    for qw, qz, s in (q, k, v):
        n = qw.size(-1) * 8
        if qz.numel() * 8 != (K // group_size) * n or s.numel() != (K // group_size) * n:
            raise ValueError("qzeros / scales shape does not match qweight")
    n = n_q + 2 * n_kv
    A = torch.empty((K, n // 8), dtype=torch.int32, device=q[0].device)
    Q = torch.empty((K // group_size, n), dtype=torch.int32, device=q[0].device)
    arr = lambda i: (ctypes.c_void_p * 3)(*(_ptr(t[i]) for t in (q, k, v)))
    check(lib.w4a16_deploy_qkv(_ptr(A), _ptr(Q), arr(0), arr(1), arr(2), n_q, n_kv, K, size_per_head, group_size, _stream()))
    return A, Q


def deploy_w13(w1, w3, group_size: int = 128):
    """The deployable fused gate|up matrix from the AWQ triples of gate_proj (w1) and up_proj (w3):
    fuse_w1_w3_s4 + convert_s4 (deploy.py:641-670) in one pass; returns (A, Q)."""
    K, n = w1[0].size(0), w1[0].size(-1) * 8
    for a, b in zip(w1, w3):
        if a.shape != b.shape:
            raise ValueError("w1 and w3 shapes differ")
    if w1[1].numel() * 8 != (K // group_size) * n or w1[2].numel() != (K // group_size) * n:
        raise ValueError("qzeros / scales shape does not match qweight")
    A = torch.empty((K, 2 * n // 8), dtype=torch.int32, device=w1[0].device)
    Q = torch.empty((K // group_size, 2 * n), dtype=torch.int32, device=w1[0].device)
    check(lib.w4a16_deploy_w13(_ptr(A), _ptr(Q), _ptr(w1[0]), _ptr(w3[0]), _ptr(w1[1]), _ptr(w3[1]), _ptr(w1[2]),
                               _ptr(w3[2]), n, K, group_size, _stream()))
    return A, Q


def dequantize_s4(src, dst) -> None:
    """bind.cpp:458-465.  int32 words -> fp16 raw nibble values (8 per word)."""
    if src.numel() * 8 != dst.numel():
        raise ValueError("FT_CHECK(src_count * 8 == dst_count) failed")
    check(lib.w4a16_dequantize_s4(_ptr(dst), _ptr(src), src.numel(), _stream()))


def unpack_repacked(A, Q, m: int, k: int, group_size: int = 128):
    """Inverse of convert_s4_k_m8: returns (qweight, qzeros, scales) as the AWQ tensors."""
    g = k // group_size
    qweight = torch.empty((k, m // 8), dtype=torch.int32, device=A.device)
    qzeros = torch.empty((g, m // 8), dtype=torch.int32, device=A.device)
    scales = torch.empty((g, m), dtype=torch.float16, device=A.device)
    check(lib.w4a16_unpack_repacked(_ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(A), _ptr(Q), m, k, group_size,
                                    _stream()))
    return qweight, qzeros, scales


def dequantize_repacked(A, Q, m: int, k: int, group_size: int = 128):
    """fp16 W[k, m] with the reference kernel's arithmetic: fp16((q - z) * s)."""
    W = torch.empty((k, m), dtype=torch.float16, device=A.device)
    check(lib.w4a16_dequantize_repacked(_ptr(W), _ptr(A), _ptr(Q), m, k, group_size, _stream()))
    return W


def from_reference_layout(A_ref, m: int, k: int):
    """Weights in the reference's own tiled layout -> the gfx950 layout."""
    out = torch.empty_like(A_ref)
    check(lib.w4a16_from_reference_layout(_ptr(out), _ptr(A_ref), m, k, _stream()))
    return out


def gemm_static(C, A, B, Q, m: int, n: int, k: int, group_size: int, type: int = 0, algo_id: int = -1,
                residual=None, stream: Optional[int] = None) -> None:
    """`GemmS4F16.Run` without a handle and without any allocation: split-K kernels use the scratch
    buffer inside the library (8 MiB per GPU, shared by all calls on that GPU)."""
    check(lib.w4a16_gemm_static(_ptr(C), _ptr(A), _ptr(B), _ptr(Q), _ptr(residual), m, n, k, group_size, type,
                                algo_id, _stream() if stream is None else stream))


class GemmS4F16:
    """gemm_s4_f16.h:17-56.  `Run(C, A, B, Q, m, n, k, group_size, type, algo_id)` with m = output
    features, n = tokens; B is the fp16 activation matrix [n, k]."""
    kGemm = _lib.GEMM
    kFusedSiluFfn = _lib.FUSED_SILU_FFN
    kFusedAdd = _lib.FUSED_ADD  # extension: C = residual + gemm

    def __init__(self):
        h = ctypes.c_void_p()
        check(lib.w4a16_create(ctypes.byref(h)))
        self._h = h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and lib is not None:  # `lib` is already gone at interpreter shutdown
            lib.w4a16_destroy(h)

    def Run(self, C, A, B, Q, m: int, n: int, k: int, group_size: int, type: int = 0, algo_id: int = -1,
            residual=None, stream: Optional[int] = None) -> None:
        check(lib.w4a16_gemm(self._h, _ptr(C), _ptr(A), _ptr(B), _ptr(Q), _ptr(residual), m, n, k, group_size, type,
                             algo_id, _stream() if stream is None else stream))

    def Measure(self, C, A, B, Q, m: int, n: int, k: int, group_size: int, type: int = 0,
                residual=None) -> List[Metric]:
        cap = lib.w4a16_algo_count()
        buf = (Metric * cap)()
        cnt = check(lib.w4a16_measure(self._h, _ptr(C), _ptr(A), _ptr(B), _ptr(Q), _ptr(residual), m, n, k,
                                      group_size, type, buf, cap, _stream()))
        return [buf[i] for i in range(cnt)]

    @staticmethod
    def algo_count() -> int:
        return lib.w4a16_algo_count()

    def ffn(self, ffn_output, gating_buf, ffn_input, A13, Q13, A2, Q2, hidden_units: int, inter_size: int, n: int,
            group_size: int = 128, residual=None, stream: Optional[int] = None) -> None:
        """The int4 branch of LlamaFfnLayer<T>::forward (LlamaFfnLayer.cc:67-116): SiLU-gated fused
        gate/up GEMM into `gating_buf` [n, inter_size], then w2 into `ffn_output` [n, hidden_units],
        plus `residual` if given (may alias `ffn_output`)."""
        check(lib.w4a16_ffn(self._h, _ptr(ffn_output), _ptr(gating_buf), _ptr(ffn_input), _ptr(A13), _ptr(Q13),
                            _ptr(A2), _ptr(Q2), _ptr(residual), hidden_units, inter_size, n, group_size,
                            _stream() if stream is None else stream))

    def sequence(self, gemms, n: int, group_size: int = 128, persistent: bool = False, stream: Optional[int] = None):
        """A list of GEMMs with a common token count `n` in one call.  `gemms`: tuples
        (C, A, B, Q, m, k, type, residual, depends) in execution order; `depends` says that the GEMM reads
        what an earlier one of the list writes.  `persistent`: up to 16 tokens, one persistent launch for the
        whole list instead of one launch per GEMM.  Returns the descriptor array (the tensors must stay
        alive while a captured call is replayed)."""
        arr = (GemmDesc * len(gemms))()
        for d, (C, A, B, Q, m, k, type_, residual, depends) in zip(arr, gemms):
            d.C, d.A, d.X, d.Q, d.R = _ptr(C), _ptr(A), _ptr(B), _ptr(Q), _ptr(residual)
            d.n_out, d.k, d.epilogue, d.depends = m, k, type_, int(bool(depends))
        check(lib.w4a16_gemm_sequence(self._h, arr, len(gemms), n, group_size,
                                      _lib.SEQ_PERSISTENT if persistent else 0, _stream() if stream is None else stream))
        return arr

    def sequence_status(self, stream: Optional[int] = None) -> None:
        """Synchronises and raises W4A16Error (code -7) if a barrier of an earlier `sequence` gave up."""
        check(lib.w4a16_sequence_status(self._h, _stream() if stream is None else stream))

    def set_barrier_timeout(self, seconds: float) -> None:
        check(lib.w4a16_set_barrier_timeout(self._h, seconds))

    def probe_read(self, t, stream: Optional[int] = None) -> None:
        """Measurement aid: a plain streaming read of tensor `t`, launched like the decode kernels."""
        check(lib.w4a16_probe_read(self._h, _ptr(t), t.numel() * t.element_size(), _stream() if stream is None else stream))

    def probe_stream(self, t, wg_per_cu: int, in_flight: int, hint: int, stream: Optional[int] = None) -> None:
        """Measurement aid: the same read with the GEMM kernels' load pipeline (`in_flight` 16-byte loads per
        lane waited for by count, `wg_per_cu` workgroups per CU, hint 0 plain / 1 non-temporal / 2 system scope)."""
        check(lib.w4a16_probe_stream(self._h, _ptr(t), t.numel() * t.element_size(), wg_per_cu, in_flight, hint,
                                     _stream() if stream is None else stream))

    def probe_barrier(self, iters: int, tree: bool = True, stream: Optional[int] = None) -> None:
        """Measurement aid: one persistent launch that crosses `iters` device-wide barriers and nothing else."""
        check(lib.w4a16_probe_barrier(self._h, iters, int(tree), _stream() if stream is None else stream))

    def probe_mfma(self, waves_per_cu: int, iters: int, stream: Optional[int] = None) -> int:
        """Measurement aid: nothing but matrix instructions, one workgroup of `waves_per_cu` waves per CU;
        returns the flop the launch executes."""
        check(lib.w4a16_probe_mfma(self._h, waves_per_cu, iters, _stream() if stream is None else stream))
        return torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count * waves_per_cu * iters * 65536

    def clock_begin(self, stream: Optional[int] = None) -> None:
        """Measurement aid: from now on the decode strip kernels and the probes launched through this
        operator record the engine cycles and constant-rate ticks they take (`clock_end` reads them)."""
        check(lib.w4a16_probe_clock_begin(self._h, _stream() if stream is None else stream))

    def clock_end(self, stream: Optional[int] = None) -> dict:
        """Synchronises, stops the recording and returns {"MHz", "us_per_launch", "launches"} of the kernels
        that recorded since `clock_begin` (zeros if none did)."""
        c, t, n, r = ctypes.c_ulonglong(), ctypes.c_ulonglong(), ctypes.c_ulonglong(), ctypes.c_longlong()
        check(lib.w4a16_probe_clock_end(self._h, ctypes.byref(c), ctypes.byref(t), ctypes.byref(n), ctypes.byref(r),
                                        _stream() if stream is None else stream))
        if not t.value or not n.value:
            return {"MHz": 0.0, "us_per_launch": 0.0, "launches": int(n.value)}
        return {"MHz": c.value / t.value * r.value / 1e6, "us_per_launch": t.value / n.value / r.value * 1e6,
                "launches": int(n.value)}

    def pick(self, m: int, n: int, k: int) -> int:
        """The algo_id that `Run(..., algo_id=-1)` uses for this shape: the fastest one a previous
        `Measure` of exactly this shape found, else the heuristic's choice."""
        return check(lib.w4a16_pick(self._h, m, n, k))

    def clear_tuning(self) -> None:
        check(lib.w4a16_clear_tuning(self._h))

    def save_tuning(self, path: str) -> int:
        """Writes the kernels `Measure` found fastest to a text file; returns the number of shapes."""
        return check(lib.w4a16_save_tuning(self._h, os.fsencode(path)))

    def load_tuning(self, path: str) -> int:
        """Reads such a file (W4A16Error code -8 if it was written by another library version or GPU)."""
        return check(lib.w4a16_load_tuning(self._h, os.fsencode(path)))
