"""CPU oracle for the W4A16 GEMM path (TEST INFRASTRUCTURE ONLY).

This module restates, in numpy, the algorithm of TurboMind's `GemmS4F16` path and of
its `convert_s4` weight repack.  It is the checker that the HIP library is compared
with; nothing in the product (`lmdeploy_amd/`) may import it.  Only `tests/`, the
smoke check and the `cpu_baseline` leg of the benchmark use it.

All citations are into the reference tree (lmdeploy v0.0.9):

  linear.py   = lmdeploy/pytorch/modules/linear.py
  common.h    = src/turbomind/kernels/gemm_s_f16/common.h
  format.cu   = src/turbomind/kernels/gemm_s_f16/format.cu
  gemm_s4_f16.cu, gemm_template.h, warp_iterator.h  (same directory)
  llama_decoder_kernels.cu = src/turbomind/models/llama/llama_decoder_kernels.cu

Conventions: T tokens, K in-features, N out-features, g group size, G = K / g.
"Logical" tensors are un-packed: q[K, N] and z[G, N] hold integers 0..15.

How each function is pinned (see tests/test_oracle.py): the pack/unpack pair by
exhaustive enumeration of one word; the two magic-number dequantisers by evaluating
the reference's instruction sequence in IEEE fp16 for every nibble value and
position; the nibble permutations by index tagging against the derived element map
and by their defining invariants; the dequantised weight by the identity
"fp16 multiply == one rounding of the exact product"; the GEMM and its epilogues by
special cases with exact answers (identity activations, one-hot rows, q == z,
power-of-two scales) and by float64 evaluation.  The reference holds no golden
vectors for this path, so none are used.
"""
from __future__ import annotations

import numpy as np

# linear.py:85 -- nibble i of a packed word holds logical column 8*j + AWQ_ORDER[i]
AWQ_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)
# common.h:47-113 -- output position p of the unpack comes from nibble UNPACK_NIBBLE[p]
UNPACK_NIBBLE = (0, 4, 1, 5, 2, 6, 3, 7)

FP16_MIN_NORMAL = 2.0 ** -14


# ---------------------------------------------------------------------------
# nibble helpers
# ---------------------------------------------------------------------------
def words_to_nibbles(words: np.ndarray) -> np.ndarray:
    """uint32[...] -> uint8[..., 8]; entry i is bits 4i..4i+3 (format.cu:19-22 `read_u4`)."""
    w = np.asarray(words).astype(np.uint32, copy=False)
    shifts = (np.arange(8, dtype=np.uint32) * 4)
    return ((w[..., None] >> shifts) & np.uint32(0xF)).astype(np.uint8)


def nibbles_to_words(nib: np.ndarray) -> np.ndarray:
    """uint8[..., 8] -> uint32[...]; inverse of words_to_nibbles."""
    n = np.asarray(nib).astype(np.uint32)
    shifts = (np.arange(8, dtype=np.uint32) * 4)
    return np.bitwise_or.reduce(n << shifts, axis=-1).astype(np.uint32)


# ---------------------------------------------------------------------------
# A1 / R1: AWQ pack  (linear.py:85,105-108,118-121)
# ---------------------------------------------------------------------------
def awq_pack(logical: np.ndarray) -> np.ndarray:
    """logical uint8 [R, C] (values 0..15, C % 8 == 0) -> uint32 [R, C/8].

    word[r, j] = OR_i (logical[r, 8j + AWQ_ORDER[i]] & 0xF) << 4i
    """
    a = np.asarray(logical)
    assert a.ndim == 2 and a.shape[1] % 8 == 0
    blocks = a.reshape(a.shape[0], a.shape[1] // 8, 8)
    nib = blocks[..., list(AWQ_ORDER)]          # nibble i <- column AWQ_ORDER[i]
    return nibbles_to_words(nib & 0xF)


# ---------------------------------------------------------------------------
# A2 / R2: the reference's own unpack  (common.h:47-113, format.cu:132-142)
# ---------------------------------------------------------------------------
def awq_unpack(words: np.ndarray) -> np.ndarray:
    """uint32 [R, C/8] -> uint8 [R, C]; position p of each word <- nibble UNPACK_NIBBLE[p]."""
    nib = words_to_nibbles(words)
    out = nib[..., list(UNPACK_NIBBLE)]
    return out.reshape(*words.shape[:-1], words.shape[-1] * 8)


def dequantize_s4(words: np.ndarray) -> np.ndarray:
    """`dequantize_s4` (format.cu:132-142): uint32[count] -> fp16[count*8] raw nibble values."""
    return awq_unpack(np.asarray(words).reshape(1, -1)).astype(np.float16).reshape(-1)


def _f16_from_bits(bits: np.ndarray) -> np.ndarray:
    return np.asarray(bits, dtype=np.uint16).view(np.float16)


def dequantize_s4_bittrick(words: np.ndarray) -> np.ndarray:
    """The literal instruction sequence of `dequantize_s4_to_fp16x2` (common.h:55-110),
    evaluated in IEEE fp16: lop3 = (x & mask) | magic, then sub / fma per half.
    Returns fp16 [..., 8] in the order h[0].lo, h[0].hi, h[1].lo, ...
    """
    x = np.asarray(words, dtype=np.uint32)
    top = x >> np.uint32(8)
    BOT, TOP, MAGIC = np.uint32(0x000F000F), np.uint32(0x00F000F0), np.uint32(0x64006400)
    h = [(x & BOT) | MAGIC, (x & TOP) | MAGIC, (top & BOT) | MAGIC, (top & TOP) | MAGIC]
    out = np.empty(x.shape + (8,), dtype=np.float16)
    for i, hv in enumerate(h):
        lo = _f16_from_bits(hv & np.uint32(0xFFFF))
        hi = _f16_from_bits(hv >> np.uint32(16))
        for j, v in enumerate((lo, hi)):
            if i % 2 == 0:      # sub.f16x2 h, h, {1024,1024}
                r = (v.astype(np.float64) - 1024.0).astype(np.float16)
            else:               # fma.rn.f16x2 h, {1/16,1/16}, {-64,-64}
                r = (v.astype(np.float64) * 0.0625 - 64.0).astype(np.float16)
            out[..., 2 * i + j] = r
    return out


# ---------------------------------------------------------------------------
# A3: offset-64 form used for the zeros and inside the kernel (common.h:115-156)
# ---------------------------------------------------------------------------
def dequantize_s4_v2_bits(words: np.ndarray) -> np.ndarray:
    """`dequantize_s4_to_fp16x2_v2` (common.h:144-151): uint32[...] -> uint16[..., 8],
    the fp16 BIT PATTERNS of 64 + q in unpack order."""
    x = np.asarray(words, dtype=np.uint32)
    top = x >> np.uint32(8)
    BOT, TOP = np.uint32(0x000F000F), np.uint32(0x00F000F0)
    M1 = np.uint32(0x54005400)
    M2 = np.uint32(0x54005400 >> 4)
    h0 = ((x & BOT) | M2) << np.uint32(4)
    h1 = (x & TOP) | M1
    h2 = ((top & BOT) | M2) << np.uint32(4)
    h3 = (top & TOP) | M1
    out = np.empty(x.shape + (8,), dtype=np.uint16)
    for i, hv in enumerate((h0, h1, h2, h3)):
        out[..., 2 * i] = (hv & np.uint32(0xFFFF)).astype(np.uint16)
        out[..., 2 * i + 1] = (hv >> np.uint32(16)).astype(np.uint16)
    return out


# ---------------------------------------------------------------------------
# A7 / R3: Q = half2(64 + z, s)   (format.cu:77-95, FMA variant off: common.h:13-15)
# ---------------------------------------------------------------------------
def merge_q(qzeros: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """qzeros uint32 [G, N/8] (AWQ packed), scales fp16 [G, N] -> uint32 [G, N].

    Low half = fp16 bits of 64 + z (== 0x5400 | z << 4), high half = scale bits.
    """
    G, N = scales.shape
    zbits = dequantize_s4_v2_bits(qzeros).reshape(G, N).astype(np.uint32)
    sbits = np.ascontiguousarray(scales, dtype=np.float16).view(np.uint16).astype(np.uint32)
    return (zbits | (sbits << np.uint32(16))).astype(np.uint32)


def split_q(Q: np.ndarray):
    """uint32 [G, N] -> (z uint8 [G, N], s fp16 [G, N]); inverse of merge_q."""
    Q = np.asarray(Q, dtype=np.uint32)
    z = ((Q >> np.uint32(4)) & np.uint32(0xF)).astype(np.uint8)
    s = (Q >> np.uint32(16)).astype(np.uint16).view(np.float16)
    return z, s


# ---------------------------------------------------------------------------
# generic nibble-tensor transpose  (format.cu:24-59 `permute_u4`)
# ---------------------------------------------------------------------------
def permute_u4(src_words: np.ndarray, dims, order) -> np.ndarray:
    """Nibble i of the flat source (nibble i%8 of word i/8) is the element with row-major
    index i in a tensor of shape `dims`; it is written to the flat destination at the
    row-major index of the same element in the tensor transposed by `order`."""
    flat = words_to_nibbles(np.asarray(src_words, dtype=np.uint32).reshape(-1)).reshape(-1)
    assert flat.size == int(np.prod(dims)), (flat.size, dims)
    t = flat.reshape(dims).transpose(order)
    return nibbles_to_words(np.ascontiguousarray(t).reshape(-1, 8))


def reformat_s4_k_m8(src: np.ndarray, m: int, k: int) -> np.ndarray:
    """The REFERENCE's tiled weight layout (format.cu:69-75); needed for format-compat only."""
    dims = (k // 32, 2, 2, 4, 2, m // 32, 2, 2, 2, 4)
    return permute_u4(src, dims, (0, 5, 9, 8, 3, 1, 6, 4, 2, 7))


def fuse_w1_w3_s4_k_m8(src: np.ndarray, m: int, k: int) -> np.ndarray:
    """format.cu:123-130: AWQ-packed cat(w1, w3) [2, k, m/8] -> AWQ-packed [k, 2m/8]
    with logical column 2j = w1 column j, 2j+1 = w3 column j."""
    dims = (2, k, m // 8, 2, 2, 2)
    return permute_u4(src, dims, (1, 2, 4, 0, 5, 3)).reshape(k, 2 * m // 8)


def transpose_qk_s4_k_m8_hf(src: np.ndarray, m: int, k: int, size_per_head: int) -> np.ndarray:
    """format.cu:115-121: within each head of D columns, dst[2i + r] = src[r*D/2 + i]."""
    dims = (k, m // size_per_head, 2, size_per_head // 2 // 8, 2, 2, 2)
    return permute_u4(src, dims, (0, 1, 3, 5, 2, 6, 4)).reshape(k, m // 8)


def convert_s4_k_m8_reference(qweight, scales, qzeros, m, k, group_size):
    """format.cu:97-113 as the reference does it: (A_dst in the reference layout, Q)."""
    assert scales.shape == (k // group_size, m)
    return reformat_s4_k_m8(qweight, m, k), merge_q(qzeros, scales)


def reference_layout_element(kt, nt, lane, word, nib):
    """Element map of the reference layout: which logical (k, n) sits in nibble `nib` of
    word ((kt*(N/32) + nt)*32 + lane)*4 + word.  Derived from format.cu:69-75 together
    with the A-fragment order of mma.m16n8k16 (warp_iterator.h:44-84)."""
    k16, n16 = word >> 1, word & 1
    klo, k8, n8 = (nib >> 2) & 1, (nib >> 1) & 1, nib & 1
    kk = 32 * kt + 16 * k16 + 8 * k8 + 2 * (lane % 4) + klo
    nn = 32 * nt + 16 * n16 + 8 * n8 + lane // 4
    return kk, nn


# ---------------------------------------------------------------------------
# A5 / R5: dequantised weight, bit exact
# ---------------------------------------------------------------------------
def _ftz16(x: np.ndarray) -> np.ndarray:
    """Flush fp16 subnormals to signed zero (the `.ftz` of common.h:229-230)."""
    x = np.asarray(x, dtype=np.float16)
    bits = x.view(np.uint16)
    sub = (bits & np.uint16(0x7C00)) == 0
    return np.where(sub, bits & np.uint16(0x8000), bits).astype(np.uint16).view(np.float16)


def dequant_weights(q: np.ndarray, z: np.ndarray, s: np.ndarray, group_size: int) -> np.ndarray:
    """W[k, n] = mul.ftz.f16( sub.ftz.f16(64 + q, 64 + z), s )  (common.h:218-235,
    warp_iterator.h:68-83).  The subtraction is exact (|q - z| <= 15); the product of
    two fp16 numbers is exact in fp32, so one fp32 -> fp16 rounding equals the fp16
    multiply.  Inputs: q uint8 [K, N], z uint8 [G, N], s fp16 [G, N]."""
    K, N = q.shape
    G = K // group_size
    assert z.shape == (G, N) and s.shape == (G, N)
    d = q.astype(np.int16).reshape(G, group_size, N) - z.astype(np.int16)[:, None, :]
    sf = _ftz16(s).astype(np.float32)[:, None, :]
    w = (d.astype(np.float32) * sf).astype(np.float16)
    return _ftz16(w).reshape(K, N)


def dequant_from_awq(qweight, qzeros, scales, group_size) -> np.ndarray:
    """AWQ tensors -> fp16 W[K, N] via the reference unpack (R2) and the closed form (R5)."""
    return dequant_weights(awq_unpack(qweight), awq_unpack(qzeros),
                           np.asarray(scales, dtype=np.float16), group_size)


# ---------------------------------------------------------------------------
# A6, A8, A9 / R8-R10: GEMM and epilogues
# ---------------------------------------------------------------------------
EPI_GEMM, EPI_SILU, EPI_ADD = 0, 1, 2


def _matmul_f32(x32: np.ndarray, w32: np.ndarray) -> np.ndarray:
    try:  # torch's CPU matmul is much faster than numpy's here; same fp32 arithmetic
        import torch
        return torch.matmul(torch.from_numpy(np.ascontiguousarray(x32)),
                            torch.from_numpy(np.ascontiguousarray(w32))).numpy()
    except ImportError:  # pragma: no cover
        return x32 @ w32


def gemm_acc(X: np.ndarray, W: np.ndarray) -> np.ndarray:
    """fp32 accumulators: acc[t, n] = sum_k fp32(X[t, k]) * fp32(W[k, n])  (gemm_template.h:12-27)."""
    return _matmul_f32(X.astype(np.float32), W.astype(np.float32))


def epilogue(acc: np.ndarray, kind: int, residual: np.ndarray | None = None) -> np.ndarray:
    """acc fp32 [T, N] -> fp16 output.

    EPI_GEMM (gemm_s4_f16.cu:22-29):  C = fp16_rn(acc)
    EPI_SILU (gemm_s4_f16.cu:31-42):  g, u = fp16_rn(acc[:, 2j]), fp16_rn(acc[:, 2j+1]);
                                      C[:, j] = fp16_rn(g / (1 + exp(-g)) * u) in fp32
    EPI_ADD  (llama_decoder_kernels.cu:52-57 applied to the fp16 GEMM output, bias = 0):
                                      C = fp16_rn(float(R) + float(fp16_rn(acc)))
    """
    y = acc.astype(np.float16)
    if kind == EPI_GEMM:
        return y
    if kind == EPI_SILU:
        g = y[:, 0::2].astype(np.float32)
        u = y[:, 1::2].astype(np.float32)
        with np.errstate(over="ignore"):
            silu = g / (np.float32(1.0) + np.exp(-g))
        return (silu * u).astype(np.float16)
    if kind == EPI_ADD:
        assert residual is not None and residual.shape == y.shape
        return (residual.astype(np.float32) + y.astype(np.float32)).astype(np.float16)
    raise ValueError("unknown epilogue")


def gemm_s4_f16(X, qweight, qzeros, scales, group_size, kind=EPI_GEMM, residual=None):
    """The whole reference CPU path: unpack, dequantise, fp32 matmul, epilogue."""
    W = dequant_from_awq(qweight, qzeros, scales, group_size)
    return epilogue(gemm_acc(np.asarray(X, dtype=np.float16), W), kind, residual)


def max_abs_rel(y: np.ndarray, yref: np.ndarray) -> float:
    """max |y - yref| / max |yref| : the reading of "max-abs-rel error" used by the gate."""
    y64, r64 = y.astype(np.float64), yref.astype(np.float64)
    den = float(np.max(np.abs(r64)))
    return float(np.max(np.abs(y64 - r64))) / (den if den > 0 else 1.0)


def elementwise_pass_rate(y: np.ndarray, yref: np.ndarray, rtol: float = 1e-2) -> float:
    """Share of the outputs with |y - yref| <= rtol * |yref| + rtol * rms(yref): the elementwise
    reading of the tolerance, which unlike the max-norm gate also holds small outputs to account."""
    y64, r64 = y.astype(np.float64), yref.astype(np.float64)
    rms = float(np.sqrt(np.mean(r64 * r64))) if r64.size else 0.0
    ok = np.abs(y64 - r64) <= rtol * np.abs(r64) + rtol * rms
    return float(np.mean(ok)) if ok.size else 1.0


# ---------------------------------------------------------------------------
# The gfx950 tiled layout produced by this build's convert_s4_k_m8 (specification).
# ---------------------------------------------------------------------------
# Weights: one tile = 16 columns x 128 rows (one quantisation group) = 1024 bytes, stored as
# 64 lanes x one 16-byte vector.  Tile index = kt * (N/16) + nt (all column tiles of a group
# are contiguous, so that waves working on neighbouring columns read neighbouring DRAM
# pages).  Lane l = 16*b + c holds
# column n = 16*nt + c; its word j (0..3) holds rows k = 128*kt + 32*j + 8*b + e, e = 0..7,
# with row offset e in nibble p where e = AWQ_ORDER[p].  That is exactly one operand of
# v_mfma_f32_16x16x32_f16 per word, and the in-register unpack needs a single shift.
TILE_N, TILE_K = 16, 128


def gfx950_layout_element(N: int, K: int, word_index: int, nib: int):
    """(k, n) held by nibble `nib` of word `word_index` of the repacked weight buffer."""
    NT = N // TILE_N
    j = word_index & 3
    lane = (word_index >> 2) & 63
    tile = word_index >> 8
    kt, nt = divmod(tile, NT)
    c, b = lane & 15, lane >> 4
    return TILE_K * kt + 32 * j + 8 * b + AWQ_ORDER[nib], TILE_N * nt + c


def repack_gfx950(qweight: np.ndarray, N: int, K: int) -> np.ndarray:
    """AWQ qweight uint32 [K, N/8] -> uint32 [K*N/8] in the gfx950 tiled layout."""
    assert N % TILE_N == 0 and K % TILE_K == 0
    q = awq_unpack(qweight)                                    # [K, N] logical
    NT, KT = N // TILE_N, K // TILE_K
    # k = 128 kt + 32 j + 8 b + e ; n = 16 nt + c
    t = q.reshape(KT, 4, 4, 8, NT, 16)                         # kt, j, b, e, nt, c
    t = t.transpose(0, 4, 2, 5, 1, 3)                          # kt, nt, b, c, j, e
    nib = t[..., list(AWQ_ORDER)]                              # nibble p <- e = AWQ_ORDER[p]
    return nibbles_to_words(np.ascontiguousarray(nib)).reshape(-1)


def unrepack_gfx950(A: np.ndarray, N: int, K: int) -> np.ndarray:
    """Inverse of repack_gfx950: tiled words -> logical q uint8 [K, N]."""
    NT, KT = N // TILE_N, K // TILE_K
    nib = words_to_nibbles(np.asarray(A, dtype=np.uint32).reshape(KT, NT, 4, 16, 4))
    e = np.empty_like(nib)
    e[..., list(AWQ_ORDER)] = nib                              # e index <- nibble p
    t = e.transpose(0, 4, 2, 5, 1, 3)                          # kt, j, b, e, nt, c
    return np.ascontiguousarray(t).reshape(K, N)


def convert_s4_k_m8(qweight, scales, qzeros, m, k, group_size):
    """This build's convert: (A in the gfx950 layout, Q identical to the reference's Q)."""
    return repack_gfx950(qweight, m, k), merge_q(qzeros, scales)


# ---------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations
# ---------------------------------------------------------------------------
def make_inputs(seed: int, T: int, K: int, N: int, group_size: int = 128, residual: bool = False):
    """int4 weights/zeros uniform 0..15 AWQ-packed, scales fp16(|N(0,1)|*0.01 + 1e-3),
    activations (and residual) fp16 N(0,1)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    G = K // group_size
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    s = (np.abs(rng.standard_normal((G, N))) * 0.01 + 1e-3).astype(np.float16)
    X = rng.standard_normal((T, K)).astype(np.float16)
    out = dict(qweight=awq_pack(q), qzeros=awq_pack(z), scales=s, X=X, q=q, z=z)
    if residual:
        out["R"] = rng.standard_normal((T, N)).astype(np.float16)
    return out
