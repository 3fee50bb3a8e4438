"""Pins the CPU oracle by what the mathematics fixes, independent of its own formulas:
exhaustive enumeration, the reference's literal bit tricks evaluated in IEEE fp16,
index tagging of the nibble permutations, and GEMM special cases with exact answers.
The reference holds no golden vectors for this path (its tests never touch it)."""
import numpy as np
import pytest

from oracle import w4a16_oracle as O


# ---------------------------------------------------------------- R1 / R2 pack + unpack
def test_pack_layout_exhaustive_one_word():
    # every (position, value): exactly the nibble linear.py:105-108 shifts it to
    for col in range(8):
        for v in range(16):
            row = np.zeros((1, 8), dtype=np.uint8)
            row[0, col] = v
            word = int(O.awq_pack(row)[0, 0])
            i = [0, 2, 4, 6, 1, 3, 5, 7].index(col)      # pack_order[i] == col
            assert word == v << (4 * i)


def test_unpack_is_inverse_of_pack():
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(37, 64), dtype=np.uint8)
    assert np.array_equal(O.awq_unpack(O.awq_pack(q)), q)
    # and the two index tables are inverse permutations of each other
    assert [O.AWQ_ORDER[O.UNPACK_NIBBLE[p]] for p in range(8)] == list(range(8))


def test_unpack_closed_form_equals_reference_bit_trick():
    # nibbles are independent, so 16 values x 8 positions (+ random words) cover the map
    words = [v << (4 * i) for i in range(8) for v in range(16)]
    rng = np.random.default_rng(1)
    words = np.array(words + list(rng.integers(0, 2 ** 32, size=500, dtype=np.uint64)), dtype=np.uint32)
    trick = O.dequantize_s4_bittrick(words)                     # fp16 [n, 8]
    closed = O.awq_unpack(words.reshape(-1, 1)).astype(np.float16)
    assert np.array_equal(trick, closed)
    assert np.array_equal(O.dequantize_s4(words).reshape(-1, 8), closed)


def test_v2_offset64_bits():
    rng = np.random.default_rng(2)
    words = rng.integers(0, 2 ** 32, size=300, dtype=np.uint64).astype(np.uint32)
    bits = O.dequantize_s4_v2_bits(words)
    vals = bits.view(np.float16).astype(np.float32)
    q = O.awq_unpack(words.reshape(-1, 1)).astype(np.float32)
    assert np.array_equal(vals, q + 64.0)
    assert np.array_equal(bits, (0x5400 | (q.astype(np.uint16) << 4)))


# ---------------------------------------------------------------- R3 Q
def test_merge_q_words():
    rng = np.random.default_rng(3)
    G, N = 3, 32
    z = rng.integers(0, 16, size=(G, N), dtype=np.uint8)
    s = (np.abs(rng.standard_normal((G, N))) * 0.01 + 1e-3).astype(np.float16)
    Q = O.merge_q(O.awq_pack(z), s)
    lo = (Q & 0xFFFF).astype(np.uint16)
    hi = (Q >> 16).astype(np.uint16)
    assert np.array_equal(lo.view(np.float16).astype(np.float32), 64.0 + z)
    assert np.array_equal(hi, s.view(np.uint16))
    z2, s2 = O.split_q(Q)
    assert np.array_equal(z2, z) and np.array_equal(s2.view(np.uint16), s.view(np.uint16))


# ---------------------------------------------------------------- R4 reference layout
def _tagged(K, N):
    """Three AWQ-packed tensors whose nibbles carry 4 bits each of the logical linear index."""
    idx = (np.arange(K)[:, None] * N + np.arange(N)[None, :]).astype(np.int64)
    return [O.awq_pack(((idx >> (4 * p)) & 0xF).astype(np.uint8)) for p in range(4)], idx


@pytest.mark.parametrize("K,N", [(32, 32), (64, 96)])
def test_reference_layout_element_map(K, N):
    planes, _ = _tagged(K, N)
    outs = [O.words_to_nibbles(O.reformat_s4_k_m8(p, N, K)) for p in planes]
    tag = sum(o.astype(np.int64) << (4 * i) for i, o in enumerate(outs))     # [words, 8]
    assert sorted(tag.reshape(-1).tolist()) == list(range(K * N))            # bijection
    for w in range(tag.shape[0]):
        word, lane = w & 3, (w >> 2) & 31
        kt, nt = divmod(w >> 7, N // 32)
        for nib in range(8):
            kk, nn = O.reference_layout_element(kt, nt, lane, word, nib)
            assert tag[w, nib] == kk * N + nn


def test_reference_layout_matches_mma_fragment():
    # mma.m16n8k16 A fragment (row-major 16x16): register r of lane l holds
    # row = l/4 + 8*(r%2), cols = 2*(l%4) + 8*(r/2) + {0,1}.  warp_iterator.h:68-83 feeds
    # word (k16*2 + n16) through the unpack, whose outputs 0..7 are nibbles [0,4,1,5,2,6,3,7].
    for lane in range(32):
        for word in range(4):
            for p in range(8):
                nib = O.UNPACK_NIBBLE[p]
                kk, nn = O.reference_layout_element(0, 0, lane, word, nib)
                r, h = divmod(p, 2)
                assert nn == 16 * (word & 1) + lane // 4 + 8 * (r % 2)
                assert kk == 16 * (word >> 1) + 2 * (lane % 4) + 8 * (r // 2) + h


# ---------------------------------------------------------------- R5 dequantised weights
def test_fp16_multiply_is_single_rounding_of_product():
    # all 31 differences x a dense sweep of fp16 scales, against float64 (exact product)
    d = np.arange(-15, 16, dtype=np.float64)
    s = np.arange(0x0400, 0x7C00, 7, dtype=np.uint16).view(np.float16)      # normal, finite
    exact = (d[:, None] * s.astype(np.float64)[None, :])
    with np.errstate(over="ignore"):
        want = exact.astype(np.float16)
        got = (d.astype(np.float32)[:, None] * s.astype(np.float32)[None, :]).astype(np.float16)
    assert np.array_equal(want.view(np.uint16), got.view(np.uint16))


def test_dequant_weights_closed_form_and_ftz():
    rng = np.random.default_rng(5)
    K, N, g = 256, 32, 128
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = (np.abs(rng.standard_normal((K // g, N))) * 0.01 + 1e-3).astype(np.float16)
    W = O.dequant_weights(q, z, s, g)
    for k in (0, 1, 127, 128, 255):
        for n in (0, 7, 31):
            want = np.float16(np.float64(int(q[k, n]) - int(z[k // g, n])) * np.float64(s[k // g, n]))
            assert W[k, n] == want
    # subnormal products and subnormal scales are flushed to zero (mul.ftz / sub.ftz)
    s_small = np.full((K // g, N), 2.0 ** -16, dtype=np.float16)             # subnormal input
    assert not np.any(O.dequant_weights(q, z, s_small, g))
    s_edge = np.full((K // g, N), 2.0 ** -14, dtype=np.float16)              # min normal
    W2 = O.dequant_weights(q, z, s_edge, g)
    assert np.all((W2 == 0) | (np.abs(W2.astype(np.float64)) >= 2.0 ** -14))
    assert np.any(W2 != 0)


# ---------------------------------------------------------------- R6 / R7 fuse + transpose_qk
def test_fuse_w1_w3_invariant():
    rng = np.random.default_rng(6)
    K, N1 = 16, 48
    w1 = rng.integers(0, 16, size=(K, N1), dtype=np.uint8)
    w3 = rng.integers(0, 16, size=(K, N1), dtype=np.uint8)
    src = np.concatenate([O.awq_pack(w1), O.awq_pack(w3)])                   # [2K, N1/8]
    U = O.awq_unpack(O.fuse_w1_w3_s4_k_m8(src, N1, K))
    assert U.shape == (K, 2 * N1)
    assert np.array_equal(U[:, 0::2], w1) and np.array_equal(U[:, 1::2], w3)


@pytest.mark.parametrize("D", [16, 32, 128])
def test_transpose_qk_invariant(D):
    rng = np.random.default_rng(7)
    K, heads = 8, 3
    N = heads * D
    w = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    U = O.awq_unpack(O.transpose_qk_s4_k_m8_hf(O.awq_pack(w), N, K, D))
    for h in range(heads):
        for i in range(D // 2):
            for r in range(2):
                assert np.array_equal(U[:, h * D + 2 * i + r], w[:, h * D + r * D // 2 + i])
    # == deploy.py:371-377 `permute` on the unpacked matrix
    perm = w.reshape(K, heads, 2, D // 2).transpose(0, 1, 3, 2).reshape(K, N)
    assert np.array_equal(U, perm)


# ---------------------------------------------------------------- gfx950 layout (this build's)
@pytest.mark.parametrize("K,N", [(128, 16), (256, 48), (384, 32)])
def test_gfx950_layout_bijection_and_element_map(K, N):
    planes, _ = _tagged(K, N)
    outs = [O.words_to_nibbles(O.repack_gfx950(p, N, K)) for p in planes]
    tag = sum(o.astype(np.int64) << (4 * i) for i, o in enumerate(outs))
    assert sorted(tag.reshape(-1).tolist()) == list(range(K * N))
    for w in range(0, tag.shape[0], 3):
        for nib in range(8):
            kk, nn = O.gfx950_layout_element(N, K, w, nib)
            assert tag[w, nib] == kk * N + nn
    rng = np.random.default_rng(8)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    assert np.array_equal(O.unrepack_gfx950(O.repack_gfx950(O.awq_pack(q), N, K), N, K), q)


# ---------------------------------------------------------------- R8-R10 GEMM + epilogues
def _small(seed, T, K, N, residual=False):
    return O.make_inputs(seed, T, K, N, 128, residual)


def test_gemm_identity_activations_return_weights_bit_exact():
    d = _small(10, 128, 128, 32)
    X = np.eye(128, dtype=np.float16)
    Y = O.gemm_s4_f16(X, d["qweight"], d["qzeros"], d["scales"], 128)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    assert np.array_equal(Y.view(np.uint16), W.view(np.uint16))


def test_gemm_one_hot_rows_and_zero_weights():
    d = _small(11, 4, 256, 32)
    X = np.zeros((4, 256), dtype=np.float16)
    rows = [0, 17, 128, 255]
    for t, k in enumerate(rows):
        X[t, k] = 1.0
    Y = O.gemm_s4_f16(X, d["qweight"], d["qzeros"], d["scales"], 128)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    assert np.array_equal(Y, W[rows])
    # q == z everywhere  =>  W == 0  =>  Y == 0
    zfull = np.repeat(d["z"], 128, axis=0)
    Y0 = O.gemm_s4_f16(d["X"], O.awq_pack(zfull), d["qzeros"], d["scales"], 128)
    assert not np.any(Y0)


def test_gemm_exact_integer_case():
    # power-of-two scales and small integer activations: every partial sum is an integer
    # multiple of 2^-3 far below 2^24, so fp32 accumulation is exact in any order
    rng = np.random.default_rng(12)
    T, K, N, g = 5, 256, 32, 128
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // g, N), dtype=np.uint8)
    s = (2.0 ** rng.integers(-3, 2, size=(K // g, N))).astype(np.float16)
    X = rng.integers(-3, 4, size=(T, K)).astype(np.float16)
    Y = O.gemm_s4_f16(X, O.awq_pack(q), O.awq_pack(z), s, g)
    Wi = (q.astype(np.int64).reshape(K // g, g, N) - z[:, None, :]).reshape(K, N) * np.repeat(
        s.astype(np.float64), g, axis=0)
    want = (X.astype(np.float64) @ Wi)
    assert np.array_equal(Y.astype(np.float64), want.astype(np.float16).astype(np.float64))


def test_gemm_against_float64():
    d = _small(13, 7, 512, 64)
    Y = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128).astype(np.float64)
    want = d["X"].astype(np.float64) @ W
    assert O.max_abs_rel(Y, want) < 1e-3


def test_silu_epilogue_closed_form():
    rng = np.random.default_rng(14)
    acc = rng.standard_normal((6, 32)).astype(np.float32) * 4
    out = O.epilogue(acc, O.EPI_SILU)
    assert out.shape == (6, 16)
    y = acc.astype(np.float16).astype(np.float64)
    g, u = y[:, 0::2], y[:, 1::2]
    want = g / (1.0 + np.exp(-g)) * u
    assert O.max_abs_rel(out, want) < 2e-3
    # even column is the gate: swapping the pair changes the result
    assert not np.array_equal(out, O.epilogue(acc[:, ::-1].copy(), O.EPI_SILU)[:, ::-1])
    import torch
    tw = torch.nn.functional.silu(torch.from_numpy(g)) * torch.from_numpy(u)
    assert O.max_abs_rel(out, tw.numpy()) < 2e-3


def test_add_epilogue_special_cases():
    d = _small(15, 3, 128, 32, residual=True)
    Yg = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128)
    R0 = np.zeros_like(d["R"])
    assert np.array_equal(O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, O.EPI_ADD, R0), Yg)
    X0 = np.zeros_like(d["X"])
    out = O.gemm_s4_f16(X0, d["qweight"], d["qzeros"], d["scales"], 128, O.EPI_ADD, d["R"])
    assert np.array_equal(out.view(np.uint16), d["R"].view(np.uint16))
    full = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, O.EPI_ADD, d["R"])
    want = (d["R"].astype(np.float64) + Yg.astype(np.float64)).astype(np.float16)
    assert np.array_equal(full, want)


def test_convert_keeps_byte_budgets():
    d = _small(16, 1, 256, 64)
    A, Q = O.convert_s4_k_m8(d["qweight"], d["scales"], d["qzeros"], 64, 256, 128)
    assert A.nbytes == 256 * 64 // 2 and Q.nbytes == (256 // 128) * 64 * 4   # LlamaDecoderLayerWeight.cc:103-110
    Ar, Qr = O.convert_s4_k_m8_reference(d["qweight"], d["scales"], d["qzeros"], 64, 256, 128)
    assert np.array_equal(Q, Qr) and Ar.nbytes == A.nbytes
