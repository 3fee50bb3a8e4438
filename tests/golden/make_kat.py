"""Writes tests/golden/w4a16_kat.npz: a small known-answer set for the W4A16 path.

The reference holds no golden vectors, fixtures or known-answer tests for this path, so these are
derived here from the definitions alone, with plain Python loops over single elements (no
vectorised index arithmetic, nothing imported from the oracle or the library):

* the AWQ packing rule (lmdeploy/pytorch/modules/linear.py:85,105-108),
* the (64 + z, s) word of convert_s4_k_m8's merge_Q (format.cu:84-95),
* the dequantised weight fp16((q - z) * s) (common.h:218-235),
* the gfx950 tile layout (16 columns x 128 rows per 1 KiB tile, group-major),
* GEMM results in float64, and the SiLU / residual epilogues on the fp16-rounded product
  (gemm_s4_f16.cu:22-42, llama_decoder_kernels.cu:52-57).

Both the CPU oracle and the GPU library are checked against the file (tests/test_golden.py).
Run from the repository root:  python tests/golden/make_kat.py
"""
import math
import os

import numpy as np

K, N, T, GROUP = 256, 64, 5, 128
ORDER = [0, 2, 4, 6, 1, 3, 5, 7]          # nibble i of a word holds logical column 8j + ORDER[i]
ROW_NIBBLE = [0, 4, 1, 5, 2, 6, 3, 7]     # row offset e of a gfx950 word sits in nibble ROW_NIBBLE[e]


def main():
    rng = np.random.default_rng(20240229)
    G = K // GROUP
    q = rng.integers(0, 16, size=(K, N))
    z = rng.integers(0, 16, size=(G, N))
    s = (np.abs(rng.standard_normal((G, N))) * 0.01 + 1e-3).astype(np.float16)
    X = rng.standard_normal((T, K)).astype(np.float16)
    R = rng.standard_normal((T, N)).astype(np.float16)

    qweight = np.zeros((K, N // 8), dtype=np.uint32)
    for k in range(K):
        for j in range(N // 8):
            word = 0
            for i in range(8):
                word |= int(q[k, 8 * j + ORDER[i]]) << (4 * i)
            qweight[k, j] = word
    qzeros = np.zeros((G, N // 8), dtype=np.uint32)
    for g in range(G):
        for j in range(N // 8):
            word = 0
            for i in range(8):
                word |= int(z[g, 8 * j + ORDER[i]]) << (4 * i)
            qzeros[g, j] = word

    Q = np.zeros((G, N), dtype=np.uint32)
    W = np.zeros((K, N), dtype=np.float16)
    for g in range(G):
        for n in range(N):
            s_bits = int(s[g, n:n + 1].view(np.uint16)[0])
            Q[g, n] = (0x5400 | (int(z[g, n]) << 4)) | (s_bits << 16)
    for k in range(K):
        for n in range(N):
            g = k // GROUP
            W[k, n] = np.float16(np.float32(int(q[k, n]) - int(z[g, n])) * np.float32(s[g, n]))

    A = np.zeros(K * N // 8, dtype=np.uint32)
    for k in range(K):
        for n in range(N):
            kt, r = divmod(k, 128)
            nt, c = divmod(n, 16)
            j, r32 = divmod(r, 32)
            b, e = divmod(r32, 8)
            lane = 16 * b + c
            word = ((kt * (N // 16) + nt) * 64 + lane) * 4 + j
            A[word] |= np.uint32(int(q[k, n]) << (4 * ROW_NIBBLE[e]))

    Y = np.zeros((T, N), dtype=np.float64)
    for t in range(T):
        for n in range(N):
            acc = 0.0
            for k in range(K):
                acc += float(X[t, k]) * float(W[k, n])
            Y[t, n] = acc
    Yh = Y.astype(np.float16)                       # the single rounding of the accumulator
    silu = np.zeros((T, N // 2), dtype=np.float64)
    for t in range(T):
        for j in range(N // 2):
            gate, up = float(Yh[t, 2 * j]), float(Yh[t, 2 * j + 1])
            silu[t, j] = gate / (1.0 + math.exp(-gate)) * up
    add = np.zeros((T, N), dtype=np.float64)
    for t in range(T):
        for n in range(N):
            add[t, n] = float(R[t, n]) + float(Yh[t, n])

    # The same weights and activations with a zero point and a scale per 32 rows (group size 32; drawn after
    # everything above, so that the arrays above keep their values): Q words, dequantised weights and the plain
    # GEMM, by the same element-wise rules.  The weight layout does not depend on the group size.
    G32 = K // 32
    z32 = rng.integers(0, 16, size=(G32, N))
    s32 = (np.abs(rng.standard_normal((G32, N))) * 0.01 + 1e-3).astype(np.float16)
    qzeros32 = np.zeros((G32, N // 8), dtype=np.uint32)
    for g in range(G32):
        for j in range(N // 8):
            word = 0
            for i in range(8):
                word |= int(z32[g, 8 * j + ORDER[i]]) << (4 * i)
            qzeros32[g, j] = word
    Q32 = np.zeros((G32, N), dtype=np.uint32)
    for g in range(G32):
        for n in range(N):
            Q32[g, n] = (0x5400 | (int(z32[g, n]) << 4)) | (int(s32[g, n:n + 1].view(np.uint16)[0]) << 16)
    W32 = np.zeros((K, N), dtype=np.float16)
    for k in range(K):
        for n in range(N):
            W32[k, n] = np.float16(np.float32(int(q[k, n]) - int(z32[k // 32, n])) * np.float32(s32[k // 32, n]))
    Y32 = np.zeros((T, N), dtype=np.float64)
    for t in range(T):
        for n in range(N):
            acc = 0.0
            for k in range(K):
                acc += float(X[t, k]) * float(W32[k, n])
            Y32[t, n] = acc

    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "w4a16_kat.npz")
    np.savez_compressed(out, K=K, N=N, T=T, q=q.astype(np.uint8), z=z.astype(np.uint8), scales=s, X=X, R=R,
                        qweight=qweight, qzeros=qzeros, Q=Q, W_bits=W.view(np.uint16), A_gfx950=A,
                        Y=Y, Y_silu=silu, Y_add=add,
                        z32=z32.astype(np.uint8), scales32=s32, qzeros32=qzeros32, Q32=Q32, W32_bits=W32.view(np.uint16), Y32=Y32)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
