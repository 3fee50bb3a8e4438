"""Known-answer vectors in tests/golden/w4a16_kat.npz (made by tests/golden/make_kat.py from the
definitions, one element at a time).  The CPU oracle must reproduce them, and so must the GPU
library - the GPU half of this file does not import the oracle."""
import os

import numpy as np
import pytest

KAT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "w4a16_kat.npz")
TOL = 1e-2


@pytest.fixture(scope="module")
def kat():
    return dict(np.load(KAT))          # plain arrays, no pickled objects


def rel(y, yref):
    return float(np.max(np.abs(y.astype(np.float64) - yref)) / np.max(np.abs(yref)))


# ------------------------------------------------------------------ the oracle against the vectors (CPU)
def test_oracle_pack_unpack_and_q(kat):
    from oracle import w4a16_oracle as O
    assert np.array_equal(O.awq_pack(kat["q"]), kat["qweight"])
    assert np.array_equal(O.awq_pack(kat["z"]), kat["qzeros"])
    assert np.array_equal(O.awq_unpack(kat["qweight"]), kat["q"])
    assert np.array_equal(O.merge_q(kat["qzeros"], kat["scales"]), kat["Q"])


def test_oracle_weights_and_layout(kat):
    from oracle import w4a16_oracle as O
    K, N = int(kat["K"]), int(kat["N"])
    W = O.dequant_from_awq(kat["qweight"], kat["qzeros"], kat["scales"], 128)
    assert np.array_equal(W.view(np.uint16), kat["W_bits"])
    assert np.array_equal(O.repack_gfx950(kat["qweight"], N, K), kat["A_gfx950"])
    A, Q = O.convert_s4_k_m8(kat["qweight"], kat["scales"], kat["qzeros"], N, K, 128)
    assert np.array_equal(A, kat["A_gfx950"]) and np.array_equal(Q, kat["Q"])


@pytest.mark.parametrize("kind,key", [(0, "Y"), (1, "Y_silu"), (2, "Y_add")])
def test_oracle_gemm(kat, kind, key):
    from oracle import w4a16_oracle as O
    got = O.gemm_s4_f16(kat["X"], kat["qweight"], kat["qzeros"], kat["scales"], 128, kind, kat["R"] if kind == 2 else None)
    assert got.shape == kat[key].shape and rel(got, kat[key]) <= 2e-3      # fp16 output against float64


def test_oracle_group_size_32(kat):
    from oracle import w4a16_oracle as O
    K, N = int(kat["K"]), int(kat["N"])
    assert np.array_equal(O.awq_pack(kat["z32"]), kat["qzeros32"])
    W = O.dequant_from_awq(kat["qweight"], kat["qzeros32"], kat["scales32"], 32)
    assert np.array_equal(W.view(np.uint16), kat["W32_bits"])
    A, Q = O.convert_s4_k_m8(kat["qweight"], kat["scales32"], kat["qzeros32"], N, K, 32)
    assert np.array_equal(A, kat["A_gfx950"]) and np.array_equal(Q, kat["Q32"])
    got = O.gemm_s4_f16(kat["X"], kat["qweight"], kat["qzeros32"], kat["scales32"], 32)
    assert rel(got, kat["Y32"]) <= 2e-3


# ------------------------------------------------------------------ the library against the vectors (GPU)
@pytest.fixture(scope="module")
def gpu(kat):
    import torch
    import lmdeploy_amd.turbomind as tm

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a.view(np.int32) if a.dtype == np.uint32 else a)).cuda()

    K, N = int(kat["K"]), int(kat["N"])
    qw, qz, s = dev(kat["qweight"]), dev(kat["qzeros"]), dev(kat["scales"])
    A, Q, ws = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32), torch.zeros_like(s)
    tm.convert_s4_k_m8(A, Q, ws, qw, s, qz, N, K, 128)
    torch.cuda.synchronize()
    return dict(torch=torch, tm=tm, dev=dev, A=A, Q=Q, K=K, N=N)


@pytest.mark.gpu
def test_library_convert_and_weights(kat, gpu):
    assert np.array_equal(gpu["A"].cpu().numpy().view(np.uint32).reshape(-1), kat["A_gfx950"])
    assert np.array_equal(gpu["Q"].cpu().numpy().view(np.uint32), kat["Q"])
    W = gpu["tm"].dequantize_repacked(gpu["A"], gpu["Q"], gpu["N"], gpu["K"]).cpu().numpy()
    assert np.array_equal(W.view(np.uint16), kat["W_bits"])


@pytest.mark.gpu
@pytest.mark.parametrize("kind,key", [(0, "Y"), (1, "Y_silu"), (2, "Y_add")])
def test_library_gemm_every_kernel(kat, gpu, kind, key):
    torch, tm = gpu["torch"], gpu["tm"]
    K, N, T = gpu["K"], gpu["N"], int(kat["T"])
    gemm = tm.GemmS4F16()
    X, R = gpu["dev"](kat["X"]), gpu["dev"](kat["R"])
    ran = 0
    for algo in [-1] + list(range(gemm.algo_count())):
        C = torch.full(kat[key].shape, float("nan"), dtype=torch.float16, device="cuda")
        try:
            gemm.Run(C, gpu["A"], X, gpu["Q"], N, T, K, 128, kind, algo, residual=R if kind == 2 else None)
        except tm.W4A16Error as e:
            assert e.code == -2, e
            continue
        torch.cuda.synchronize()
        got = C.cpu().numpy()
        assert np.isfinite(got).all() and rel(got, kat[key]) <= TOL, (algo, rel(got, kat[key]))
        ran += 1
    assert ran >= 10


@pytest.mark.gpu
def test_library_group_size_32(kat, gpu):
    torch, tm, dev = gpu["torch"], gpu["tm"], gpu["dev"]
    K, N, T = gpu["K"], gpu["N"], int(kat["T"])
    qw, qz, s = dev(kat["qweight"]), dev(kat["qzeros32"]), dev(kat["scales32"])
    A, Q = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32)
    tm.convert_s4_k_m8(A, Q, torch.zeros_like(s), qw, s, qz, N, K, 32)
    assert np.array_equal(A.cpu().numpy().view(np.uint32).reshape(-1), kat["A_gfx950"])
    assert np.array_equal(Q.cpu().numpy().view(np.uint32), kat["Q32"])
    W = tm.dequantize_repacked(A, Q, N, K, 32).cpu().numpy()
    assert np.array_equal(W.view(np.uint16), kat["W32_bits"])
    C = torch.full((T, N), float("nan"), dtype=torch.float16, device="cuda")
    tm.GemmS4F16().Run(C, A, dev(kat["X"]), Q, N, T, K, 32, 0, -1)
    torch.cuda.synchronize()
    got = C.cpu().numpy()
    assert np.isfinite(got).all() and rel(got, kat["Y32"]) <= TOL
