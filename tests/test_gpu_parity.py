"""GPU parity: the HIP library, called through its C ABI, against the CPU oracle.

Integer work (repack, unpack, fuse, transpose, dequantised weights) must be bit exact.
GEMM outputs must satisfy max|y - yref| / max|yref| <= 1e-2 in fp16 (the stated tolerance),
and are exact in the special cases where the mathematics fixes the answer.  On the benchmark
configurations every single output must also satisfy |y - yref| <= 1e-2 |yref| + 1e-2 rms(yref)."""
import numpy as np
import pytest
import torch

from oracle import w4a16_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(scope="module")
def tm():
    import lmdeploy_amd.turbomind as tm
    return tm


@pytest.fixture(scope="module")
def gemm(tm):
    return tm.GemmS4F16()


def dev(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host_u32(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint32)


def assert_close(got, want, what):
    """The max-norm gate plus the elementwise criterion (pass rate must be 100 %)."""
    err = O.max_abs_rel(got, want)
    rate = O.elementwise_pass_rate(got, want, TOL)
    assert np.isfinite(got).all() and err <= TOL and rate == 1.0, (what, err, rate)


def convert(tm, d, N, K):
    qw, qz, s = dev(d["qweight"]), dev(d["qzeros"]), dev(d["scales"])
    A = torch.zeros_like(qw)
    Q = torch.zeros_like(s, dtype=torch.int32)
    ws = torch.zeros_like(s)
    tm.convert_s4_k_m8(A, Q, ws, qw, s, qz, N, K, 128)
    return A, Q


def run(tm, gemm, d, A, Q, T, K, N, kind=0, algo=-1):
    X = dev(d["X"])
    R = dev(d["R"]) if kind == 2 else None
    n_out = N // 2 if kind == 1 else N
    C = torch.full((T, n_out), float("nan"), dtype=torch.float16, device="cuda")
    gemm.Run(C, A, X, Q, N, T, K, 128, kind, algo, residual=R)
    torch.cuda.synchronize()
    return C.cpu().numpy()


# ------------------------------------------------------------------ repack (integer, bit exact)
@pytest.mark.parametrize("K,N", [(128, 16), (256, 48), (512, 4096), (4096, 4096), (11008, 4096), (4096, 22016)])
def test_convert_bit_exact_and_round_trip(tm, K, N):
    d = O.make_inputs(100 + K + N, 1, K, N)
    A, Q = convert(tm, d, N, K)
    A_ref, Q_ref = O.convert_s4_k_m8(d["qweight"], d["scales"], d["qzeros"], N, K, 128)
    assert np.array_equal(host_u32(A).reshape(-1), A_ref)
    assert np.array_equal(host_u32(Q), Q_ref)
    qw, qz, s = tm.unpack_repacked(A, Q, N, K)
    assert np.array_equal(host_u32(qw), d["qweight"])          # == the reference's own unpack of the input
    assert np.array_equal(host_u32(qz), d["qzeros"])
    assert np.array_equal(s.cpu().numpy().view(np.uint16), d["scales"].view(np.uint16))


@pytest.mark.parametrize("K,N", [(256, 48), (4096, 4096), (11008, 4096)])
def test_dequantised_weights_bit_exact(tm, K, N):
    d = O.make_inputs(200 + K + N, 1, K, N)
    A, Q = convert(tm, d, N, K)
    W = tm.dequantize_repacked(A, Q, N, K).cpu().numpy()
    W_ref = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    assert np.array_equal(W.view(np.uint16), W_ref.view(np.uint16))


def test_dequantised_weights_flush_subnormals(tm):
    K, N = 256, 32
    d = O.make_inputs(7, 1, K, N)
    s = d["scales"].copy()
    s[0, :] = np.float16(2.0 ** -16)      # subnormal scale
    s[1, :] = np.float16(2.0 ** -14)      # products with |q - z| >= 1 are normal, 0 stays 0
    s[1, ::3] = np.float16(3.0e-5)        # subnormal scale again
    d["scales"] = s
    A, Q = convert(tm, d, N, K)
    W = tm.dequantize_repacked(A, Q, N, K).cpu().numpy()
    W_ref = O.dequant_from_awq(d["qweight"], d["qzeros"], s, 128)
    assert np.array_equal(W.view(np.uint16), W_ref.view(np.uint16))


def test_dequantize_s4_bit_exact(tm):
    rng = np.random.default_rng(3)
    words = rng.integers(0, 2 ** 32, size=4099, dtype=np.uint64).astype(np.uint32)
    dst = torch.empty(words.size * 8, dtype=torch.float16, device="cuda")
    tm.dequantize_s4(dev(words), dst)
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy(), O.dequantize_s4(words))
    with pytest.raises(ValueError):
        tm.dequantize_s4(dev(words), dst[:-8])


@pytest.mark.parametrize("K,N1", [(16, 48), (4096, 11008)])
def test_fuse_w1_w3(tm, K, N1):
    rng = np.random.default_rng(4)
    w1 = rng.integers(0, 16, size=(K, N1), dtype=np.uint8)
    w3 = rng.integers(0, 16, size=(K, N1), dtype=np.uint8)
    src = np.concatenate([O.awq_pack(w1), O.awq_pack(w3)])
    dst = torch.zeros(K, 2 * N1 // 8, dtype=torch.int32, device="cuda")
    tm.fuse_w1_w3_s4_k_m8(dev(src), dst, N1, K)
    torch.cuda.synchronize()
    got = host_u32(dst)
    assert np.array_equal(got, O.fuse_w1_w3_s4_k_m8(src, N1, K))
    U = O.awq_unpack(got)
    assert np.array_equal(U[:, 0::2], w1) and np.array_equal(U[:, 1::2], w3)


@pytest.mark.parametrize("K,N,D", [(8, 96, 32), (512, 4096, 128)])
def test_transpose_qk(tm, K, N, D):
    rng = np.random.default_rng(5)
    w = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    src = O.awq_pack(w)
    dst = torch.zeros(K, N // 8, dtype=torch.int32, device="cuda")
    tm.transpose_qk_s4_k_m8(dev(src), dst, N, K, D)
    torch.cuda.synchronize()
    assert np.array_equal(host_u32(dst), O.transpose_qk_s4_k_m8_hf(src, N, K, D))


@pytest.mark.parametrize("K,N", [(128, 32), (512, 4096)])
def test_from_reference_layout(tm, K, N):
    d = O.make_inputs(6, 1, K, N)
    A_ref_layout, _ = O.convert_s4_k_m8_reference(d["qweight"], d["scales"], d["qzeros"], N, K, 128)
    ours = tm.from_reference_layout(dev(A_ref_layout), N, K)
    torch.cuda.synchronize()
    assert np.array_equal(host_u32(ours).reshape(-1), O.repack_gfx950(d["qweight"], N, K))


# ------------------------------------------------------------------ GEMM, every kernel
def _algos(gemm):
    return list(range(gemm.algo_count()))


@pytest.mark.parametrize("T", [1, 3, 16, 17, 33, 125])
def test_every_kernel_small_shape(tm, gemm, T):
    K, N = 1024, 256
    d = O.make_inputs(300 + T, T, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    want = {k: O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, k, d.get("R")) for k in (0, 1, 2)}
    ran = 0
    for algo in _algos(gemm):
        for kind in (0, 1, 2):
            try:
                got = run(tm, gemm, d, A, Q, T, K, N, kind, algo)
            except tm.W4A16Error as e:
                assert e.code == -2, e     # infeasible for this shape is the only acceptable failure
                continue
            ran += 1
            err = O.max_abs_rel(got, want[kind])
            assert np.isfinite(got).all() and err <= TOL, (algo, kind, err)
    assert ran >= 20


@pytest.mark.parametrize("K", [128, 640, 1408])
def test_every_kernel_odd_number_of_groups(tm, gemm, K):
    # K / 128 odd: the prefill kernels, which walk K two groups at a time, must pad with a group
    # that adds nothing; with K split across workgroups some splits are odd and some even
    N = 256
    for T in (40, 130):
        d = O.make_inputs(700 + K + T, T, K, N, residual=True)
        A, Q = convert(tm, d, N, K)
        want = {k: O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, k, d.get("R")) for k in (0, 1, 2)}
        ran = 0
        for algo in _algos(gemm):
            for kind in (0, 1, 2):
                try:
                    got = run(tm, gemm, d, A, Q, T, K, N, kind, algo)
                except tm.W4A16Error as e:
                    assert e.code == -2, e
                    continue
                ran += 1
                err = O.max_abs_rel(got, want[kind])
                assert np.isfinite(got).all() and err <= TOL, (algo, kind, T, err)
        assert ran >= 20


def test_identity_activations_return_weights(tm, gemm):
    # X = I  =>  Y == W.  The prefill kernels use the reference's exact fp16 weight, so they are
    # bit exact; the decode kernels scale after the group sum: (q - z) * s rounded once from fp32,
    # which is the same single rounding.
    K, N = 256, 128
    d = O.make_inputs(9, K, K, N)
    d["X"] = np.eye(K, dtype=np.float16)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    for algo in _algos(gemm):
        try:
            got = run(tm, gemm, d, A, Q, K, K, N, 0, algo)
        except tm.W4A16Error:
            continue
        assert np.array_equal(got.view(np.uint16), W.view(np.uint16)), algo


def test_exact_integer_case_and_zero_weights(tm, gemm):
    rng = np.random.default_rng(12)
    T, K, N = 5, 512, 64
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // 128, N), dtype=np.uint8)
    s = (2.0 ** rng.integers(-3, 2, size=(K // 128, N))).astype(np.float16)
    X = rng.integers(-3, 4, size=(T, K)).astype(np.float16)
    d = dict(qweight=O.awq_pack(q), qzeros=O.awq_pack(z), scales=s, X=X)
    A, Q = convert(tm, d, N, K)
    want = O.gemm_s4_f16(X, d["qweight"], d["qzeros"], s, 128)
    for algo in _algos(gemm):
        try:
            got = run(tm, gemm, d, A, Q, T, K, N, 0, algo)
        except tm.W4A16Error:
            continue
        assert np.array_equal(got, want), algo
    # q == z  =>  Y == 0 ; with the residual epilogue  =>  Y == R bit for bit
    d0 = dict(d, qweight=O.awq_pack(np.repeat(z, 128, axis=0)), R=rng.standard_normal((T, N)).astype(np.float16))
    A0, Q0 = convert(tm, d0, N, K)
    assert not np.any(run(tm, gemm, d0, A0, Q0, T, K, N, 0))
    assert np.array_equal(run(tm, gemm, d0, A0, Q0, T, K, N, 2).view(np.uint16), d0["R"].view(np.uint16))


def test_residual_in_place(tm, gemm):
    T, K, N = 8, 512, 128
    d = O.make_inputs(21, T, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, O.EPI_ADD, d["R"])
    C = dev(d["R"])
    gemm.Run(C, A, dev(d["X"]), Q, N, T, K, 128, gemm.kFusedAdd, -1, residual=C)   # C aliases R
    torch.cuda.synchronize()
    assert O.max_abs_rel(C.cpu().numpy(), want) <= TOL


@pytest.fixture(scope="module")
def algo_table(tm, gemm):
    """id -> (kind, tokens per workgroup, K parts) of every kernel configuration (they do not depend on the shape)."""
    T, K, N = 4, 256, 64
    d = O.make_inputs(1, T, K, N)
    A, Q = convert(tm, d, N, K)
    ms = gemm.Measure(torch.empty(T, N, dtype=torch.float16, device="cuda"), A, dev(d["X"]), Q, N, T, K, 128)
    gemm.clear_tuning()
    return {m.id: (m.kind, m.tile_t, m.slices) for m in ms}


@pytest.mark.parametrize("N", [16384, 32768, 22016, 17600, 12288, 36864, 57344])
def test_strip_kernels_on_wide_matrices(tm, gemm, algo_table, N):
    """Strips of several column tiles (2 to 8 per workgroup, even and uneven deals of the column tiles to
    256 and 512 workgroups, and - for more than 2048 column tiles - to 256 workgroups that take two strips one
    after the other), every strip configuration forced by id, few groups (so that some waves of a workgroup have
    none), 16- and 32-token variants, every epilogue."""
    K = 256
    strips = [i for i, (kind, _, _) in algo_table.items() if kind == 2]
    assert len(strips) == 5
    in_turn = sorted(i for i in strips if algo_table[i][1] == 16)[2]   # one workgroup per CU, several strips in turn
    Ts = (1, 8, 16, 20, 32)
    d = O.make_inputs(4000 + N, max(Ts), K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    ran = 0
    for T in Ts:
        dd = dict(d, X=d["X"][:T], R=d["R"][:T])
        acc = O.gemm_acc(dd["X"], W)
        for kind in (0, 1, 2):
            want = O.epilogue(acc, kind, dd["R"] if kind == 2 else None)
            for algo in strips:
                try:
                    got = run(tm, gemm, dd, A, Q, T, K, N, kind, algo)
                except tm.W4A16Error as e:
                    assert e.code == -2, e       # the 32-token strips do not take 16 tokens or fewer
                    # ... and the strips-in-turn kernel only takes matrices too wide for one strip of 8 tiles per CU
                    assert (algo_table[algo][1] == 32 and T <= 16) or (algo == in_turn and N // 16 <= 2048), (algo, T)
                    continue
                ran += 1
                assert_close(got, want, (N, T, kind, algo))
    assert ran >= 3 * (3 * 2 + 2 * 4) + (3 * 5 if N // 16 > 2048 else 0)


@pytest.mark.parametrize("name,K,N,kind", [("qkv", 4096, 12288, 0), ("gate_up", 4096, 22016, 1)])
def test_llama7b_wide_shapes_at_17_to_32_tokens_take_the_32_token_strips(tm, gemm, algo_table, name, K, N, kind):
    """qkv (strips of 3 tiles) and gate_up (strips of 6 and 5 on 256 workgroups, of 3 and 2 on 512) with 32 token
    rows per workgroup, four groups per wave (so every LDS patch is refilled while the other one is in use):
    what the default dispatch picks at 17 and 24 tokens, and forced by id at 32 (where the dispatch may prefer
    an MFMA tile)."""
    d = O.make_inputs(4100 + kind, 32, K, N)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    strip32 = [i for i, (k, tile_t, _) in sorted(algo_table.items()) if (k, tile_t) == (2, 32)]
    for T in (17, 24, 32):
        dd = dict(d, X=d["X"][:T])
        want = O.epilogue(O.gemm_acc(dd["X"], W), kind)
        k, tile_t, _ = algo_table[gemm.pick(N, T, K)]
        if T < 32:
            assert (k, tile_t) == (2, 32), (name, T, k, tile_t)
        assert_close(run(tm, gemm, dd, A, Q, T, K, N, kind), want, (name, T, "default"))
        for algo in strip32:
            assert_close(run(tm, gemm, dd, A, Q, T, K, N, kind, algo), want, (name, T, algo))


def test_subnormal_scales_count_as_zero_in_the_gemm(tm, gemm):
    """The reference multiplies with flush-to-zero (common.h:229-230): a subnormal scale is read as zero, so such a
    group contributes nothing (a normal scale times a non-zero integer is never subnormal, so nothing else is ever
    flushed).  The GEMM kernels do the same; without it this case fails the elementwise criterion."""
    K, N = 512, 256
    for T in (4, 100):
        d = O.make_inputs(4200 + T, T, K, N, residual=True)
        s = d["scales"].copy()
        s[1, :] = np.float16(2.0 ** -16)       # every product of this group is subnormal (or zero)
        s[2, ::2] = np.float16(3.0e-5)
        d["scales"] = s
        A, Q = convert(tm, d, N, K)
        for kind in (0, 1, 2):
            want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], s, 128, kind, d["R"])
            assert_close(run(tm, gemm, d, A, Q, T, K, N, kind), want, (T, kind))


# ------------------------------------------------------------------ the benchmark configurations
LLAMA7B = [("qkv", 4096, 12288, 0), ("o", 4096, 4096, 0), ("gate_up", 4096, 22016, 1), ("down", 11008, 4096, 2)]
SEED = {"qkv": 11, "o": 22, "gate_up": 33, "down": 44}


@pytest.mark.parametrize("name,K,N,kind", LLAMA7B)
def test_llama7b_decode_shapes(tm, gemm, name, K, N, kind):
    d = O.make_inputs(SEED[name], 16, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    for T in (1, 4, 8, 16):
        dd = dict(d, X=d["X"][:T], R=d["R"][:T])
        want = O.epilogue(O.gemm_acc(dd["X"], W), kind, dd["R"] if kind == 2 else None)
        got = run(tm, gemm, dd, A, Q, T, K, N, kind)
        assert_close(got, want, (name, T))


@pytest.mark.parametrize("name,K,N,kind", LLAMA7B)
def test_llama7b_prefill_shapes_sampled_rows(tm, gemm, name, K, N, kind):
    # T = 2048 on the GPU; the oracle checks 96 of the 2048 token rows (first, last and random
    # rows: output rows are independent, so this covers every column and every tile row class)
    T = 2048
    d = O.make_inputs(SEED[name] + 1, T, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    got = run(tm, gemm, d, A, Q, T, K, N, kind)
    rng = np.random.default_rng(0)
    rows = np.unique(np.concatenate([[0, 1, 15, 16, 255, 256, T - 1], rng.integers(0, T, 89)]))
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    want = O.epilogue(O.gemm_acc(d["X"][rows], W), kind, d["R"][rows] if kind == 2 else None)
    assert np.isfinite(got).all()
    assert_close(got[rows], want, name)


def test_llama7b_o_prefill_every_output_row(tm, gemm):
    # The sampled comparisons of the T = 2048 shapes rest on this one: the smallest of them (o, 4096 x 4096)
    # with all 2048 x 4096 outputs held against the oracle, for the default kernel and every large prefill tile.
    T, K, N = 2048, 4096, 4096
    d = O.make_inputs(SEED["o"] + 2, T, K, N)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    want = O.epilogue(O.gemm_acc(d["X"], W), 0)
    assert_close(run(tm, gemm, d, A, Q, T, K, N, 0), want, "o, default kernel")
    ms = gemm.Measure(torch.empty(T, N, dtype=torch.float16, device="cuda"), A, dev(d["X"]), Q, N, T, K, 128)
    gemm.clear_tuning()
    large = [m.id for m in ms if m.feasible and m.kind == 1 and m.slices == 1 and m.tile_t >= 128]
    assert len(large) >= 3
    for algo in large:
        assert_close(run(tm, gemm, d, A, Q, T, K, N, 0, algo), want, ("o", algo))


LLAMA70B = [("qkv70", 8192, 10240, 0), ("o70", 8192, 8192, 0), ("gate_up70", 8192, 57344, 1), ("down70", 28672, 8192, 2)]


@pytest.mark.parametrize("name,K,N,kind", LLAMA70B)
def test_llama70b_shapes_sampled_columns(tm, gemm, name, K, N, kind):
    """Llama-2-70B GQA layer shapes, unsharded, at M in {1, 16, 2048}.  The GPU computes everything;
    the oracle dequantises 512 sampled column pairs (first, last and random ones: output columns are
    independent, and pairs keep gate/up together for the SiLU epilogue) and, at 2048 tokens, 48
    sampled token rows."""
    Tmax = 2048
    d = O.make_inputs(700 + kind + K // 1024, Tmax, K, N, residual=kind == 2)
    A, Q = convert(tm, d, N, K)
    rng = np.random.default_rng(5)
    pairs = np.unique(np.concatenate([[0, 1, 7, 8, N // 2 - 1], rng.integers(0, N // 2, 507)]))
    cols = np.stack([2 * pairs, 2 * pairs + 1], axis=1).reshape(-1)
    Wc = O.dequant_weights(d["q"][:, cols], d["z"][:, cols], d["scales"][:, cols], 128)
    for T in (1, 16, Tmax):
        dd = dict(d, X=d["X"][:T])
        if kind == 2:
            dd["R"] = d["R"][:T]
        got = run(tm, gemm, dd, A, Q, T, K, N, kind)
        rows = np.arange(T) if T <= 16 else np.unique(np.concatenate([[0, 15, 16, T - 1], rng.integers(0, T, 44)]))
        want = O.epilogue(O.gemm_acc(dd["X"][rows], Wc), kind, dd["R"][rows][:, cols] if kind == 2 else None)
        sel = got[rows][:, pairs] if kind == 1 else got[rows][:, cols]
        assert np.isfinite(got).all()
        assert_close(sel, want, (name, T))


def test_llama7b_32_layer_decode_sequence(tm, gemm):
    """The full 32-layer Llama-2-7B GEMM sequence of one decode step at M = 8: per layer
    qkv -> o -> gate_up (SiLU) -> down (+ residual), every layer with its own random int4 weights
    (3.5 GB packed), outputs feeding the next GEMM.  Attention and norms are not part of this path:
    o_proj reads the first 4096 features of the qkv output, and every GEMM input is rescaled to unit
    variance on the host side of the test so that 128 chained GEMMs stay in fp16 range.  The oracle
    replays layers 0 and 31 from the GPU's own inputs to those layers."""
    T, H, F, L = 8, 4096, 11008, 32
    gen = torch.Generator(device="cuda").manual_seed(1234)

    def rand_w(K, N):
        A = torch.randint(-2 ** 31, 2 ** 31 - 1, (K * N // 8,), dtype=torch.int32, device="cuda", generator=gen)
        s = (torch.randn((K // 128, N), device="cuda", generator=gen).abs() * 0.01 + 1e-3).half()
        z = torch.randint(0, 16, (K // 128, N), device="cuda", generator=gen, dtype=torch.int32)
        Q = (s.view(torch.int16).to(torch.int32) << 16) | (0x5400 | (z << 4))
        return A, Q

    shapes = [(H, 3 * H, 0), (H, H, 0), (H, 2 * F, 1), (F, H, 2)]
    layers = [[rand_w(K, N) for K, N, _ in shapes] for _ in range(L)]
    x = torch.randn(T, H, device="cuda", generator=gen).half()
    keep = {}

    def norm(t):
        return (t.float() / t.float().std()).half()

    for li, ws in enumerate(layers):
        x_in = norm(x)
        qkv = torch.empty(T, 3 * H, dtype=torch.float16, device="cuda")
        gemm.Run(qkv, ws[0][0], x_in, ws[0][1], 3 * H, T, H, 128, 0)
        o_in = norm(qkv[:, :H]).contiguous()
        o = torch.empty(T, H, dtype=torch.float16, device="cuda")
        gemm.Run(o, ws[1][0], o_in, ws[1][1], H, T, H, 128, 0)
        f_in = norm(o)
        act = torch.empty(T, F, dtype=torch.float16, device="cuda")
        gemm.Run(act, ws[2][0], f_in, ws[2][1], 2 * F, T, H, 128, 1)
        d_in = norm(act)
        out = x_in.clone()
        gemm.Run(out, ws[3][0], d_in, ws[3][1], H, T, F, 128, 2, -1, residual=out)
        if li in (0, L - 1):
            keep[li] = [t.cpu().numpy() for t in (x_in, qkv, o_in, o, f_in, act, d_in, out)]
        x = out
    torch.cuda.synchronize()
    assert torch.isfinite(x).all()

    for li in (0, L - 1):
        x_in, qkv, o_in, o, f_in, act, d_in, out = keep[li]
        for (K, N, kind), (A, Q), xin, got, res in zip(shapes, layers[li], (x_in, o_in, f_in, d_in),
                                                       (qkv, o, act, out), (None, None, None, x_in)):
            qw, qz, sc = tm.unpack_repacked(A, Q, N, K, 128)
            W = O.dequant_from_awq(host_u32(qw), host_u32(qz), sc.cpu().numpy(), 128)
            want = O.epilogue(O.gemm_acc(xin, W), kind, res)
            assert_close(got, want, (li, K, N, kind))


@pytest.mark.parametrize("K,N", [(1024, 3072), (512, 4112), (128, 16), (2048, 2064), (4224, 1024)])
def test_default_dispatch_over_token_counts(tm, gemm, K, N):
    """`algo_id = -1` across the hand-over points between the decode, strip and prefill kernels,
    on shapes with and without the divisibility the wider tiles need (4112 = 16 * 257, 2064 = 16 * 129),
    and on a deep narrow one (33 groups) where the prefill tiles split K across workgroups."""
    Ts = (1, 5, 16, 17, 24, 32, 33, 48, 64, 100, 129, 192, 300, 1000)
    d = O.make_inputs(900 + K + N, max(Ts), K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    for kind in ((0, 2) if N % 32 else (0, 1, 2)):
        for T in Ts:
            dd = dict(d, X=d["X"][:T], R=d["R"][:T])
            want = O.epilogue(O.gemm_acc(dd["X"], W), kind, dd["R"] if kind == 2 else None)
            got = run(tm, gemm, dd, A, Q, T, K, N, kind)
            err = O.max_abs_rel(got, want)
            assert np.isfinite(got).all() and err <= TOL, (K, N, kind, T, gemm.pick(N, T, K), err)


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_token_tails_of_the_reference_test(tm, gemm, kind):
    """The token counts that the reference's mixed-GEMM test sweeps
    (tests/csrc/gemm_dequantize/th_gemm_dequantize.py:170: 256, 177, 195, 125, 66, 33, 8, 2, 1) plus a few
    odd ones, through the default dispatch, all three epilogues."""
    K, N = 1024, 1024
    Ts = (1, 2, 3, 7, 8, 9, 17, 33, 66, 125, 177, 195, 256)
    d = O.make_inputs(1700 + kind, max(Ts), K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    for T in Ts:
        dd = dict(d, X=d["X"][:T], R=d["R"][:T])
        want = O.epilogue(O.gemm_acc(dd["X"], W), kind, dd["R"] if kind == 2 else None)
        got = run(tm, gemm, dd, A, Q, T, K, N, kind)
        err = O.max_abs_rel(got, want)
        assert np.isfinite(got).all() and err <= TOL, (kind, T, gemm.pick(N, T, K), err)


def test_graph_replays_of_kernels_that_use_the_handle_scratch(tm, gemm):
    """The split-K kernels keep arrival counters in the handle and reset them themselves (no memset node).
    A captured graph holding one GEMM per such kernel is replayed several times, with new activations
    written eagerly between the replays, and every replay must equal the eager result bit for bit."""
    K, N, T = 4224, 1024, 100
    d = O.make_inputs(777, T, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    X, R = dev(d["X"]), dev(d["R"])
    ms = gemm.Measure(torch.empty((T, N), dtype=torch.float16, device="cuda"), A, X, Q, N, T, K, 128, gemm.kGemm)
    algos = [m.id for m in ms if m.feasible]           # every kernel that can run the shape, split-K ones included
    assert sum(1 for m in ms if m.feasible and m.kind == 1 and m.slices > 1) >= 4
    gemm.clear_tuning()
    outs = [torch.empty((T, N), dtype=torch.float16, device="cuda") for _ in algos]
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        st = torch.cuda.current_stream().cuda_stream
        for a, C in zip(algos, outs):
            gemm.Run(C, A, X, Q, N, T, K, 128, gemm.kFusedAdd, a, residual=R, stream=st)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    for rep in range(5):
        X.copy_(torch.randn((T, K), device="cuda", generator=gen).half())       # eager work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for a, C in zip(algos, outs):
            E = torch.empty_like(C)
            gemm.Run(E, A, X, Q, N, T, K, 128, gemm.kFusedAdd, a, residual=R)
            torch.cuda.synchronize()
            assert torch.equal(E.view(torch.int16), C.view(torch.int16)), (rep, a)


def test_every_kernel_is_deterministic(tm, gemm):
    """Sliced and split K sums are added in a fixed order (as the reference's sum_slices, gemm_template.h:288-333),
    so repeated launches must agree bit for bit, whichever workgroup happens to arrive last."""
    K, N, T = 4224, 1024, 100
    d = O.make_inputs(4242, T, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    X, R = dev(d["X"]), dev(d["R"])
    ran = 0
    for algo in _algos(gemm):
        first = None
        for rep in range(8):
            C = torch.full((T, N), float("nan"), dtype=torch.float16, device="cuda")
            try:
                gemm.Run(C, A, X, Q, N, T, K, 128, gemm.kFusedAdd, algo, residual=R)
            except tm.W4A16Error:
                break
            got = C.view(torch.int16)
            if first is None:
                first = got.clone()
            else:
                assert torch.equal(got, first), (algo, rep)
        ran += first is not None
    assert ran >= 30


def test_random_shapes_every_kernel(tm, gemm):
    """Seeded random (K, N, T) x every kernel configuration x every epilogue, against an fp32 torch matmul on
    the library's own dequantised weights (which test_dequantised_weights_bit_exact pins to the oracle)."""
    import random
    rng = random.Random(5)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    ran = 0
    for case in range(24):
        K, N = 128 * rng.randint(1, 44), 64 * rng.randint(1, 40)
        T = rng.choice([1, 2, 5, 8, 13, 16, 17, 20, 31, 32, 33, 47, 64, 65, 100, 128, 129, 200, 257])
        G = K // 128
        qw = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        qz = torch.randint(-2**31, 2**31 - 1, (G, N // 8), dtype=torch.int32, device="cuda", generator=gen)
        s = (torch.randn((G, N), device="cuda", generator=gen).abs() * 0.01 + 1e-3).half()
        A, Q = torch.empty_like(qw), torch.empty((G, N), dtype=torch.int32, device="cuda")
        tm.convert_s4_k_m8(A, Q, s, qw, s, qz, N, K, 128)
        W = tm.dequantize_repacked(A, Q, N, K).float()
        X = torch.randn((T, K), device="cuda", generator=gen).half()
        R = torch.randn((T, N), device="cuda", generator=gen).half()
        y = (X.float() @ W).half().float()                       # the single rounding of the accumulator
        want = {0: y, 1: y[:, 0::2] / (1 + torch.exp(-y[:, 0::2])) * y[:, 1::2], 2: R.float() + y}
        for algo in [-1] + _algos(gemm):
            for kind in (0, 1, 2):
                C = torch.full((T, N // 2 if kind == 1 else N), float("nan"), dtype=torch.float16, device="cuda")
                try:
                    gemm.Run(C, A, X, Q, N, T, K, 128, kind, algo, residual=R if kind == 2 else None)
                except tm.W4A16Error as e:
                    assert e.code == -2, e
                    continue
                err = ((C.float() - want[kind]).abs().max() / want[kind].abs().max()).item()
                assert err <= TOL, (K, N, T, algo, kind, err)
                ran += 1
    assert ran >= 1000


def test_ffn_block(tm, gemm):
    """LlamaFfnLayer's int4 branch as one call: fused gate/up + SiLU into the gating buffer, then w2
    (+ residual, in place), against the oracle chained through the same fp16 intermediate."""
    T, H, F = 6, 512, 768
    d13 = O.make_inputs(31, T, H, 2 * F)
    d2 = O.make_inputs(32, T, F, H, residual=True)
    A13, Q13 = convert(tm, d13, 2 * F, H)
    A2, Q2 = convert(tm, d2, H, F)
    x = dev(d13["X"])
    gating = torch.empty((T, F), dtype=torch.float16, device="cuda")
    out = torch.empty((T, H), dtype=torch.float16, device="cuda")
    gemm.ffn(out, gating, x, A13, Q13, A2, Q2, H, F, T)
    torch.cuda.synchronize()
    want_g = O.gemm_s4_f16(d13["X"], d13["qweight"], d13["qzeros"], d13["scales"], 128, O.EPI_SILU)
    assert O.max_abs_rel(gating.cpu().numpy(), want_g) <= TOL
    g_host = gating.cpu().numpy()               # the second GEMM is checked on the GPU's own intermediate
    want = O.gemm_s4_f16(g_host, d2["qweight"], d2["qzeros"], d2["scales"], 128)
    assert O.max_abs_rel(out.cpu().numpy(), want) <= TOL
    res = dev(d2["R"])
    gemm.ffn(res, gating, x, A13, Q13, A2, Q2, H, F, T, residual=res)     # output aliases the residual
    torch.cuda.synchronize()
    want = O.gemm_s4_f16(g_host, d2["qweight"], d2["qzeros"], d2["scales"], 128, O.EPI_ADD, d2["R"])
    assert O.max_abs_rel(res.cpu().numpy(), want) <= TOL
    with pytest.raises(tm.W4A16Error):
        gemm.ffn(out, gating, x, A13, Q13, A2, Q2, H, F, T, group_size=256)


def test_errors(tm, gemm):
    T, K, N = 4, 256, 64
    d = O.make_inputs(1, T, K, N)
    A, Q = convert(tm, d, N, K)
    X = dev(d["X"])
    C = torch.empty(T, N, dtype=torch.float16, device="cuda")
    with pytest.raises(tm.W4A16Error, match="unsupported group size") as e:
        gemm.Run(C, A, X, Q, N, T, K, 256)
    assert e.value.code == -1
    with pytest.raises(tm.W4A16Error, match="no feasible kernel found") as e:
        gemm.Run(C, A, X, Q, N + 8, T, K, 128)
    assert e.value.code == -2
    with pytest.raises(tm.W4A16Error) as e:
        gemm.Run(C, A, X, Q, N, T, K, 128, 0, 10 ** 6)
    assert e.value.code == -5
    with pytest.raises(tm.W4A16Error) as e:
        gemm.Run(C, A, X, Q, N, T, K, 128, gemm.kFusedAdd)        # residual missing
    assert e.value.code == -4
    gemm.Run(C, A, X, Q, N, 0, K, 128)                            # zero tokens: no-op


def test_measure_reports_all_kernels(tm, gemm):
    T, K, N = 8, 1024, 256
    d = O.make_inputs(2, T, K, N)
    A, Q = convert(tm, d, N, K)
    C = torch.empty(T, N, dtype=torch.float16, device="cuda")
    ms = gemm.Measure(C, A, dev(d["X"]), Q, N, T, K, 128)
    assert len(ms) == gemm.algo_count()
    feas = [m for m in ms if m.feasible]
    assert feas and all(np.isfinite(m.ms) and m.count == 100 for m in feas)
    assert [m.ms for m in ms] == sorted(m.ms for m in ms)
    assert sum(m.best for m in ms) == 1
    # the handle remembers the winner for exactly this shape and Run(algo_id=-1) uses it
    assert gemm.pick(N, T, K) == ms[0].id
    got = run(tm, gemm, d, A, Q, T, K, N, 0)
    assert O.max_abs_rel(got, O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128)) <= TOL
    other = tm.GemmS4F16()                      # a fresh handle knows nothing: heuristic choice
    heuristic = other.pick(N, T, K)
    gemm.clear_tuning()
    assert gemm.pick(N, T, K) == heuristic
    with pytest.raises(tm.W4A16Error):
        gemm.pick(N + 8, T, K)


@pytest.mark.parametrize("K,N,tokens", [(4224, 64, (1, 3, 4)), (4224, 4096, (1, 2, 4)), (4224, 22016, (1, 4, 8, 16)),
                                         (11008, 4096, (1, 4))])
def test_narrow_and_wide_strip_variants(tm, gemm, K, N, tokens):
    """The strip kernel's variants that the launcher picks by strip width: sixteen waves for one-tile strips at up to
    four tokens (64 and 4096 columns), one group in flight per wave for wide strips (22016 columns); 33 groups of K
    do not divide by the waves of either."""
    d0 = O.make_inputs(900 + N, max(tokens), K, N, residual=True)
    A, Q = convert(tm, d0, N, K)
    for T in tokens:
        d = dict(d0, X=d0["X"][:T], R=d0["R"][:T])
        for kind in (0, 1, 2):
            want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, kind, d["R"])
            assert_close(run(tm, gemm, d, A, Q, T, K, N, kind), want, (K, N, T, kind))


def test_clock_recording_changes_no_result_and_reads_a_plausible_clock(tm):
    """The measurement aid that records the engine clock inside the strip kernels: same outputs with and without it,
    a clock between 1 and 3 GHz, one record per launch; and the MFMA probe runs and records too."""
    g = tm.GemmS4F16()
    K, N, T = 1024, 4096, 5
    d = O.make_inputs(77, T, K, N)
    A, Q = convert(tm, d, N, K)
    plain = run(tm, g, d, A, Q, T, K, N, 0)
    g.clock_begin()
    rec = [run(tm, g, d, A, Q, T, K, N, 0) for _ in range(3)]
    c = g.clock_end()
    assert all(np.array_equal(r, plain) for r in rec)
    assert c["launches"] == 3 and 1000 < c["MHz"] < 3000 and 0 < c["us_per_launch"] < 1000, c
    again = run(tm, g, d, A, Q, T, K, N, 0)       # recording is off again
    assert np.array_equal(again, plain) and g.clock_end()["launches"] == 3
    g.clock_begin()
    flop = g.probe_mfma(8, 1000)
    c = g.clock_end()
    assert flop > 0 and c["launches"] == 1 and 1000 < c["MHz"] < 3000, c


def test_measured_choices_survive_in_a_file(tm, tmp_path):
    """w4a16_measure -> w4a16_save_tuning -> a fresh handle -> w4a16_load_tuning: the fresh handle then picks
    what was measured; a file written for another library version or CU count is refused and changes nothing."""
    T, K, N = 24, 1024, 512
    d = O.make_inputs(8800, T, K, N)
    A, Q = convert(tm, d, N, K)
    g1 = tm.GemmS4F16()
    ms = g1.Measure(torch.empty(T, N, dtype=torch.float16, device="cuda"), A, dev(d["X"]), Q, N, T, K, 128)
    fastest = ms[0].id
    assert g1.pick(N, T, K) == fastest
    path = str(tmp_path / "tuning.txt")
    assert g1.save_tuning(path) == 1
    g2 = tm.GemmS4F16()
    heuristic = g2.pick(N, T, K)
    assert g2.load_tuning(path) == 1
    assert g2.pick(N, T, K) == fastest
    want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128)
    assert_close(run(tm, g2, d, A, Q, T, K, N), want, "tuned pick")
    # another version / another GPU: refused
    text = open(path).read()
    other = str(tmp_path / "other.txt")
    open(other, "w").write(text.replace("cus=", "cus=9", 1))
    g3 = tm.GemmS4F16()
    with pytest.raises(tm.W4A16Error) as e:
        g3.load_tuning(other)
    assert e.value.code == -8 and g3.pick(N, T, K) == heuristic
    open(other, "w").write("hello\n")
    with pytest.raises(tm.W4A16Error) as e:
        g3.load_tuning(other)
    assert e.value.code == -4
    # an entry whose kernel cannot run its shape is skipped, the others are taken
    lines = text.splitlines()
    open(other, "w").write("\n".join([lines[0], "72 4 256 0", lines[1]]) + "\n")
    assert g3.load_tuning(other) == 1 and g3.pick(N, T, K) == fastest


# ------------------------------------------------------------------ group sizes 64 and 32
@pytest.mark.parametrize("gs", [64, 32])
def test_group_sizes_64_and_32_conversion_is_bit_exact(tm, gs):
    """The weight layout does not depend on the group size; Q has K / gs rows.  Repack, Q, the inverse and the
    dequantised weights, word for word against the oracle."""
    K, N = 640, 256
    d = O.make_inputs(6400 + gs, 1, K, N, gs)
    qw, qz, s = dev(d["qweight"]), dev(d["qzeros"]), dev(d["scales"])
    A, Q = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32)
    tm.convert_s4_k_m8(A, Q, torch.zeros_like(s), qw, s, qz, N, K, gs)
    A_ref, Q_ref = O.convert_s4_k_m8(d["qweight"], d["scales"], d["qzeros"], N, K, gs)
    assert np.array_equal(host_u32(A).reshape(-1), A_ref)
    assert np.array_equal(host_u32(Q), Q_ref)
    qw2, qz2, s2 = tm.unpack_repacked(A, Q, N, K, gs)
    assert torch.equal(qw2, qw) and torch.equal(qz2, qz) and torch.equal(s2.view(torch.int16), s.view(torch.int16))
    W = tm.dequantize_repacked(A, Q, N, K, gs).cpu().numpy()
    W_ref = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], gs)
    assert np.array_equal(W.view(np.uint16), W_ref.view(np.uint16))


@pytest.mark.parametrize("gs", [64, 32])
@pytest.mark.parametrize("K,N", [(1024, 256), (640, 4096), (256, 22016), (384, 57344), (128, 48)])
def test_group_sizes_64_and_32_gemm(tm, gemm, gs, K, N):
    """One kernel family serves these group sizes (strips of up to four column tiles, the scale applied per
    quantisation group inside the tile): narrow and wide matrices, uneven deals, one and several strips per CU,
    token counts on both sides of the 16-token block, every epilogue, against the oracle."""
    Ts = (1, 5, 16, 17, 40) if N > 8192 else (1, 5, 16, 17, 40, 130)
    d = O.make_inputs(6500 + gs + N, max(Ts), K, N, gs, residual=True)
    qw, qz, s = dev(d["qweight"]), dev(d["qzeros"]), dev(d["scales"])
    A, Q = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32)
    tm.convert_s4_k_m8(A, Q, torch.zeros_like(s), qw, s, qz, N, K, gs)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], gs)
    for T in Ts:
        X, R = dev(d["X"][:T]), dev(d["R"][:T])
        acc = O.gemm_acc(d["X"][:T], W)
        for kind in (0, 1, 2):
            want = O.epilogue(acc, kind, d["R"][:T] if kind == 2 else None)
            C = torch.full((T, N // 2 if kind == 1 else N), float("nan"), dtype=torch.float16, device="cuda")
            gemm.Run(C, A, X, Q, N, T, K, gs, kind, -1, residual=R if kind == 2 else None)
            torch.cuda.synchronize()
            assert_close(C.cpu().numpy(), want, (gs, K, N, T, kind))
            if T in (5, 40):   # the entry point without a handle runs the same kernel
                Cs = torch.empty_like(C)
                tm.gemm_static(Cs, A, X, Q, N, T, K, gs, kind, -1, residual=R if kind == 2 else None)
                torch.cuda.synchronize()
                assert torch.equal(Cs.view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("gs", [64, 32])
def test_group_sizes_64_and_32_many_tokens(tm, gemm, gs):
    """Above a few hundred tokens these group sizes run on the 256 x 128 MFMA tile (the reference's exact fp16
    weight, scale and zero point changing inside the K step): token counts on both sides of a tile boundary, odd
    numbers of K steps, every epilogue, every output against the oracle; a matrix whose width is not a multiple of
    128 and a misaligned output stay with the strips."""
    for K, N, Ts in ((640, 512, (300, 512, 700)), (1024, 2048, (1000,)), (256, 400, (600,))):
        d = O.make_inputs(6800 + gs + N, max(Ts), K, N, gs, residual=True)
        qw, qz, s = dev(d["qweight"]), dev(d["qzeros"]), dev(d["scales"])
        A, Q = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32)
        tm.convert_s4_k_m8(A, Q, torch.zeros_like(s), qw, s, qz, N, K, gs)
        W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], gs)
        for T in Ts:
            X, R = dev(d["X"][:T]), dev(d["R"][:T])
            acc = O.gemm_acc(d["X"][:T], W)
            for kind in (0, 1, 2):
                want = O.epilogue(acc, kind, d["R"][:T] if kind == 2 else None)
                C = torch.full((T, N // 2 if kind == 1 else N), float("nan"), dtype=torch.float16, device="cuda")
                gemm.Run(C, A, X, Q, N, T, K, gs, kind, -1, residual=R if kind == 2 else None)
                torch.cuda.synchronize()
                assert_close(C.cpu().numpy(), want, (gs, K, N, T, kind))
            if N % 128 == 0:
                buf = torch.zeros(T * N + 8, dtype=torch.float16, device="cuda")
                C1 = buf[2:2 + T * N].view(T, N)      # 4-byte aligned only
                gemm.Run(C1, A, X, Q, N, T, K, gs, 0, -1)
                torch.cuda.synchronize()
                assert_close(C1.cpu().numpy(), O.epilogue(acc, 0), (gs, K, N, T, "misaligned"))


def test_group_size_errors(tm, gemm):
    K, N, T = 256, 64, 4
    d = O.make_inputs(6600, T, K, N, 64)
    qw, qz, s = dev(d["qweight"]), dev(d["qzeros"]), dev(d["scales"])
    A, Q = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32)
    tm.convert_s4_k_m8(A, Q, torch.zeros_like(s), qw, s, qz, N, K, 64)
    C = torch.empty((T, N), dtype=torch.float16, device="cuda")
    for bad in (256, 16, 96, 0):      # gemm_s4_f16.cu:119,233: the reference's message
        with pytest.raises(tm.W4A16Error, match="unsupported group size") as e:
            gemm.Run(C, A, dev(d["X"]), Q, N, T, K, bad)
        assert e.value.code == -1
    with pytest.raises(tm.W4A16Error, match="kernel ids belong to group size 128") as e:
        gemm.Run(C, A, dev(d["X"]), Q, N, T, K, 64, 0, 0)
    assert e.value.code == -5
    with pytest.raises(tm.W4A16Error) as e:
        gemm.Measure(C, A, dev(d["X"]), Q, N, T, K, 64)
    assert e.value.code == -1


def test_group_size_64_ffn_block(tm, gemm):
    """w4a16_ffn (two GEMMs planned as a list) with group size 64, against the oracle."""
    H, F, T, gs = 512, 1408, 9, 64
    d13 = O.make_inputs(6700, T, H, 2 * F, gs, residual=True)
    d2 = O.make_inputs(6701, T, F, H, gs)

    def conv(dd, N, K):
        qw, qz, s = dev(dd["qweight"]), dev(dd["qzeros"]), dev(dd["scales"])
        A, Q = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32)
        tm.convert_s4_k_m8(A, Q, torch.zeros_like(s), qw, s, qz, N, K, gs)
        return A, Q
    A13, Q13 = conv(d13, 2 * F, H)
    A2, Q2 = conv(d2, H, F)
    gating = torch.empty((T, F), dtype=torch.float16, device="cuda")
    out = torch.empty((T, H), dtype=torch.float16, device="cuda")
    res = dev(d13["R"][:, :H].copy())
    gemm.ffn(out, gating, dev(d13["X"]), A13, Q13, A2, Q2, H, F, T, gs, residual=res)
    torch.cuda.synchronize()
    g_ref = O.gemm_s4_f16(d13["X"], d13["qweight"], d13["qzeros"], d13["scales"], gs, O.EPI_SILU)
    assert_close(gating.cpu().numpy(), g_ref, "gating")
    want = O.gemm_s4_f16(gating.cpu().numpy(), d2["qweight"], d2["qzeros"], d2["scales"], gs, O.EPI_ADD, d13["R"][:, :H])
    assert_close(out.cpu().numpy(), want, "ffn output")
