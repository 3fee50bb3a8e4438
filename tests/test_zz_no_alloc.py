"""`w4a16_gemm_static`, the entry point that allocates nothing: its split-K kernels keep partial tiles
and arrival counters in a device array inside the library instead of a handle's workspace.  Its
output must equal `w4a16_gemm`'s (bit for bit when both run the same kernel, which sums the splits
in a fixed order), on two calls in a row, the second on a smaller problem, and both must agree with
the CPU oracle within the GEMM tolerance."""
import numpy as np
import pytest
import torch

from oracle import w4a16_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-2


def dev(a):
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def convert(tm, d, N, K):
    qw, qz, s = dev(d["qweight"]), dev(d["qzeros"]), dev(d["scales"])
    A, Q = torch.zeros_like(qw), torch.zeros_like(s, dtype=torch.int32)
    tm.convert_s4_k_m8(A, Q, torch.zeros_like(s), qw, s, qz, N, K, 128)
    return A, Q


def split_k_algos(gemm, A, Q, X, N, T, K):
    """ids of the MFMA kernels that split K across workgroups (they are the ones that use scratch)"""
    C = torch.empty((T, N), dtype=torch.float16, device="cuda")
    ms = gemm.Measure(C, A, X, Q, N, T, K, 128, gemm.kGemm)
    gemm.clear_tuning()
    return [(m.id, m.slices) for m in ms if m.feasible and m.kind == 1 and m.slices > 1]


def test_static_scratch_entry_point_equals_the_handle_entry_point():
    import lmdeploy_amd.turbomind as tm
    gemm = tm.GemmS4F16()
    used_scratch = 0
    # two problems in a row through the same static buffer, the second smaller in every dimension
    for seed, (K, N, T) in enumerate([(4224, 1024, 100), (2176, 512, 40)]):
        d = O.make_inputs(5150 + seed, T, K, N, residual=True)
        A, Q = convert(tm, d, N, K)
        X, R = dev(d["X"]), dev(d["R"])
        algos = split_k_algos(gemm, A, Q, X, N, T, K)
        assert len(algos) >= 4, algos
        for kind in (0, 1, 2):
            want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, kind, d["R"])
            res = R if kind == 2 else None
            shape = (T, N // 2 if kind == 1 else N)
            for algo in [-1] + [a for a, _ in algos]:
                print("static-scratch case", (K, N, T), "epilogue", kind, "algo", algo, flush=True)
                Ch = torch.full(shape, float("nan"), dtype=torch.float16, device="cuda")
                Cs = torch.full(shape, float("nan"), dtype=torch.float16, device="cuda")
                gemm.Run(Ch, A, X, Q, N, T, K, 128, kind, algo, residual=res)
                tm.gemm_static(Cs, A, X, Q, N, T, K, 128, kind, algo, residual=res)
                torch.cuda.synchronize()
                got = Cs.cpu().numpy()
                assert np.isfinite(got).all() and O.max_abs_rel(got, want) <= TOL, (K, N, T, kind, algo)
                assert O.max_abs_rel(got, Ch.cpu().numpy()) <= TOL
                if algo >= 0:   # same kernel, same number of splits, fixed summation order
                    assert torch.equal(Cs.view(torch.int16), Ch.view(torch.int16)), (K, N, T, kind, algo)
                    used_scratch += 1
    assert used_scratch >= 24


def test_static_scratch_decode_kernels_that_split_k_across_workgroups():
    """Narrow matrices at up to 16 tokens take the column-block decode kernel with K split across workgroups,
    whose partial tiles and counters also come from the static buffer: every such configuration, and the default
    choice, bit for bit against the handle's workspace; then replayed from a graph."""
    import lmdeploy_amd.turbomind as tm
    gemm = tm.GemmS4F16()
    K, N, T = 5632, 1024, 12
    d = O.make_inputs(5180, T, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    X, R = dev(d["X"]), dev(d["R"])
    ms = gemm.Measure(torch.empty((T, N), dtype=torch.float16, device="cuda"), A, X, Q, N, T, K, 128, gemm.kGemm)
    gemm.clear_tuning()
    # a column-block kernel that launches more workgroups than it has column blocks splits K across them
    split = [m.id for m in ms if m.feasible and m.kind == 0 and m.grid > N // m.tile_n]
    assert len(split) >= 3, split
    picked = gemm.pick(N, T, K)
    assert picked in split, (picked, split)      # what algo_id = -1 runs for this shape
    want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128, O.EPI_ADD, d["R"])
    outs = []
    for algo in [-1] + split:
        Ch = torch.full((T, N), float("nan"), dtype=torch.float16, device="cuda")
        Cs = torch.full((T, N), float("nan"), dtype=torch.float16, device="cuda")
        gemm.Run(Ch, A, X, Q, N, T, K, 128, gemm.kFusedAdd, algo, residual=R)
        tm.gemm_static(Cs, A, X, Q, N, T, K, 128, gemm.kFusedAdd, algo, residual=R)
        torch.cuda.synchronize()
        assert O.max_abs_rel(Cs.cpu().numpy(), want) <= TOL, algo
        assert torch.equal(Cs.view(torch.int16), Ch.view(torch.int16)), algo
        outs.append(Cs)
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    caps = [torch.empty((T, N), dtype=torch.float16, device="cuda") for _ in outs]
    with torch.cuda.graph(g, stream=stream):
        st = torch.cuda.current_stream().cuda_stream
        for algo, C in zip([-1] + split, caps):
            tm.gemm_static(C, A, X, Q, N, T, K, 128, gemm.kFusedAdd, algo, residual=R, stream=st)
    for rep in range(3):
        g.replay()
        torch.cuda.synchronize()
        for C, E in zip(caps, outs):
            assert torch.equal(C.view(torch.int16), E.view(torch.int16)), rep


def test_static_scratch_rejects_what_does_not_fit():
    import lmdeploy_amd.turbomind as tm
    gemm = tm.GemmS4F16()
    K, N, T = 2048, 4096, 128
    d = O.make_inputs(5160, T, K, N)
    A, Q = convert(tm, d, N, K)
    X = dev(d["X"])
    big = [a for a, s in split_k_algos(gemm, A, Q, X, N, T, K) if s == 8]   # 4096 x 128 x 8 splits x 4 B = 16 MiB
    assert big
    C = torch.empty((T, N), dtype=torch.float16, device="cuda")
    gemm.Run(C, A, X, Q, N, T, K, 128, 0, big[0])                            # the handle's 64 MiB holds it
    with pytest.raises(tm.W4A16Error, match="static buffer holds") as e:
        tm.gemm_static(C, A, X, Q, N, T, K, 128, 0, big[0])
    assert e.value.code == -6
    E = torch.empty_like(C)
    tm.gemm_static(E, A, X, Q, N, T, K, 128, 0, -1)                         # the default choice always fits
    torch.cuda.synchronize()
    want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128)
    assert O.max_abs_rel(E.cpu().numpy(), want) <= TOL
    with pytest.raises(tm.W4A16Error) as e:
        tm.gemm_static(C, A, X, Q, N, T, K, 256)
    assert e.value.code == -1


def test_static_scratch_entry_point_under_graph_capture():
    """The reason the entry point exists: it can be recorded into a HIP graph by a caller that has no handle and
    has allocated nothing.  A graph holding split-K launches (their counters are cleared by a fill kernel, not a
    memset node) is replayed several times with new activations written eagerly in between; every replay must equal
    the eager result bit for bit."""
    import lmdeploy_amd.turbomind as tm
    K, N, T = 2176, 512, 40
    d = O.make_inputs(5170, T, K, N, residual=True)
    A, Q = convert(tm, d, N, K)
    X, R = dev(d["X"]), dev(d["R"])
    algos = [a for a, _ in split_k_algos(tm.GemmS4F16(), A, Q, X, N, T, K)][:4] + [-1]
    outs = [torch.empty((T, N), dtype=torch.float16, device="cuda") for _ in algos]
    tm.gemm_static(outs[0], A, X, Q, N, T, K, 128, tm.GemmS4F16.kFusedAdd, -1, residual=R)   # first call on the device: outside capture
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        st = torch.cuda.current_stream().cuda_stream
        for a, C in zip(algos, outs):
            tm.gemm_static(C, A, X, Q, N, T, K, 128, tm.GemmS4F16.kFusedAdd, a, residual=R, stream=st)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    for rep in range(4):
        X.copy_(torch.randn((T, K), device="cuda", generator=gen).half())
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for a, C in zip(algos, outs):
            E = torch.empty_like(C)
            tm.gemm_static(E, A, X, Q, N, T, K, 128, tm.GemmS4F16.kFusedAdd, a, residual=R)
            torch.cuda.synchronize()
            assert torch.equal(E.view(torch.int16), C.view(torch.int16)), (rep, a)
    want = O.gemm_s4_f16(X.cpu().numpy(), d["qweight"], d["qzeros"], d["scales"], 128, O.EPI_ADD, d["R"])
    assert O.max_abs_rel(outs[-1].cpu().numpy(), want) <= TOL
