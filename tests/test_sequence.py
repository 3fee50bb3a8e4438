"""`w4a16_gemm_sequence` / `w4a16_ffn`: lists of dependent GEMMs, as one launch per GEMM and as one
persistent launch with device-wide barriers, against the CPU oracle chained through the same fp16
intermediates, and the persistent launch bit for bit against the one-GEMM strip kernel whose code it shares."""
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


def close(got, want, what):
    err, rate = O.max_abs_rel(got, want), O.elementwise_pass_rate(got, want, TOL)
    assert np.isfinite(got).all() and err <= TOL and rate == 1.0, (what, err, rate)


@pytest.fixture(scope="module")
def tm():
    import lmdeploy_amd.turbomind as tm
    return tm


@pytest.fixture(scope="module")
def strip_id(tm):
    """algo id of the strip kernel with one strip per CU and 16 token rows (ids do not depend on the shape)"""
    g = tm.GemmS4F16()
    d = O.make_inputs(1, 4, 256, 64)
    A, Q = convert(tm, d, 64, 256)
    ms = g.Measure(torch.empty(4, 64, dtype=torch.float16, device="cuda"), A, dev(d["X"]), Q, 64, 4, 256, 128)
    return min(m.id for m in ms if m.kind == 2 and m.tile_t == 16)


@pytest.mark.parametrize("H,F,Ts", [(4096, 11008, (1, 8, 16)), (640, 1408, (3, 16)), (128, 256, (5,))])
def test_ffn_against_the_oracle(tm, H, F, Ts):
    """LlamaFfnLayer's int4 branch (LlamaFfnLayer.cc:67-116) on the Llama-2-7B shapes and on shapes with odd
    numbers of groups and fewer column tiles than CUs: `ffn` (two launches) and the persistent launch."""
    gemm = tm.GemmS4F16()
    Tmax = max(Ts)
    d13 = O.make_inputs(61, Tmax, H, 2 * F)
    d2 = O.make_inputs(62, Tmax, F, H, residual=True)
    A13, Q13 = convert(tm, d13, 2 * F, H)
    A2, Q2 = convert(tm, d2, H, F)
    W13 = O.dequant_from_awq(d13["qweight"], d13["qzeros"], d13["scales"], 128)
    W2 = O.dequant_from_awq(d2["qweight"], d2["qzeros"], d2["scales"], 128)
    for T in Ts:
        x = dev(d13["X"][:T])
        want_g = O.epilogue(O.gemm_acc(d13["X"][:T], W13), O.EPI_SILU)
        for persistent in (False, True):
            gating = torch.full((T, F), float("nan"), dtype=torch.float16, device="cuda")
            out = dev(d2["R"][:T])                                    # residual added in place
            print("ffn case", (H, F, T), "persistent" if persistent else "two launches", flush=True)
            if persistent:
                gemm.sequence([(gating, A13, x, Q13, 2 * F, H, gemm.kFusedSiluFfn, None, False),
                               (out, A2, gating, Q2, H, F, gemm.kFusedAdd, out, True)], T, persistent=True)
            else:
                gemm.ffn(out, gating, x, A13, Q13, A2, Q2, H, F, T, residual=out)
            gemm.sequence_status()
            g_host = gating.cpu().numpy()
            close(g_host, want_g, (H, F, T, persistent, "gating"))
            want = O.epilogue(O.gemm_acc(g_host, W2), O.EPI_ADD, d2["R"][:T])   # chained through the GPU's own intermediate
            close(out.cpu().numpy(), want, (H, F, T, persistent, "output"))


def test_persistent_layers_equal_the_strip_kernel_bit_for_bit(tm, strip_id):
    """Three decoder layers' worth of GEMMs (qkv, o, gate/up + SiLU, down + residual in place) chained through
    the same four buffers, so that every barrier guards a true dependency and every buffer is overwritten and
    re-read several times within one launch: a stale cache line anywhere changes the result."""
    gemm = tm.GemmS4F16()
    T, H, F, L = 7, 1024, 2816, 3
    gen = torch.Generator(device="cuda").manual_seed(99)

    def rand_w(K, N):
        A = torch.randint(-2 ** 31, 2 ** 31 - 1, (K * N // 8,), dtype=torch.int32, device="cuda", generator=gen)
        s = (torch.randn((K // 128, N), device="cuda", generator=gen).abs() * 0.004 + 1e-3).half()
        z = torch.randint(0, 16, (K // 128, N), device="cuda", generator=gen, dtype=torch.int32)
        return A, (s.view(torch.int16).to(torch.int32) << 16) | (0x5400 | (z << 4))

    shapes = [(H, 3 * H), (H, H), (H, 2 * F), (F, H)]
    layers = [[rand_w(K, N) for K, N in shapes] for _ in range(L)]
    x0 = (torch.randn(T, H, device="cuda", generator=gen) * 0.1).half()

    def run(persistent):
        b = dict(x=x0.clone(), qkv=torch.zeros(T, 3 * H, dtype=torch.float16, device="cuda"),
                 o=torch.zeros(T, H, dtype=torch.float16, device="cuda"), act=torch.zeros(T, F, dtype=torch.float16, device="cuda"))
        descs = []
        for li, ws in enumerate(layers):
            # (attention is not part of this path: o_proj reads the layer input again, but is ordered after qkv)
            descs += [(b["qkv"], ws[0][0], b["x"], ws[0][1], 3 * H, H, 0, None, li > 0),
                      (b["o"], ws[1][0], b["x"], ws[1][1], H, H, 0, None, True),
                      (b["act"], ws[2][0], b["o"], ws[2][1], 2 * F, H, 1, None, True),
                      (b["x"], ws[3][0], b["act"], ws[3][1], H, F, 2, b["x"], True)]
        if persistent:
            gemm.sequence(descs, T, persistent=True)
        else:
            for C, A, X, Q, m, k, typ, res, _ in descs:
                gemm.Run(C, A, X, Q, m, T, k, 128, typ, strip_id, residual=res)
        gemm.sequence_status()
        return b

    want = run(False)
    for rep in range(3):
        got = run(True)
        for k in want:
            assert torch.isfinite(got[k]).all() and got[k].abs().max() > 0
            assert torch.equal(got[k].view(torch.int16), want[k].view(torch.int16)), (rep, k)


def test_sequences_longer_than_one_launch_and_above_16_tokens(tm):
    gemm = tm.GemmS4F16()
    K = N = 256
    d = O.make_inputs(77, 40, K, N)
    A, Q = convert(tm, d, N, K)
    W = O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], 128)
    for T, count in ((4, 70), (40, 3)):           # 70 GEMMs: three persistent launches; 40 tokens: one launch per GEMM
        X = dev(d["X"][:T])
        outs = [torch.full((T, N), float("nan"), dtype=torch.float16, device="cuda") for _ in range(count)]
        gemm.sequence([(C, A, X, Q, N, K, 0, None, i % 2) for i, C in enumerate(outs)], T, persistent=True)
        gemm.sequence_status()
        want = O.epilogue(O.gemm_acc(d["X"][:T], W), 0)
        for C in outs:
            close(C.cpu().numpy(), want, (T, count))
    gemm.sequence([], 4)                           # empty list: nothing to do
    with pytest.raises(tm.W4A16Error) as e:
        gemm.sequence([(outs[0], A, X, Q, N + 8, K, 0, None, False)], 4)
    assert e.value.code == -2


def test_a_barrier_that_gives_up_is_reported_and_every_workgroup_still_finishes(tm):
    """The wait at the device-wide barrier is bounded.  With a time limit of zero every workgroup that is not
    the last to arrive gives up at once: the launch still runs to its end (nothing hangs), the handle reports
    the timeout once, and works again afterwards."""
    gemm = tm.GemmS4F16()
    T, K, N = 8, 2048, 8192
    d = O.make_inputs(78, T, K, N)
    A, Q = convert(tm, d, N, K)
    X = dev(d["X"])
    outs = [torch.empty((T, N), dtype=torch.float16, device="cuda") for _ in range(4)]
    descs = [(C, A, X, Q, N, K, 0, None, True) for C in outs]
    gemm.set_barrier_timeout(0.0)
    gemm.sequence(descs, T, persistent=True)
    with pytest.raises(tm.W4A16Error, match="gave up waiting") as e:
        gemm.sequence_status()
    assert e.value.code == -7
    gemm.sequence_status()                         # reported once
    gemm.set_barrier_timeout(2.0)
    gemm.sequence(descs, T, persistent=True)
    gemm.sequence_status()
    want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128)
    for C in outs:
        close(C.cpu().numpy(), want, "after the timeout")
    with pytest.raises(tm.W4A16Error):
        gemm.set_barrier_timeout(-1.0)


def test_a_list_that_cannot_run_as_a_whole_launches_nothing(tm):
    """Every GEMM of a list is planned (kernel, workspace, alignment) before the first one is launched: a second
    GEMM whose output pointer is misaligned for the MFMA kernels (8 bytes above 32 tokens) fails the call, and the
    first GEMM's output is still untouched."""
    T, K, N = 512, 1024, 2048
    d = O.make_inputs(9100, T, K, N)
    A, Q = convert(tm, d, N, K)
    X = dev(d["X"])
    C0 = torch.full((T, N), float("nan"), dtype=torch.float16, device="cuda")
    buf = torch.zeros(T * N + 8, dtype=torch.float16, device="cuda")
    C1 = buf[2:2 + T * N].view(T, N)          # 4-byte aligned only
    gemm = tm.GemmS4F16()
    with pytest.raises(tm.W4A16Error, match="misaligned") as e:
        gemm.sequence([(C0, A, X, Q, N, K, 0, None, False), (C1, A, X, Q, N, K, 0, None, False)], T)
    assert e.value.code == -4
    torch.cuda.synchronize()
    assert torch.isnan(C0).all()
    gemm.sequence([(C0, A, X, Q, N, K, 0, None, False)], T)
    torch.cuda.synchronize()
    want = O.gemm_s4_f16(d["X"], d["qweight"], d["qzeros"], d["scales"], 128)
    assert O.max_abs_rel(C0.cpu().numpy(), want) <= 1e-2
