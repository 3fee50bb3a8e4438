"""The AWQ checkpoint converter and the workspace loader (GPU: they run the library's repack kernels).

A tiny synthetic "checkpoint" with the reference's tensor names goes through `deploy_awq_weights`;
the files must have the reference's names and exact sizes, and the weights they hold, dequantised
by the library, must equal bit for bit what the oracle derives from the checkpoint tensors with the
defining formulas of the deploy steps (rotary re-ordering of q/k columns, q|k|v concatenation,
gate/up interleave).  A workspace in the reference's own layout, written by the oracle's
restatement of the reference's convert, must load into the same tensors."""
import configparser
import os

import numpy as np
import pytest
import torch

from oracle import w4a16_oracle as O

pytestmark = pytest.mark.gpu

H, F, L, G = 256, 384, 2, 128   # hidden (2 heads of 128), intermediate, layers, group size


def _awq(rng, K, N, G=G):
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // G, N), dtype=np.uint8)
    s = (np.abs(rng.standard_normal((K // G, N))) * 0.01 + 1e-3).astype(np.float16)
    return O.awq_pack(q), O.awq_pack(z), s


@pytest.fixture(scope="module")
def checkpoint():
    rng = np.random.default_rng(2024)
    sd = {}
    for i in range(L):
        for proj, (K, N) in {"self_attn.q_proj": (H, H), "self_attn.k_proj": (H, H), "self_attn.v_proj": (H, H),
                             "self_attn.o_proj": (H, H), "mlp.gate_proj": (H, F), "mlp.up_proj": (H, F),
                             "mlp.down_proj": (F, H)}.items():
            qw, qz, s = _awq(rng, K, N)
            base = "model.layers.%d.%s." % (i, proj)
            sd[base + "qweight"] = torch.from_numpy(qw.view(np.int32))
            sd[base + "qzeros"] = torch.from_numpy(qz.view(np.int32))
            sd[base + "scales"] = torch.from_numpy(s)
        sd["model.layers.%d.input_layernorm.weight" % i] = torch.ones(H, dtype=torch.float16)
    return sd


def _W(sd, i, proj):
    base = "model.layers.%d.%s." % (i, proj)
    return O.dequant_from_awq(sd[base + "qweight"].numpy().view(np.uint32), sd[base + "qzeros"].numpy().view(np.uint32),
                              sd[base + "scales"].numpy(), G)


def _rotary_permute_cols(W):
    # deploy.py:371-377 applied to the columns of the dequantised [K, dim] matrix
    K, dim = W.shape
    return W.reshape(K, dim // 128, 2, 64).transpose(0, 1, 3, 2).reshape(K, dim)


def test_deploy_writes_reference_named_files_with_exact_sizes(tmp_path, checkpoint):
    from lmdeploy_amd import deploy
    wdir = deploy.deploy_awq_weights(checkpoint, L, str(tmp_path))
    sizes = {"attention.w_qkv": (H, 3 * H), "attention.wo": (H, H), "feed_forward.w13": (H, 2 * F), "feed_forward.w2": (F, H)}
    for i in range(L):
        for key, (K, N) in sizes.items():
            assert os.path.getsize(os.path.join(wdir, "layers.%d.%s.0.qweight" % (i, key))) == K * N // 2
            assert os.path.getsize(os.path.join(wdir, "layers.%d.%s.0.scales_zeros" % (i, key))) == K // G * N * 4
        assert os.path.getsize(os.path.join(wdir, "layers.%d.attention_norm.weight" % i)) == H * 2
    cfg = configparser.ConfigParser()
    cfg.read(os.path.join(wdir, "config.ini"))
    assert cfg["llama"]["weight_type"] == "int4" and cfg["llama"]["group_size"] == "128"
    assert cfg["llama"]["inter_size"] == str(F) and cfg["llama"]["num_layer"] == str(L)
    assert deploy.workspace_layout(wdir) == deploy.LAYOUT_GFX950
    with pytest.raises(NotImplementedError):
        deploy.deploy_awq_weights(checkpoint, L, str(tmp_path), tp=2)


def test_deployed_weights_equal_the_defining_formulas(tmp_path, checkpoint):
    from lmdeploy_amd import deploy
    import lmdeploy_amd.turbomind as tm
    wdir = deploy.deploy_awq_weights(checkpoint, L, str(tmp_path))
    gemm = tm.GemmS4F16()
    rng = np.random.default_rng(7)
    for i in range(L):
        want = {
            "attention.w_qkv": np.concatenate([_rotary_permute_cols(_W(checkpoint, i, "self_attn.q_proj")),
                                               _rotary_permute_cols(_W(checkpoint, i, "self_attn.k_proj")),
                                               _W(checkpoint, i, "self_attn.v_proj")], axis=1),
            "attention.wo": _W(checkpoint, i, "self_attn.o_proj"),
            "feed_forward.w13": np.stack([_W(checkpoint, i, "mlp.gate_proj"), _W(checkpoint, i, "mlp.up_proj")],
                                         axis=2).reshape(H, 2 * F),
            "feed_forward.w2": _W(checkpoint, i, "mlp.down_proj"),
        }
        for key, Wref in want.items():
            K, N = Wref.shape
            A, Q = deploy.load_workspace_linear(wdir, "layers.%d.%s" % (i, key), K, N)
            got = tm.dequantize_repacked(A, Q, N, K).cpu().numpy()
            assert np.array_equal(got.view(np.uint16), Wref.view(np.uint16)), (i, key)
            # and the loaded pair runs: one GEMM against the oracle on the expected matrix
            T = 5
            X = rng.standard_normal((T, K)).astype(np.float16)
            kind = 1 if key == "feed_forward.w13" else 0
            C = torch.empty((T, N // 2 if kind else N), dtype=torch.float16, device="cuda")
            gemm.Run(C, A, torch.from_numpy(X).cuda(), Q, N, T, K, G, kind)
            torch.cuda.synchronize()
            assert O.max_abs_rel(C.cpu().numpy(), O.epilogue(O.gemm_acc(X, Wref), kind)) <= 1e-2


def test_reference_written_workspace_loads_into_the_same_tensors(tmp_path):
    from lmdeploy_amd import deploy
    import lmdeploy_amd.turbomind as tm
    K, N = 512, 384
    d = O.make_inputs(99, 1, K, N)
    A_ref, Q_ref = O.convert_s4_k_m8_reference(d["qweight"], d["scales"], d["qzeros"], N, K, G)
    wdir = tmp_path / "weights"
    wdir.mkdir()
    np.asarray(A_ref, dtype=np.uint32).tofile(wdir / "layers.0.attention.wo.0.qweight")
    np.asarray(Q_ref, dtype=np.uint32).tofile(wdir / "layers.0.attention.wo.0.scales_zeros")
    (wdir / "config.ini").write_text("[llama]\nweight_type = int4\ngroup_size = 128\n")   # as the reference writes it
    assert deploy.workspace_layout(str(wdir)) == "reference"
    A, Q = deploy.load_workspace_linear(str(wdir), "layers.0.attention.wo", K, N)
    A_ours, Q_ours = O.convert_s4_k_m8(d["qweight"], d["scales"], d["qzeros"], N, K, G)
    assert np.array_equal(A.cpu().numpy().view(np.uint32).reshape(-1), np.asarray(A_ours, dtype=np.uint32).reshape(-1))
    assert np.array_equal(Q.cpu().numpy().view(np.uint32).reshape(-1), np.asarray(Q_ours, dtype=np.uint32).reshape(-1))
    W = tm.dequantize_repacked(A, Q, N, K).cpu().numpy()
    assert np.array_equal(W.view(np.uint16), O.dequant_from_awq(d["qweight"], d["qzeros"], d["scales"], G).view(np.uint16))
    with pytest.raises(ValueError, match="file size"):
        deploy.load_workspace_linear(str(wdir), "layers.0.attention.wo", K, N + 16)


@pytest.mark.parametrize("G", [128, 64, 32])
def test_fused_tensor_entry_points_equal_the_reference_steps_bit_for_bit(G):
    """`w4a16_deploy_qkv` / `w4a16_deploy_w13` against the oracle's restatement of the reference's separate
    steps (format.cu:115-130 on qweight and qzeros, deploy.py:371-383 and :651-652 on the scales, then
    convert_s4_k_m8), with grouped-query widths (k and v narrower than q) and several heads."""
    import lmdeploy_amd.turbomind as tm
    rng = np.random.default_rng(77)
    K, D = 512, 128
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a.view(np.int32) if a.dtype == np.uint32 else a)).cuda()

    def rot_scales(s):       # deploy.py:371-377
        g, dim = s.shape
        return s.reshape(g, dim // D, 2, D // 2).transpose(0, 1, 3, 2).reshape(g, dim)

    for n_q, n_kv in ((1024, 256), (256, 256)):
        q, k, v = _awq(rng, K, n_q, G), _awq(rng, K, n_kv, G), _awq(rng, K, n_kv, G)
        A, Q = tm.deploy_qkv(tuple(map(dev, q)), tuple(map(dev, k)), tuple(map(dev, v)), D, G)
        qw = np.concatenate([O.transpose_qk_s4_k_m8_hf(q[0], n_q, K, D), O.transpose_qk_s4_k_m8_hf(k[0], n_kv, K, D), v[0]], axis=1)
        qz = np.concatenate([O.transpose_qk_s4_k_m8_hf(q[1], n_q, K // G, D), O.transpose_qk_s4_k_m8_hf(k[1], n_kv, K // G, D),
                             v[1]], axis=1)
        s = np.concatenate([rot_scales(q[2]), rot_scales(k[2]), v[2]], axis=1)
        N = n_q + 2 * n_kv
        A_ref, Q_ref = O.convert_s4_k_m8(np.ascontiguousarray(qw), np.ascontiguousarray(s), np.ascontiguousarray(qz), N, K, G)
        assert np.array_equal(A.cpu().numpy().view(np.uint32).reshape(-1), A_ref)
        assert np.array_equal(Q.cpu().numpy().view(np.uint32), Q_ref)
    F1 = 1408
    w1, w3 = _awq(rng, K, F1, G), _awq(rng, K, F1, G)
    A, Q = tm.deploy_w13(tuple(map(dev, w1)), tuple(map(dev, w3)), G)
    qw = O.fuse_w1_w3_s4_k_m8(np.concatenate([w1[0], w3[0]]), F1, K)
    qz = O.fuse_w1_w3_s4_k_m8(np.concatenate([w1[1], w3[1]]), F1, K // G)
    s = np.stack([w1[2], w3[2]], axis=-1).reshape(K // G, 2 * F1)      # deploy.py:651-652
    A_ref, Q_ref = O.convert_s4_k_m8(qw, np.ascontiguousarray(s), qz, 2 * F1, K, G)
    assert np.array_equal(A.cpu().numpy().view(np.uint32).reshape(-1), A_ref)
    assert np.array_equal(Q.cpu().numpy().view(np.uint32), Q_ref)
    with pytest.raises(tm.W4A16Error):
        tm.deploy_qkv(tuple(map(dev, q)), tuple(map(dev, k)), tuple(map(dev, v)), 96, G)     # 256 is not a multiple of 96
