"""AWQ checkpoint -> deployable W4A16 weights, and the loader for such a workspace.

The W4A16 part of `deploy_awq` (`lmdeploy/serve/turbomind/deploy.py:554-783`) and of `export`
(`:110-240`), with the library's repack functions in place of `_turbomind`'s, plus the raw-file
loading of `loadWeights` (`src/turbomind/models/llama/LlamaDecoderLayerWeight.cc:207-218`).

What is kept from the reference: tensor names (`model.layers.{i}.self_attn.q_proj.qweight` ...),
the q/k rotary re-ordering (`transpose_qk_s4` on qweight and qzeros, `permute` on scales,
`:371-383`), `merge_qkv` (`:251-260`), `fuse_w1_w3_s4` (`:641-658`), `convert_s4` (`:660-670`), the
output file names `layers.{i}.attention.w_qkv.{rank}.qweight` / `.scales_zeros` (`:717-757`,
`:172-192`) with their exact byte sizes (`.qweight` K*N/2, `.scales_zeros` K/128*N*4,
`utils/memory_utils.cu:332-346`), and the `config.ini` keys `weight_type = int4`,
`group_size = 128` (`:223-224`).

What differs: the `.qweight` files hold the gfx950 tiled layout, announced by the extra key
`weight_layout = gfx950_tiled_v1` in `config.ini`.  A workspace without that key was written by
the reference; `load_workspace_linear` then converts its `.qweight` files with
`from_reference_layout` while loading (the `.scales_zeros` files are bit-identical in both).
Tensor parallel export is out of scope (one GPU): `tp` other than 1 is refused.
"""
from __future__ import annotations

import configparser
import os
from typing import Callable, Dict, Mapping, Optional, Tuple

import torch

from . import turbomind as tm

LAYOUT_KEY = "weight_layout"
LAYOUT_GFX950 = "gfx950_tiled_v1"
SIZE_PER_HEAD = 128


# ---------------------------------------------------------------------------------------------
# the W4A16 steps of deploy_awq, on GPU tensors
# ---------------------------------------------------------------------------------------------
def transpose_qk_s4(src: torch.Tensor, group_size: int = 128) -> torch.Tensor:
    """deploy.py:633-639 (the reference passes group_size where the binding expects
    size_per_head; both are 128)."""
    assert src.is_contiguous()
    dst = torch.empty_like(src)
    tm.transpose_qk_s4_k_m8(src, dst, src.size(-1) * 8, src.size(0), group_size)
    return dst


def permute(x: torch.Tensor) -> torch.Tensor:
    """deploy.py:371-383: interleaved rotary pairs -> half-split order, per head of 128."""
    if x.shape[-1] > 1:
        dim = x.shape[-1]
        n_heads = dim // SIZE_PER_HEAD
        return x.view(-1, n_heads, 2, dim // n_heads // 2).transpose(2, 3).reshape(-1, dim)
    dim = x.shape[0]
    n_heads = dim // SIZE_PER_HEAD
    return x.view(n_heads, 2, dim // n_heads // 2, 1).transpose(1, 2).reshape(dim, 1)


def merge_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, tp: int, dim: int) -> torch.Tensor:
    """deploy.py:251-260."""
    def reshape(x):
        return x.view(x.size(0), tp, -1) if dim == 2 else x.view(tp, -1)
    qkv = torch.cat((reshape(q), reshape(k), reshape(v)), dim=-1)
    return qkv.view(q.size(0), -1)


def fuse_w1_w3_s4(w1_qw, w1_qz, w1_s, w3_qw, w3_qz, w3_s):
    """deploy.py:641-658: gate and up columns interleaved (weights, zeros and scales alike)."""
    def fuse(a: torch.Tensor, b: torch.Tensor):
        ab = torch.cat((a, b)).contiguous()
        out = torch.empty_like(ab)
        tm.fuse_w1_w3_s4_k_m8(ab, out, a.size(-1) * 8, a.size(0))
        return out.view(a.size(0), -1)

    w13_s = torch.cat((w1_s, w3_s)).view(2, w1_s.size(0), -1)
    w13_s = w13_s.permute(1, 2, 0).contiguous().view(w1_s.size(0), -1)
    return fuse(w1_qw, w3_qw), fuse(w1_qz, w3_qz), w13_s


def convert_s4(qw: torch.Tensor, qz: torch.Tensor, s: torch.Tensor, group_size: int):
    """deploy.py:660-670."""
    assert qw.is_contiguous() and qz.is_contiguous() and s.is_contiguous()
    A = torch.empty_like(qw)
    Q = torch.empty_like(s, dtype=torch.int32)  # half2
    tm.convert_s4_k_m8(A, Q, torch.empty(0, device=qw.device), qw, s, qz, qw.size(-1) * 8, qw.size(0), group_size)
    return A, Q


def convert_awq_layer(get: Callable[[str], torch.Tensor], i: int, group_size: int = 128) -> Dict[str, torch.Tensor]:
    """The int4 tensors of decoder layer `i` (deploy.py:676-757): `get(name)` returns the
    checkpoint tensor of that name on the GPU.  Returns the eight deployable tensors keyed by the
    reference's parameter names (without the rank infix)."""
    p = "model.layers.%d." % i
    att, mlp = p + "self_attn.", p + "mlp."
    q_qw, k_qw, v_qw, o_qw = (get(att + n + "_proj.qweight") for n in "qkvo")
    q_qz, k_qz, v_qz, o_qz = (get(att + n + "_proj.qzeros") for n in "qkvo")
    q_s, k_s, v_s, o_s = (get(att + n + "_proj.scales") for n in "qkvo")
    q_qw, k_qw = transpose_qk_s4(q_qw, group_size), transpose_qk_s4(k_qw, group_size)
    q_qz, k_qz = transpose_qk_s4(q_qz, group_size), transpose_qk_s4(k_qz, group_size)
    q_s, k_s = permute(q_s), permute(k_s)
    out = {}
    qkv = (merge_qkv(q_qw, k_qw, v_qw, 1, 2), merge_qkv(q_qz, k_qz, v_qz, 1, 2), merge_qkv(q_s, k_s, v_s, 1, 2))
    out["layers.%d.attention.w_qkv.qweight" % i], out["layers.%d.attention.w_qkv.scales_zeros" % i] = \
        convert_s4(*(t.contiguous() for t in qkv), group_size)
    out["layers.%d.attention.wo.qweight" % i], out["layers.%d.attention.wo.scales_zeros" % i] = \
        convert_s4(o_qw, o_qz, o_s, group_size)
    w13 = fuse_w1_w3_s4(get(mlp + "gate_proj.qweight"), get(mlp + "gate_proj.qzeros"), get(mlp + "gate_proj.scales"),
                        get(mlp + "up_proj.qweight"), get(mlp + "up_proj.qzeros"), get(mlp + "up_proj.scales"))
    out["layers.%d.feed_forward.w13.qweight" % i], out["layers.%d.feed_forward.w13.scales_zeros" % i] = \
        convert_s4(*(t.contiguous() for t in w13), group_size)
    out["layers.%d.feed_forward.w2.qweight" % i], out["layers.%d.feed_forward.w2.scales_zeros" % i] = \
        convert_s4(get(mlp + "down_proj.qweight"), get(mlp + "down_proj.qzeros"), get(mlp + "down_proj.scales"),
                   group_size)
    return out


# ---------------------------------------------------------------------------------------------
# export: raw files + config.ini
# ---------------------------------------------------------------------------------------------
def _ranked(name: str, rank: int) -> str:
    prefix, ext = os.path.splitext(name)
    return "%s.%d%s" % (prefix, rank, ext)


def deploy_awq_weights(params: Mapping[str, torch.Tensor], num_layer: int, out_dir: str, tp: int = 1,
                       group_size: int = 128, extra_config: Optional[Mapping[str, object]] = None) -> str:
    """Writes `<out_dir>/weights/` for the int4 linear layers of an AWQ checkpoint given as a
    name -> tensor mapping (a state dict; tensors may live on the CPU).  Norm, embedding and
    output weights present in `params` are passed through as fp16 files under the reference's
    names (deploy.py:759-771).  Returns the weights directory."""
    if tp != 1:
        raise NotImplementedError("tensor-parallel export is not part of this one-GPU build: cut the tiled "
                                  "weights on 16-column / 128-row tile boundaries per rank")
    if group_size != 128:
        raise ValueError("unsupported group size")
    wdir = os.path.join(out_dir, "weights")
    os.makedirs(wdir, exist_ok=True)

    def get(name: str) -> torch.Tensor:
        return params[name].cuda().contiguous()

    def save_bin(t: torch.Tensor, name: str) -> None:
        if t.dtype in (torch.float, torch.bfloat16):
            t = t.half()
        t.contiguous().cpu().numpy().tofile(os.path.join(wdir, name))

    inter_size = 0
    for i in range(num_layer):
        for name, t in convert_awq_layer(get, i, group_size).items():
            key = name.split(".")[-2]
            if key == "w13":
                inter_size = max(inter_size, (t.shape[-1] * (8 if name.endswith("qweight") else 1)) // 2)
            save_bin(t, _ranked(name, 0))  # every int4 tensor is split (w_qkv, w13 along N; wo, w2 along K): rank 0 of 1
        for ours, hf in (("attention_norm.weight", "input_layernorm.weight"),
                         ("ffn_norm.weight", "post_attention_layernorm.weight")):
            full = "model.layers.%d.%s" % (i, hf)
            if full in params:
                save_bin(params[full], "layers.%d.%s" % (i, ours))
    for ours, hf in (("tok_embeddings.weight", "model.embed_tokens.weight"), ("norm.weight", "model.norm.weight"),
                     ("output.weight", "lm_head.weight")):
        if hf in params:
            save_bin(params[hf], ours)

    cfg = dict(num_layer=num_layer, inter_size=inter_size, weight_type="int4", group_size=group_size,
               tensor_para_size=tp, size_per_head=SIZE_PER_HEAD)
    cfg[LAYOUT_KEY] = LAYOUT_GFX950
    if extra_config:
        cfg.update(extra_config)
    config = configparser.ConfigParser()
    config["llama"] = {k: str(v) for k, v in cfg.items()}
    with open(os.path.join(wdir, "config.ini"), "w") as f:
        config.write(f)
    return wdir


# ---------------------------------------------------------------------------------------------
# loading a workspace (ours or the reference's)
# ---------------------------------------------------------------------------------------------
def workspace_layout(wdir: str) -> str:
    """`gfx950_tiled_v1` for a workspace written by `deploy_awq_weights`, `reference` otherwise."""
    config = configparser.ConfigParser()
    config.read(os.path.join(wdir, "config.ini"))
    if "llama" in config and config["llama"].get("weight_type", "int4") != "int4":
        raise ValueError("workspace is not int4")
    if "llama" in config and config["llama"].get(LAYOUT_KEY) == LAYOUT_GFX950:
        return LAYOUT_GFX950
    return "reference"


def _read_exact(path: str, nbytes: int) -> torch.Tensor:
    """Raw file -> int32 GPU tensor, with the reference's exact-size check
    (utils/memory_utils.cu:332-346)."""
    size = os.path.getsize(path)
    if size != nbytes:
        raise ValueError("%s: file size %d does not match the expected %d bytes" % (path, size, nbytes))
    import numpy as np
    return torch.from_numpy(np.fromfile(path, dtype=np.int32)).cuda()


def load_workspace_linear(wdir: str, prefix: str, k: int, m: int, group_size: int = 128, rank: int = 0,
                          layout: Optional[str] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """`loadWeights` for one int4 linear layer (LlamaDecoderLayerWeight.cc:207-218): reads
    `<prefix>.<rank>.qweight` (k*m/2 bytes) and `<prefix>.<rank>.scales_zeros` (k/g*m*4 bytes) and
    returns (A, Q) ready for `GemmS4F16.Run`.  A reference-written workspace is converted to the
    gfx950 layout on the way in."""
    if layout is None:
        layout = workspace_layout(wdir)
    A = _read_exact(os.path.join(wdir, "%s.%d.qweight" % (prefix, rank)), k * m // 2)
    Q = _read_exact(os.path.join(wdir, "%s.%d.scales_zeros" % (prefix, rank)), k // group_size * m * 4)
    if layout != LAYOUT_GFX950:
        A = tm.from_reference_layout(A, m, k)
    return A, Q.view(k // group_size, m)
