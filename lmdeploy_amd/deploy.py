"""AWQ checkpoint -> deployable W4A16 weights, and the loader for such a workspace.

The W4A16 part of `deploy_awq` (`lmdeploy/serve/turbomind/deploy.py:554-783`) and of `export`
(`:110-240`), with the library's repack functions in place of `_turbomind`'s, plus the raw-file
loading of `loadWeights` (`src/turbomind/models/llama/LlamaDecoderLayerWeight.cc:207-218`).

What is kept from the reference: tensor names (`model.layers.{i}.self_attn.q_proj.qweight` ...),
the result of its deploy steps - q/k rotary re-ordering (`:371-383`, `:633-639`), q|k|v side by side
(`:251-260`), gate/up columns interleaved (`:641-658`), conversion (`:660-670`) - which the library
computes per fused tensor in one gather (`w4a16_deploy_qkv`, `w4a16_deploy_w13`), the
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
# the W4A16 part of deploy_awq for one decoder layer
# ---------------------------------------------------------------------------------------------
def convert_awq_layer(get: Callable[[str], torch.Tensor], i: int, group_size: int = 128) -> Dict[str, torch.Tensor]:
    """The int4 tensors of decoder layer `i` (deploy.py:676-757): `get(name)` returns the
    checkpoint tensor of that name on the GPU, contiguous.  Returns the eight deployable tensors
    keyed by the reference's parameter names (without the rank infix).  The library builds each fused
    tensor in one pass from the checkpoint's tensors (`w4a16_deploy_qkv`, `w4a16_deploy_w13`); wo and
    w2 need only the layout conversion."""
    def awq(prefix: str):
        return tuple(get(prefix + "." + part) for part in ("qweight", "qzeros", "scales"))

    def plain(prefix: str):
        qw, qz, s = awq(prefix)
        A, Q = torch.empty_like(qw), torch.empty_like(s, dtype=torch.int32)   # Q: half2 per (group, feature)
        tm.convert_s4_k_m8(A, Q, torch.empty(0, device=qw.device), qw, s, qz, qw.size(-1) * 8, qw.size(0), group_size)
        return A, Q

    att, mlp = "model.layers.%d.self_attn." % i, "model.layers.%d.mlp." % i
    made = {"attention.w_qkv": tm.deploy_qkv(awq(att + "q_proj"), awq(att + "k_proj"), awq(att + "v_proj"),
                                             SIZE_PER_HEAD, group_size),
            "attention.wo": plain(att + "o_proj"),
            "feed_forward.w13": tm.deploy_w13(awq(mlp + "gate_proj"), awq(mlp + "up_proj"), group_size),
            "feed_forward.w2": plain(mlp + "down_proj")}
    out = {}
    for key, (A, Q) in made.items():
        out["layers.%d.%s.qweight" % (i, key)] = A
        out["layers.%d.%s.scales_zeros" % (i, key)] = Q
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
    if group_size not in (128, 64, 32):
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
