"""CPU oracle for the 10-layer experimental BiBo forward around the sparse-MoE block.  TEST INFRASTRUCTURE ONLY.

Restates, with explicit per-head loops and explicit masks, the forward pass of the reference's experimental model
(`exp/modeling_bibo.py` of IsNoobgrammer/BiBo) in the one topology its throughput probe runs
(`ablate/tools/tps_probe.sh:30-41`): Block Attention Residuals with one depth mix per layer, the carry write
`attn_read + c * attn_out` with a raw per-channel `c`, hybrid [global, window, window] attention with NoPE on the
global layers and full RoPE on the windowed ones, QK-norm, XSA with a learnable per-head strength, dense SwiGLU in
`mlp_only_layers` and the sparse-MoE block everywhere else.  Nothing in the product package may import it.

`params` is a dict keyed like the reference's `state_dict()`; `cfg` any object with the reference's config
attribute names.  Everything is evaluated in `dtype` (fp32 or fp64) whatever the parameters' storage dtype.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

from . import bibo_moe_oracle as M


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """BiBoRMSNorm.forward (src/modeling/norm.py:19-24) in x's dtype (no intermediate rounding: x is fp32/fp64)."""
    return weight.to(x.dtype) * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))


def rope_tables(positions: torch.Tensor, dim: int, base: float, dtype=torch.float64):
    """cos, sin [S, dim]: BiBoRotaryEmbedding.forward (src/modeling/embed.py:49-74): inverse frequencies
    base^(-2i/dim), angles position * frequency, the half-width table repeated twice."""
    inv = torch.tensor([base ** (-(2.0 * i) / dim) for i in range(dim // 2)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * inv[None, :]
    ang = torch.cat((ang, ang), dim=-1)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """(-x2, x1) over the two halves of the last dim (embed.py:10-14)."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def attention_residual(prefix: torch.Tensor, blocks, proj_w: torch.Tensor, norm_w: torch.Tensor, eps: float) -> torch.Tensor:
    """apply_attention_residual (exp/modeling_bibo.py:119-232), softmax scores, dense: every candidate (the completed
    blocks, then the current prefix sum) is RMS-normalised with `norm_w`, scored by the pseudo-query `proj_w`, and
    the candidates are averaged with the softmax of the scores.  prefix [T,H]; blocks: list of [T,H]."""
    values = torch.stack(list(blocks) + [prefix], dim=1)                       # [T, N+1, H]
    keys = rmsnorm(values, norm_w, eps)
    scores = (keys * proj_w.to(values.dtype).reshape(1, 1, -1)).sum(-1)        # [T, N+1]
    return (scores.softmax(-1).unsqueeze(-1) * values).sum(1)


def attention(x, p, pre, cfg, is_swa, cos, sin, dtype):
    """BiBoAttention.forward (src/modeling/attn/base.py:62-128) without cache or padding: projections, QK-norm over
    the head dim, RoPE on windowed layers only, causal (and banded) softmax attention per head with grouped keys,
    XSA (src/modeling/attn/xsa.py:11-54), output projection.  x [B,S,H] -> [B,S,H]."""
    B, S, _ = x.shape
    nh, nkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    g = nh // nkv
    W = lambda n: p[pre + n].to(dtype)
    q = (x @ W("q_proj.weight").t()).view(B, S, nh, d)
    k = (x @ W("k_proj.weight").t()).view(B, S, nkv, d)
    v = (x @ W("v_proj.weight").t()).view(B, S, nkv, d)
    if pre + "q_norm.weight" in p:                                              # QK-norm (base.py:62-64)
        q = rmsnorm(q, p[pre + "q_norm.weight"], cfg.rms_norm_eps)
        k = rmsnorm(k, p[pre + "k_norm.weight"], cfg.rms_norm_eps)
    if is_swa:                                                                  # full RoPE, windowed layers only (base.py:87-91)
        c, s = cos[None, :, None, :], sin[None, :, None, :]
        q = q * c + rotate_half(q) * s
        k = k * c + rotate_half(k) * s
    i = torch.arange(S)[:, None]
    j = torch.arange(S)[None, :]
    allow = j <= i                                                              # causal
    if is_swa:
        allow = allow & ((i - j) < cfg.sliding_window)                          # band (attn/utils.py:35-40)
    out = torch.zeros(B, S, nh, d, dtype=dtype)
    alpha = p.get(pre + "xsa_alpha")
    for h in range(nh):
        kv = h // g                                                             # head h reads kv head h // g (repeat_kv order)
        sc = torch.einsum("bqd,bkd->bqk", q[:, :, h], k[:, :, kv]) * (d ** -0.5)
        sc = sc.masked_fill(~allow[None], float("-inf"))
        y = torch.einsum("bqk,bkd->bqd", sc.softmax(-1), v[:, :, kv])
        if alpha is not None:                                                   # Y <- Y - tanh(alpha_h) (Y.Vn) Vn
            vn = v[:, :, kv] / v[:, :, kv].norm(dim=-1, keepdim=True).clamp_min(1e-12)
            y = y - math.tanh(float(alpha[h])) * (y * vn).sum(-1, keepdim=True) * vn
        out[:, :, h] = y
    return out.reshape(B, S, nh * d) @ W("o_proj.weight").t()


def dense_mlp(x, p, pre, dtype):
    """BiBoMLP.forward (src/modeling/ffn/mlp.py:34-35) with hidden_act = silu."""
    W = lambda n: p[pre + n].to(dtype)
    return (F.silu(x @ W("gate_proj.weight").t()) * (x @ W("up_proj.weight").t())) @ W("down_proj.weight").t()


def moe_block(xn, p, pre, cfg, dtype, routing=None):
    """BiBoMoELayer.forward in eval mode (src/modeling/ffn/moe.py:157-183) on normalised rows xn [T,H]; `routing` =
    (idx, w) replaces the router's decision (the parity protocol: routing is compared separately, bit for bit)."""
    if routing is None:
        logits = (xn.to(torch.float32) @ p[pre + "gate.gate_proj.weight"].float().t()).numpy()
        idx, w, _ = M.route_from_logits(logits, p[pre + "gate.bias"].float().numpy(), cfg.num_experts_per_tok)
    else:
        idx, w = routing
    return M.experts_forward(xn, idx, w, p[pre + "experts.gate_up_proj"], p[pre + "experts.down_proj"],
                             p[pre + "experts.radial_theta"].float(), dtype=dtype)


def forward(input_ids: torch.Tensor, p: dict, cfg, dtype=torch.float32, routing=None, return_hidden=False):
    """Logits [B,S,V] of the experimental BiBoForCausalLM (exp/modeling_bibo.py:765-943, 466-671) for the config
    described in the module docstring.  routing: optional {layer_idx: (idx [T,k], w [T,k])}."""
    B, S = input_ids.shape
    H = cfg.hidden_size
    T = B * S
    eps = cfg.rms_norm_eps
    bs = cfg.attn_res_block_size
    h = p["model.embed_tokens.weight"].to(dtype)[input_ids]                     # [B,S,H]
    cos, sin = rope_tables(torch.arange(S), cfg.head_dim, cfg.rope_theta, dtype)
    blocks = []                                                                 # completed block representatives, [T,H] each
    for l in range(cfg.num_hidden_layers):
        pre = f"model.layers.{l}."
        prefix = h.reshape(T, H)
        hs = prefix
        if blocks:                                                              # depth-mix read (:484-492)
            hs = attention_residual(prefix, blocks, p[pre + "self_attention_res_proj.weight"].reshape(-1),
                                    p[pre + "self_attention_res_norm.weight"], eps)
        attn_read = hs
        if l % bs == 0:                                                         # block boundary (:526-531)
            blocks = blocks + [prefix]
            prefix = None
        a = attention(rmsnorm(hs, p[pre + "input_layernorm.weight"], eps).view(B, S, H), p, pre + "self_attn.", cfg,
                      bool(cfg.hybrid_layer_pattern[l]), cos, sin, dtype).reshape(T, H)
        prefix = a if prefix is None else prefix + a
        c = p[pre + "attn_res_carry_theta"].to(dtype)                           # raw per-channel carry scale (:640-648)
        hs = attn_read + c * a
        xn = rmsnorm(hs, p[pre + "post_attention_layernorm.weight"], eps)       # _attn_res_mlp_forward (:429-431)
        if l in cfg.mlp_only_layers:
            m = dense_mlp(xn, p, pre + "mlp.", dtype)
        else:
            m = moe_block(xn, p, pre + "mlp.", cfg, dtype, None if routing is None else routing.get(l))
        h = (prefix + m).view(B, S, H)                                          # prefix_sum += mlp_out (:666)
    hf = attention_residual(h.reshape(T, H), blocks, p["model.output_attn_res_proj.weight"].reshape(-1),
                            p["model.output_attn_res_norm.weight"], eps)       # final depth mix (:916-920)
    hf = rmsnorm(hf, p["model.norm.weight"], eps)
    logits = (hf @ p["lm_head.weight"].to(dtype).t()).view(B, S, -1)
    return (logits, hf.view(B, S, H)) if return_hidden else logits
