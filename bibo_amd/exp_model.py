"""The 10-layer experimental BiBo forward around the sparse-MoE block, assembled on the host.

This is the model the reference's throughput probe runs (`ablate/tools/tps_probe.sh:30-41` on `exp/modeling_bibo.py`):
Block Attention Residuals with one depth mix per layer and the carry write `attn_read + c * attn_out`, hybrid
[global, window, window] attention (NoPE on global layers, full RoPE on windowed ones), QK-norm, XSA, dense SwiGLU in
`mlp_only_layers` and `BiBoMoELayer` everywhere else.  Only the MoE block runs on this package's HIP kernels, one
library call per layer: `out = prefix_sum + moe(rmsnorm(h))` (`bibo_moe_ffn_forward` with its own residual operand).
Everything around it is stock PyTorch tensor operations: attention through `scaled_dot_product_attention` (the
windowed layers as block-local attention over a two-block key window instead of the reference's eager S x S band
mask, `src/modeling/attn/swa.py:93-112`), the depth mix in fp32 as `apply_attention_residual` spells it out.

Parameter names follow the reference's `state_dict()` (`model.layers.N.self_attn.q_proj.weight`, ...,
`model.layers.N.attn_res_carry_theta`, `model.output_attn_res_proj.weight`, tied `lm_head.weight`), so a checkpoint
of the reference's experimental model in this topology loads.  Forward only, no KV cache, no padding mask.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .config import BiBoMoEConfig
from . import ops
from .moe import BiBoMoELayer

__all__ = ["BiBoExpConfig", "BiBoExpForCausalLM"]


class BiBoExpConfig(BiBoMoEConfig):
    """The fields of the reference's experimental BiBoConfig this forward reads, with the probe's values as defaults
    (`ablate/tools/tps_probe.sh:30-41`, `ablate/common/configs.py:63-73`); MoE fields as in BiBoMoEConfig."""

    def __init__(self, vocab_size=32000, hidden_size=768, num_hidden_layers=10, num_attention_heads=4,
                 num_key_value_heads=2, head_dim=None, intermediate_size=2304, moe_intermediate_size=384,
                 num_routed_experts=64, num_experts_per_tok=6, special_expert_pairs=0, mlp_only_layers=(0, 9),
                 hybrid_layer_pattern=None, sliding_window=128, rms_norm_eps=1e-6, rope_theta=10000.0, use_xsa=True,
                 xsa_alpha_init=0.0, swa_qk_norm=True, attn_res_block_size=3, attn_res_sites=1, attn_res_carry=True,
                 attn_res_carry_per_dim=True, attn_res_carry_scale="raw", tie_word_embeddings=True,
                 bf16_residual_stream=True, **kw):
        super().__init__(hidden_size=hidden_size, intermediate_size=intermediate_size,
                         moe_intermediate_size=moe_intermediate_size, num_experts_per_tok=num_experts_per_tok,
                         num_routed_experts=num_routed_experts, special_expert_pairs=special_expert_pairs, **kw)
        self.vocab_size = vocab_size
        self.num_hidden_layers = num_hidden_layers
        self.num_attention_heads = num_attention_heads
        self.num_key_value_heads = num_key_value_heads
        self.head_dim = head_dim if head_dim is not None else hidden_size // num_attention_heads
        self.mlp_only_layers = list(mlp_only_layers)
        # [global, window, window] blocks plus a global tail (configs.py:63-73)
        self.hybrid_layer_pattern = (list(hybrid_layer_pattern) if hybrid_layer_pattern is not None else
                                     [0 if i % 3 == 0 else 1 for i in range(num_hidden_layers - 1)] + [0])
        self.sliding_window = sliding_window
        self.rms_norm_eps = rms_norm_eps
        self.rope_theta = rope_theta
        self.use_xsa = use_xsa
        self.xsa_alpha_init = xsa_alpha_init
        self.swa_qk_norm = swa_qk_norm
        self.attn_res_block_size = attn_res_block_size
        self.attn_res_sites = attn_res_sites
        self.attn_res_carry = attn_res_carry
        self.attn_res_carry_per_dim = attn_res_carry_per_dim
        self.attn_res_carry_scale = attn_res_carry_scale
        self.tie_word_embeddings = tie_word_embeddings
        self.bf16_residual_stream = bf16_residual_stream
        if len(self.hybrid_layer_pattern) != num_hidden_layers:
            raise ValueError("hybrid_layer_pattern needs one entry per layer")
        if num_attention_heads % num_key_value_heads:
            raise ValueError("num_attention_heads must be a multiple of num_key_value_heads")
        if (attn_res_block_size is None or attn_res_sites != 1 or not attn_res_carry
                or attn_res_carry_scale not in ("raw", "unbounded", "none")):
            raise NotImplementedError("only the probe's residual topology is assembled here: attn_res_block_size set, "
                                      "attn_res_sites=1, attn_res_carry=True, attn_res_carry_scale raw or none")


class RMSNorm(nn.Module):
    """BiBoRMSNorm (src/modeling/norm.py:8-24): fp32 statistics, the normalised row rounded to the input dtype, then
    the weight."""

    def __init__(self, n, eps):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(n))
        self.variance_epsilon = eps

    def forward(self, x):
        if _hip_ok(x) and x.shape[-1] % 8 == 0:
            # the library's row norm (bibo_moe_rmsnorm_fwd): the same arithmetic in one launch
            w32 = _fp32_copy(self, "weight")
            return ops.rmsnorm_fwd(x.reshape(-1, x.shape[-1]).contiguous(), w32, float(self.variance_epsilon)).view(x.shape)
        xf = x.float()
        return self.weight * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)).to(x.dtype)


def _hip_ok(x) -> bool:
    """bf16 on the GPU with no autograd graph to build: the cases the library's caller-side kernels serve."""
    return x.is_cuda and x.dtype == torch.bfloat16 and not (torch.is_grad_enabled() and x.requires_grad)


def _fp32_copy(module, name):
    """fp32 copy of a small parameter, refreshed when the parameter changes (storage address or version counter)."""
    p = getattr(module, name)
    tag = (p.data_ptr(), p._version, p.device)
    hit = module.__dict__.get("_fp32_" + name)
    if hit is None or hit[0] != tag:
        hit = (tag, p.detach().float().contiguous())
        module.__dict__["_fp32_" + name] = hit
    return hit[1]


def _rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def attention_residual(prefix, blocks, proj_w, norm_w, eps):
    """apply_attention_residual (exp/modeling_bibo.py:119-232): fp32 scores `inv_rms * (v . (norm_w * proj_w))` per
    candidate, softmax over the candidates, fp32 weighted sum, result in prefix's dtype.  blocks: list of [T,H]."""
    sw = norm_w.float() * proj_w.reshape(-1).float()
    if (_hip_ok(prefix) and prefix.shape[-1] % 8 == 0 and prefix.shape[-1] <= 1024 and len(blocks) < 8
            and not (torch.is_grad_enabled() and (norm_w.requires_grad or proj_w.requires_grad))):
        return ops.attn_res_fwd([b.contiguous() for b in blocks] + [prefix.contiguous()], sw.contiguous(), float(eps))
    cands = [b.float() for b in blocks] + [prefix.float()]
    scores = torch.stack([(c @ sw) * torch.rsqrt(c.pow(2).mean(-1) + eps) for c in cands], dim=-1)
    prob = scores.softmax(-1)
    mixed = prob[:, 0:1] * cands[0]
    for i in range(1, len(cands)):
        mixed = mixed + prob[:, i:i + 1] * cands[i]
    return mixed.to(prefix.dtype)


def _band_attention(q, k, v, window, scale):
    """Causal attention restricted to the last `window` keys, as block-local attention: queries in blocks of
    `window`, each block against its own and the previous block of keys (every allowed key lies there), with the
    exact band mask inside the 2*window key window.  q [B,H,S,d], k, v [B,H,S,d] (heads already expanded)."""
    B, H, S, d = q.shape
    W = window
    nb = (S + W - 1) // W
    pad = nb * W - S
    if pad:
        q, k, v = (F.pad(t, (0, 0, 0, pad)) for t in (q, k, v))
    qb = q.view(B, H, nb, W, d)
    kb = k.view(B, H, nb, W, d)
    vb = v.view(B, H, nb, W, d)
    kw = torch.cat((F.pad(kb, (0, 0, 0, 0, 1, 0))[:, :, :-1], kb), dim=3)       # previous block, then own block
    vw = torch.cat((F.pad(vb, (0, 0, 0, 0, 1, 0))[:, :, :-1], vb), dim=3)
    blk = torch.arange(nb, device=q.device)[:, None, None]
    qi = blk * W + torch.arange(W, device=q.device)[None, :, None]
    kj = (blk - 1) * W + torch.arange(2 * W, device=q.device)[None, None, :]
    allow = (kj >= 0) & (kj <= qi) & ((qi - kj) < W)                            # attn/utils.py:35-40 in absolute positions
    out = F.scaled_dot_product_attention(qb, kw, vw, attn_mask=allow, scale=scale)
    return out.reshape(B, H, nb * W, d)[:, :, :S]


class BiBoExpAttention(nn.Module):
    """BiBoAttention (src/modeling/attn/base.py:19-128) without cache: GQA projections, QK-norm, RoPE on windowed
    layers only, causal / banded attention, XSA with tanh(alpha) per head, output projection."""

    def __init__(self, config, layer_idx):
        super().__init__()
        self.num_heads = config.num_attention_heads
        self.num_key_value_heads = config.num_key_value_heads
        self.head_dim = config.head_dim
        self.scaling = self.head_dim ** -0.5
        self.is_swa = bool(config.hybrid_layer_pattern[layer_idx])
        self.sliding_window = config.sliding_window if self.is_swa else None
        H, d = config.hidden_size, self.head_dim
        self.q_proj = nn.Linear(H, self.num_heads * d, bias=False)
        self.k_proj = nn.Linear(H, self.num_key_value_heads * d, bias=False)
        self.v_proj = nn.Linear(H, self.num_key_value_heads * d, bias=False)
        self.o_proj = nn.Linear(self.num_heads * d, H, bias=False)
        qk_norm = (not self.is_swa) or config.swa_qk_norm
        self.q_norm = RMSNorm(d, config.rms_norm_eps) if qk_norm else nn.Identity()
        self.k_norm = RMSNorm(d, config.rms_norm_eps) if qk_norm else nn.Identity()
        self.xsa_alpha = (nn.Parameter(torch.full((self.num_heads,), float(config.xsa_alpha_init)))
                          if config.use_xsa else None)

    def forward(self, x, cos, sin):
        B, S, _ = x.shape
        nh, nkv, d = self.num_heads, self.num_key_value_heads, self.head_dim
        g = nh // nkv
        q = self.q_norm(self.q_proj(x).view(B, S, nh, d)).transpose(1, 2)
        k = self.k_norm(self.k_proj(x).view(B, S, nkv, d)).transpose(1, 2)
        v = self.v_proj(x).view(B, S, nkv, d).transpose(1, 2)
        if self.is_swa:                                                         # base.py:87-91
            c, s = cos[None, None], sin[None, None]
            q = q * c + _rotate_half(q) * s
            k = k * c + _rotate_half(k) * s
        kx = k[:, :, None].expand(B, nkv, g, S, d).reshape(B, nh, S, d)         # repeat_kv order: head h reads kv h // g
        vx = v[:, :, None].expand(B, nkv, g, S, d).reshape(B, nh, S, d)
        if self.is_swa:
            y = _band_attention(q, kx, vx, self.sliding_window, self.scaling)
        else:
            y = F.scaled_dot_product_attention(q, kx, vx, is_causal=S > 1, scale=self.scaling)
        if self.xsa_alpha is not None:                                          # xsa.py:41-54
            vn = F.normalize(v, dim=-1)[:, :, None]                             # [B,nkv,1,S,d]
            yg = y.view(B, nkv, g, S, d)
            coeff = (yg * vn).sum(-1, keepdim=True) * torch.tanh(self.xsa_alpha.float()).to(y.dtype).view(1, nkv, g, 1, 1)
            y = (yg - coeff * vn).reshape(B, nh, S, d)
        return self.o_proj(y.transpose(1, 2).reshape(B, S, nh * d))


class BiBoExpMLP(nn.Module):
    """BiBoMLP (src/modeling/ffn/mlp.py:9-35), SwiGLU."""

    def __init__(self, config):
        super().__init__()
        self.gate_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.up_proj = nn.Linear(config.hidden_size, config.intermediate_size, bias=False)
        self.down_proj = nn.Linear(config.intermediate_size, config.hidden_size, bias=False)

    def forward(self, x):
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class BiBoExpDecoderLayer(nn.Module):
    """One layer of `_forward_attention_residuals` (exp/modeling_bibo.py:466-671) with sites = 1 and carry."""

    def __init__(self, config, layer_idx):
        super().__init__()
        self.layer_idx = layer_idx
        self.attn_res_block_size = config.attn_res_block_size
        self.self_attn = BiBoExpAttention(config, layer_idx)
        self.is_moe_layer = layer_idx not in config.mlp_only_layers
        self.mlp = BiBoMoELayer(config) if self.is_moe_layer else BiBoExpMLP(config)
        self.input_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.self_attention_res_norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.self_attention_res_proj = nn.Linear(config.hidden_size, 1, bias=False)
        shape = (config.hidden_size,) if config.attn_res_carry_per_dim else (1,)
        self.attn_res_carry_theta = (nn.Parameter(torch.ones(shape))
                                     if config.attn_res_carry_scale in ("raw", "unbounded") else None)
        self.last_routing = None

    def forward(self, hidden_states, blocks, cos, sin, collect_routing=False):
        B, S, H = hidden_states.shape
        prefix = hidden_states
        hs = hidden_states
        if blocks:                                                              # depth-mix read (:484-492)
            hs = attention_residual(prefix.reshape(-1, H), blocks, self.self_attention_res_proj.weight,
                                    self.self_attention_res_norm.weight,
                                    self.self_attention_res_norm.variance_epsilon).view(B, S, H)
        attn_read = hs
        if self.layer_idx % self.attn_res_block_size == 0:                      # block boundary (:526-531)
            blocks = blocks + [prefix.reshape(-1, H)]
            prefix = None
        a = self.self_attn(self.input_layernorm(hs), cos, sin)
        prefix = a if prefix is None else prefix + a
        if self.attn_res_carry_theta is not None:                               # carry write (:640-648)
            hs = attn_read + self.attn_res_carry_theta.float().to(a.dtype) * a
        else:
            hs = attn_read + a
        ln = self.post_attention_layernorm
        if self.is_moe_layer:
            # prefix_sum + mlp(post_attention_layernorm(hs)) (:429-431, :666) as one library call
            if collect_routing:
                out = self._moe_with_routing(hs, prefix)
            else:
                # the reference's block returns its output in the stream's dtype (moe.py:101) before `prefix_sum +
                # mlp_output` (exp/modeling_bibo.py:666): on a bf16 stream the block is rounded, then the sum
                out = self.mlp.ffn_forward(hs, ln.weight, ln.variance_epsilon, residual=prefix,
                                           bf16_moe_out=hs.dtype == torch.bfloat16)
        else:
            out = prefix + self.mlp(ln(hs))
        return out, blocks

    def _moe_with_routing(self, hs, prefix):
        """The same call through the tensor-level wrapper, keeping the routing decision for parity checks."""
        from . import ops
        from .moe import _compute_dtype
        m, ln = self.mlp, self.post_attention_layernorm
        B, S, H = hs.shape
        cd = _compute_dtype(hs)
        gu, dn, th = m.experts._weights(cd)
        out, idx, w, _ = ops.ffn_forward(hs.reshape(-1, H).to(cd).contiguous(), ln.weight.detach().float().contiguous(),
                                         float(ln.variance_epsilon), m.gate._cache.get("w", m.gate.gate_proj.weight, cd),
                                         m.gate._cache.get("b", m.gate.bias, torch.float32), gu, dn, th,
                                         m.num_experts_per_tok, norm=m.gate.norm_topk_prob, algo=m.experts.algo,
                                         want_routing=True, act=m.experts.act, round_block_out=cd == torch.bfloat16,
                                         residual=prefix.reshape(-1, H).to(cd).contiguous())
        self.last_routing = (idx, w)
        return out.view(B, S, H).to(hs.dtype)


class BiBoExpModel(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([BiBoExpDecoderLayer(config, i) for i in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.output_attn_res_norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.output_attn_res_proj = nn.Linear(config.hidden_size, 1, bias=False)
        inv = 1.0 / (config.rope_theta ** (torch.arange(0, config.head_dim, 2, dtype=torch.int64).float() / config.head_dim))
        self.register_buffer("inv_freq", inv, persistent=False)                 # embed.py:43-47

    def forward(self, input_ids, collect_routing=False):
        B, S = input_ids.shape
        H = self.config.hidden_size
        h = self.embed_tokens(input_ids)
        if self.config.bf16_residual_stream:                                    # exp/modeling_bibo.py:858-859
            h = h.to(torch.bfloat16)
        ang = torch.arange(S, device=h.device, dtype=torch.float32)[:, None] * self.inv_freq.float()[None, :]
        ang = torch.cat((ang, ang), dim=-1)
        cos, sin = ang.cos().to(h.dtype), ang.sin().to(h.dtype)                 # embed.py:63-74
        blocks = []
        for layer in self.layers:
            h, blocks = layer(h, blocks, cos, sin, collect_routing)
        h = attention_residual(h.reshape(-1, H), blocks, self.output_attn_res_proj.weight, self.output_attn_res_norm.weight,
                               self.output_attn_res_norm.variance_epsilon).view(B, S, H)     # :916-920
        return self.norm(h)


class BiBoExpForCausalLM(nn.Module):
    """Trunk + tied language-model head (exp/modeling_bibo.py:946-1046, forward only)."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.model = BiBoExpModel(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.model.embed_tokens.weight
        std = config.initializer_range
        for name, p in self.named_parameters():
            if name.endswith("proj.weight") or name.endswith("embed_tokens.weight") or name.endswith("lm_head.weight"):
                nn.init.normal_(p, mean=0.0, std=std)

    @torch.no_grad()
    def forward(self, input_ids, collect_routing=False):
        return self.lm_head(self.model(input_ids, collect_routing))

    def routing(self):
        """{layer index: (idx int32 [T,k], w fp32 [T,k])} of the last forward(collect_routing=True)."""
        return {i: l.last_routing for i, l in enumerate(self.model.layers) if l.is_moe_layer and l.last_routing is not None}
