"""The 10-layer experimental forward (config 5): the oracle pinned by closed forms the reference's own tests use
(tests/test_exp_attn_res.py:48-75, tests/test_attention.py:41-49, tests/test_rope.py:28-38 of the reference), the
host assembly in bibo_amd.exp_model against the oracle on the CPU where no MoE layer is involved, and, on the GPU,
the whole model with the HIP MoE block in layers 1-8 against the oracle."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from bibo_amd import exp_model as X
from oracle import bibo_exp_oracle as XO
from conftest import rel_err


def small_config(**kw):
    base = dict(vocab_size=97, hidden_size=64, num_hidden_layers=10, num_attention_heads=4, num_key_value_heads=2,
                intermediate_size=96, moe_intermediate_size=32, num_routed_experts=8, num_experts_per_tok=2,
                sliding_window=8, bf16_residual_stream=False)
    base.update(kw)
    return X.BiBoExpConfig(**base)


def randomize(model, seed=0):
    """Move every parameter off its neutral initial value, so that each one's path through the forward is live."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
                p.copy_(torch.rand(p.shape, generator=g) + 0.5)
            elif name.endswith("xsa_alpha"):
                p.copy_(torch.randn(p.shape, generator=g))
            elif name.endswith("attn_res_carry_theta"):
                p.copy_(torch.rand(p.shape, generator=g) * 1.5 + 0.25)
            elif name.endswith("res_proj.weight"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.5)
            elif name.endswith("radial_theta"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.5)
            elif name.endswith("gate.bias"):
                p.copy_(torch.rand(p.shape, generator=g) * 0.02 - 0.01)
            else:
                p.copy_(torch.randn(p.shape, generator=g) * (0.3 if p.ndim <= 2 else 0.2))
    return model


# ------------------------------------------------------------------ oracle pins
def test_attention_residual_closed_forms():
    torch.manual_seed(0)
    T, N, H = 6, 3, 16
    prefix = torch.randn(T, H, dtype=torch.float64)
    blocks = [torch.randn(T, H, dtype=torch.float64) for _ in range(N)]
    nw, pw = torch.rand(H, dtype=torch.float64) + 0.5, torch.randn(H, dtype=torch.float64)
    out = XO.attention_residual(prefix, blocks, pw, nw, 1e-6)
    # the folded form of the reference: inv_rms * (v . (norm_w * proj_w)) per candidate
    vals = torch.stack(blocks + [prefix], 1)
    sc = (vals @ (nw * pw)) * torch.rsqrt(vals.pow(2).mean(-1) + 1e-6)
    assert torch.allclose(out, (sc.softmax(-1)[..., None] * vals).sum(1), atol=1e-12)
    # a zero pseudo-query is an exact uniform average over depth (tests/test_exp_attn_res.py:64-74)
    z = XO.attention_residual(torch.tensor([[7.0, 8.0]]), [torch.tensor([[1.0, 2.0]]), torch.tensor([[4.0, 5.0]])],
                              torch.zeros(2), torch.ones(2), 1e-6)
    assert torch.equal(z, torch.tensor([[4.0, 5.0]]))
    # the score of a candidate does not depend on its scale (RMS-normalised keys): rescaling one candidate moves the
    # output only through the values, not the weights
    blocks2 = [blocks[0] * 7.0] + blocks[1:]
    vals2 = torch.stack(blocks2 + [prefix], 1)
    out2 = XO.attention_residual(prefix, blocks2, pw, nw, 1e-6)
    assert torch.allclose(out2, (sc.softmax(-1)[..., None] * vals2).sum(1), atol=1e-4)    # up to the 1e-6 under the root
    # a dominating score picks its candidate
    big = XO.attention_residual(prefix, blocks, pw * 1e4, nw, 1e-6)
    pick = sc.argmax(-1)
    assert torch.allclose(big, vals[torch.arange(T), pick], atol=1e-6)


def test_rope_tables_and_rotation():
    cos, sin = XO.rope_tables(torch.arange(16), 8, 10000.0)
    inv = 1.0 / (10000.0 ** (torch.arange(0, 8, 2, dtype=torch.int64).double() / 8))     # tests/test_rope.py:28-38
    fr = torch.arange(16).double()[:, None] * inv[None]
    emb = torch.cat((fr, fr), -1)
    assert torch.allclose(cos, emb.cos(), atol=1e-12) and torch.allclose(sin, emb.sin(), atol=1e-12)
    x = torch.randn(16, 8, dtype=torch.float64)
    r = x * cos + XO.rotate_half(x) * sin
    assert torch.allclose(r.norm(dim=-1), x.norm(dim=-1))                 # a rotation
    assert torch.allclose(r[0], x[0])                                     # position 0 is the identity
    # relative property: <R_m q, R_n k> depends on m - n only
    q, k = torch.randn(8, dtype=torch.float64), torch.randn(8, dtype=torch.float64)
    rot = lambda v, m: v * cos[m] + XO.rotate_half(v) * sin[m]
    assert math.isclose(float(rot(q, 9) @ rot(k, 4)), float(rot(q, 12) @ rot(k, 7)), rel_tol=1e-9)


def _attn_params(cfg, seed=1, alpha=None):
    g = torch.Generator().manual_seed(seed)
    H, d, nh, nkv = cfg.hidden_size, cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads
    p = {"a.q_proj.weight": torch.randn(nh * d, H, generator=g, dtype=torch.float64) * 0.3,
         "a.k_proj.weight": torch.randn(nkv * d, H, generator=g, dtype=torch.float64) * 0.3,
         "a.v_proj.weight": torch.randn(nkv * d, H, generator=g, dtype=torch.float64) * 0.3,
         "a.o_proj.weight": torch.eye(H, dtype=torch.float64),
         "a.q_norm.weight": torch.ones(d, dtype=torch.float64), "a.k_norm.weight": torch.ones(d, dtype=torch.float64)}
    if alpha is not None:
        p["a.xsa_alpha"] = alpha
    return p


def test_oracle_attention_band_causality_and_xsa():
    cfg = small_config(sliding_window=4)
    S = 12
    x = torch.randn(1, S, 64, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    cos, sin = XO.rope_tables(torch.arange(S), cfg.head_dim, cfg.rope_theta)
    p = _attn_params(cfg)
    y = XO.attention(x, p, "a.", cfg, True, cos, sin, torch.float64)
    # band: position q sees inputs q-3..q only (tests/test_attention.py:41-49)
    for qpos in (5, 9):
        x2 = x.clone(); x2[0, :qpos - 3] += 1.0; x2[0, qpos + 1:] -= 2.0
        y2 = XO.attention(x2, p, "a.", cfg, True, cos, sin, torch.float64)
        assert torch.allclose(y2[0, qpos], y[0, qpos], atol=1e-12)
        x3 = x.clone(); x3[0, qpos - 3] += 1.0
        assert not torch.allclose(XO.attention(x3, p, "a.", cfg, True, cos, sin, torch.float64)[0, qpos], y[0, qpos])
    # global layer: causal, and NoPE (a shift of all positions changes nothing: no position enters)
    yg = XO.attention(x, p, "a.", cfg, False, cos, sin, torch.float64)
    x4 = x.clone(); x4[0, 7:] += 1.0
    assert torch.allclose(XO.attention(x4, p, "a.", cfg, False, cos, sin, torch.float64)[0, :7], yg[0, :7], atol=1e-12)
    cos9, sin9 = XO.rope_tables(torch.arange(S) + 9, cfg.head_dim, cfg.rope_theta)
    assert torch.allclose(XO.attention(x, p, "a.", cfg, False, cos9, sin9, torch.float64), yg)
    assert torch.allclose(XO.attention(x, p, "a.", cfg, True, cos9, sin9, torch.float64), y, atol=1e-9)   # RoPE is relative
    # the first position attends to itself only: output = v_0 of its kv head (o_proj is the identity here)
    v = (x @ p["a.v_proj.weight"].t()).view(1, S, 2, 16)
    assert torch.allclose(yg[0, 0].view(4, 16), v[0, 0][[0, 0, 1, 1]], atol=1e-12)        # head h reads kv head h // 2
    # XSA: alpha = 0 is a no-op; a large alpha removes the whole component along the token's own value
    assert torch.allclose(XO.attention(x, _attn_params(cfg, alpha=torch.zeros(4)), "a.", cfg, False, cos, sin, torch.float64), yg)
    yx = XO.attention(x, _attn_params(cfg, alpha=torch.full((4,), 20.0)), "a.", cfg, False, cos, sin, torch.float64)
    dots = (yx.view(1, S, 4, 16) * v[:, :, [0, 0, 1, 1]]).sum(-1)
    assert dots.abs().max() < 1e-9


# ------------------------------------------------------------------ host assembly vs oracle, CPU (no MoE layer)
def test_host_building_blocks_match_the_oracle():
    cfg = small_config()
    torch.manual_seed(4)
    for layer_idx in (0, 1):                                             # a global and a windowed layer
        att = X.BiBoExpAttention(cfg, layer_idx).double()
        randomize(att, 5)
        S = 21                                                           # not a multiple of the window
        x = torch.randn(2, S, 64, dtype=torch.float64)
        cos, sin = XO.rope_tables(torch.arange(S), cfg.head_dim, cfg.rope_theta)
        p = {"a." + k: v for k, v in att.state_dict().items()}
        ref = XO.attention(x, p, "a.", cfg, bool(layer_idx), cos, sin, torch.float64)
        got = att(x, cos, sin)
        assert rel_err(got, ref) < 1e-6, layer_idx                       # (the norms compute in fp32 whatever the input)
    prefix = torch.randn(9, 64)
    blocks = [torch.randn(9, 64) for _ in range(3)]
    nw, pw = torch.rand(64) + 0.5, torch.randn(1, 64)
    assert torch.allclose(X.attention_residual(prefix, blocks, pw, nw, 1e-6),
                          XO.attention_residual(prefix, blocks, pw.reshape(-1), nw, 1e-6), atol=1e-5)


def test_dense_only_model_matches_the_oracle_on_cpu():
    """Every layer dense (mlp_only_layers = all): the whole assembly, block boundaries, carry write, depth mixes and
    the tied head, runs without the HIP library and must equal the oracle."""
    cfg = small_config(mlp_only_layers=list(range(10)))
    model = randomize(X.BiBoExpForCausalLM(cfg), 6).double().eval()
    ids = torch.randint(0, 97, (2, 19), generator=torch.Generator().manual_seed(7))
    logits = model(ids)
    sd = model.state_dict()
    assert sd["lm_head.weight"].data_ptr() == sd["model.embed_tokens.weight"].data_ptr()        # tied
    ref = XO.forward(ids, sd, cfg, dtype=torch.float64)
    assert logits.shape == (2, 19, 97) and rel_err(logits, ref) < 1e-4      # norms and depth mixes compute in fp32
    # the depth mix really is in the path: a different pseudo-query changes the logits
    with torch.no_grad():
        model.model.layers[4].self_attention_res_proj.weight.mul_(-1.0)
    assert rel_err(model(ids), ref) > 1e-4


def test_block_boundaries_follow_the_layer_index():
    """Blocks are committed at layers 0, 3, 6, 9 for block size 3 (exp/modeling_bibo.py:526-531): layer l reads
    ceil(l / 3) completed blocks and the final mix reads 4."""
    cfg = small_config(mlp_only_layers=list(range(10)))
    model = X.BiBoExpForCausalLM(cfg).eval()
    seen = []
    orig = X.attention_residual
    X.attention_residual = lambda prefix, blocks, *a: (seen.append(len(blocks)), orig(prefix, blocks, *a))[1]
    try:
        model(torch.randint(0, 97, (1, 5)))
    finally:
        X.attention_residual = orig
    assert seen == [1, 1, 1, 2, 2, 2, 3, 3, 3, 4]                        # layers 1..9, then the output mix


def test_state_dict_keys_follow_the_reference():
    sd = X.BiBoExpForCausalLM(small_config()).state_dict()
    for k in ("model.embed_tokens.weight", "lm_head.weight", "model.norm.weight", "model.output_attn_res_norm.weight",
              "model.output_attn_res_proj.weight", "model.layers.0.mlp.gate_proj.weight",
              "model.layers.1.mlp.gate.gate_proj.weight", "model.layers.1.mlp.gate.bias",
              "model.layers.1.mlp.experts.gate_up_proj", "model.layers.1.mlp.experts.radial_theta",
              "model.layers.1.mlp.accumulated_tpe", "model.layers.1.self_attn.q_norm.weight",
              "model.layers.1.self_attn.xsa_alpha", "model.layers.1.attn_res_carry_theta",
              "model.layers.1.self_attention_res_norm.weight", "model.layers.1.self_attention_res_proj.weight",
              "model.layers.9.post_attention_layernorm.weight"):
        assert k in sd, k
    assert sd["model.layers.1.attn_res_carry_theta"].shape == (64,) and not any("inv_freq" in k for k in sd)
    with pytest.raises(NotImplementedError):
        small_config(attn_res_sites=2)


# ------------------------------------------------------------------ GPU: HIP MoE block in layers 1-8
def _gpu_case(dtype, seed):
    cfg = small_config(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, intermediate_size=384,
                       moe_intermediate_size=128, num_routed_experts=64, num_experts_per_tok=6, vocab_size=503,
                       sliding_window=16, bf16_residual_stream=dtype == torch.bfloat16)
    model = randomize(X.BiBoExpForCausalLM(cfg), seed)
    with torch.no_grad():
        for n, p in model.named_parameters():                           # keep the stream at O(1) through ten layers
            if p.ndim >= 2 and "res_proj" not in n:
                p.mul_(0.25)
            elif "res_proj" in n and dtype == torch.bfloat16:
                # depth scores of O(1): with scores of +-10 the depth softmax is a hard selection that a bf16
                # rounding can flip, and the comparison would measure that chaos instead of the arithmetic
                p.mul_(0.1)
    model = model.to("cuda:0").to(dtype).eval()
    ids = torch.randint(0, 503, (2, 150), generator=torch.Generator().manual_seed(seed))
    return cfg, model, ids


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 5e-2)])
def test_model_with_hip_moe_layers_matches_the_oracle(dtype, tol):
    """Logits of the whole model against the fp32 oracle evaluated with the routing decisions the kernels made
    (routing itself is bit-exact against the oracle at the layer level; feeding it keeps one near-tie from turning into
    an expert-sized difference ten layers later).  fp32: the assembly is exact to rounding.  bf16: the stream,
    attention and the MoE kernels all round to bf16."""
    cfg, model, ids = _gpu_case(dtype, 11)
    logits = model(ids.to("cuda:0"), collect_routing=True)
    fast = model(ids.to("cuda:0"))                                       # the path without routing outputs
    torch.cuda.synchronize()
    assert torch.equal(logits, fast)
    routing = {l: (i.cpu().numpy(), w.cpu().numpy()) for l, (i, w) in model.routing().items()}
    assert sorted(routing) == list(range(1, 9))
    sd = {k: v.detach().cpu() for k, v in model.state_dict().items()}
    ref = XO.forward(ids, sd, cfg, dtype=torch.float32, routing=routing)
    err = rel_err(logits.cpu(), ref)
    print(f"reduced config 5, {dtype}: rel err {err:.3e} (bar {tol:g})")
    assert torch.isfinite(logits).all() and err <= tol


@pytest.mark.gpu
def test_hip_depth_mix_and_row_norm_match_the_stock_operations():
    """The two caller-side kernels of the 10-layer forward against the tensor-operation versions they replace:
    bibo_moe_exp_attn_res_fwd (depth mix, 1 to 5 candidates) and bibo_moe_rmsnorm_fwd on head-sized rows."""
    from bibo_amd import exp_model as X
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(8)
    T, H = 1000, 768
    rows = [(torch.randn(T, H, generator=g) * (1 + i)).to(torch.bfloat16).to(dev) for i in range(5)]
    proj = torch.randn(1, H, generator=g).to(dev) * 0.2
    nw = (1 + 0.1 * torch.randn(H, generator=g)).to(dev)
    for n in range(0, 5):
        blocks, prefix = rows[:n], rows[4]
        got = X.attention_residual(prefix, blocks, proj, nw, 1e-6)                       # HIP kernel
        with torch.enable_grad():                                                        # the tensor-operation path
            ref = X.attention_residual(prefix.clone().requires_grad_(True), blocks, proj, nw, 1e-6).detach()
        assert float((got.float() - ref.float()).abs().max()) <= 2e-2 * float(ref.float().abs().max())
    x = torch.randn(4, 50, 4, 192, generator=g).to(torch.bfloat16).to(dev)
    norm = X.RMSNorm(192, 1e-6).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        norm.weight.copy_((1 + 0.1 * torch.randn(192, generator=g)).to(torch.bfloat16))
    got = norm(x)
    with torch.enable_grad():
        ref = norm(x.clone().requires_grad_(True)).detach()
    assert got.shape == x.shape and float((got.float() - ref.float()).abs().max()) <= 1e-2 * float(ref.float().abs().max())


# ------------------------------------------------------------------ GPU: config 5 at its real dimensions
def _full_size_case(dtype, seed):
    """The probe's model as the reference configures it (ablate/tools/tps_probe.sh:30-41, ablate/common/configs.py:63-73):
    H = 768, 4 query / 2 KV heads of 192, window 128, dense layers 0 and 9 at 2304, E = 64, top-6, I = 384, vocabulary
    32000, tied head, N(0, 0.02) initialisation.  The parameters that start at a neutral value (norm weights, XSA alpha,
    carry theta, radial theta, balancing bias) are moved off it so that their paths are live."""
    cfg = X.BiBoExpConfig(bf16_residual_stream=dtype == torch.bfloat16)
    assert (cfg.hidden_size, cfg.head_dim, cfg.sliding_window, cfg.moe_intermediate_size, cfg.vocab_size) == (768, 192, 128, 384, 32000)
    torch.manual_seed(seed)
    model = X.BiBoExpForCausalLM(cfg)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
                p.copy_(torch.rand(p.shape, generator=g) + 0.5)
            elif name.endswith("xsa_alpha"):
                p.copy_(torch.randn(p.shape, generator=g))
            elif name.endswith("attn_res_carry_theta"):
                p.copy_(torch.rand(p.shape, generator=g) * 1.5 + 0.25)
            elif name.endswith("radial_theta"):
                p.copy_(torch.randn(p.shape, generator=g) * 0.5)
            elif name.endswith("gate.bias"):
                p.copy_(torch.rand(p.shape, generator=g) * 0.02 - 0.01)
    model = model.to("cuda:0").to(dtype).eval()
    ids = torch.randint(0, cfg.vocab_size, (1, 330), generator=torch.Generator().manual_seed(seed))   # 2.6 windows
    return cfg, model, ids


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 5e-2)])
def test_full_size_model_matches_the_oracle(dtype, tol):
    """Config 5 at its real dimensions, one sequence of 330 tokens (more than two windows, no multiple of the window):
    logits of the whole model against the fp32 oracle evaluated with the kernels' routing decisions."""
    cfg, model, ids = _full_size_case(dtype, 21)
    logits = model(ids.to("cuda:0"), collect_routing=True)
    fast = model(ids.to("cuda:0"))
    torch.cuda.synchronize()
    assert torch.equal(logits, fast)
    routing = {l: (i.cpu().numpy(), w.cpu().numpy()) for l, (i, w) in model.routing().items()}
    assert sorted(routing) == list(range(1, 9))
    sd = {k: v.detach().cpu() for k, v in model.state_dict().items()}
    ref = XO.forward(ids, sd, cfg, dtype=torch.float32, routing=routing)
    err = rel_err(logits.cpu(), ref)
    print(f"full-size config 5, {dtype}: rel err {err:.3e} (bar {tol:g})")
    assert logits.shape == (1, 330, 32000) and torch.isfinite(logits).all() and err <= tol
