"""The drop-in modules on the GPU: same behaviours the reference's tests/test_moe.py checks on
BiBoMoELayer / BiBoMoERouter, plus parity of the whole layer with the oracle."""
import numpy as np
import pytest
import torch

import bibo_amd
from oracle import bibo_moe_oracle as O
from bibo_amd import ops
from conftest import rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def make_config(**kw):
    base = dict(hidden_size=64, intermediate_size=96, moe_intermediate_size=96, num_routed_experts=8,
                special_expert_pairs=0, num_experts_per_tok=2)
    base.update(kw)
    return bibo_amd.BiBoMoEConfig(**base)


def _layer_from(p, dtype=torch.bfloat16, **cfg):
    E, two_i, H = p["w_gate_up"].shape
    c = bibo_amd.BiBoMoEConfig(hidden_size=H, moe_intermediate_size=two_i // 2, num_routed_experts=E,
                               special_expert_pairs=0, num_experts_per_tok=p["k"], **cfg)
    layer = bibo_amd.BiBoMoELayer(c)
    sd = {"gate.gate_proj.weight": p["w_router"].float(), "gate.bias": p["bias"],
          "experts.gate_up_proj": p["w_gate_up"].float(), "experts.down_proj": p["w_down"].float(),
          "experts.radial_theta": p["theta"], "accumulated_tpe": torch.zeros(E)}
    layer.load_state_dict(sd, strict=True)
    return layer.to(DEV).to(dtype).eval()


@pytest.mark.parametrize("name", ["c1", "c3"])
def test_layer_matches_oracle(name):
    cfg = O.CONFIGS[name]
    p = O.make_inputs(**cfg)
    layer = _layer_from(p)
    x3 = p["x"].view(cfg["B"], -1, cfg["H"]).to(DEV)
    with torch.no_grad():
        out = layer(x3)
        logits = layer.gate.router_logits(x3)
        idx, w = layer.gate(x3)
    assert out.shape == x3.shape and out.dtype == torch.bfloat16
    assert idx.dtype == torch.int64 and w.dtype == torch.float32 and idx.shape == (cfg["B"], cfg["T"] // cfg["B"], 6)
    ref, oi, ow = O.moe_forward(**p, logits=logits.cpu().numpy())
    assert np.array_equal(idx.view(-1, 6).cpu().numpy(), oi)
    assert np.array_equal(w.view(-1, 6).cpu().numpy(), ow)
    assert rel_err(out.view(-1, cfg["H"]).cpu(), ref) <= 2e-2
    # the same layer evaluated with the oracle's own logits: routing flips only at ulp-level near-ties
    ref2, oi2, _ = O.moe_forward(**p)
    assert (oi2 != oi).any(1).mean() < 0.01


def test_hooked_path_equals_fused_path_and_replays_hooks():
    p = O.make_inputs(**O.CONFIGS["c1"])
    layer = _layer_from(p)
    x3 = p["x"].view(1, -1, 512).to(DEV)
    with torch.no_grad():
        fused = layer(x3)
    seen = {}
    h1 = layer.experts.register_forward_pre_hook(lambda m, a: seen.__setitem__("experts", a))
    h2 = layer.gate.register_forward_hook(lambda m, a, o: seen.__setitem__("gate", (a, o)))
    layer.gate._probe_gap = True
    with torch.no_grad():
        hooked = layer(x3)
    h1.remove(); h2.remove(); layer.gate._probe_gap = False
    assert torch.equal(fused, hooked)
    flat, idx, w = seen["experts"]                              # (hidden, idx.long(), w): router_trace.py of the reference
    assert flat.shape == (512, 512) and idx.dtype == torch.int64 and idx.shape == (512, 6) and w.dtype == torch.float32
    (gin,), (gidx, gw) = seen["gate"]
    assert gin.shape == (1, 512, 512) and gidx.shape == (1, 512, 6) and gw.shape == (1, 512, 6)
    gap = layer.gate.boundary_gap
    assert gap is not None and gap.ndim == 0 and 0 < float(gap) < 1


def test_router_module_contract():
    """tests/test_moe.py:138-202 of the reference: fp32 positive weights with unit mass, raw scores without
    normalisation, bias only moves selection."""
    for norm in ("sum", "softmax"):
        r = bibo_amd.BiBoMoERouter(make_config(norm_topk_prob=norm)).to(DEV)
        with torch.no_grad():
            idx, w = r(torch.randn(2, 5, 64, device=DEV) * 3)
        assert w.dtype == torch.float32 and (w > 0).all() and idx.min() >= 0 and idx.max() < 8
        assert torch.allclose(w.sum(-1), torch.ones(2, 5, device=DEV), atol=1e-6)
    r = bibo_amd.BiBoMoERouter(make_config(norm_topk_prob=False)).to(DEV)
    x = torch.randn(2, 5, 64, device=DEV) * 3
    with torch.no_grad():
        _, w = r(x)
        scores = torch.sigmoid(r.router_logits(x))
    assert not torch.allclose(w.sum(-1), torch.ones(2, 5, device=DEV), atol=1e-3)
    assert torch.allclose(w.flatten().sort().values, scores.topk(2, -1).values.flatten().sort().values, atol=1e-6)
    with torch.no_grad():
        r.bias[0] = 5.0
        idx, w = r(x)
    assert (idx == 0).any(-1).all() and w.max() <= 1.0 + 1e-6


def test_dtype_regimes():
    """fp32 module: fp32 kernels, tight tolerance; .to(bfloat16) module keeps routing fp32 and returns bf16
    (tests/test_moe.py:252-259); bf16 autocast over fp32 masters runs the bf16 kernels and returns fp32."""
    p = O.make_inputs(T=40, H=64, E=8, k=2, I=96, bias="uniform", theta="normal", seed=4, dtype=torch.float32)
    layer = _layer_from(p, dtype=torch.float32)
    x3 = p["x"].view(2, 20, 64).to(DEV)
    with torch.no_grad():
        out = layer(x3)
        logits = layer.gate.router_logits(x3)
    idx, w, _ = O.route_from_logits(logits.cpu().numpy(), p["bias"].numpy(), 2)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"], dtype=torch.float64)
    assert out.dtype == torch.float32 and rel_err(out.view(-1, 64).cpu(), ref) < 1e-5
    half = _layer_from(p, dtype=torch.bfloat16)
    with torch.no_grad():
        _, wh = half.gate(x3.bfloat16())
        oh = half(x3.bfloat16())
    assert wh.dtype == torch.float32 and oh.dtype == torch.bfloat16
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        oa = layer(x3)
        la = layer.gate.router_logits(x3)
    pb = {k_: (v.bfloat16() if k_ in ("x", "w_router", "w_gate_up", "w_down") else v) for k_, v in p.items()}
    ref_a, _, _ = O.moe_forward(**pb, logits=la.cpu().numpy())
    assert oa.dtype == torch.float32 and rel_err(oa.view(-1, 64).cpu(), ref_a) <= 2e-2


def test_training_mode_balances_once_per_forward_and_eval_never():
    p = O.make_inputs(T=64, H=64, E=8, k=2, I=96, seed=6)
    layer = _layer_from(p, bias_update_factor=0.4, bias_update_threshold=64 * 2)
    x3 = p["x"].view(2, 32, 64).to(DEV)
    with torch.no_grad():
        layer(x3)
    assert layer._fwd_step == 0 and float(layer.accumulated_tpe.sum()) == 0         # eval: never
    layer.train()
    with torch.no_grad():
        layer(x3)
    assert layer._fwd_step == 1 and float(layer.accumulated_tpe.sum()) == 64 * 2    # T*k slots counted once
    idx, _, _ = O.route_from_logits(layer.gate.router_logits(x3).cpu().numpy(), p["bias"].numpy(), 2)
    assert np.array_equal(layer.accumulated_tpe.float().cpu().numpy(), np.bincount(idx.reshape(-1), minlength=8))
    bias_before = layer.gate.bias.clone()
    with torch.no_grad():
        layer(x3)                                                                    # second forward fires
    assert layer._fwd_step == 2 and float(layer.accumulated_tpe.sum()) == 0
    assert not torch.equal(bias_before, layer.gate.bias) and abs(float(layer.gate.bias.float().mean())) < 1e-3
    # hooked path takes the same counts
    layer2 = _layer_from(p, bias_update_factor=0.4, bias_update_threshold=64 * 2).train()
    h = layer2.experts.register_forward_pre_hook(lambda m, a: None)
    with torch.no_grad():
        layer2(x3)
    h.remove()
    assert np.array_equal(layer2.accumulated_tpe.float().cpu().numpy(), np.bincount(idx.reshape(-1), minlength=8))


def test_experts_module_seam_takes_int64_indices():
    p = O.make_inputs(T=50, H=64, E=8, k=2, I=96, theta="normal", seed=8)
    layer = _layer_from(p)
    idx, w, _ = O.route_from_logits(O.router_logits(p["x"], p["w_router"]), p["bias"].numpy(), 2)
    with torch.no_grad():
        out = layer.experts(p["x"].to(DEV), torch.from_numpy(idx).long().to(DEV), torch.from_numpy(w).to(DEV))
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    assert out.dtype == torch.bfloat16 and rel_err(out.cpu(), ref) <= 2e-2


@pytest.mark.parametrize("T", [1, 17, 64, 65, 200])
def test_fused_forward_routing_equals_standalone_router(T):
    """bibo_moe_forward takes a one-launch router+permutation path for T <= 64; its routing, logits and
    counts must equal the standalone router's bit for bit, and the output must match the oracle."""
    from bibo_amd import ops
    p = O.make_inputs(T=T, H=1024, E=64, k=6, I=512, bias="uniform", theta="normal", seed=100 + T)
    d = {k_: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k_, v in p.items()}
    out, idx, w, counts, logits = ops.moe_forward(d["x"], d["w_router"], d["bias"], d["w_gate_up"], d["w_down"],
                                                  d["theta"], 6, want_routing=True, want_counts=True, want_logits=True)
    idx2, w2, logits2, _ = ops.router_fwd(d["x"], d["w_router"], d["bias"], 6, want_logits=True)
    torch.cuda.synchronize()
    assert torch.equal(logits, logits2) and torch.equal(idx, idx2) and torch.equal(w, w2)
    oi, ow, _ = O.route_from_logits(logits.cpu().numpy(), p["bias"].numpy(), 6)
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(w.cpu().numpy(), ow)
    assert np.array_equal(counts.cpu().numpy(), O.permute(oi, 64)[0])
    ref = O.experts_forward(p["x"], oi, ow, p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(out.cpu(), ref) <= 2e-2


# ------------------------------------------------------------------ the caller's seam: RMSNorm in front, residual behind
@pytest.mark.parametrize("T,H,I,algo", [(64, 1024, 512, "auto"), (700, 768, 384, "auto"), (300, 256, 128, "generic"),
                                        (300, 200, 72, "auto")])
def test_ffn_forward_matches_oracle(T, H, I, algo):
    """bibo_moe_ffn_forward = h + moe(rmsnorm(h)) (layers.py:57-67): routing bit-exact on the kernel's own
    normalised input, output within the bf16 tolerance of the fp32 oracle."""
    p = O.make_inputs(T=T, H=H, E=64, k=6, I=I, bias="uniform", theta="normal", seed=T + H)
    g = torch.Generator().manual_seed(T)
    nw = torch.rand(H, generator=g) + 0.5
    h = (p["x"].float() * 3).bfloat16()
    dev = torch.device("cuda:0")
    out, idx, w, counts = ops.ffn_forward(h.to(dev), nw.to(dev), 1e-6, p["w_router"].to(dev), p["bias"].to(dev),
                                          p["w_gate_up"].to(dev), p["w_down"].to(dev), p["theta"].to(dev), 6, algo=algo,
                                          want_routing=True, want_counts=True)
    # the norm kernel against the oracle: equal up to one bf16 step where the fp32 statistics round differently
    xn_k = ops.rmsnorm_fwd(h.to(dev), nw.to(dev), 1e-6)
    torch.cuda.synchronize()
    xn = O.rmsnorm(h, nw, 1e-6)
    d = (xn_k.cpu().float() - xn.float()).abs()
    assert (d <= xn.float().abs() * 2.0 ** -7 + 1e-30).all() and (d > 0).float().mean() < 0.01
    # the parity protocol on the kernel's own normalised rows: routing from the router kernel's logits on them
    _, _, logits, _ = ops.router_fwd(xn_k, p["w_router"].to(dev), p["bias"].to(dev), 6, want_logits=True)
    y, oi, ow = O.moe_forward(xn_k.cpu(), p["w_router"], p["bias"], p["w_gate_up"], p["w_down"], p["theta"], 6,
                              logits=logits.cpu().numpy())
    ref = h.float() + y.float()
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(w.cpu().numpy(), ow)
    assert np.array_equal(counts.cpu().numpy(), np.bincount(oi.reshape(-1), minlength=64))
    assert rel_err(out.cpu(), ref) <= 2e-2


def test_ffn_forward_fp32_isolates_the_block_contribution():
    """In fp32 the sum is not rounded to bf16, so out - h must be the block's output itself (in the bf16 case
    above it is mostly below the resolution of the residual)."""
    p = O.make_inputs(T=90, H=96, E=16, k=3, I=40, bias="uniform", theta="normal", seed=8, dtype=torch.float32)
    nw = torch.rand(96, generator=torch.Generator().manual_seed(1)) + 0.5
    h = p["x"] * 2
    dev = torch.device("cuda:0")
    out, idx, w, _ = ops.ffn_forward(h.to(dev), nw.to(dev), 1e-6, p["w_router"].to(dev), p["bias"].to(dev),
                                     p["w_gate_up"].to(dev), p["w_down"].to(dev), p["theta"].to(dev), 3, want_routing=True)
    xn_k = ops.rmsnorm_fwd(h.to(dev), nw.to(dev), 1e-6)
    torch.cuda.synchronize()
    assert torch.allclose(xn_k.cpu(), O.rmsnorm(h, nw, 1e-6), rtol=1e-5, atol=1e-6)
    y = O.experts_forward(xn_k.cpu(), idx.cpu().numpy(), w.cpu().numpy(), p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(out.cpu() - h, y) <= 1e-4


def test_layer_ffn_forward_equals_norm_block_residual_composition():
    torch.manual_seed(3)
    cfg = make_config(hidden_size=256, moe_intermediate_size=128, num_routed_experts=64, num_experts_per_tok=6)
    layer = bibo_amd.BiBoMoELayer(cfg).to("cuda:0").bfloat16().eval()
    with torch.no_grad():
        layer.experts.radial_theta.normal_(0, 0.5)
    h = (torch.randn(2, 100, 256, device="cuda:0") * 2).bfloat16()
    nw = (torch.rand(256, device="cuda:0") + 0.5).bfloat16()
    with torch.no_grad():
        fused = layer.ffn_forward(h, nw, 1e-6)
        hf = h.float()
        xn = (hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
        composed = h + layer(nw * xn)                              # layers.py:59-64 with stock ops around the block
    assert fused.dtype == torch.bfloat16 and fused.shape == h.shape
    assert rel_err(fused.cpu(), composed.cpu().float()) <= 1e-2     # one rounding less on the fused side
    # an fp32 stream under bf16 autocast keeps its fp32 residual
    layer32 = bibo_amd.BiBoMoELayer(cfg).to("cuda:0").eval()
    h32 = torch.randn(1, 50, 256, device="cuda:0")
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        o32 = layer32.ffn_forward(h32, torch.ones(256, device="cuda:0"), 1e-6)
    assert o32.dtype == torch.float32
    assert (o32 - h32).abs().max() < 1.0 and torch.isfinite(o32).all()


def test_ffn_forward_bf16_moe_out_rounds_the_block_before_the_sum():
    """bf16_moe_out (src/modeling/layers.py:37,62-63): the block's output is rounded to bf16 before it enters the
    residual sum.  With a residual of zero the two roundings collapse, so out == round(block); with a real residual
    the result equals bf16(residual + bf16(block)) exactly, which the fp32-sum path does not."""
    torch.manual_seed(5)
    cfg = make_config(hidden_size=256, moe_intermediate_size=128, num_routed_experts=64, num_experts_per_tok=6)
    layer = bibo_amd.BiBoMoELayer(cfg).to("cuda:0").bfloat16().eval()
    h = (torch.randn(2, 150, 256, device="cuda:0") * 2).bfloat16()
    nw = (torch.rand(256, device="cuda:0") + 0.5).bfloat16()
    with torch.no_grad():
        hf = h.float()
        xn = (hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
        blk = layer(nw * xn)                                   # bf16 block output, rounded once
        rounded = layer.ffn_forward(h, nw, 1e-6, bf16_moe_out=True)
        plain = layer.ffn_forward(h, nw, 1e-6)
    assert torch.equal(rounded, h + blk)                        # bf16 + bf16: one more rounding of the sum
    assert not torch.equal(plain, rounded)                      # the fp32 sum keeps bits the rounded block lost
    assert rel_err(plain.cpu(), rounded.cpu().float()) <= 1e-2
    # an fp32 stream: stock tensor operations around the block, same contract
    layer32 = bibo_amd.BiBoMoELayer(cfg).to("cuda:0").eval()
    h32 = torch.randn(2, 50, 256, device="cuda:0")
    with torch.no_grad():
        a = layer32.ffn_forward(h32, nw.float(), 1e-6, bf16_moe_out=True)
        hf = h32
        xn = hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + 1e-6)
        b = h32 + layer32(nw.float() * xn).bfloat16().float()
    assert a.dtype == torch.float32 and torch.equal(a, b)


def test_layer_with_tanh_exponent_and_conv_shared_expert():
    """Module-level switches: radial_p='tanh' reaches the kernels; the conv shared expert is added to the routed
    output (moe.py:174-176 with experts.py:11-34)."""
    p = O.make_inputs(T=96, H=256, E=64, k=6, I=128, bias="uniform", theta="normal", seed=31)
    p["theta"] = p["theta"] * 3 - 0.5
    c = bibo_amd.BiBoMoEConfig(hidden_size=256, moe_intermediate_size=128, num_routed_experts=64, special_expert_pairs=0,
                               num_experts_per_tok=6, use_shared_expert=True, shared_expert_type="conv", kernel_size=3)
    layer = bibo_amd.BiBoMoELayer(c)
    missing = layer.load_state_dict({"gate.gate_proj.weight": p["w_router"].float(), "gate.bias": p["bias"],
                                     "experts.gate_up_proj": p["w_gate_up"].float(),
                                     "experts.down_proj": p["w_down"].float(), "experts.radial_theta": p["theta"],
                                     "accumulated_tpe": torch.zeros(64)}, strict=False)
    assert sorted(missing.missing_keys) == ["shared_experts_list.0.down_proj.weight",
                                            "shared_experts_list.0.gate_conv.weight", "shared_experts_list.0.up_proj.weight"]
    with torch.no_grad():
        for q in layer.shared_experts_list.parameters():       # keep the shared term at the routed term's magnitude
            q.mul_(0.7)
    layer = layer.to(DEV).bfloat16().eval()
    layer.experts.radial_p = "tanh"
    x3 = p["x"].view(2, 48, 256).to(DEV)
    with torch.no_grad():
        out = layer(x3)
        logits = layer.gate.router_logits(x3)
        shared = layer.shared_experts_list[0](x3)
    # .bfloat16() rounded the selection bias and theta too (a quirk the reference shares, tests/test_moe.py:252-259):
    # the oracle gets the module's values
    idx, w, _ = O.route_from_logits(logits.cpu().numpy(), layer.gate.bias.float().cpu().numpy(), 6)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], layer.experts.radial_theta.float().cpu(), act="tanh")
    sh = shared.float().view(-1, 256).cpu()
    assert 0.2 < sh.abs().max() / ref.abs().max() < 5                                    # neither term hides the other
    assert rel_err(out.view(-1, 256).cpu(), ref + sh) <= 2e-2
    assert rel_err(out.view(-1, 256).cpu(), sh) > 0.1 and rel_err(out.view(-1, 256).cpu(), ref) > 0.1
