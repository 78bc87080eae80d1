"""+/-Identity special experts (moe.py:39-44,95-99) and the shared expert (moe.py:118-127,174-176) on the GPU,
through the C ABI and the layer mirror."""
import numpy as np
import pytest
import torch

import bibo_amd
from bibo_amd import ops
from oracle import bibo_moe_oracle as O
from conftest import rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _inputs(T, H, I, Eg, n_pos, n_neg, k, seed):
    """GLU weights for Eg experts, router rows / bias for Eg + n_pos + n_neg."""
    p = O.make_inputs(T=T, H=H, E=Eg, k=min(k, Eg), I=I, theta="normal", seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    E = Eg + n_pos + n_neg
    p["w_router"] = (torch.randn(E, H, generator=g) * 0.02).bfloat16()
    p["bias"] = torch.rand(E, generator=g) * 0.02 - 0.01
    return p, E


@pytest.mark.parametrize("algo,T,H,I", [("generic", 60, 128, 64), ("mfma", 500, 256, 128), ("fused", 500, 256, 128),
                                        ("stream", 40, 256, 128), ("auto", 1100, 768, 384)])
@pytest.mark.parametrize("n_pos,n_neg", [(1, 1), (3, 0), (0, 2)])
def test_whole_layer_with_specials_matches_oracle(algo, T, H, I, n_pos, n_neg):
    Eg, k = 16 - n_pos - n_neg, 4
    p, E = _inputs(T, H, I, Eg, n_pos, n_neg, k, seed=T + n_pos)
    p["bias"][Eg:] += 0.3                                   # make sure the specials get picked often
    out, idx, w, counts, logits = ops.moe_forward(p["x"].to(DEV), p["w_router"].to(DEV), p["bias"].to(DEV),
                                                  p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), k,
                                                  algo=algo, want_routing=True, want_counts=True, want_logits=True,
                                                  n_pos=n_pos, n_neg=n_neg)
    torch.cuda.synchronize()
    ref, oi, ow = O.moe_forward(p["x"], p["w_router"], p["bias"], p["w_gate_up"], p["w_down"], p["theta"], k,
                                logits=logits.cpu().numpy(), n_pos=n_pos, n_neg=n_neg)
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(w.cpu().numpy(), ow)
    assert (oi >= Eg).mean() > 0.1, "the test must exercise the specials"
    assert np.array_equal(counts.cpu().numpy(), np.bincount(oi.reshape(-1), minlength=E))
    assert rel_err(out.cpu(), ref) <= 2e-2


def test_only_specials_is_a_signed_copy_of_the_input():
    """Every slot on a special: no GLU row exists at all, and the output is (sum of signed weights) * x."""
    T, H, Eg = 100, 256, 6                                        # few rows per expert keep the streaming kernels eligible
    p, E = _inputs(T, H, 128, Eg, 1, 1, 2, seed=5)
    idx = np.tile(np.array([[6, 7]], np.int32), (T, 1))            # +Identity, -Identity
    w = np.stack([np.full(T, 0.75, np.float32), np.full(T, 0.25, np.float32)], 1)
    for algo in ("generic", "mfma", "fused", "stream"):
        out, counts = ops.experts_fwd(p["x"].to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV),
                                      p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), algo=algo,
                                      want_counts=True, n_pos=1, n_neg=1)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), (0.5 * p["x"].float()).bfloat16()), algo
        assert counts.cpu().tolist() == [0] * 6 + [T, T]


def test_stage_combine_with_specials_and_residual():
    T, H, k, Eg = 50, 64, 3, 4
    g = torch.Generator().manual_seed(8)
    yw = torch.randn(T * k, H, generator=g)
    x = torch.randn(T, H, generator=g)
    res = torch.randn(T, H, generator=g)
    idx = torch.randint(0, Eg + 2, (T, k), generator=g, dtype=torch.int32)
    idx[::7, 0] = 99                                                 # padding slots
    w = torch.rand(T, k, generator=g)
    want = res.clone()
    for t in range(T):
        for j in range(k):
            e = int(idx[t, j])
            if e < Eg: want[t] += yw[t * k + j]
            elif e == Eg: want[t] += w[t, j] * x[t]
            elif e == Eg + 1: want[t] -= w[t, j] * x[t]
    got = ops.combine_fwd(yw.to(DEV), T, k, idx=idx.to(DEV), w=w.to(DEV), x=x.to(DEV), n_glu=Eg, n_pos=1, n_neg=1,
                          residual=res.to(DEV))
    torch.cuda.synchronize()
    assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-5)


def test_layer_with_default_style_config_specials_and_shared_expert():
    """The reference's default config has one +/-Identity pair; with a shared expert on top the layer output is
    routed(x) + shared(x) (moe.py:174-176)."""
    torch.manual_seed(4)
    cfg = bibo_amd.BiBoMoEConfig(hidden_size=256, moe_intermediate_size=128, num_routed_experts=16, num_experts_per_tok=4,
                                 special_expert_pairs=1, use_shared_expert=True, num_shared_experts=2)
    layer = bibo_amd.BiBoMoELayer(cfg).to(DEV).bfloat16().eval()
    with torch.no_grad():
        layer.experts.radial_theta.normal_(0, 0.5)
        layer.gate.bias[14:] += 0.3
    x = torch.randn(2, 150, 256, device=DEV).bfloat16()
    with torch.no_grad():
        out = layer(x)
        idx, w = layer.gate(x)
    sd = {k_: v.detach().cpu() for k_, v in layer.state_dict().items()}
    xf = x.cpu().reshape(-1, 256)
    routed = O.experts_forward(xf, idx.cpu().reshape(-1, 4).numpy(), w.cpu().reshape(-1, 4).numpy(),
                               sd["experts.gate_up_proj"], sd["experts.down_proj"], sd["experts.radial_theta"].float(),
                               n_pos=1, n_neg=1)
    shared = O.shared_mlp(xf, sd["shared_experts_list.0.gate_proj.weight"], sd["shared_experts_list.0.up_proj.weight"],
                          sd["shared_experts_list.0.down_proj.weight"])
    assert (idx >= 14).float().mean() > 0.05
    assert rel_err(out.cpu().reshape(-1, 256), routed + shared) <= 2e-2
    # the caller's seam composes around it
    nw = torch.ones(256, device=DEV).bfloat16()
    with torch.no_grad():
        seam = layer.ffn_forward(x, nw, 1e-6)
        xf32 = x.float()
        xn = (xf32 * torch.rsqrt(xf32.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
        assert rel_err(seam.cpu(), (x + layer(nw * xn)).cpu().float()) <= 1e-2


def test_reference_tiny_config_six_glu_plus_identity_pair():
    """The reference's own test configuration (tests/conftest.py:30-43 there): H=64, 8 routed experts = 6 GLU + one
    +/-Identity pair, k=2.  Same checks as its tests/test_moe.py:81-126,138-145: router weights positive and
    summing to one, indices in range, the layer equal to the oracle, and a bias that forces the specials gives
    out = (w_pos - w_neg) * x."""
    torch.manual_seed(0)
    cfg = bibo_amd.BiBoMoEConfig(hidden_size=64, intermediate_size=96, moe_intermediate_size=96, num_routed_experts=8,
                                 special_expert_pairs=1, num_experts_per_tok=2)
    layer = bibo_amd.BiBoMoELayer(cfg).to(DEV).eval()                # fp32 module: generic kernels
    x = torch.randn(2, 33, 64, device=DEV)
    with torch.no_grad():
        out = layer(x)
        idx, w = layer.gate(x)
    assert idx.dtype == torch.int64 and w.dtype == torch.float32 and idx.min() >= 0 and idx.max() < 8
    assert (w > 0).all() and torch.allclose(w.sum(-1), torch.ones_like(w.sum(-1)), atol=1e-6)
    sd = {k_: v.detach().cpu() for k_, v in layer.state_dict().items()}
    ref = O.experts_forward(x.cpu().reshape(-1, 64), idx.cpu().reshape(-1, 2).numpy(), w.cpu().reshape(-1, 2).numpy(),
                            sd["experts.gate_up_proj"], sd["experts.down_proj"], sd["experts.radial_theta"], n_pos=1,
                            n_neg=1)
    assert rel_err(out.cpu().reshape(-1, 64), ref) <= 1e-5
    with torch.no_grad():
        layer.gate.bias[6:] += 5.0                                  # selection only: both specials always win
        out2 = layer(x)
        idx2, w2 = layer.gate(x)
    assert (idx2 == torch.tensor([6, 7], device=DEV)).all()
    assert torch.allclose(out2, (w2[..., :1] - w2[..., 1:]) * x, atol=1e-6)
