"""Backward pass of the layer through the C ABI (bibo_moe_backward) against the oracle's autograd gradients, which
are pinned on the CPU by central differences and closed forms (tests/test_oracle.py).  The oracle differentiates the
fp64 forward with the selection the kernel made; the kernel works in bf16 with fp32 accumulation, so gradients are
compared by max |difference| relative to max |reference| per tensor."""
import numpy as np
import pytest
import torch

from bibo_amd import ops
from oracle import bibo_moe_oracle as O

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
TOL = 2e-2          # bf16 operands, fp32 accumulation, bf16 results
F32_TOL = 1e-5      # fp32 operands and arithmetic against the fp64 oracle (measured below 1e-6)


def _rel(a, ref):
    return float((a.double().cpu() - ref.double()).abs().max() / ref.double().abs().max().clamp_min(1e-30))


def _run(T, H, E, k, I, norm="sum", act="radial", seed=0, theta="normal", scale=1.0):
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, bias="uniform", theta=theta, seed=seed)
    g = torch.Generator().manual_seed(seed + 100)
    d_out = (torch.randn(T, H, generator=g) * scale).to(torch.bfloat16)
    dev = lambda t: t.to(DEV)
    _, idx, w, _, logits = ops.moe_forward(dev(p["x"]), dev(p["w_router"]), dev(p["bias"]), dev(p["w_gate_up"]),
                                           dev(p["w_down"]), dev(p["theta"]), k, norm=norm, act=act, want_routing=True,
                                           want_logits=True)
    got = ops.moe_backward(dev(p["x"]), dev(d_out), dev(p["w_router"]), dev(p["bias"]), dev(p["w_gate_up"]), dev(p["w_down"]),
                           dev(p["theta"]), k, norm=norm, act=act, want_dw=True)
    torch.cuda.synchronize()
    ref = O.moe_backward(p["x"], p["w_router"], p["w_gate_up"], p["w_down"], p["theta"], idx.cpu().numpy(), d_out, norm=norm,
                         act=act)
    return dict(zip(("x", "w_router", "w_gate_up", "w_down", "theta", "w"), got)), ref, idx.cpu().numpy()


@pytest.mark.parametrize("T,H,E,k,I", [(300, 256, 16, 4, 128), (512, 512, 64, 6, 256), (64, 384, 8, 2, 384), (1000, 768, 64, 6, 384),
                                       (200, 1024, 16, 4, 512),      # the widest rows the backward pass takes
                                       (600, 256, 4, 2, 128), (700, 768, 5, 3, 384)])   # 300 / 420 rows per expert: 256-row tiles
def test_backward_matches_oracle(T, H, E, k, I):
    got, ref, _ = _run(T, H, E, k, I, seed=T)
    for name in ("w", "x", "w_down", "w_gate_up", "w_router", "theta"):
        assert _rel(got[name], ref[name]) <= TOL, (name, _rel(got[name], ref[name]))


@pytest.mark.parametrize("T,H,Eg,n_pos,n_neg,k,I,norm", [(300, 256, 6, 1, 1, 3, 128, "sum"), (1000, 768, 62, 1, 1, 6, 384, "sum"),
                                                         (200, 256, 5, 2, 0, 4, 128, "softmax"), (64, 384, 3, 0, 2, 2, 256, False)])
def test_backward_with_identity_experts_matches_oracle(T, H, Eg, n_pos, n_neg, k, I, norm):
    """+/-Identity experts (moe.py:95-99, on by default in the reference's configuration): a slot routed to one sends
    +/- w d_out to d_x and +/- <d_out, x> to its combine weight, hence to the router; its router row gets a gradient,
    the GLU experts' tensors keep their shapes."""
    E = Eg + n_pos + n_neg
    p = O.make_inputs(T=T, H=H, E=Eg, k=k, I=I, theta="normal", seed=T + E)
    g = torch.Generator().manual_seed(T)
    p["w_router"] = (torch.randn(E, H, generator=g) * 0.02).bfloat16()
    p["bias"] = torch.rand(E, generator=g) * 0.02 - 0.01
    p["bias"][Eg:] += 0.05                                         # the specials get their share of the slots
    d_out = torch.randn(T, H, generator=g).to(torch.bfloat16)
    dev = lambda t: t.to(DEV)
    args = [dev(p[n]) for n in ("w_router", "bias", "w_gate_up", "w_down", "theta")]
    _, idx, w, _, _ = ops.moe_forward(dev(p["x"]), *args, k, norm=norm, want_routing=True, n_pos=n_pos, n_neg=n_neg)
    got = ops.moe_backward(dev(p["x"]), dev(d_out), *args, k, norm=norm, want_dw=True, n_pos=n_pos, n_neg=n_neg)
    torch.cuda.synchronize()
    idx = idx.cpu().numpy()
    assert (idx >= Eg).sum() > 0                                   # the case does route to specials
    ref = O.moe_backward(p["x"], p["w_router"], p["w_gate_up"], p["w_down"], p["theta"], idx, d_out, norm=norm, n_pos=n_pos,
                         n_neg=n_neg)
    got = dict(zip(("x", "w_router", "w_gate_up", "w_down", "theta", "w"), got))
    assert got["w_router"].shape == (E, H) and got["w_gate_up"].shape == (Eg, 2 * I, H) and got["theta"].shape == (Eg,)
    for name in ("w", "x", "w_down", "w_gate_up", "w_router", "theta"):
        assert _rel(got[name], ref[name]) <= TOL, (name, _rel(got[name], ref[name]))
    # the experts alone, with the routing as the caller's: same d_x up to the router's share, same d_w
    gx, gw, ggu, gdn, gth = ops.experts_backward(dev(p["x"]), dev(d_out), dev(torch.from_numpy(idx)), w, dev(p["w_gate_up"]),
                                                 dev(p["w_down"]), dev(p["theta"]), n_pos=n_pos, n_neg=n_neg)
    torch.cuda.synchronize()
    assert torch.equal(gw, got["w"]) and torch.equal(ggu, got["w_gate_up"]) and torch.equal(gdn, got["w_down"])


def test_layer_with_identity_experts_trains():
    """The reference's default configuration has one +Identity and one -Identity expert: the module's forward under
    autograd reaches every parameter, with or without hooks on the submodules."""
    from bibo_amd.config import BiBoMoEConfig
    from bibo_amd.moe import BiBoMoELayer
    layer = BiBoMoELayer(BiBoMoEConfig(hidden_size=256, moe_intermediate_size=128, num_routed_experts=8,
                                       num_experts_per_tok=3, special_expert_pairs=1)).to(DEV).bfloat16()
    assert layer.experts.num_pos == 1 and layer.experts.num_neg == 1
    x = torch.randn(2, 40, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    layer(x).float().square().sum().backward()
    assert x.grad is not None and bool(torch.isfinite(x.grad.float()).all())
    grads = {n: prm.grad.clone() for n, prm in layer.named_parameters() if prm.requires_grad}
    assert all(g is not None and bool(torch.isfinite(g.float()).all()) for g in grads.values())
    assert float(grads["gate.gate_proj.weight"][-2:].abs().max()) > 0      # the specials' router rows learn
    # the same through the experts seam (a hook makes the layer call its submodules one by one)
    for prm in layer.parameters():
        prm.grad = None
    hook = layer.experts.register_forward_hook(lambda m, a, o: None)
    x2 = x.detach().clone().requires_grad_(True)
    layer(x2).float().square().sum().backward()
    hook.remove()
    assert _rel(x2.grad, x.grad.cpu()) <= TOL
    for n, prm in layer.named_parameters():
        if prm.requires_grad:
            assert _rel(prm.grad, grads[n].cpu()) <= TOL, n


@pytest.mark.parametrize("norm,act", [("softmax", "radial"), (False, "tanh"), ("sum", "silu"), ("sum", "tanh")])
def test_backward_norm_modes_and_activations(norm, act):
    got, ref, _ = _run(320, 256, 16, 3, 128, norm=norm, act=act, seed=7)
    for name in ("w", "x", "w_down", "w_gate_up", "w_router"):
        assert _rel(got[name], ref[name]) <= TOL, (name, _rel(got[name], ref[name]))
    if act == "silu":
        assert float(got["theta"].abs().max()) == 0.0            # plain SwiGLU: theta is not read
    else:
        assert _rel(got["theta"], ref["theta"]) <= TOL


def test_backward_idle_experts_and_ragged_rows():
    """Experts that get no row have zero weight gradients; row counts that are no multiple of any tile size."""
    T, H, E, k, I = 37, 256, 64, 2, 128
    got, ref, idx = _run(T, H, E, k, I, seed=5)
    idle = np.setdiff1d(np.arange(E), np.unique(idx))
    assert idle.size > 0
    for name in ("w_down", "w_gate_up", "w_router"):
        assert float(got[name][torch.from_numpy(idle).to(DEV)].abs().max()) == 0.0
        assert _rel(got[name], ref[name]) <= TOL, name
    assert _rel(got["x"], ref["x"]) <= TOL and _rel(got["theta"], ref["theta"]) <= TOL


@pytest.mark.parametrize("H,I,dtype", [(256, 128, torch.bfloat16), (48, 40, torch.float32)])
def test_backward_of_a_few_tokens_and_of_none(H, I, dtype):
    """One token, three tokens (far fewer rows than a tile holds) and an empty batch, in both kernel families: an
    empty batch gives zero gradients for every parameter."""
    E, k = 8, 2
    tol = TOL if dtype == torch.bfloat16 else F32_TOL
    for T in (1, 3):
        got, ref, _ = _run_generic(T, H, E, k, I, dtype, seed=T)
        for name in ("w", "x", "w_down", "w_gate_up", "w_router", "theta"):
            assert _rel(got[name], ref[name]) <= tol, (T, name, _rel(got[name], ref[name]))
    p = O.make_inputs(T=4, H=H, E=E, k=k, I=I, seed=0)
    dev = lambda t: (t.to(dtype) if t.dtype == torch.bfloat16 else t).to(DEV)
    none = torch.empty(0, H, dtype=dtype, device=DEV)
    ops.workspace(DEV, 1 << 20).fill_(0x7f)
    got = ops.moe_backward(none, none, dev(p["w_router"]), dev(p["bias"]), dev(p["w_gate_up"]), dev(p["w_down"]),
                           dev(p["theta"]), k)
    torch.cuda.synchronize()
    assert got[0].shape == (0, H)
    for g in got[1:5]:
        assert float(g.float().abs().max()) == 0.0


@pytest.mark.parametrize("T,H,Eg,n_pos,n_neg,k,I,norm,act", [(700, 768, 5, 0, 0, 3, 384, "sum", "radial"),
                                                              (300, 256, 6, 1, 1, 3, 128, "softmax", "tanh"),
                                                              (37, 256, 64, 0, 0, 2, 128, "sum", "radial"),
                                                              (1, 384, 8, 0, 0, 2, 256, False, "silu"),
                                                              (0, 256, 8, 0, 0, 2, 128, "sum", "radial")])
def test_training_forward_keeps_what_the_backward_would_recompute(T, H, Eg, n_pos, n_neg, k, I, norm, act):
    """bibo_moe_forward_train gives the output of bibo_moe_forward with the fused kernels bit for bit, and
    bibo_moe_backward_saved, reading routing, permutation and pre-activations from its state buffer, the gradients of
    bibo_moe_backward bit for bit (tall and short tiles, +/-Identity experts, idle experts, one token, no token)."""
    E = Eg + n_pos + n_neg
    p = O.make_inputs(T=T, H=H, E=Eg, k=k, I=I, theta="normal", seed=T + 1)
    g = torch.Generator().manual_seed(T)
    p["w_router"] = (torch.randn(E, H, generator=g) * 0.05).bfloat16()
    p["bias"] = torch.rand(E, generator=g) * 0.02 - 0.01
    d_out = torch.randn(T, H, generator=g).to(torch.bfloat16).to(DEV)
    dev = lambda t: t.to(DEV)
    x, wr, b, gu, dn, th = (dev(p[n]) for n in ("x", "w_router", "bias", "w_gate_up", "w_down", "theta"))
    kw = dict(norm=norm, act=act, n_pos=n_pos, n_neg=n_neg)
    ref_out, _, _, ref_counts, _ = ops.moe_forward(x, wr, b, gu, dn, th, k, algo="fused", want_counts=True, **kw)
    ref = ops.moe_backward(x, d_out, wr, b, gu, dn, th, k, want_dw=True, **kw)
    out, counts, state = ops.moe_forward_train(x, wr, b, gu, dn, th, k, want_counts=True, **kw)
    ops.workspace(DEV, 1 << 20).fill_(0x7f)                            # nothing may be left over in the workspace
    got = ops.moe_backward_saved(x, d_out, wr, gu, dn, th, k, state, want_dw=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(out, ref_out) and torch.equal(counts, ref_counts)
    for a, r, name in zip(got, ref, ("x", "w_router", "w_gate_up", "w_down", "theta", "w")):
        assert torch.equal(a, r), name


def test_layer_trains_the_same_with_and_without_kept_activations():
    """The module's two ways through the library (keep_activations) give the same output and gradients, and what has
    no state-keeping pair (fp32, odd sizes) is reported as such instead of failing."""
    assert ops.train_state_bytes(64, 256, 8, 2, 128, torch.float32) is None
    assert ops.train_state_bytes(64, 200, 8, 2, 128, torch.bfloat16) is None
    assert ops.train_state_bytes(64, 256, 8, 2, 512, torch.bfloat16) is None      # I = 512: MFMA backward, no fused forward
    assert ops.train_state_bytes(64, 256, 8, 2, 128, torch.bfloat16) > 64 * 2 * 2 * 128 * 2
    res = []
    for keep in (True, False):
        torch.manual_seed(5)
        layer = _layer()
        layer.keep_activations = keep
        x = torch.randn(2, 400, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)   # 200 rows per expert: the fused kernel either way
        out = layer(x)
        out.float().square().sum().backward()
        res.append((out.detach(), x.grad, {n: p_.grad for n, p_ in layer.named_parameters() if p_.grad is not None}))
    (o1, g1, p1), (o2, g2, p2) = res
    assert torch.equal(o1, o2) and torch.equal(g1, g2) and sorted(p1) == sorted(p2)
    for n in p1:
        assert torch.equal(p1[n], p2[n]), n


def test_backward_with_a_few_experts_holding_most_rows():
    """Four experts that every token selects (selection bias + 2): their rows are cut into chunks by the weight-gradient
    GEMMs and the chunks' partial tiles are added up; every gradient against the oracle, and twice the same bits."""
    T, H, E, k, I = 1500, 256, 16, 6, 128                  # 1500 rows on each hot expert, 250 on average elsewhere
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, bias="hot4", theta="normal", seed=44)
    g = torch.Generator().manual_seed(45)
    d_out = torch.randn(T, H, generator=g).to(torch.bfloat16)
    dev = lambda t: t.to(DEV)
    args = [dev(p[n]) for n in ("w_router", "bias", "w_gate_up", "w_down", "theta")]
    _, idx, _, counts, _ = ops.moe_forward(dev(p["x"]), *args, k, want_routing=True, want_counts=True)
    assert int(counts.max()) == T and int(counts.max()) > 2 * (T * k // E)      # cut into chunks: above 1.5 x the average
    got = ops.moe_backward(dev(p["x"]), dev(d_out), *args, k, want_dw=True)
    again = ops.moe_backward(dev(p["x"]), dev(d_out), *args, k, want_dw=True)
    torch.cuda.synchronize()
    ref = O.moe_backward(p["x"], p["w_router"], p["w_gate_up"], p["w_down"], p["theta"], idx.cpu().numpy(), d_out)
    for a, b_, name in zip(got, again, ("x", "w_router", "w_gate_up", "w_down", "theta", "w")):
        assert torch.equal(a, b_), name
        assert _rel(a, ref[name]) <= TOL, (name, _rel(a, ref[name]))


def test_backward_is_linear_in_the_upstream_gradient():
    """Size-independent property at the full c2 shape: the gradients of 2 d are twice those of d (every path is linear
    in d_out), to bf16 rounding; and nothing is accumulated between calls."""
    T, H, E, k, I = 8192, 768, 64, 6, 384
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, bias="uniform", theta="normal", seed=20262)
    g = torch.Generator().manual_seed(1)
    d = torch.randn(T, H, generator=g).to(torch.bfloat16).to(DEV)
    args = [p[n].to(DEV) for n in ("w_router", "bias", "w_gate_up", "w_down", "theta")]
    x = p["x"].to(DEV)
    a = ops.moe_backward(x, d, *args, k)
    b = ops.moe_backward(x, (2 * d.float()).to(torch.bfloat16), *args, k)
    a2 = ops.moe_backward(x, d, *args, k)
    torch.cuda.synchronize()
    for u, v, u2 in zip(a[:5], b[:5], a2[:5]):
        assert torch.equal(u, u2)
        assert _rel(v.float(), 2 * u.float().cpu()) <= 1e-2
    assert all(bool(torch.isfinite(t.float()).all()) for t in a[:5])


def test_backward_families_and_what_neither_covers():
    """bf16 with H and I multiples of 128 runs the MFMA backward; other sizes and fp32 run the generic kernels, whose
    workspace holds fp32 intermediates; a row of more than 64 KB (2H + 5I floats) is refused."""
    from bibo_amd import _lib as L
    import ctypes
    n = ctypes.c_size_t(0)
    size = lambda *a: (L.lib().bibo_moe_backward_workspace_bytes(ctypes.byref(L.Shape(*a)), ctypes.byref(n)), n.value)
    rc_fast, fast = size(64, 256, 8, 2, 128, L.DTYPE_BF16)
    rc_odd, odd = size(64, 200, 8, 2, 128, L.DTYPE_BF16)           # H no multiple of 128: generic
    rc_f32, f32 = size(64, 256, 8, 2, 128, L.DTYPE_F32)            # fp32: generic
    assert (rc_fast, rc_odd, rc_f32) == (0, 0, 0) and min(fast, odd, f32) > 0
    assert size(64, 256, 8, 2, 128, L.DTYPE_BF16, 1, 1)[0] == 0    # +/-Identity experts are covered
    assert size(64, 4096, 8, 2, 2048, L.DTYPE_BF16)[0] == -6       # MFMA family: I > 512; generic: 72 KB per row


def _run_generic(T, H, E, k, I, dtype, norm="sum", act="radial", seed=0, n_pos=0, n_neg=0):
    """bibo_moe_backward on a shape or dtype the generic kernels take, against the fp64 autograd oracle."""
    Et = E + n_pos + n_neg
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, theta="normal", seed=seed)
    g = torch.Generator().manual_seed(seed + 50)
    p["w_router"] = (torch.randn(Et, H, generator=g) * 0.05).bfloat16()
    p["bias"] = torch.rand(Et, generator=g) * 0.02 - 0.01
    if n_pos + n_neg:
        p["bias"][E:] += 0.05
    d_out = torch.randn(T, H, generator=g).to(torch.bfloat16)
    dev = lambda t: (t.to(dtype) if t.dtype == torch.bfloat16 else t).to(DEV)     # bf16-representable values either way
    args = [dev(p[n]) for n in ("w_router", "bias", "w_gate_up", "w_down", "theta")]
    _, idx, w, _, _ = ops.moe_forward(dev(p["x"]), *args, k, norm=norm, act=act, want_routing=True, n_pos=n_pos, n_neg=n_neg)
    got = ops.moe_backward(dev(p["x"]), dev(d_out), *args, k, norm=norm, act=act, want_dw=True, n_pos=n_pos, n_neg=n_neg)
    torch.cuda.synchronize()
    ref = O.moe_backward(p["x"], p["w_router"], p["w_gate_up"], p["w_down"], p["theta"], idx.cpu().numpy(), d_out, norm=norm,
                         act=act, n_pos=n_pos, n_neg=n_neg)
    return dict(zip(("x", "w_router", "w_gate_up", "w_down", "theta", "w"), got)), ref, idx.cpu().numpy()


@pytest.mark.parametrize("T,H,E,k,I", [(40, 48, 6, 2, 40), (130, 100, 16, 4, 72), (64, 256, 8, 2, 128)])
def test_generic_backward_in_fp32_matches_oracle(T, H, E, k, I):
    """fp32 operands, fp32 arithmetic, sizes that are no multiples of anything: every gradient against the fp64 oracle
    at 1e-5 of each tensor's maximum."""
    got, ref, _ = _run_generic(T, H, E, k, I, torch.float32, seed=T)
    errs = {name: _rel(got[name], ref[name]) for name in ("w", "x", "w_down", "w_gate_up", "w_router", "theta")}
    print("fp32 backward", (T, H, E, k, I), {n: f"{e:.1e}" for n, e in errs.items()})
    for name, err in errs.items():
        assert got[name].dtype == torch.float32
        assert err <= F32_TOL, (name, err)


@pytest.mark.parametrize("norm,act,n_pos,n_neg", [("softmax", "tanh", 0, 0), (False, "silu", 0, 0), ("sum", "radial", 1, 1)])
def test_generic_backward_modes_and_identity_experts(norm, act, n_pos, n_neg):
    got, ref, idx = _run_generic(90, 72, 6, 3, 48, torch.float32, norm=norm, act=act, seed=11, n_pos=n_pos, n_neg=n_neg)
    if n_pos + n_neg:
        assert (idx >= 6).sum() > 0
    for name in ("w", "x", "w_down", "w_gate_up", "w_router") + (() if act == "silu" else ("theta",)):
        assert _rel(got[name], ref[name]) <= F32_TOL, (name, _rel(got[name], ref[name]))


def test_generic_backward_in_bf16_on_odd_sizes():
    """bf16 operands whose sizes the MFMA tiles do not divide: the generic kernels, bf16 results."""
    got, ref, idx = _run_generic(150, 200, 8, 3, 96, torch.bfloat16, seed=3)
    for name in ("w", "x", "w_down", "w_gate_up", "w_router", "theta"):
        assert _rel(got[name], ref[name]) <= TOL, (name, _rel(got[name], ref[name]))
    idle = np.setdiff1d(np.arange(8), np.unique(idx))
    for e in idle:
        assert float(got["w_down"][e].abs().max()) == 0.0


def test_generic_backward_at_the_lds_limit():
    """The longest rows the generic kernels take: 2H + 5I floats just under 64 KB of LDS."""
    got, ref, _ = _run_generic(4, 4096, 2, 1, 1616, torch.bfloat16, seed=9)
    for name in ("w", "x", "w_down", "w_gate_up", "w_router", "theta"):
        assert _rel(got[name], ref[name]) <= TOL, (name, _rel(got[name], ref[name]))
    assert not ops.backward_supported(4096, 1664, 2, torch.bfloat16)


def test_generic_experts_backward_with_padded_slots():
    """The experts alone in fp32 with padding ids in a caller's indices: zero combine-weight gradient for those slots,
    nothing of theirs in d_x (workspace poisoned first)."""
    T, H, E, k, I = 60, 40, 5, 3, 24
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, theta="normal", seed=2)
    g = torch.Generator().manual_seed(6)
    idx = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32)
    idx[:, 0] = -1
    w = torch.rand(T, k, generator=g) + 0.1
    d_out = torch.randn(T, H, generator=g)
    f = lambda t: t.float().to(DEV)
    ops.workspace(DEV, 64 << 20).fill_(0x7f)
    got = ops.experts_backward(f(p["x"]), f(d_out), idx.to(DEV), f(w), f(p["w_gate_up"]), f(p["w_down"]), f(p["theta"]))
    torch.cuda.synchronize()
    pad = idx < 0
    w0, idx0 = w.clone(), idx.clone()
    w0[pad] = 0.0
    idx0[pad] = 0
    leaf = lambda t: t.double().clone().requires_grad_(True)
    x, wl, gu, dn, th = leaf(p["x"]), leaf(w0), leaf(p["w_gate_up"]), leaf(p["w_down"]), leaf(p["theta"])
    (O.experts_forward(x, idx0, wl, gu, dn, th, dtype=torch.float64) * d_out.double()).sum().backward()
    ref_w = wl.grad.clone()
    ref_w[pad] = 0.0
    assert float(got[1].cpu()[pad].abs().max()) == 0.0
    for a, r, name in zip(got, (x.grad, ref_w, gu.grad, dn.grad, th.grad), ("x", "w", "w_gate_up", "w_down", "theta")):
        assert bool(torch.isfinite(a.float()).all()) and _rel(a, r) <= F32_TOL, (name, _rel(a, r))


# ---- the module: BiBoMoELayer.forward under autograd ----
def _layer(H=256, I=128, E=8, k=2, **kw):
    from bibo_amd.config import BiBoMoEConfig
    from bibo_amd.moe import BiBoMoELayer
    cfg = BiBoMoEConfig(hidden_size=H, moe_intermediate_size=I, num_routed_experts=E, num_experts_per_tok=k,
                        special_expert_pairs=0, **kw)
    torch.manual_seed(0)
    return BiBoMoELayer(cfg).to(DEV).bfloat16()


def test_radial_theta_is_a_real_learnable_parameter():
    """The reference's regression test (tests/test_moe.py:53-63): theta requires grad, starts at 0, and a backward
    through the layer leaves a non-zero gradient in it."""
    layer = _layer()
    th = layer.experts.radial_theta
    assert th.requires_grad and float(th.detach().abs().max()) == 0.0
    x = torch.randn(2, 6, 256, device=DEV, dtype=torch.bfloat16)
    (layer(x) * torch.randn(2, 6, 256, device=DEV, dtype=torch.bfloat16)).sum().backward()
    assert th.grad is not None and float(th.grad.abs().max()) > 0


def test_layer_gradients_match_oracle():
    layer = _layer(H=256, I=128, E=16, k=4)
    with torch.no_grad():
        layer.experts.radial_theta.copy_(torch.linspace(-2, 3, 16))
        layer.gate.bias.copy_(torch.linspace(-0.01, 0.01, 16))
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 50, 256, generator=g).to(torch.bfloat16).to(DEV).requires_grad_(True)
    d = torch.randn(3, 50, 256, generator=g).to(torch.bfloat16).to(DEV)
    layer.train()
    out = layer(x)
    out.backward(d)
    torch.cuda.synchronize()
    p = {n: v.detach().cpu() for n, v in (("wr", layer.gate.gate_proj.weight), ("b", layer.gate.bias),
                                          ("gu", layer.experts.gate_up_proj), ("dn", layer.experts.down_proj),
                                          ("th", layer.experts.radial_theta))}
    x2 = x.detach().cpu().reshape(150, 256)
    _, idx, _, _, _ = ops.moe_forward(x.detach().reshape(150, 256), layer.gate.gate_proj.weight.detach(), layer.gate.bias.detach().float(),
                                      layer.experts.gate_up_proj.detach(), layer.experts.down_proj.detach(),
                                      layer.experts.radial_theta.detach().float(), 4, want_routing=True)
    ref = O.moe_backward(x2, p["wr"], p["gu"], p["dn"], p["th"].float(), idx.cpu().numpy(), d.cpu().reshape(150, 256))
    assert _rel(x.grad.reshape(150, 256), ref["x"]) <= TOL
    assert _rel(layer.gate.gate_proj.weight.grad, ref["w_router"]) <= TOL
    assert _rel(layer.experts.gate_up_proj.grad, ref["w_gate_up"]) <= TOL
    assert _rel(layer.experts.down_proj.grad, ref["w_down"]) <= TOL
    assert _rel(layer.experts.radial_theta.grad, ref["theta"]) <= TOL
    assert layer.gate.bias.grad is None                          # selection only (router.py:38)
    assert float(layer.accumulated_tpe.sum()) == 150 * 4        # the training forward still feeds the balancing state


def test_seam_and_shared_expert_under_autograd():
    """ffn_forward with autograd on: norm and residual become ordinary differentiable operations around the block, and
    the shared expert's parameters get gradients as well."""
    layer = _layer(H=256, I=128, E=8, k=2, use_shared_expert=True)
    nw = torch.ones(256, device=DEV, requires_grad=True)
    h = torch.randn(2, 20, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    out = layer.ffn_forward(h, nw, 1e-6)
    out.float().square().sum().backward()
    assert h.grad is not None and nw.grad is not None and float(nw.grad.abs().max()) > 0
    for prm in layer.parameters():
        if prm.requires_grad:
            assert prm.grad is not None and bool(torch.isfinite(prm.grad.float()).all())


def test_fp32_and_odd_sized_layers_train():
    """The regimes of the reference's own gradient tests (tests/test_moe.py:53-63, ablate/common/test_eager_radial.py:
    63-89): an fp32 layer of small, odd sizes under autograd.  theta starts at 0, receives a non-zero gradient, and
    moving it moves the output; fp32 master weights under bf16 autocast train as well; only rows too long for the
    generic kernels' LDS are refused."""
    from bibo_amd.config import BiBoMoEConfig
    from bibo_amd.moe import BiBoMoELayer
    torch.manual_seed(1)
    layer = BiBoMoELayer(BiBoMoEConfig(hidden_size=96, moe_intermediate_size=40, num_routed_experts=6,
                                       num_experts_per_tok=2, special_expert_pairs=0)).to(DEV)
    th = layer.experts.radial_theta
    assert th.requires_grad and float(th.detach().abs().max()) == 0.0
    x = torch.randn(2, 6, 96, device=DEV, requires_grad=True)
    out = layer(x)
    assert out.dtype == torch.float32
    (out * torch.randn(2, 6, 96, device=DEV)).sum().backward()
    assert th.grad is not None and float(th.grad.abs().max()) > 0 and x.grad is not None
    for prm in layer.parameters():
        if prm.requires_grad:
            assert prm.grad is not None and prm.grad.dtype == torch.float32 and bool(torch.isfinite(prm.grad).all())
    with torch.no_grad():
        base = layer(x).clone()
        th += 2.0
        assert float((layer(x) - base).abs().max()) > 1e-5
    bf = BiBoMoELayer(BiBoMoEConfig(hidden_size=192, moe_intermediate_size=128, num_routed_experts=8,
                                    num_experts_per_tok=2)).to(DEV).bfloat16()
    xb = torch.randn(1, 8, 192, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    bf(xb).float().square().sum().backward()                       # hidden size no multiple of 128: generic kernels
    assert xb.grad is not None and bf.experts.down_proj.grad is not None
    fp32 = _layer().float()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        fp32(torch.randn(1, 8, 256, device=DEV)).sum().backward()  # fp32 master weights under bf16 autocast
    assert fp32.experts.gate_up_proj.grad is not None and fp32.experts.gate_up_proj.grad.dtype == torch.float32
    huge = BiBoMoELayer(BiBoMoEConfig(hidden_size=4096, moe_intermediate_size=2048, num_routed_experts=2,
                                      num_experts_per_tok=1, special_expert_pairs=0)).to(DEV).bfloat16()
    with pytest.raises(NotImplementedError):
        huge(torch.randn(1, 4, 4096, device=DEV, dtype=torch.bfloat16))
    with torch.no_grad():
        huge(torch.randn(1, 4, 4096, device=DEV, dtype=torch.bfloat16))


def test_experts_backward_with_caller_owned_routing():
    """bibo_moe_experts_backward: the experts alone, routing handed in (an expert may repeat inside a token); d_w is the
    gradient of the combine weights."""
    T, H, E, k, I = 200, 256, 8, 3, 128
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, theta="normal", seed=9)
    g = torch.Generator().manual_seed(4)
    idx = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32)
    w = torch.rand(T, k, generator=g) + 0.1
    d_out = torch.randn(T, H, generator=g).to(torch.bfloat16)
    dev = lambda t: t.to(DEV)
    got = ops.experts_backward(dev(p["x"]), dev(d_out), dev(idx), dev(w), dev(p["w_gate_up"]), dev(p["w_down"]), dev(p["theta"]))
    torch.cuda.synchronize()
    leaf = lambda t: t.double().clone().requires_grad_(True)
    x, wl, gu, dn, th = leaf(p["x"]), leaf(w), leaf(p["w_gate_up"]), leaf(p["w_down"]), leaf(p["theta"])
    (O.experts_forward(x, idx, wl, gu, dn, th, dtype=torch.float64) * d_out.double()).sum().backward()
    for a, r, name in zip(got, (x.grad, wl.grad, gu.grad, dn.grad, th.grad), ("x", "w", "w_gate_up", "w_down", "theta")):
        assert _rel(a, r) <= TOL, (name, _rel(a, r))


def test_hooks_path_trains_module_by_module():
    """With a hook present the layer calls router and experts as modules; both carry autograd graphs, and the
    gradients agree with the single-node path."""
    layer = _layer(H=256, I=128, E=16, k=4)
    with torch.no_grad():
        layer.experts.radial_theta.copy_(torch.linspace(-1, 1, 16))
    g = torch.Generator().manual_seed(6)
    x = torch.randn(2, 40, 256, generator=g).to(torch.bfloat16).to(DEV)
    d = torch.randn(2, 40, 256, generator=g).to(torch.bfloat16).to(DEV)
    layer(x).backward(d)
    ref = {n: p.grad.clone() for n, p in layer.named_parameters() if p.grad is not None}
    layer.zero_grad()
    seen = []
    h = layer.gate.register_forward_hook(lambda m, i, o: seen.append(o[0].shape))
    layer(x).backward(d)
    h.remove()
    assert seen == [torch.Size([2, 40, 4])]
    for n, p in layer.named_parameters():
        if n in ref:
            assert _rel(p.grad, ref[n].cpu()) <= 3e-2, n


def test_experts_backward_with_padded_slots():
    """Routing indices outside [0, E) (padding in a caller's indices): the forward pass skips those slots, and the
    backward pass gives them a zero combine-weight gradient and leaves them out of d_x.  The workspace is poisoned
    first, so a slot row nobody wrote cannot pass by luck."""
    T, H, E, k, I = 150, 256, 8, 3, 128
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, theta="normal", seed=12)
    g = torch.Generator().manual_seed(5)
    idx = torch.randint(0, E, (T, k), generator=g, dtype=torch.int32)
    idx[:, 1] = E                                                  # one padded slot per token
    idx[::7, 2] = -1
    w = torch.rand(T, k, generator=g) + 0.1
    d_out = torch.randn(T, H, generator=g).to(torch.bfloat16)
    dev = lambda t: t.to(DEV)
    ops.workspace(DEV, 256 << 20).fill_(0x7f)                      # bf16 0x7f7f = 3.4e38, fp32 0x7f7f7f7f = 3.4e38
    got = ops.experts_backward(dev(p["x"]), dev(d_out), dev(idx), dev(w), dev(p["w_gate_up"]), dev(p["w_down"]), dev(p["theta"]))
    torch.cuda.synchronize()
    pad = (idx < 0) | (idx >= E)
    w0, idx0 = w.clone(), idx.clone()
    w0[pad] = 0.0                                                  # the same slots with weight zero on a real expert
    idx0[pad] = 0
    leaf = lambda t: t.double().clone().requires_grad_(True)
    x, wl, gu, dn, th = leaf(p["x"]), leaf(w0), leaf(p["w_gate_up"]), leaf(p["w_down"]), leaf(p["theta"])
    (O.experts_forward(x, idx0, wl, gu, dn, th, dtype=torch.float64) * d_out.double()).sum().backward()
    ref_w = wl.grad.clone()
    ref_w[pad] = 0.0
    assert float(got[1].cpu()[pad].abs().max()) == 0.0
    for a, r, name in zip(got, (x.grad, ref_w, gu.grad, dn.grad, th.grad), ("x", "w", "w_gate_up", "w_down", "theta")):
        assert bool(torch.isfinite(a.float()).all()), name
        assert _rel(a, r) <= TOL, (name, _rel(a, r))
    # the module under autograd takes the same indices
    from bibo_amd.config import BiBoMoEConfig
    from bibo_amd.moe import BiBoFusedExperts
    ex = BiBoFusedExperts(BiBoMoEConfig(hidden_size=H, moe_intermediate_size=I, num_routed_experts=E, num_experts_per_tok=k,
                                        special_expert_pairs=0)).to(DEV).bfloat16()
    with torch.no_grad():
        ex.gate_up_proj.copy_(p["w_gate_up"]); ex.down_proj.copy_(p["w_down"])
    ex.radial_theta.data = dev(p["theta"])                         # fp32, so both calls see the same exponents
    xg, wg = dev(p["x"]).requires_grad_(True), dev(w).requires_grad_(True)
    ex(xg, dev(idx).long(), wg).backward(dev(d_out))
    assert torch.equal(xg.grad, got[0]) and torch.equal(wg.grad, got[1])


def test_fp32_master_weights_train_while_the_balancing_bias_moves():
    """fp32 master weights under bf16 autocast with a balancing step that fires in the same forward (token count at the
    threshold, moe.py:139-155): update_bias writes gate.bias in place after the block ran, the backward pass still
    routes with the bias the forward saw, and the gradients are those of that selection."""
    T, H, E, k, I = 256, 256, 16, 4, 128
    layer = _layer(H=H, I=I, E=E, k=k, bias_update_threshold=T).float().train()
    with torch.no_grad():
        layer.gate.bias.copy_(torch.linspace(-0.2, 0.2, E))        # far from balance: the update moves every entry
        layer.experts.radial_theta.copy_(torch.linspace(-1, 2, E))
    bias0 = layer.gate.bias.detach().clone()
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, T // 2, H, generator=g).to(DEV).requires_grad_(True)
    d = torch.randn(2, T // 2, H, generator=g).to(DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = layer(x)
    assert not torch.equal(layer.gate.bias.detach(), bias0)         # the balancing step fired inside the forward
    out.backward(d.to(out.dtype))
    torch.cuda.synchronize()
    bf = lambda t: t.detach().to(torch.bfloat16)
    xb = bf(x).reshape(T, H)
    _, idx, _, _, _ = ops.moe_forward(xb, bf(layer.gate.gate_proj.weight), bias0.float(), bf(layer.experts.gate_up_proj),
                                      bf(layer.experts.down_proj), layer.experts.radial_theta.detach().float(), k,
                                      want_routing=True)
    _, idx_new, _, _, _ = ops.moe_forward(xb, bf(layer.gate.gate_proj.weight), layer.gate.bias.detach().float(),
                                          bf(layer.experts.gate_up_proj), bf(layer.experts.down_proj),
                                          layer.experts.radial_theta.detach().float(), k, want_routing=True)
    assert not torch.equal(idx, idx_new)                            # the moved bias would select differently
    ref = O.moe_backward(xb.cpu(), bf(layer.gate.gate_proj.weight).cpu(), bf(layer.experts.gate_up_proj).cpu(),
                         bf(layer.experts.down_proj).cpu(), layer.experts.radial_theta.detach().float().cpu(),
                         idx.cpu().numpy(), bf(d).cpu().reshape(T, H))
    assert x.grad.dtype == torch.float32 and layer.experts.gate_up_proj.grad.dtype == torch.float32
    assert _rel(x.grad.reshape(T, H), ref["x"]) <= TOL
    assert _rel(layer.gate.gate_proj.weight.grad, ref["w_router"]) <= TOL
    assert _rel(layer.experts.gate_up_proj.grad, ref["w_gate_up"]) <= TOL
    assert _rel(layer.experts.down_proj.grad, ref["w_down"]) <= TOL
    assert _rel(layer.experts.radial_theta.grad, ref["theta"]) <= TOL


@pytest.mark.parametrize("seam", ["layer", "ffn"])
def test_layer_under_activation_checkpointing(seam):
    """The reference wraps its decoder layers in torch.utils.checkpoint (src/modeling/layers.py:97-98): the block runs
    once in the forward pass and once more when the backward pass recomputes it.  Gradients equal those of the plain
    run bit for bit (the kernels are deterministic), and the balancing state stays consistent."""
    from torch.utils.checkpoint import checkpoint
    H = 256
    layer = _layer(H=H, I=128, E=16, k=4, bias_update_threshold=10 ** 9).train()   # no bias step inside this test
    nw = (1 + 0.1 * torch.randn(H, device=DEV)).requires_grad_(True)
    g = torch.Generator().manual_seed(9)
    x0 = torch.randn(2, 60, H, generator=g).to(torch.bfloat16).to(DEV)
    d = torch.randn(2, 60, H, generator=g).to(torch.bfloat16).to(DEV)
    fn = (lambda t: layer(t)) if seam == "layer" else (lambda t: layer.ffn_forward(t, nw, 1e-6))

    def run(wrapped):
        layer.zero_grad()
        nw.grad = None
        layer.accumulated_tpe.zero_()
        layer._fwd_step = 0
        x = x0.clone().requires_grad_(True)
        out = checkpoint(fn, x, use_reentrant=False) if wrapped else fn(x)
        out.backward(d)
        torch.cuda.synchronize()
        grads = {n: p.grad.clone() for n, p in layer.named_parameters() if p.grad is not None}
        return (out.detach(), x.grad.clone(), grads, (None if nw.grad is None else nw.grad.clone()),
                (layer._fwd_step, float(layer.accumulated_tpe.sum())))

    out_a, gx_a, gp_a, gn_a, steps_a = run(False)
    out_b, gx_b, gp_b, gn_b, steps_b = run(True)
    assert torch.equal(out_a, out_b) and torch.equal(gx_a, gx_b)
    assert sorted(gp_a) == sorted(gp_b) and all(torch.equal(gp_a[n], gp_b[n]) for n in gp_a)
    if seam == "ffn":
        assert gn_a is not None and torch.equal(gn_a, gn_b)
    # The balancing state counts calls of the layer.  The recomputation calls it again, but torch stops it as soon as
    # the last tensor the backward pass needs exists again, which may be before the balancing step: one or two steps,
    # each with all of the forward's 120 * 4 selections.
    assert steps_a == (1, 120.0 * 4) and steps_b in ((1, 120.0 * 4), (2, 2 * 120.0 * 4))
