"""The composite entry points at the sizes bench.py times: bibo_moe_forward and bibo_moe_ffn_forward on the full
prefill workloads c2 (T=8192) and c4 (T=16384, four hot experts), where the router runs 32 tokens per workgroup,
leaves its per-workgroup histograms and the permutation consumes them.  Routing, counts and the permutation the
counts imply are bit-exact against the oracle evaluated on the kernel's own fp32 logits; the output is checked
against the fp32 oracle on a token sample (a token's output depends only on its own row and routing).
Reference: BiBoMoELayer.forward, src/modeling/ffn/moe.py:157-183; caller src/modeling/layers.py:57-67."""
import numpy as np
import pytest
import torch

from bibo_amd import ops
from oracle import bibo_moe_oracle as O
from conftest import rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
BF16_TOL = 2e-2


def _dev(p):
    return {n: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for n, v in p.items()}


def _check_forward(p, sample_tokens=256, seed=0):
    """moe_forward with every optional output; returns (out, idx) on the host."""
    d = _dev(p)
    T, k, E = p["x"].shape[0], p["k"], p["w_router"].shape[0]
    out, idx, w, counts, logits = ops.moe_forward(d["x"], d["w_router"], d["bias"], d["w_gate_up"], d["w_down"],
                                                  d["theta"], k, want_routing=True, want_counts=True, want_logits=True)
    torch.cuda.synchronize()
    idx, w, counts, logits, out = idx.cpu().numpy(), w.cpu().numpy(), counts.cpu().numpy(), logits.cpu().numpy(), out.cpu()
    # logits against an fp64 GEMM; routing from the kernel's own logits, bit for bit
    ref_lg = p["x"].double() @ p["w_router"].double().t()
    assert np.abs(logits - ref_lg.numpy()).max() < 1e-5 * max(1.0, float(ref_lg.abs().max()))
    oi, ow, _ = O.route_from_logits(logits, p["bias"].numpy(), k)
    assert np.array_equal(idx, oi), "expert indices differ from the oracle"
    assert np.array_equal(w, ow), "routing weights differ from the oracle"
    assert np.array_equal(counts, O.permute(oi, E)[0]), "per-expert counts differ from the oracle"
    sample = np.random.default_rng(seed).choice(T, min(T, sample_tokens), replace=False)
    ref = O.experts_forward(p["x"][sample], oi[sample], ow[sample], p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(out[sample], ref) <= BF16_TOL
    assert torch.isfinite(out.float()).all()
    return out, oi, ow, logits


@pytest.mark.parametrize("name", ["c2", "c4"])
def test_layer_forward_at_full_prefill_size(name):
    p = O.make_inputs(**O.CONFIGS[name])
    assert ops.select_algo(p["x"].shape[0], p["x"].shape[1], 64, 6, p["w_down"].shape[2]) == "fused"
    out, oi, ow, _ = _check_forward(p)
    # the composite call and the experts seam fed with the same routing agree bit for bit
    d = _dev(p)
    seam, _ = ops.experts_fwd(d["x"], torch.from_numpy(oi).to(DEV), torch.from_numpy(ow).to(DEV), d["w_gate_up"],
                              d["w_down"], d["theta"])
    torch.cuda.synchronize()
    assert torch.equal(seam.cpu(), out)
    if name == "c4":                                   # +2.0 on a sigmoid score: the four hot experts win every token
        assert (np.bincount(oi.reshape(-1), minlength=64)[:4] == p["x"].shape[0]).all()


def test_layer_forward_with_idle_experts_at_full_size():
    """T=8192 with eight experts that never win (bias -2 on a score in (0,1)): empty segments in the permutation."""
    p = O.make_inputs(**O.CONFIGS["c2"])
    p["bias"][5:61:7] = -2.0
    out, oi, _, _ = _check_forward(p, seed=1)
    cnt = np.bincount(oi.reshape(-1), minlength=64)
    assert (cnt[5:61:7] == 0).all() and (cnt > 0).sum() == 56


@pytest.mark.parametrize("T", [8193, 8192 + 33])
def test_layer_forward_with_a_ragged_last_router_tile(T):
    """One and 33 tokens past a multiple of the router's 32-token tile (and of the permutation's 128-token chunk)."""
    p = O.make_inputs(**{**O.CONFIGS["c2"], "T": T})
    out, _, _, logits = _check_forward(p, seed=2)
    tail = slice(T - 40, T)                            # the last tokens, whatever the sample picked
    ref, _, _ = O.moe_forward(p["x"][tail], p["w_router"], p["bias"], p["w_gate_up"], p["w_down"], p["theta"], 6,
                              logits=logits[tail])
    assert rel_err(out[tail], ref) <= BF16_TOL


@pytest.mark.parametrize("name", ["c2", "c4"])
def test_ffn_forward_at_full_prefill_size(name):
    """out = h + moe(rmsnorm(h)) in one call at full size: routing bit-exact on the normalised rows the norm kernel
    produces, output within tolerance on a token sample."""
    p = O.make_inputs(**O.CONFIGS[name])
    T, H = p["x"].shape
    nw = torch.rand(H, generator=torch.Generator().manual_seed(7)) + 0.5
    h = (p["x"].float() * 3).bfloat16()
    d = _dev(p)
    out, idx, w, counts = ops.ffn_forward(h.to(DEV), nw.to(DEV), 1e-6, d["w_router"], d["bias"], d["w_gate_up"],
                                          d["w_down"], d["theta"], 6, want_routing=True, want_counts=True)
    xn_k = ops.rmsnorm_fwd(h.to(DEV), nw.to(DEV), 1e-6)
    _, _, logits, _ = ops.router_fwd(xn_k, d["w_router"], d["bias"], 6, want_logits=True)
    torch.cuda.synchronize()
    oi, ow, _ = O.route_from_logits(logits.cpu().numpy(), p["bias"].numpy(), 6)
    assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(w.cpu().numpy(), ow)
    assert np.array_equal(counts.cpu().numpy(), np.bincount(oi.reshape(-1), minlength=64))
    sample = np.random.default_rng(3).choice(T, 256, replace=False)
    xs = xn_k.cpu()[sample]
    y = O.experts_forward(xs, oi[sample], ow[sample], p["w_gate_up"], p["w_down"], p["theta"])
    ref = h[sample].float() + y.float()
    assert rel_err(out.cpu()[sample], ref) <= BF16_TOL
    # the block's own contribution, which the residual would otherwise hide
    blk = out.cpu()[sample].float() - h[sample].float()
    assert (blk - y.float()).abs().max() <= 2.0 ** -7 * ref.abs().max() + BF16_TOL * y.abs().max()


@pytest.mark.parametrize("algo", ["auto", "stream"])
def test_every_slot_on_one_expert_with_repeats(algo):
    """A caller's indices may name one expert in every slot of every token (the reference's loop accepts that,
    moe.py:46-71): 2560 rows on expert 9, more than the row list of a streaming workgroup holds.  `auto` does not
    pick the streaming kernels for such a call and `stream` is refused before anything is launched."""
    T, k, H, I, E = 320, 8, 256, 256, 64
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, theta="normal", seed=320)
    idx = np.full((T, k), 9, np.int32)
    w = np.random.default_rng(4).random((T, k)).astype(np.float32)
    assert ops.select_algo(T, H, E, k, I) == "fused"           # 40 slots per expert on average: past the streaming range
    args = (p["x"].to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV), p["w_gate_up"].to(DEV),
            p["w_down"].to(DEV), p["theta"].to(DEV))
    if algo == "stream":
        with pytest.raises(RuntimeError, match="does not support"):
            ops.experts_fwd(*args, algo="stream")
        return
    ops.workspace(DEV, 64 << 20).fill_(0x7f)
    out, counts = ops.experts_fwd(*args, algo="auto", want_counts=True)
    torch.cuda.synchronize()
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(out.cpu(), ref) <= BF16_TOL
    assert counts.cpu().numpy()[9] == T * k and counts.cpu().numpy().sum() == T * k


def test_streaming_kernels_take_repeats_that_fit_their_row_list():
    """Repeated experts within the row list's capacity still run the streaming kernels (T*k <= 2048)."""
    T, k, H, I, E = 200, 8, 256, 256, 64
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, theta="normal", seed=200)
    idx = np.full((T, k), 3, np.int32)
    idx[:, 4:] = 40
    w = np.random.default_rng(5).random((T, k)).astype(np.float32)
    out, _ = ops.experts_fwd(p["x"].to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV),
                             p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), algo="stream")
    torch.cuda.synchronize()
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(out.cpu(), ref) <= BF16_TOL


def test_half_a_million_tokens_cross_the_4_gib_offsets():
    """T = 524288 at the prefill shape: 3.1 M routed rows, so the slot rows, the pre-activations and the per-slot input
    gradients each hold more than 2^31 elements (4.8 GB) and every row offset near the end needs 64 bits.  A token's
    output and input gradient depend on its own row, its routing and the weights alone, so chunks of the big call equal
    the same tokens run by themselves bit for bit (first, middle and last chunk); the weight gradients of the big call
    equal the sum over all 64 chunks' to bf16 rounding."""
    T, H, E, k, I, CH = 524288, 768, 64, 6, 384, 8192
    p = O.make_inputs(T=64, H=H, E=E, k=k, I=I, bias="uniform", theta="normal", seed=77)
    wts = [p[n].to(DEV) for n in ("w_router", "bias", "w_gate_up", "w_down", "theta")]
    g = torch.Generator(device=DEV).manual_seed(78)
    x = torch.randn(T, H, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    d = torch.randn(T, H, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    assert T * k * H > 2 ** 31
    try:
        out, idx, w, _, _ = ops.moe_forward(x, *wts, k, want_routing=True)
        grads = ops.moe_backward(x, d, *wts, k)
        torch.cuda.synchronize()
        assert all(bool(torch.isfinite(t.float()).all()) for t in (out,) + tuple(grads[:5]))
        sums = [torch.zeros_like(t, dtype=torch.float64) for t in grads[1:5]]
        for a in range(0, T, CH):
            gc = ops.moe_backward(x[a:a + CH], d[a:a + CH], *wts, k)
            for s_, t_ in zip(sums, gc[1:5]):
                s_ += t_.double()
            if a in (0, T // 2, T - CH):
                oc, ic, wc, _, _ = ops.moe_forward(x[a:a + CH], *wts, k, want_routing=True)
                assert torch.equal(ic, idx[a:a + CH]) and torch.equal(wc, w[a:a + CH]), f"routing of chunk {a}"
                assert torch.equal(oc, out[a:a + CH]), f"output of chunk {a}"
                assert torch.equal(gc[0], grads[0][a:a + CH]), f"input gradient of chunk {a}"
        for name, s_, t_ in zip(("d_w_router", "d_w_gate_up", "d_w_down", "d_theta"), sums, grads[1:5]):
            err = ((t_.double() - s_).abs().max() / s_.abs().max()).item()
            assert err <= BF16_TOL, f"{name}: big call against the sum over chunks, rel err {err:.3e}"
        # the last tokens against the fp32 oracle
        tail = slice(T - 64, T)
        oi, ow = idx[tail].cpu().numpy(), w[tail].cpu().numpy()
        ref = O.experts_forward(x[tail].cpu(), oi, ow, p["w_gate_up"], p["w_down"], p["theta"])
        assert rel_err(out[tail].cpu(), ref) <= BF16_TOL
    finally:
        ops._workspaces.clear()                      # 20 GB of workspace: not kept for the tests that follow
        del x, d
        torch.cuda.empty_cache()


@pytest.mark.parametrize("T", [32768, 32768 + 40, 70000])
def test_block_sums_of_the_router_histograms_from_1024_on(T):
    """From 1024 router histograms on (32768 tokens) the permutation adds them up in two levels: counts and the
    permutation against the oracle, bit for bit, and the ends of the output against the same tokens run alone."""
    H, E, k, I, CH = 256, 64, 6, 128, 4096
    p = O.make_inputs(T=64, H=H, E=E, k=k, I=I, bias="uniform", theta="normal", seed=91)
    wts = [p[n].to(DEV) for n in ("w_router", "bias", "w_gate_up", "w_down", "theta")]
    g = torch.Generator(device=DEV).manual_seed(T)
    x = torch.randn(T, H, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    out, idx, w, counts, _ = ops.moe_forward(x, *wts, k, want_routing=True, want_counts=True)
    torch.cuda.synchronize()
    idx_np = idx.cpu().numpy()
    oc, _, oslot, otoken = O.permute(idx_np, E)
    assert np.array_equal(counts.cpu().numpy(), oc)
    # the permutation itself, through the stage entry point fed with the same indices (hist_kernel's histograms)
    c2_, _, ps, pt = ops.permute(idx, E)
    assert np.array_equal(c2_.cpu().numpy(), oc) and np.array_equal(ps.cpu().numpy(), oslot)
    assert np.array_equal(pt.cpu().numpy(), otoken)
    for a in (0, (T // 2) & ~127, T - CH):
        oc_, ic_, wc_, _, _ = ops.moe_forward(x[a:a + CH], *wts, k, want_routing=True)
        assert torch.equal(ic_, idx[a:a + CH]) and torch.equal(wc_, w[a:a + CH])
        assert torch.equal(oc_, out[a:a + CH]), f"output of chunk {a}"
