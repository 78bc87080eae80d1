"""Kernels 3 and 4 (grouped gate/up + Radial NormSiLU, grouped down + weighted combine) against the
oracle, for the generic and the MFMA kernel families, through the C ABI.

Tolerances: fp32 kernels vs the fp64 oracle 1e-5 (reference: ablate/common/test_eager_radial.py:61);
bf16 kernels vs the fp32 oracle max|d|/max|ref| <= 2e-2 (reference: ablate/common/test_act_silu.py:65-66)."""
import numpy as np
import pytest
import torch

from bibo_amd import ops
from oracle import bibo_moe_oracle as O
from conftest import rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
BF16_TOL = 2e-2


def _route(p):
    idx, w, _ = O.route_from_logits(O.router_logits(p["x"], p["w_router"]), p["bias"].numpy(), p["k"])
    return idx, w


def _gpu_experts(p, idx, w, algo):
    out, counts = ops.experts_fwd(p["x"].to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV),
                                  p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), algo=algo,
                                  want_counts=True)
    torch.cuda.synchronize()
    return out.cpu(), counts.cpu().numpy()


def _stages(p, idx, w, algo):
    """The two expert kernels called separately, returning the intermediate activations too."""
    E = p["w_gate_up"].shape[0]
    idx_d = torch.from_numpy(idx).to(DEV)
    counts, offsets, perm_slot, perm_token = ops.permute(idx_d, E)
    hidden = ops.gateup_fwd(p["x"].to(DEV), p["w_gate_up"].to(DEV), p["theta"].to(DEV), offsets, perm_token,
                            idx.shape[1], algo=algo)
    out = ops.down_combine_fwd(hidden, p["w_down"].to(DEV), torch.from_numpy(w).to(DEV), offsets, perm_slot,
                               idx.shape[0], algo=algo)
    torch.cuda.synchronize()
    return hidden.cpu(), out.cpu()


# ------------------------------------------------------------------ fp32 generic kernels vs fp64
def test_fp32_kernels_match_the_fp64_closed_form():
    """theta = -2/0/1.5/3 (p = .12/.50/.82/.95), every row through one expert with weight 1
    (tests/test_moe.py:35-50 of the reference)."""
    g = torch.Generator().manual_seed(0)
    E, H, I, N = 4, 64, 96, 40
    p = dict(x=torch.randn(N, H, generator=g), w_gate_up=torch.randn(E, 2 * I, H, generator=g) * 0.1,
             w_down=torch.randn(E, H, I, generator=g) * 0.1, theta=torch.tensor([-2.0, 0.0, 1.5, 3.0]))
    for e in range(E):
        idx = np.full((N, 1), e, dtype=np.int32)
        w = np.ones((N, 1), dtype=np.float32)
        out, counts = _gpu_experts(p, idx, w, "generic")
        ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"], dtype=torch.float64)
        assert rel_err(out, ref) < 1e-5
        assert counts.tolist() == [N if j == e else 0 for j in range(E)]


def test_fp32_kernels_at_p_zero_are_normsilu_and_theta_moves_the_output():
    g = torch.Generator().manual_seed(1)
    E, H, I, N = 4, 32, 64, 40                                   # ablate/common/test_eager_radial.py:34
    x = torch.randn(N, H, generator=g)
    wgu = torch.randn(E, 2 * I, H, generator=g) * 0.2
    wd = torch.randn(E, H, I, generator=g) * 0.2
    idx = np.zeros((N, 1), dtype=np.int32); w = np.ones((N, 1), dtype=np.float32)
    p = dict(x=x, w_gate_up=wgu, w_down=wd, theta=torch.tensor([-40.0, 0, 0, 0]))
    out, _ = _gpu_experts(p, idx, w, "generic")
    gate, up = (x.double() @ wgu[0].double().t()).chunk(2, -1)
    ns = torch.nn.functional.silu(gate * torch.rsqrt(gate.square().mean(-1, keepdim=True) + 1e-6)) * up
    assert (out.double() - ns @ wd[0].double().t()).abs().max() < 1e-4
    p2 = dict(p, theta=torch.tensor([-38.0, 0, 0, 0]))
    assert (_gpu_experts(p2, idx, w, "generic")[0] - out).abs().max() < 1e-5      # still the p=0 floor
    p3 = dict(p, theta=torch.tensor([2.0, 0, 0, 0]))
    assert (_gpu_experts(p3, idx, w, "generic")[0] - out).abs().max() > 1e-4      # theta is live


def test_fp32_combine_is_linear_and_handles_repeated_experts():
    g = torch.Generator().manual_seed(2)
    E, H, I, N = 6, 48, 40, 33
    p = dict(x=torch.randn(N, H, generator=g), w_gate_up=torch.randn(E, 2 * I, H, generator=g) * 0.1,
             w_down=torch.randn(E, H, I, generator=g) * 0.1, theta=torch.randn(E, generator=g))
    one = lambda e: _gpu_experts(p, np.full((N, 1), e, np.int32), np.ones((N, 1), np.float32), "generic")[0]
    idx = np.tile(np.array([[1, 4]], np.int32), (N, 1))
    w = np.tile(np.array([[0.3, 0.7]], np.float32), (N, 1))
    both, _ = _gpu_experts(p, idx, w, "generic")
    assert torch.allclose(both, 0.3 * one(1) + 0.7 * one(4), atol=1e-6)
    rep, _ = _gpu_experts(p, np.tile(np.array([[2, 2]], np.int32), (N, 1)), w, "generic")
    assert torch.allclose(rep, one(2), atol=1e-6)                 # 0.3*E2 + 0.7*E2


# ------------------------------------------------------------------ bf16 kernels vs fp32 oracle
@pytest.mark.parametrize("algo", ["generic", "mfma"])
@pytest.mark.parametrize("name", ["c1", "c3"])
def test_bf16_experts_match_oracle_on_named_workloads(name, algo):
    p = O.make_inputs(**O.CONFIGS[name])
    idx, w = _route(p)
    ref, ref_hidden = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"], return_hidden=True)
    hidden, out_staged = _stages(p, idx, w, algo)
    assert rel_err(hidden, ref_hidden) <= BF16_TOL
    out, counts = _gpu_experts(p, idx, w, algo)
    assert out.dtype == torch.bfloat16
    assert rel_err(out, ref) <= BF16_TOL
    assert torch.equal(out, out_staged), "composite and staged entry points must agree exactly"
    assert np.array_equal(counts, O.permute(idx, 64)[0])


@pytest.mark.parametrize("algo", ["generic", "mfma"])
@pytest.mark.parametrize("T,H,I,bias,theta", [(1024, 768, 384, "uniform", "normal"), (1024, 768, 384, "hot4", "normal"),
                                              (7, 1024, 512, "zero", "normal"), (333, 256, 128, "uniform", "normal"),
                                              (300, 384, 256, "uniform", "normal"),
                                              (130, 128, 256, "zero", "zero")])
def test_bf16_experts_reduced_prefill_and_ragged_shapes(T, H, I, bias, theta, algo):
    p = O.make_inputs(T=T, H=H, E=64, k=6, I=I, bias=bias, theta=theta, seed=T + H)
    idx, w = _route(p)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    out, _ = _gpu_experts(p, idx, w, algo)
    assert rel_err(out, ref) <= BF16_TOL


@pytest.mark.parametrize("T,H,I,k,theta", [(64, 1024, 512, 6, "zero"), (7, 1024, 512, 6, "normal"), (1, 768, 384, 6, "normal"),
                                           (200, 256, 128, 6, "normal"), (130, 128, 256, 2, "normal"),
                                           (40, 64, 64, 1, "normal"), (341, 512, 256, 6, "normal")])
def test_streaming_kernels_match_oracle(T, H, I, k, theta):
    """Weight-streaming (decode) kernels: few rows per expert, several 16-row passes, idle experts."""
    p = O.make_inputs(T=T, H=H, E=64, k=k, I=I, bias="uniform", theta=theta, seed=T + I)
    idx, w = _route(p)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    out, counts = _gpu_experts(p, idx, w, "stream")
    assert rel_err(out, ref) <= BF16_TOL
    assert np.array_equal(counts, O.permute(idx, 64)[0])
    gen, _ = _gpu_experts(p, idx, w, "generic")
    assert rel_err(out, gen) <= 1e-2


@pytest.mark.parametrize("T,H,I,E,k", [(69, 1536, 512, 64, 8), (36, 1024, 576, 4, 1), (56, 1088, 128, 64, 1),
                                       (61, 192, 1024, 8, 2), (5, 768, 64, 4, 2), (19, 64, 384, 64, 6),
                                       (77, 512, 1024, 64, 6), (39, 64, 512, 8, 6), (18, 1536, 1024, 8, 2),
                                       (15, 256, 576, 4, 4)])
def test_streaming_kernels_over_odd_shapes(T, H, I, E, k):
    """Rows that are not whole 256-element chunks, I above the fused-activation width (activation as its own launch),
    rows longer than the two register chunks (refilled every pass), few experts with many rows each."""
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, bias="uniform", theta="normal", seed=T * 7 + H)
    idx, w = _route(p)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    out, counts = _gpu_experts(p, idx, w, "stream")
    assert rel_err(out, ref) <= BF16_TOL
    assert np.array_equal(counts, O.permute(idx, E)[0])
    gen, _ = _gpu_experts(p, idx, w, "generic")
    assert rel_err(out, gen) <= 1e-2


def test_streaming_kernels_without_the_permutation_pass():
    """Without a counts request the composite call launches no permutation: the streaming kernels scan the
    routing indices themselves.  Same bits either way."""
    p = O.make_inputs(T=64, H=1024, E=64, k=6, I=512, bias="uniform", theta="normal", seed=99)
    idx, w = _route(p)
    args = (p["x"].to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV), p["w_gate_up"].to(DEV),
            p["w_down"].to(DEV), p["theta"].to(DEV))
    with_counts, _ = ops.experts_fwd(*args, algo="stream", want_counts=True)
    without, none = ops.experts_fwd(*args, algo="stream", want_counts=False)
    torch.cuda.synchronize()
    assert none is None and torch.equal(with_counts, without)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(without.cpu(), ref) <= BF16_TOL


@pytest.mark.parametrize("algo,T,H,I", [("generic", 40, 256, 128), ("mfma", 400, 256, 128), ("fused", 400, 256, 128),
                                        ("stream", 40, 256, 128)])
def test_slots_without_an_expert_contribute_nothing(algo, T, H, I):
    """Routing indices outside [0,E) (the reference never produces them; a caller might use them as padding) get
    no row, and the combine skips their slot."""
    p = O.make_inputs(T=T, H=H, E=64, k=6, I=I, bias="uniform", theta="normal", seed=T + 1)
    idx, w = _route(p)
    bad = idx.copy()
    bad[::3, 1] = 64
    bad[1::5, 4] = -1
    w0 = w.copy()
    w0[::3, 1] = 0.0
    w0[1::5, 4] = 0.0
    ref = O.experts_forward(p["x"], idx, w0, p["w_gate_up"], p["w_down"], p["theta"])   # same slots, weight zero
    # poison the workspace so that an unwritten slot row cannot pass by luck
    ops.workspace(DEV, 64 << 20).fill_(0x7f)
    out, counts = _gpu_experts(p, bad, w, algo)
    assert torch.isfinite(out.float()).all()
    assert rel_err(out, ref) <= BF16_TOL
    keep = (bad >= 0) & (bad < 64)
    assert np.array_equal(counts, np.bincount(bad[keep], minlength=64))


def test_streaming_kernels_with_a_crowded_expert():
    """Every row on two experts (far more than 16 rows each): the pass loop re-streams the weights."""
    p = O.make_inputs(T=90, H=512, E=64, k=2, I=256, theta="normal", seed=21)
    idx = np.tile(np.array([[3, 60]], np.int32), (90, 1))
    w = np.random.default_rng(2).random((90, 2)).astype(np.float32)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    out, _ = _gpu_experts(p, idx, w, "stream")
    assert rel_err(out, ref) <= BF16_TOL


def test_mfma_and_generic_families_agree():
    p = O.make_inputs(T=777, H=768, E=64, k=6, I=384, bias="uniform", theta="normal", seed=5)
    idx, w = _route(p)
    h_g, o_g = _stages(p, idx, w, "generic")
    h_m, o_m = _stages(p, idx, w, "mfma")
    assert rel_err(h_m, h_g) <= 1e-2 and rel_err(o_m, o_g) <= 1e-2


@pytest.mark.parametrize("T,H,I,k,bias", [(1024, 768, 384, 6, "uniform"), (1024, 768, 384, 6, "hot4"),
                                          (333, 256, 128, 6, "uniform"), (130, 128, 256, 6, "zero"),
                                          (777, 512, 256, 6, "uniform"), (515, 640, 384, 8, "uniform"),
                                          (600, 768, 256, 6, "uniform"), (400, 1024, 128, 6, "uniform"),
                                          (450, 640, 256, 6, "uniform"), (1, 768, 384, 6, "zero")])
def test_fused_kernel_matches_oracle_and_the_two_kernel_family(T, H, I, k, bias):
    """One launch for both GEMMs (activations never leave the CU): same operand rounding as the two MFMA
    kernels, another accumulation order in the down projection."""
    p = O.make_inputs(T=T, H=H, E=64, k=k, I=I, bias=bias, theta="normal", seed=T + H + I)
    idx, w = _route(p)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    out, counts = _gpu_experts(p, idx, w, "fused")
    assert rel_err(out, ref) <= BF16_TOL
    assert np.array_equal(counts, O.permute(idx, 64)[0])
    two, _ = _gpu_experts(p, idx, w, "mfma")
    assert rel_err(out, two) <= 1e-2


@pytest.mark.parametrize("H,I", [(768, 384), (512, 256), (256, 128)])
def test_fused_kernel_tiles_of_every_height(H, I):
    """The fused kernel has one code path per number of 32-row blocks a tile holds (1 to 4) and leaves the missing
    blocks out of all three phases: experts with 1, 31, 32, 33, 64, 65, 96, 97, 128, 129, 160 and 200 rows make last
    tiles of every height next to full ones, and every row still matches the oracle and the generic family."""
    counts = [1, 31, 32, 33, 64, 65, 96, 97, 128, 129, 160, 200, 0, 5]
    E, k = len(counts), 1
    T = sum(counts)
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, theta="normal", seed=H + I)
    rng = np.random.default_rng(H)
    idx = np.repeat(np.arange(E, dtype=np.int32), counts)
    rng.shuffle(idx)
    idx = idx.reshape(T, 1)
    w = rng.uniform(0.2, 1.0, size=(T, 1)).astype(np.float32)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    out, cnt = _gpu_experts(p, idx, w, "fused")
    assert np.array_equal(cnt, np.asarray(counts))
    assert rel_err(out, ref) <= BF16_TOL
    # row by row, so that a block left out by mistake (zeros or stale rows) cannot hide behind a large row elsewhere
    err = (out.double() - ref.double()).abs().amax(dim=1) / ref.double().abs().amax(dim=1).clamp_min(1e-30)
    assert float(err.max()) <= 2 * BF16_TOL, int(err.argmax())
    gen, _ = _gpu_experts(p, idx, w, "generic")
    assert rel_err(out, gen) <= 1e-2


def test_fused_stage_entry_points_compose_to_the_composite_call():
    """permute -> gateup_down -> combine through the stage ABI equals bibo_moe_experts_fwd(fused) bit for bit;
    the slot buffer holds w[t,j] * expert_j(x_t) (checked against the oracle per slot)."""
    p = O.make_inputs(T=300, H=768, E=64, k=6, I=384, bias="uniform", theta="normal", seed=77)
    idx, w = _route(p)
    idx_d, w_d = torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV)
    counts, offsets, perm_slot, perm_token = ops.permute(idx_d, 64)
    yw = ops.gateup_down_fwd(p["x"].to(DEV), p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), w_d,
                             offsets, perm_slot, perm_token)
    out = ops.combine_fwd(yw, 300, 6)
    torch.cuda.synchronize()
    ref_out, _ = _gpu_experts(p, idx, w, "fused")
    assert torch.equal(out.cpu(), ref_out)
    # one-hot routing weights isolate single slots in the oracle
    for t, j in [(0, 0), (123, 5), (299, 3)]:
        w1 = np.zeros_like(w[t:t + 1]); w1[0, j] = w[t, j]
        ref = O.experts_forward(p["x"][t:t + 1], idx[t:t + 1], w1, p["w_gate_up"], p["w_down"], p["theta"])
        assert rel_err(yw[t * 6 + j].cpu()[None], ref) <= BF16_TOL
    # fp32 slot rows through the same combine entry point
    y32 = yw.float()
    out32 = ops.combine_fwd(y32, 300, 6)
    torch.cuda.synchronize()
    assert torch.allclose(out32.cpu(), y32.view(300, 6, 768).cpu().sum(1), atol=1e-5, rtol=1e-5)


def test_mfma_with_empty_experts_and_one_hot_expert():
    """Only experts {5, 9} get rows (everything else empty), one of them with a ragged last tile."""
    g = torch.Generator().manual_seed(11)
    T, H, I, E = 201, 512, 256, 64
    p = O.make_inputs(T=T, H=H, E=E, k=2, I=I, theta="normal", seed=11)
    idx = np.tile(np.array([[5, 9]], np.int32), (T, 1))
    w = torch.rand(T, 2, generator=g).numpy().astype(np.float32)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    for algo in ("generic", "mfma", "fused"):
        out, counts = _gpu_experts(p, idx, w, algo)
        assert rel_err(out, ref) <= BF16_TOL
        assert counts[5] == T and counts[9] == T and counts.sum() == 2 * T


@pytest.mark.parametrize("algo", ["mfma", "fused"])
@pytest.mark.parametrize("name", ["c2", "c4"])
def test_full_size_prefill_properties(name, algo):
    """Full T: (a) oracle parity on a 256-token sample (a token's output depends only on its own row and
    routing); (b) doubling the routing weights doubles the bf16 output exactly; (c) permuting the tokens
    permutes the output rows exactly."""
    p = O.make_inputs(**O.CONFIGS[name])
    T = p["x"].shape[0]
    idx, w = _route(p)
    out, counts = _gpu_experts(p, idx, w, algo)
    assert counts.sum() == T * 6 and np.array_equal(counts, np.bincount(idx.reshape(-1), minlength=64))
    sample = np.random.default_rng(0).choice(T, 256, replace=False)
    ref = O.experts_forward(p["x"][sample], idx[sample], w[sample], p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(out[sample], ref) <= BF16_TOL
    out2, _ = _gpu_experts(p, idx, (2 * w).astype(np.float32), algo)
    assert torch.equal(out2.float(), 2 * out.float())
    perm = torch.randperm(T, generator=torch.Generator().manual_seed(1))
    pp = dict(p, x=p["x"][perm].contiguous())
    outp, _ = _gpu_experts(pp, idx[perm.numpy()], w[perm.numpy()], algo)
    assert torch.equal(outp, out[perm])


# ------------------------------------------------------------------ activation variants (act codes 10 and 0)
@pytest.mark.parametrize("act", ["tanh", "silu"])
@pytest.mark.parametrize("algo,T,H,I", [("generic", 60, 96, 40), ("mfma", 400, 256, 128), ("fused", 400, 256, 128),
                                        ("stream", 40, 256, 128), ("stream", 30, 256, 576), ("mfma", 300, 256, 512)])
def test_activation_variants_match_oracle(algo, T, H, I, act):
    """p = tanh(theta) (negative exponents shrink high-rms rows) and plain SwiGLU, the two activations the
    reference's harness can switch its external kernel to (ablate/common/patches.py:53-69), in every family."""
    E = 8 if algo == "generic" else 64
    p = O.make_inputs(T=T, H=H, E=E, k=2 if E == 8 else 6, I=I, bias="uniform", theta="normal", seed=T + I)
    p["theta"] = p["theta"] * 3 - 0.5                       # tanh(theta) spread over (-1, 1), mostly away from 0
    idx, w = _route(p)
    ref = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"], act=act)
    other = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"])
    assert rel_err(other, ref) > 0.05                        # the variants really differ from the default activation
    out, _ = ops.experts_fwd(p["x"].to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV),
                             p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), algo=algo, act=act)
    torch.cuda.synchronize()
    assert rel_err(out.cpu(), ref) <= BF16_TOL


def test_activation_variants_through_the_stage_entry_points():
    p = O.make_inputs(T=300, H=256, E=64, k=6, I=128, bias="uniform", theta="normal", seed=12)
    p["theta"] = p["theta"] * 3 - 0.5
    idx, w = _route(p)
    idx_d, w_d = torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV)
    counts, offsets, perm_slot, perm_token = ops.permute(idx_d, 64)
    for act in ("tanh", "silu"):
        ref, ref_hidden = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"], return_hidden=True,
                                            act=act)
        for algo in ("generic", "mfma"):
            hidden = ops.gateup_fwd(p["x"].to(DEV), p["w_gate_up"].to(DEV), p["theta"].to(DEV), offsets, perm_token, 6,
                                    algo=algo, act=act)
            torch.cuda.synchronize()
            assert rel_err(hidden.cpu(), ref_hidden) <= BF16_TOL
        yw = ops.gateup_down_fwd(p["x"].to(DEV), p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), w_d,
                                 offsets, perm_slot, perm_token, act=act)
        out = ops.combine_fwd(yw, 300, 6)
        torch.cuda.synchronize()
        assert rel_err(out.cpu(), ref) <= BF16_TOL


def test_fp32_tanh_exponent_matches_the_fp64_closed_form():
    g = torch.Generator().manual_seed(3)
    E, H, I, N = 4, 64, 96, 40
    p = dict(x=torch.randn(N, H, generator=g), w_gate_up=torch.randn(E, 2 * I, H, generator=g) * 0.1,
             w_down=torch.randn(E, H, I, generator=g) * 0.1, theta=torch.tensor([-2.0, -0.4, 0.0, 1.5]))
    for e in range(E):
        idx = np.full((N, 1), e, dtype=np.int32)
        w = np.ones((N, 1), dtype=np.float32)
        out, _ = ops.experts_fwd(p["x"].to(DEV), torch.from_numpy(idx).to(DEV), torch.from_numpy(w).to(DEV),
                                 p["w_gate_up"].to(DEV), p["w_down"].to(DEV), p["theta"].to(DEV), algo="generic", act="tanh")
        gate, up = (p["x"].double() @ p["w_gate_up"][e].double().t()).chunk(2, -1)
        r = (gate.square().mean(-1, keepdim=True) + 1e-6).sqrt()
        ref = (torch.nn.functional.silu(gate / r) * r.pow(np.tanh(float(p["theta"][e]))) * up) @ p["w_down"][e].double().t()
        assert rel_err(out.cpu(), ref) < 1e-5
