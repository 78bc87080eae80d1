"""Pins for the CPU oracle.  The reference stores no golden vectors for this path
(its tests are closed forms and invariants: tests/test_moe.py, ablate/common/test_eager_radial.py),
so each oracle function is pinned by library routines, special cases, invariants and tiny brute force
written independently of the oracle's own expressions."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import bibo_moe_oracle as O


def _ulp_diff(a, b):
    return np.abs(a.view(np.int32).astype(np.int64) - b.view(np.int32).astype(np.int64))


# ------------------------------------------------------------------ sigmoid
def test_canonical_exp_matches_libm():
    y = np.linspace(-200, 200, 200001)
    assert np.max(np.abs(O.exp64_canonical(y) - np.exp(y)) / np.exp(y)) < 1e-15


def test_canonical_sigmoid_is_the_correctly_rounded_one():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * 4,
                        np.linspace(-110, 110, 50001).astype(np.float32)])
    s = O.sigmoid32(x)
    # Python's math.exp on doubles, one rounding to float32: an independent evaluation
    sample = x[::97]
    ref = np.array([1.0 / (1.0 + math.exp(-float(v))) for v in sample]).astype(np.float32)
    assert np.array_equal(s[::97], ref)
    # the reference's torch.sigmoid (router.py:31) is within 2 ulp wherever the result is normal
    m = np.abs(x) <= 80
    assert _ulp_diff(s[m], torch.sigmoid(torch.from_numpy(x[m])).numpy()).max() <= 2


def test_sigmoid_special_values_and_monotonicity():
    x = np.array([0.0, -0.0, np.inf, -np.inf, 1e38, -1e38, 200.0, -200.0], dtype=np.float32)
    assert O.sigmoid32(x).tolist() == [0.5, 0.5, 1.0, 0.0, 1.0, 0.0, 1.0, 0.0]
    xs = np.sort(np.random.default_rng(1).standard_normal(100000).astype(np.float32) * 6)
    assert (np.diff(O.sigmoid32(xs)) >= 0).all()
    a = np.linspace(-30, 30, 10001).astype(np.float32)      # s(x) + s(-x) = 1
    assert np.max(np.abs(O.sigmoid32(a).astype(np.float64) + O.sigmoid32(-a) - 1.0)) < 1.2e-7


# ------------------------------------------------------------------ router
def _brute_topk(sel_row, k):
    order = sorted(range(len(sel_row)), key=lambda e: (-float(sel_row[e]), e))
    return sorted(order[:k])


@pytest.mark.parametrize("E,k", [(64, 6), (8, 2), (22, 2), (4, 1), (5, 5)])
def test_selection_matches_brute_force_and_torch_topk(E, k):
    rng = np.random.default_rng(E * 10 + k)
    logits = (rng.standard_normal((257, E)) * 2).astype(np.float32)
    bias = (rng.uniform(-0.05, 0.05, E)).astype(np.float32)
    idx, w, scores = O.route_from_logits(logits, bias, k)
    sel = scores + bias[None]
    for t in range(logits.shape[0]):
        assert idx[t].tolist() == _brute_topk(sel[t], k)
    # torch.topk (router.py:39) picks the same SET whenever the boundary is not tied
    tk = torch.topk(torch.from_numpy(sel), k, dim=-1, sorted=False).indices.sort(-1).values.numpy()
    assert np.array_equal(tk, idx)
    # reference invariants (tests/test_moe.py:138-145): fp32, positive, unit mass, indices in range
    assert w.dtype == np.float32 and idx.dtype == np.int32
    assert (w > 0).all() and idx.min() >= 0 and idx.max() < E
    if k > 1:
        assert np.allclose(w.sum(-1), 1.0, atol=1e-6)


def test_ties_go_to_the_lowest_expert_index():
    E, k = 8, 3
    logits = np.zeros((4, E), dtype=np.float32)          # all scores equal -> experts 0,1,2
    logits[1, 5] = 1.0                                    # one winner then lowest indices
    logits[2, [6, 7]] = 1.0
    logits[3, :] = [0.5, 0.7, 0.7, 0.7, 0.7, 0.2, 0.9, 0.7]
    idx, w, _ = O.route_from_logits(logits, np.zeros(E, np.float32), k)
    assert idx.tolist() == [[0, 1, 2], [0, 1, 5], [0, 6, 7], [1, 2, 6]]
    # a tie created by the bias is broken the same way
    b = np.zeros(E, np.float32); b[4] = 0.25
    lg = np.zeros((1, E), np.float32)
    idx, w, sc = O.route_from_logits(lg, b, 2)
    assert idx.tolist() == [[0, 4]]


def test_bias_moves_selection_but_never_weights():
    """tests/test_moe.py:177-185, plus: weights are the unbiased scores of the chosen experts."""
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((64, 16)).astype(np.float32)
    bias = np.zeros(16, np.float32); bias[0] = 5.0
    idx, w, scores = O.route_from_logits(logits, bias, 4, norm=False)
    assert (idx == 0).any(axis=1).all()
    assert np.array_equal(w, np.take_along_axis(scores, idx.astype(np.int64), 1))
    assert w.max() <= 1.0
    _, wn, _ = O.route_from_logits(logits, bias, 4)
    assert np.allclose(wn, w / w.sum(-1, keepdims=True), rtol=1e-6)
    _, ws, _ = O.route_from_logits(logits, bias, 4, norm="softmax")
    assert np.allclose(ws, torch.softmax(torch.from_numpy(w), -1).numpy())


def test_router_logits_and_gap():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(33, 48, generator=g).bfloat16()
    wr = (torch.randn(10, 48, generator=g) * 0.1).bfloat16()
    lg = O.router_logits(x, wr)
    assert lg.dtype == np.float32 and lg.shape == (33, 10)
    ref = np.einsum("th,eh->te", x.double().numpy(), wr.double().numpy())   # experts are the ROW dim
    assert np.max(np.abs(lg - ref)) < 1e-5
    _, _, scores = O.route_from_logits(lg, np.zeros(10, np.float32), 3)
    tk = torch.from_numpy(scores).topk(4, dim=-1).values                     # router.py:35-36
    assert np.allclose(O.boundary_gap(scores, 3), (tk[:, 2] - tk[:, 3]).numpy())


# ------------------------------------------------------------------ permutation
@pytest.mark.parametrize("T,E,k", [(1, 4, 1), (37, 8, 2), (300, 64, 6), (64, 64, 6)])
def test_permutation_matches_brute_force(T, E, k):
    rng = np.random.default_rng(T)
    idx = np.stack([np.sort(rng.choice(E, k, replace=False)) for _ in range(T)]).astype(np.int32)
    counts, offsets, perm_slot, perm_token = O.permute(idx, E)
    flat = idx.reshape(-1)
    brute = sorted(range(T * k), key=lambda s: (int(flat[s]), s // k, s % k))
    assert perm_slot.tolist() == brute
    assert perm_token.tolist() == [s // k for s in brute]
    assert counts.tolist() == [int((flat == e).sum()) for e in range(E)]
    assert offsets[0] == 0 and offsets[-1] == T * k and (np.diff(offsets) == counts).all()
    assert sorted(perm_slot.tolist()) == list(range(T * k))
    assert (np.bincount(perm_token, minlength=T) == k).all()        # every token exactly k times


def test_permutation_with_repeated_experts_and_empty_experts():
    idx = np.array([[2, 2], [0, 2], [2, 0]], dtype=np.int32)     # legal at the experts seam
    counts, offsets, perm_slot, perm_token = O.permute(idx, 4)
    assert counts.tolist() == [2, 0, 4, 0]
    assert offsets.tolist() == [0, 2, 2, 6, 6]
    assert perm_slot.tolist() == [2, 5, 0, 1, 3, 4]
    with pytest.raises(ValueError):
        O.permute(np.array([[4]], dtype=np.int32), 4)


# ------------------------------------------------------------------ experts
def _tiny(E=4, H=16, I=8, T=5, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    wgu = torch.randn(E, 2 * I, H, generator=g, dtype=torch.float64) * 0.3
    wd = torch.randn(E, H, I, generator=g, dtype=torch.float64) * 0.3
    return x, wgu, wd


def _scalar_expert(xrow, wgu_e, wd_e, theta):
    """Pure-Python scalar evaluation of one expert on one row, written from the definition
    r^p * SiLU(g/r) with r = rms(gate), p = sigmoid(theta) (tests/test_moe.py:36-37)."""
    two_i, H = len(wgu_e), len(xrow)
    I = two_i // 2
    gu = [sum(wgu_e[j][h] * xrow[h] for h in range(H)) for j in range(two_i)]
    gate, up = gu[:I], gu[I:]
    r = math.sqrt(sum(v * v for v in gate) / I + 1e-6)
    p = 1.0 / (1.0 + math.exp(-theta))
    hid = [(r ** p) * (v / r) / (1.0 + math.exp(-v / r)) * u for v, u in zip(gate, up)]
    return [sum(wd_e[o][i] * hid[i] for i in range(I)) for o in range(len(wd_e))]


def test_experts_match_scalar_brute_force():
    E, H, I, T, k = 4, 16, 8, 5, 2
    x, wgu, wd = _tiny(E, H, I, T)
    theta = torch.tensor([-2.0, 0.0, 1.5, 3.0], dtype=torch.float64)   # p = .12/.50/.82/.95
    idx = np.array([[0, 1], [1, 3], [2, 3], [0, 2], [0, 3]], dtype=np.int32)
    w = torch.tensor(np.random.default_rng(0).uniform(0.1, 1, (T, k)))
    out = O.experts_forward(x, idx, w, wgu, wd, theta, dtype=torch.float64)
    for t in range(T):
        acc = [0.0] * H
        for j in range(k):
            e = int(idx[t, j])
            y = _scalar_expert(x[t].tolist(), wgu[e].tolist(), wd[e].tolist(), float(theta[e]))
            acc = [a + float(w[t, j]) * v for a, v in zip(acc, y)]
        assert np.allclose(out[t].numpy(), acc, rtol=1e-10, atol=1e-12)


def test_radial_special_cases():
    x, wgu, wd = _tiny(seed=1)
    g = (x @ wgu[0].t())[:, :8]
    # p -> 0 is NormSiLU: SiLU(g * rsqrt(mean g^2 + eps)) (tests/test_moe.py:66-78)
    a0 = O.radial_normsilu(g, torch.tensor(-40.0))
    assert torch.allclose(a0, F.silu(g * torch.rsqrt(g.square().mean(-1, keepdim=True) + 1e-6)), rtol=1e-9)
    # p -> 1: r * SiLU(g/r) = g * sigmoid(g/r)
    r = (g.square().mean(-1, keepdim=True) + 1e-6).sqrt()
    assert torch.allclose(O.radial_normsilu(g, torch.tensor(40.0)), g * torch.sigmoid(g / r), rtol=1e-9)
    # degree-p homogeneity: act(a*g) = a^p act(g) for a > 0 (eps negligible) -- fails for r^theta
    for theta in (-2.0, 0.0, 1.5):
        p = 1 / (1 + math.exp(-theta))
        lhs = O.radial_normsilu(3.0 * g, torch.tensor(theta))
        assert torch.allclose(lhs, (3.0 ** p) * O.radial_normsilu(g, torch.tensor(theta)), rtol=1e-5)
    # the mean is over the LAST dim only: rows are independent
    assert torch.allclose(O.radial_normsilu(g[:2], torch.tensor(0.3)), O.radial_normsilu(g, torch.tensor(0.3))[:2])


def test_activation_variants_of_the_training_harness():
    """The two activations the reference's harness can switch its external kernel to
    (ablate/common/patches.py:53-69): p = tanh(theta) and plain SiLU."""
    x, wgu, wd = _tiny(seed=2)
    g = (x @ wgu[0].t())[:, :8]
    # tanh exponent: degree-p homogeneity with p = tanh(theta), which a NEGATIVE theta makes negative
    # (a sigmoid exponent, or a dropped sign, fails: 3^p would exceed 1)
    for theta in (-1.5, -0.3, 0.0, 0.9):
        pexp = math.tanh(theta)
        lhs = O.radial_normsilu(3.0 * g, torch.tensor(theta), "tanh")
        assert torch.allclose(lhs, (3.0 ** pexp) * O.radial_normsilu(g, torch.tensor(theta), "tanh"), rtol=1e-5)
    assert (O.radial_normsilu(3.0 * g, torch.tensor(-1.5), "tanh").abs().max()
            < O.radial_normsilu(g, torch.tensor(-1.5), "tanh").abs().max())         # gain r^p shrinks with r for p < 0
    # theta = 0 gives p = 0 under tanh (NormSiLU) but p = 1/2 under sigmoid
    r = (g.square().mean(-1, keepdim=True) + 1e-6).sqrt()
    assert torch.allclose(O.radial_normsilu(g, torch.tensor(0.0), "tanh"), F.silu(g / r), rtol=1e-9)
    assert torch.allclose(O.radial_normsilu(g, torch.tensor(0.0)), F.silu(g / r) * r.sqrt(), rtol=1e-9)
    # large |theta|: tanh -> +/-1
    assert torch.allclose(O.radial_normsilu(g, torch.tensor(20.0), "tanh"), g * torch.sigmoid(g / r), rtol=1e-9)
    assert torch.allclose(O.radial_normsilu(g, torch.tensor(-20.0), "tanh"), F.silu(g / r) / r, rtol=1e-9)
    # plain SwiGLU: the library routine, rows independent of theta and of the other columns
    assert torch.equal(O.radial_normsilu(g, torch.tensor(0.7), "silu"), F.silu(g))
    idx = np.zeros((x.shape[0], 1), np.int64); w = np.ones((x.shape[0], 1), np.float32)
    out = O.experts_forward(x, idx, w, wgu, wd, torch.full((wgu.shape[0],), 0.7), dtype=torch.float64, act="silu")
    gate, up = (x @ wgu[0].t()).chunk(2, -1)
    assert torch.allclose(out, (F.silu(gate) * up) @ wd[0].t(), rtol=1e-9)


def test_gate_is_the_first_half_of_gate_up_rows():
    """moe.py:85 chunk(2): rows 0..I-1 gate, I..2I-1 up.  Zeroing the up half must zero the output;
    zeroing the gate half must too (SiLU(0) = 0)."""
    x, wgu, wd = _tiny(E=1, seed=2)
    idx = np.zeros((5, 1), np.int32); w = torch.ones(5, 1, dtype=torch.float64); th = torch.zeros(1)
    a = wgu.clone(); a[:, 8:, :] = 0
    assert O.experts_forward(x, idx, w, a, wd, th, dtype=torch.float64).abs().max() == 0
    b = wgu.clone(); b[:, :8, :] = 0
    assert O.experts_forward(x, idx, w, b, wd, th, dtype=torch.float64).abs().max() == 0
    # swapping the halves changes the result (the activation is on the gate only)
    c = torch.cat([wgu[:, 8:], wgu[:, :8]], 1)
    o1 = O.experts_forward(x, idx, w, wgu, wd, th, dtype=torch.float64)
    assert (O.experts_forward(x, idx, w, c, wd, th, dtype=torch.float64) - o1).abs().max() > 1e-3


def test_combine_is_linear_in_the_weights_and_order_free():
    x, wgu, wd = _tiny(seed=3)
    th = torch.tensor([0.1, -0.3, 0.7, 0.0], dtype=torch.float64)
    one = lambda e: O.experts_forward(x, np.full((5, 1), e, np.int32), torch.ones(5, 1, dtype=torch.float64),
                                      wgu, wd, th, dtype=torch.float64)
    idx = np.tile(np.array([[1, 3]], np.int32), (5, 1))
    w = torch.tensor([[0.3, 0.7]], dtype=torch.float64).repeat(5, 1)
    both = O.experts_forward(x, idx, w, wgu, wd, th, dtype=torch.float64)
    assert torch.allclose(both, 0.3 * one(1) + 0.7 * one(3), rtol=1e-12)
    swapped = O.experts_forward(x, idx[:, ::-1].copy(), w.flip(-1), wgu, wd, th, dtype=torch.float64)
    assert torch.allclose(both, swapped, rtol=1e-12)


def test_fp32_oracle_tracks_fp64_and_eager_loop_tracks_oracle():
    p = O.make_inputs(T=96, H=64, E=8, k=2, I=32, bias="uniform", theta="normal", seed=7)
    out32, idx, w = O.moe_forward(**p)
    out64 = O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"], dtype=torch.float64)
    assert ((out32.double() - out64).abs().max() / out64.abs().max()) < 1e-5     # test_eager_radial.py:61
    # the timed bf16 eager loop agrees with the fp32 oracle at the bf16 tolerance (test_act_silu.py:65-66)
    eager = O.eager_loop_forward(**p)
    assert eager.dtype == torch.bfloat16
    assert ((eager.double() - out64).abs().max() / out64.abs().max()) < 2e-2
    # fp32 eager loop == fp32 oracle to rounding (same routing: no ties in this draw)
    pf = {k_: (v.float() if isinstance(v, torch.Tensor) else v) for k_, v in p.items()}
    assert ((O.eager_loop_forward(**pf).double() - out64).abs().max() / out64.abs().max()) < 1e-5


def test_workload_table_matches_the_named_shapes():
    c = O.CONFIGS
    assert (c["c2"]["T"], c["c2"]["H"], c["c2"]["I"]) == (8192, 768, 384)
    assert (c["c3"]["T"], c["c3"]["H"], c["c3"]["I"]) == (64, 1024, 512)
    p = O.make_inputs(**{**c["c4"], "T": 32})
    assert (p["bias"][:4] == 2.0).all() and p["bias"][4:].abs().max() <= 0.01
    assert p["x"].dtype == torch.bfloat16 and p["bias"].dtype == torch.float32


# ------------------------------------------------------------------ caller seam: RMSNorm + residual
def test_rmsnorm_matches_library_routine_and_closed_form():
    """norm.py:19-24.  Pins: torch.nn.functional.rms_norm (an independent library routine) in fp32; a scalar
    pure-Python evaluation; scale invariance rmsnorm(a*x) == rmsnorm(x) when eps is negligible; a row of
    equal magnitudes maps to sign(x) * weight."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 48, generator=g) * 3
    wgt = torch.rand(48, generator=g) + 0.5
    got = O.rmsnorm(x, wgt, 1e-6)
    lib = torch.nn.functional.rms_norm(x, (48,), wgt, 1e-6)
    assert torch.allclose(got, lib, rtol=1e-6, atol=1e-6)
    r = 2
    ms = sum(float(v) ** 2 for v in x[r]) / 48
    want = [float(wgt[c]) * float(x[r, c]) / math.sqrt(ms + 1e-6) for c in range(48)]
    assert np.allclose(got[r].numpy(), want, rtol=1e-5, atol=1e-6)
    assert torch.allclose(O.rmsnorm(7.0 * x, wgt, 1e-12), O.rmsnorm(x, wgt, 1e-12), rtol=1e-5, atol=1e-6)
    s = torch.tensor([[2.0, -2.0, 2.0, -2.0]])
    assert torch.allclose(O.rmsnorm(s, torch.tensor([1.0, 2.0, 3.0, 4.0]), 0.0), torch.tensor([[1.0, -2.0, 3.0, -4.0]]))


def test_rmsnorm_rounds_the_normalised_row_before_the_weight_in_bf16():
    """norm.py:24 multiplies the weight with the row ALREADY cast back to the input dtype."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 64, generator=g).bfloat16()
    wgt = (torch.rand(64, generator=g) + 0.5)
    xf = x.float()
    xn = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    assert torch.equal(O.rmsnorm(x, wgt, 1e-6), (wgt * xn.float()).bfloat16())
    assert O.rmsnorm(x, wgt, 1e-6).dtype == torch.bfloat16


def test_ffn_forward_is_residual_plus_block_of_the_normalised_input():
    p = O.make_inputs(T=24, H=32, E=8, k=2, I=16, bias="uniform", theta="normal", seed=12, dtype=torch.float32)
    g = torch.Generator().manual_seed(6)
    wgt = torch.rand(32, generator=g) + 0.5
    out, xn, idx, w = O.ffn_forward(p["x"], wgt, 1e-6, p["w_router"], p["bias"], p["w_gate_up"], p["w_down"], p["theta"], 2)
    y, idx2, w2 = O.moe_forward(xn, p["w_router"], p["bias"], p["w_gate_up"], p["w_down"], p["theta"], 2)
    assert np.array_equal(idx, idx2) and np.array_equal(w, w2)
    assert torch.allclose(out, p["x"] + y, rtol=0, atol=0)
    # a zero block (w_down = 0) leaves the residual untouched
    out0, *_ = O.ffn_forward(p["x"], wgt, 1e-6, p["w_router"], p["bias"], p["w_gate_up"], torch.zeros_like(p["w_down"]),
                             p["theta"], 2)
    assert torch.equal(out0, p["x"])


# ------------------------------------------------------------------ +/-Identity specials and the shared expert
def test_identity_specials_add_and_subtract_the_weighted_input():
    """moe.py:95-99.  A token routed only to a +Identity expert comes back as w*x, to a -Identity expert as -w*x;
    mixed with a GLU expert the contributions add; a +/- pair with equal weights cancels."""
    p = O.make_inputs(T=6, H=16, E=4, k=2, I=8, theta="normal", seed=2, dtype=torch.float32)
    x, gu, dn, th = p["x"], p["w_gate_up"], p["w_down"], p["theta"]          # 4 GLU experts; ids 4,5 = +I, 6 = -I
    w = np.full((6, 2), 0.25, np.float32)
    w[:, 1] = 0.5
    only_pos = O.experts_forward(x, np.tile([[4, 5]], (6, 1)), w, gu, dn, th, n_pos=2, n_neg=1)
    assert torch.allclose(only_pos, 0.75 * x, atol=1e-6)
    only_neg = O.experts_forward(x, np.tile([[6, 6]], (6, 1)), w, gu, dn, th, n_pos=2, n_neg=1)
    assert torch.allclose(only_neg, -0.75 * x, atol=1e-6)
    cancel = O.experts_forward(x, np.tile([[5, 6]], (6, 1)), np.full((6, 2), 0.3, np.float32), gu, dn, th, n_pos=2, n_neg=1)
    assert torch.allclose(cancel, torch.zeros_like(x), atol=1e-6)
    glu_only = O.experts_forward(x, np.tile([[1, 1]], (6, 1)), np.stack([w[:, 0], 0 * w[:, 1]], 1), gu, dn, th)
    mixed = O.experts_forward(x, np.tile([[1, 6]], (6, 1)), w, gu, dn, th, n_pos=2, n_neg=1)
    assert torch.allclose(mixed, glu_only - 0.5 * x, atol=1e-5)


def test_shared_mlp_is_a_swiglu():
    g = torch.Generator().manual_seed(3)
    x, wg, wu, wd = (torch.randn(5, 12, generator=g), torch.randn(20, 12, generator=g), torch.randn(20, 12, generator=g),
                     torch.randn(12, 20, generator=g))
    got = O.shared_mlp(x, wg, wu, wd)
    a = x.double() @ wg.double().t()
    want = ((a / (1 + torch.exp(-a))) * (x.double() @ wu.double().t())) @ wd.double().t()
    assert torch.allclose(got.double(), want, rtol=1e-4, atol=1e-4)


# --------------------------------------------------------------------------------------
# backward pass of the oracle: pinned by central differences and by hand-derived closed forms
# --------------------------------------------------------------------------------------
def _bwd_case(seed=11, T=24, H=32, E=6, k=3, I=16, act="radial", norm="sum"):
    p = O.make_inputs(T=T, H=H, E=E, k=k, I=I, bias="uniform", theta="normal", seed=seed, dtype=torch.float64)
    g = torch.Generator().manual_seed(seed + 1)
    p["x"] = torch.randn(T, H, generator=g, dtype=torch.float64)
    p["w_gate_up"] = torch.randn(E, 2 * I, H, generator=g, dtype=torch.float64) * 0.3
    p["w_down"] = torch.randn(E, H, I, generator=g, dtype=torch.float64) * 0.3
    p["w_router"] = torch.randn(E, H, generator=g, dtype=torch.float64) * 0.2
    logits = (p["x"] @ p["w_router"].t()).float().numpy()
    idx, _, _ = O.route_from_logits(logits, p["bias"].float().numpy(), k, norm)
    d_out = torch.randn(T, H, generator=g, dtype=torch.float64)
    return p, idx, d_out


def _loss(p, idx, d_out, norm, act):
    w = O.route_weights(p["x"] @ p["w_router"].t(), idx, norm)
    return float((O.experts_forward(p["x"], idx, w, p["w_gate_up"], p["w_down"], p["theta"], dtype=torch.float64, act=act)
                  * d_out).sum())


@pytest.mark.parametrize("act,norm", [("radial", "sum"), ("tanh", "softmax"), ("silu", False)])
def test_backward_matches_central_differences(act, norm):
    """The gradient of every operand agrees with (L(v + h d) - L(v - h d)) / 2h along random directions d: pins the
    autograd oracle against a dropped path (router, theta, norm) without retyping any derivative."""
    p, idx, d_out = _bwd_case(act=act, norm=norm)
    grads = O.moe_backward(p["x"], p["w_router"], p["w_gate_up"], p["w_down"], p["theta"], idx, d_out, norm=norm, act=act)
    g = torch.Generator().manual_seed(5)
    for name in ("x", "w_router", "w_gate_up", "w_down", "theta"):
        if act == "silu" and name == "theta":
            assert grads[name] is None or float(grads[name].abs().max()) == 0.0   # plain SiLU has no radial gain
            continue
        d = torch.randn(p[name].shape, generator=g, dtype=torch.float64)
        h = 1e-6
        base = p[name].clone()
        p[name] = base + h * d
        lp = _loss(p, idx, d_out, norm, act)
        p[name] = base - h * d
        lm = _loss(p, idx, d_out, norm, act)
        p[name] = base
        fd, an = (lp - lm) / (2 * h), float((grads[name] * d).sum())
        assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), (name, fd, an)


def test_backward_with_identity_experts_closed_form_and_differences():
    """+/-Identity experts (moe.py:95-99): out[t] += sign w[t,j] x[t] for a slot routed to one.  Closed form for the
    part of the gradients that comes from those slots alone: dw[t,j] = sign <d_out[t], x[t]>, and the x gradient of
    that term is sign w[t,j] d_out[t]; the whole gradient agrees with central differences."""
    T, H, Eg, k, I = 20, 16, 3, 3, 8
    n_pos, n_neg = 1, 1
    E = Eg + n_pos + n_neg
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=g, dtype=torch.float64)
    wr = torch.randn(E, H, generator=g, dtype=torch.float64) * 0.3
    gu = torch.randn(Eg, 2 * I, H, generator=g, dtype=torch.float64) * 0.3
    dn = torch.randn(Eg, H, I, generator=g, dtype=torch.float64) * 0.3
    th = torch.randn(Eg, generator=g, dtype=torch.float64)
    d_out = torch.randn(T, H, generator=g, dtype=torch.float64)
    idx, _, _ = O.route_from_logits((x @ wr.t()).float().numpy(), np.zeros(E, np.float32), k, "sum")
    assert (idx >= Eg).any() and (idx == Eg).any() and (idx == Eg + 1).any()
    grads = O.moe_backward(x, wr, gu, dn, th, idx, d_out, norm="sum", n_pos=n_pos, n_neg=n_neg)
    dot = (d_out * x).sum(-1)
    for t in range(T):
        for j in range(k):
            if idx[t, j] >= Eg:
                sign = 1.0 if idx[t, j] < Eg + n_pos else -1.0
                assert abs(float(grads["w"][t, j]) - sign * float(dot[t])) <= 1e-12 * max(1.0, abs(float(dot[t])))

    def loss(xv, wrv):
        w = O.route_weights(xv @ wrv.t(), idx, "sum")
        return float((O.experts_forward(xv, idx, w, gu, dn, th, dtype=torch.float64, n_pos=n_pos, n_neg=n_neg) * d_out).sum())
    for name, base in (("x", x), ("w_router", wr)):
        d = torch.randn(base.shape, generator=g, dtype=torch.float64)
        h = 1e-6
        lp = loss(x + h * d, wr) if name == "x" else loss(x, wr + h * d)
        lm = loss(x - h * d, wr) if name == "x" else loss(x, wr - h * d)
        fd, an = (lp - lm) / (2 * h), float((grads[name] * d).sum())
        assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), (name, fd, an)


def test_radial_backward_closed_form():
    """h = r^p SiLU(g/r) u, r = sqrt(mean(g^2) + eps), p = sigmoid(theta).  With a = SiLU(z), a' = s (1 + z (1 - s)),
    s = sigmoid(z), z = g / r and q = dh u (all per element):
      du = dh r^p a;   dg = q r^(p-1) a' + g / (I r) * sum_i q_i (p r^(p-1) a_i - r^(p-2) a'_i g_i);
      dtheta = p (1 - p) ln(r) sum_i q_i r^p a_i."""
    g0 = torch.Generator().manual_seed(2)
    I = 24
    gate = torch.randn(5, I, generator=g0, dtype=torch.float64, requires_grad=True)
    up = torch.randn(5, I, generator=g0, dtype=torch.float64, requires_grad=True)
    theta = torch.tensor(0.7, dtype=torch.float64, requires_grad=True)
    dh = torch.randn(5, I, generator=g0, dtype=torch.float64)
    (O.radial_normsilu(gate, theta) * up * dh).sum().backward()
    with torch.no_grad():
        r = torch.sqrt(gate.square().mean(-1, keepdim=True) + O.NORMSILU_EPS)
        p = torch.sigmoid(theta)
        z = gate / r
        s = torch.sigmoid(z)
        a, ad = z * s, s * (1 + z * (1 - s))
        q = dh * up
        du = dh * r.pow(p) * a
        inner = (q * (p * r.pow(p - 1) * a - r.pow(p - 2) * ad * gate)).sum(-1, keepdim=True)
        dg = q * r.pow(p - 1) * ad + gate / (I * r) * inner
        dth = (p * (1 - p) * torch.log(r) * (q * r.pow(p) * a).sum(-1, keepdim=True)).sum()
    assert torch.allclose(up.grad, du, rtol=1e-12, atol=1e-14)
    assert torch.allclose(gate.grad, dg, rtol=1e-10, atol=1e-13)
    assert abs(float(theta.grad) - float(dth)) <= 1e-12 * max(1.0, abs(float(dth)))


@pytest.mark.parametrize("norm", ["sum", "softmax", False])
def test_route_weight_backward_closed_form(norm):
    """sum: w = s / (S + eps), S = sum of the selected scores: ds_j = (dw_j - sum_i dw_i w_i) / (S + eps);
    softmax over the selected scores: ds_j = w_j (dw_j - sum_i dw_i w_i); none: ds = dw; dlogit = ds s (1 - s)."""
    g0 = torch.Generator().manual_seed(4)
    logits = torch.randn(7, 10, generator=g0, dtype=torch.float64, requires_grad=True)
    idx = np.stack([np.sort(np.random.default_rng(i).choice(10, 4, replace=False)) for i in range(7)])
    dw = torch.randn(7, 4, generator=g0, dtype=torch.float64)
    w = O.route_weights(logits, idx, norm)
    (w * dw).sum().backward()
    with torch.no_grad():
        s = torch.sigmoid(logits).gather(-1, torch.from_numpy(idx))
        dot = (dw * w).sum(-1, keepdim=True)
        if norm == "sum":
            ds = (dw - dot) / (s.sum(-1, keepdim=True) + O.SUM_NORM_EPS)
        elif norm == "softmax":
            ds = w * (dw - dot)
        else:
            ds = dw
        dl = torch.zeros_like(logits).scatter_(-1, torch.from_numpy(idx), ds * s * (1 - s))
    assert torch.allclose(logits.grad, dl, rtol=1e-12, atol=1e-15)
