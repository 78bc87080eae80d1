"""Kernel 1 (router) against the oracle on the GPU, through the C ABI.

Protocol: the kernel's own fp32 logits are checked against an fp32/fp64 GEMM, then the oracle
recomputes scores, selection and weights FROM THOSE LOGITS and indices must match bit for bit."""
import numpy as np
import pytest
import torch

from bibo_amd import ops
from oracle import bibo_moe_oracle as O

pytestmark = pytest.mark.gpu


def _run(x, wr, bias, k, norm="sum", gap=False):
    dev = torch.device("cuda:0")
    idx, w, logits, g = ops.router_fwd(x.to(dev), wr.to(dev), bias.to(dev), k, norm, want_logits=True, want_gap=gap)
    torch.cuda.synchronize()
    return idx.cpu().numpy(), w.cpu().numpy(), logits.cpu().numpy(), (g.cpu().numpy() if gap else None)


def _check(x, wr, bias, k, norm="sum", gap=False):
    idx, w, logits, g = _run(x, wr, bias, k, norm, gap)
    ref_logits = (x.double() @ wr.double().t()).numpy()
    assert np.max(np.abs(logits - ref_logits)) <= 1e-5 * max(1.0, np.abs(ref_logits).max())
    oi, ow, scores = O.route_from_logits(logits, bias.numpy(), k, norm)
    assert np.array_equal(idx, oi), f"{(idx != oi).any(1).sum()} tokens routed differently"
    if norm == "softmax":
        assert np.allclose(w, ow, rtol=1e-6, atol=1e-7)
    else:
        assert np.array_equal(w, ow), f"max |dw| = {np.abs(w - ow).max()}"
    if gap:
        assert np.array_equal(g, O.boundary_gap(scores, k))
    return idx, w, logits


@pytest.mark.parametrize("name", ["c1", "c3"])
def test_router_matches_oracle_on_named_workloads(name):
    p = O.make_inputs(**O.CONFIGS[name])
    _check(p["x"], p["w_router"], p["bias"], p["k"], gap=True)


@pytest.mark.parametrize("T", [1, 15, 16, 17, 1000])
def test_router_ragged_token_counts(T):
    p = O.make_inputs(T=T, H=768, E=64, k=6, I=8, bias="uniform", seed=T)
    _check(p["x"], p["w_router"] * 8, p["bias"], 6)


@pytest.mark.parametrize("T,H,E,k", [(8192, 768, 64, 6), (8209, 256, 64, 6), (8200, 128, 33, 3)])
def test_router_large_token_counts_use_the_32_token_tile(T, H, E, k):
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, H, generator=g).bfloat16()
    wr = (torch.randn(E, H, generator=g) * 0.1).bfloat16()
    bias = torch.rand(E, generator=g) * 0.02 - 0.01
    _check(x, wr, bias, k, gap=True)


@pytest.mark.parametrize("E,k,H,dtype", [(8, 2, 64, torch.bfloat16), (22, 2, 64, torch.float32),
                                         (4, 1, 40, torch.bfloat16), (5, 5, 64, torch.float32),
                                         (64, 8, 100, torch.bfloat16), (33, 3, 96, torch.bfloat16)])
def test_router_small_and_odd_shapes(E, k, H, dtype):
    g = torch.Generator().manual_seed(E * 100 + k)
    x = (torch.randn(77, H, generator=g) * 3).to(dtype)
    wr = (torch.randn(E, H, generator=g) * 0.3).to(dtype)
    bias = torch.rand(E, generator=g) * 0.1 - 0.05
    for norm in ("sum", "softmax", False):
        idx, w, _ = _check(x, wr, bias, k, norm, gap=(k < E))
        assert idx.min() >= 0 and idx.max() < E and (w > 0).all()
        if norm and k > 1:
            assert np.allclose(w.sum(-1), 1.0, atol=1e-6)        # tests/test_moe.py:138-145 of the reference


def test_exact_ties_go_to_the_lowest_expert():
    E, H, k = 64, 128, 6
    g = torch.Generator().manual_seed(9)
    wr = (torch.randn(E, H, generator=g) * 0.05).bfloat16()
    wr[40] = wr[3]; wr[41] = wr[3]; wr[63] = wr[10]            # identical rows -> identical logits
    x = torch.randn(256, H, generator=g).bfloat16()
    x[0] = 0                                                    # every logit 0: experts 0..5 win
    idx, w, logits = _check(x, wr, torch.zeros(E), k)
    assert idx[0].tolist() == [0, 1, 2, 3, 4, 5]
    assert np.array_equal(logits[:, 3], logits[:, 40]) and np.array_equal(logits[:, 3], logits[:, 41])
    # whenever the later duplicates are chosen, the earliest one is chosen too
    has = lambda e: (idx == e).any(1)
    assert (~has(41) | has(40)).all() and (~has(40) | has(3)).all() and (~has(63) | has(10)).all()
    # a tie manufactured by the bias: experts 7 and 20 duplicates, bias lifts both equally
    b = torch.zeros(E); b[7] = 0.5; b[20] = 0.5
    wr2 = wr.clone(); wr2[20] = wr2[7]
    _check(x, wr2, b, k)


def test_bias_moves_selection_but_not_weights():
    p = O.make_inputs(T=128, H=256, E=16, k=4, I=8, seed=3)
    bias = torch.zeros(16); bias[0] = 5.0
    idx, w, logits = _check(p["x"], p["w_router"], bias, 4, norm=False)
    assert (idx == 0).any(1).all() and w.max() <= 1.0
    scores = O.sigmoid32(logits)
    assert np.array_equal(w, np.take_along_axis(scores, idx.astype(np.int64), 1))


def test_sigmoid_bits_over_a_wide_logit_range():
    """Scores are returned as raw weights (norm=False, k=E): every expert's score must equal the
    canonical sigmoid of the kernel's logit bit for bit, including saturated values."""
    E, H = 8, 32
    x = torch.zeros(64, H)
    x[:, 0] = torch.linspace(-55, 55, 64)
    wr = torch.zeros(E, H); wr[:, 0] = torch.tensor([1.0, 0.5, 0.25, -1.0, 0.125, 0.01, 1.5, -0.3])
    idx, w, logits, _ = _run(x, wr, torch.zeros(E), E, norm=False)
    assert np.array_equal(idx, np.tile(np.arange(E, dtype=np.int32), (64, 1)))
    assert np.array_equal(w, O.sigmoid32(logits))


def test_full_size_prefill_routing_properties():
    """T=16384 skewed workload (hot experts via +2.0 bias): oracle parity at full size (routing is cheap
    on the CPU) plus the structural properties."""
    p = O.make_inputs(**O.CONFIGS["c4"])
    idx, w, _ = _check(p["x"], p["w_router"], p["bias"], 6)
    assert (idx[:, :4] == np.arange(4)).all(), "bias +2 on a (0,1) score makes the four hot experts win every token"
    assert (np.diff(idx, axis=1) > 0).all()
    assert np.allclose(w.sum(-1), 1.0, atol=1e-6)
