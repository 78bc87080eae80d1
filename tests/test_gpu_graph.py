"""The entry points under HIP graph capture: the library launches kernels on the caller's stream and nothing else
(no allocation, no synchronisation, no memset nodes), so a captured call can be replayed.  Every replay is checked bit
for bit against the same call made eagerly, with new inputs copied into the captured buffers and eager work and
synchronisations between the replays."""
import pytest
import torch

from bibo_amd import ops
from oracle import bibo_moe_oracle as O

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

NAMES = ("w_router", "bias", "w_gate_up", "w_down", "theta")


def _inputs(seed, **shape):
    p = O.make_inputs(bias="uniform", theta="normal", seed=seed, **shape)
    g = torch.Generator().manual_seed(seed + 100)
    d = torch.randn(p["x"].shape, generator=g).to(torch.bfloat16)
    return p, d


@pytest.mark.parametrize("shape", [dict(T=700, H=256, E=64, k=6, I=128),      # permutation + fused tile kernel
                                   dict(T=17, H=1024, E=64, k=6, I=512),      # weight-streaming kernels
                                   dict(T=300, H=128, E=8, k=2, I=128)])
def test_forward_and_backward_replay_like_eager_calls(shape):
    k = shape["k"]
    p0, d0 = _inputs(1, **shape)
    wts = [p0[n].to(DEV) for n in NAMES]
    x_s, d_s = p0["x"].to(DEV), d0.to(DEV)

    norm_w = (1.0 + 0.1 * torch.randn(shape["H"], generator=torch.Generator().manual_seed(9))).to(DEV)
    keeps = ops.train_state_bytes(shape["T"], shape["H"], shape["E"], k, shape["I"], torch.bfloat16) is not None

    def call(x, d):
        out, idx, w, counts, _ = ops.moe_forward(x, *wts, k, want_routing=True, want_counts=True)
        res = (out, idx, w, counts) + tuple(ops.moe_backward(x, d, *wts, k, want_dw=True))
        if keeps:                                      # the training pair: forward that keeps its state, backward from it
            out_t, counts_t, state = ops.moe_forward_train(x, *wts, k, want_counts=True)
            w_router, _, w_gate_up, w_down, theta = wts
            res += (out_t, counts_t) + tuple(ops.moe_backward_saved(x, d, w_router, w_gate_up, w_down, theta, k, state,
                                                                    want_dw=True))
        # the caller's seam (norm + block + residual) and the experts alone with the routing handed over
        res += tuple(ops.ffn_forward(x, norm_w, 1e-6, *wts, k, want_routing=True, want_counts=True))
        res += (ops.experts_fwd(x, idx, w, wts[2], wts[3], wts[4])[0],)
        res += tuple(ops.experts_backward(x, d, idx, w, wts[2], wts[3], wts[4]))
        return res

    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream(DEV))
    with torch.cuda.stream(side):                      # warm-up on the capturing stream: its workspace exists afterwards
        call(x_s, d_s)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = call(x_s, d_s)
    torch.cuda.synchronize()
    for seed in (2, 3, 4, 2):
        p, d = _inputs(seed, **shape)
        x, dd = p["x"].to(DEV), d.to(DEV)
        eager = call(x, dd)                            # the program's own eager work between the replays
        torch.cuda.synchronize()
        x_s.copy_(x); d_s.copy_(dd)
        graph.replay()
        torch.cuda.synchronize()
        grads = ("d_x", "d_w_router", "d_w_gate_up", "d_w_down", "d_theta", "d_w")
        names = ("out", "idx", "w", "counts") + grads
        if keeps:
            names += ("out (train)", "counts (train)") + tuple(g + " (saved)" for g in grads)
        names += ("out (seam)", "idx (seam)", "w (seam)", "counts (seam)", "out (experts)", "d_x (experts)", "d_w (experts)",
                  "d_w_gate_up (experts)", "d_w_down (experts)", "d_theta (experts)")
        assert len(captured) == len(eager) == len(names)
        for name, a, b in zip(names, captured, eager):
            assert torch.equal(a, b), f"{name} of the replay differs from the eager call (seed {seed}, {shape})"


def test_static_entry_point_replays():
    shape = dict(T=64, H=1024, E=64, k=6, I=512)
    p0, _ = _inputs(5, **shape)
    wts = [p0[n].to(DEV) for n in NAMES]
    x_s = p0["x"].to(DEV)
    out_s = torch.empty_like(x_s)
    side = torch.cuda.Stream(device=DEV)
    side.wait_stream(torch.cuda.current_stream(DEV))
    with torch.cuda.stream(side):                      # first call on the device looks up the scratch array's address
        ops.moe_forward_static(x_s, *wts, 6, out_s)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.moe_forward_static(x_s, *wts, 6, out_s)
    torch.cuda.synchronize()
    for seed in (6, 7, 8):
        p, _ = _inputs(seed, **shape)
        x = p["x"].to(DEV)
        eager = ops.moe_forward(x, *wts, 6)[0]
        torch.cuda.synchronize()
        x_s.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_s, eager), f"replay differs from the eager call (seed {seed})"
