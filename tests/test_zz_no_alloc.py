"""bibo_moe_forward_static: the whole layer without a workspace argument and without any allocation, its
intermediates in the library's static per-GPU scratch array.  Checked against bibo_moe_forward (same kernels,
caller-owned workspace) bit for bit, on two calls in a row, the second with a smaller input, so stale contents of
the shared array from the first call cannot leak into the second."""
import ctypes

import numpy as np
import pytest
import torch

from bibo_amd import _lib as L
from bibo_amd import ops
from oracle import bibo_moe_oracle as O

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _both(p, algo="auto"):
    d = {n: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for n, v in p.items()}
    T, H = p["x"].shape
    k, E = p["k"], p["w_router"].shape[0]
    ref, ridx, rw, rcounts, rlogits = ops.moe_forward(d["x"], d["w_router"], d["bias"], d["w_gate_up"], d["w_down"],
                                                      d["theta"], k, algo=algo, want_routing=True, want_counts=True,
                                                      want_logits=True)
    out = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    idx = torch.full((T, k), -7, dtype=torch.int32, device=DEV)
    w = torch.full((T, k), float("nan"), dtype=torch.float32, device=DEV)
    counts = torch.full((E,), -7, dtype=torch.int32, device=DEV)
    logits = torch.full((T, E), float("nan"), dtype=torch.float32, device=DEV)
    ops.moe_forward_static(d["x"], d["w_router"], d["bias"], d["w_gate_up"], d["w_down"], d["theta"], k, out, algo=algo,
                           idx=idx, w=w, counts=counts, logits=logits)
    torch.cuda.synchronize()
    assert torch.equal(idx, ridx) and torch.equal(w, rw) and torch.equal(counts, rcounts) and torch.equal(logits, rlogits)
    assert torch.equal(out, ref)
    return out.cpu(), idx.cpu().numpy(), w.cpu().numpy()


def test_static_entry_point_equals_the_workspace_one_on_two_calls_in_a_row():
    big = O.make_inputs(**O.CONFIGS["c3"])                                     # decode workload: streaming kernels
    out, idx, w = _both(big)
    ref = O.experts_forward(big["x"], idx, w, big["w_gate_up"], big["w_down"], big["theta"])
    assert ((out.double() - ref.double()).abs().max() / ref.double().abs().max()).item() <= 2e-2
    small = O.make_inputs(T=17, H=1024, E=64, k=6, I=512, bias="uniform", theta="normal", seed=5)
    out, idx, w = _both(small)
    ref = O.experts_forward(small["x"], idx, w, small["w_gate_up"], small["w_down"], small["theta"])
    assert ((out.double() - ref.double()).abs().max() / ref.double().abs().max()).item() <= 2e-2
    # a tile-kernel shape (permutation + fused kernel + combine) through the same array, then a smaller one again
    mid = O.make_inputs(T=700, H=256, E=64, k=6, I=128, bias="uniform", theta="normal", seed=6)
    _both(mid)
    _both(O.make_inputs(T=5, H=256, E=64, k=6, I=128, bias="uniform", theta="normal", seed=7))


def test_static_entry_point_refuses_what_does_not_fit():
    T, H, E, k, I = 8192, 768, 64, 6, 384
    assert ops.workspace_bytes(T, H, E, k, I, L.DTYPE_BF16) > L.STATIC_SCRATCH_BYTES
    sh = L.Shape(T, H, E, k, I, L.DTYPE_BF16)
    lib = L.lib()
    rc = lib.bibo_moe_forward_static(None, None, None, None, None, None, ctypes.byref(sh), L.NORM_SUM, L.ALGO_AUTO, None,
                                     None, None, None, None, None)
    assert rc == -7 and b"static scratch" in lib.bibo_moe_strerror(rc)
    # the largest decode-size shapes fit
    assert ops.workspace_bytes(256, 1024, 64, 6, 512, L.DTYPE_BF16) <= L.STATIC_SCRATCH_BYTES
