"""Edge cases of the C ABI on the GPU: empty input, misaligned operands, k at its maximum, a workspace that
is too small.  Every call goes through ctypes or the thin ops wrappers."""
import ctypes

import numpy as np
import pytest
import torch

from bibo_amd import _lib as L
from bibo_amd import ops
from oracle import bibo_moe_oracle as O
from conftest import rel_err

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
P = lambda t: ctypes.c_void_p(t.data_ptr())


def _operands(T, H, E, I, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(T + H)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.05).to(dtype).to(DEV)
    return (torch.randn(T, H, generator=g).to(dtype).to(DEV), mk(E, H), torch.zeros(E, device=DEV), mk(E, 2 * I, H),
            mk(E, H, I), torch.zeros(E, device=DEV))


def test_zero_tokens_through_every_composite_entry_point():
    x, wr, b, gu, dn, th = _operands(0, 256, 16, 128)
    out, idx, w, counts, _ = ops.moe_forward(x, wr, b, gu, dn, th, 4, want_routing=True, want_counts=True)
    torch.cuda.synchronize()
    assert out.shape == (0, 256) and idx.shape == (0, 4) and w.shape == (0, 4)
    assert counts.cpu().tolist() == [0] * 16
    out2, counts2 = ops.experts_fwd(x, idx, w, gu, dn, th, want_counts=True)
    out3, *_ = ops.ffn_forward(x, torch.ones(256, device=DEV), 1e-6, wr, b, gu, dn, th, 4)
    c, off, ps, pt = ops.permute(idx, 16)
    torch.cuda.synchronize()
    assert out2.shape == (0, 256) and out3.shape == (0, 256) and counts2.cpu().tolist() == [0] * 16
    assert c.cpu().tolist() == [0] * 16 and off.cpu().tolist() == [0] * 17 and ps.numel() == 0 and pt.numel() == 0


def test_misaligned_operands_are_reported_not_launched():
    """The MFMA / fused / streaming kernels move 16 bytes at a time; a pointer that is not 16-byte aligned is an
    argument error found on the host (the generic kernels take any alignment)."""
    T, H, E, k, I = 300, 256, 64, 6, 128
    x, wr, b, gu, dn, th = _operands(T, H, E, I)
    raw = torch.empty(x.numel() + 8, dtype=torch.bfloat16, device=DEV)
    x_off = raw[1:1 + x.numel()].view(T, H)                      # 2 bytes past an aligned address
    x_off.copy_(x)
    sh = L.Shape(T, H, E, k, I, L.DTYPE_BF16)
    ws = ops.workspace(DEV, ops.workspace_bytes(T, H, E, k, I, L.DTYPE_BF16))
    out = torch.empty(T, H, dtype=torch.bfloat16, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream(DEV).cuda_stream)
    lib = L.lib()
    def forward(xp, algo):
        return lib.bibo_moe_forward(P(xp), P(wr), P(b), P(gu), P(dn), P(th), ctypes.byref(sh), L.NORM_SUM, algo, P(out),
                                    None, None, None, None, P(ws), ws.numel(), stream)
    assert forward(x_off, L.ALGO_FUSED) == -5 and forward(x_off, L.ALGO_MFMA) == -5
    assert b"align" in lib.bibo_moe_strerror(-5)
    assert forward(x_off, L.ALGO_GENERIC) == 0
    # the workspace is carved at multiples of 256 bytes and accessed 16 bytes at a time: its base must be aligned
    big = torch.empty(ws.numel() + 256, dtype=torch.uint8, device=DEV)
    for off in (2, 16, 128):
        rc = lib.bibo_moe_forward(P(x), P(wr), P(b), P(gu), P(dn), P(th), ctypes.byref(sh), L.NORM_SUM, L.ALGO_AUTO, P(out),
                                  None, None, None, None, ctypes.c_void_p(big.data_ptr() + off), ws.numel(), stream)
        assert rc == -5
    idx = torch.zeros(T, k, dtype=torch.int32, device=DEV)
    w = torch.ones(T, k, dtype=torch.float32, device=DEV)
    assert lib.bibo_moe_experts_fwd(P(x), P(idx), P(w), P(gu), P(dn), P(th), ctypes.byref(sh), L.ALGO_AUTO, P(out), None,
                                    ctypes.c_void_p(big.data_ptr() + 16), ws.numel(), stream) == -5
    assert lib.bibo_moe_ffn_forward(P(x), P(th.new_ones(H)), ctypes.c_float(1e-6), None, P(wr), P(b), P(gu), P(dn), P(th),
                                    ctypes.byref(sh), L.NORM_SUM, L.ALGO_AUTO, P(out), None, None, None,
                                    ctypes.c_void_p(big.data_ptr() + 16), big.numel() - 16, stream) == -5
    gen = out.clone()
    assert forward(x, L.ALGO_FUSED) == 0
    torch.cuda.synchronize()
    assert rel_err(out.cpu(), gen.cpu().float()) <= 1e-2          # same answer from the aligned copy


def test_top_k_at_its_maximum_and_few_experts():
    for E, k, T in ((8, 8, 200), (9, 8, 513), (64, 8, 300)):
        p = O.make_inputs(T=T, H=256, E=E, k=k, I=128, bias="uniform", theta="normal", seed=E + T)
        dev = DEV
        out, idx, w, counts, logits = ops.moe_forward(p["x"].to(dev), p["w_router"].to(dev), p["bias"].to(dev),
                                                      p["w_gate_up"].to(dev), p["w_down"].to(dev), p["theta"].to(dev), k,
                                                      want_routing=True, want_counts=True, want_logits=True)
        torch.cuda.synchronize()
        ref, oi, ow = O.moe_forward(p["x"], p["w_router"], p["bias"], p["w_gate_up"], p["w_down"], p["theta"], k,
                                    logits=logits.cpu().numpy())
        assert np.array_equal(idx.cpu().numpy(), oi) and np.array_equal(w.cpu().numpy(), ow)
        assert counts.sum().item() == T * k
        assert rel_err(out.cpu(), ref) <= 2e-2


def test_workspace_too_small_is_an_error():
    T, H, E, k, I = 64, 256, 16, 2, 128
    x, wr, b, gu, dn, th = _operands(T, H, E, I)
    sh = L.Shape(T, H, E, k, I, L.DTYPE_BF16)
    need = ops.workspace_bytes(T, H, E, k, I, L.DTYPE_BF16)
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=DEV)
    lib = L.lib()
    rc = lib.bibo_moe_forward(P(x), P(wr), P(b), P(gu), P(dn), P(th), ctypes.byref(sh), L.NORM_SUM, L.ALGO_AUTO, P(out),
                              None, None, None, None, P(ws), need - 1, None)
    assert rc == -4
    rc = lib.bibo_moe_ffn_forward(P(x), P(th.new_ones(H)), ctypes.c_float(1e-6), None, P(wr), P(b), P(gu), P(dn), P(th),
                                  ctypes.byref(sh), L.NORM_SUM, L.ALGO_AUTO, P(out), None, None, None, P(ws), need, None)
    assert rc == -4                                                # the seam needs room for the normalised rows too
