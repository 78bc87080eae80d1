"""CPU oracle for the BiBo sparse-MoE feed-forward block.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the algorithm of the reference's MoE layer
(`src/modeling/ffn/router.py`, `src/modeling/ffn/moe.py` in IsNoobgrammer/BiBo).  It is the
checker the HIP kernels are compared against.  Nothing in the product package may import it:
only the test-suite, the smoke check and the benchmark's CPU-baseline leg do.

Conventions fixed here (the reference leaves them implementation-defined):

* top-k ties are broken by the LOWEST expert index, and the k indices of a token are emitted
  in ascending expert order (reference: `torch.topk(..., sorted=False)`, router.py:39);
* routed slots are ordered by (expert ascending, token ascending, slot ascending), i.e. a
  stable sort of the flattened `[T*k]` slot list by expert (reference: unstable
  `Tensor.sort()`, moe.py:61);
* the routing sigmoid is `float32(1 / (1 + exp64(-x)))` where `exp64` is the fixed
  sequence of IEEE-754 double multiplications and additions in `exp64_canonical` below.
  The GPU kernel executes the same sequence, so scores, and therefore selections at
  near-ties, are bit-identical on both sides.  It agrees with `torch.sigmoid` to 1 ulp.

Every function cites the reference lines it follows.
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

NORMSILU_EPS = 1e-6          # moe.py:16
SUM_NORM_EPS = 1e-20         # router.py:45

# --------------------------------------------------------------------------------------
# canonical sigmoid (router.py:31 `torch.sigmoid(logits)` on fp32 logits)
# --------------------------------------------------------------------------------------
_LOG2E = 1.4426950408889634          # 0x3FF71547652B82FE
_LN2_HI = 0.693147180369123816490    # 0x3FE62E42FEE00000: low 20 mantissa bits zero, n*LN2_HI exact
_LN2_LO = 1.90821492927058770002e-10  # 0x3DEA39EF35793C76
_EXP_CLAMP = 200.0
# Taylor coefficients 1/j!, j = 13 .. 0, evaluated by Horner with separate mul and add
_EXP_POLY = tuple(1.0 / math.factorial(j) for j in range(13, -1, -1))


def exp64_canonical(y: np.ndarray) -> np.ndarray:
    """exp(y) for float64 `y`, as a fixed sequence of IEEE double ops (no fused multiply-add).

    y is clamped to [-200, 200]; n = floor(y*log2(e) + 0.5); r = (y - n*LN2_HI) - n*LN2_LO;
    p = Horner_13(r) with one rounding after every multiply and every add; result = p * 2^n.
    Relative error is a few 1e-16, far below what a float32 rounding of the sigmoid sees.
    """
    y = np.asarray(y, dtype=np.float64)
    y = np.minimum(np.maximum(y, -_EXP_CLAMP), _EXP_CLAMP)
    n = np.floor(y * _LOG2E + 0.5)
    r = y - n * _LN2_HI
    r = r - n * _LN2_LO
    p = np.full_like(r, _EXP_POLY[0])
    for c in _EXP_POLY[1:]:
        p = p * r
        p = p + c
    return np.ldexp(p, n.astype(np.int64))


def sigmoid32(x: np.ndarray) -> np.ndarray:
    """Canonical float32 sigmoid: one rounding of 1/(1+exp64(-x)) to float32 (router.py:31)."""
    x = np.asarray(x, dtype=np.float32)
    e = exp64_canonical(-x.astype(np.float64))
    return (1.0 / (1.0 + e)).astype(np.float32)


# --------------------------------------------------------------------------------------
# router (router.py:25-51)
# --------------------------------------------------------------------------------------
def router_logits(x: torch.Tensor, w_router: torch.Tensor) -> np.ndarray:
    """fp32 logits `x @ w_router.T` (router.py:25-26).  x [T,H], w_router [E,H] (row = expert).

    Inputs are up-cast to fp32 first; the product is NOT rounded to bf16 (the build pins
    routing to fp32 logits)."""
    return (x.float() @ w_router.float().t()).numpy()


def route_from_logits(logits: np.ndarray, bias: np.ndarray, k: int, norm="sum"):
    """Scores, selection and combine weights from fp32 logits (router.py:31-47).

    Returns (idx int32 [T,k] ascending expert order, w float32 [T,k], scores float32 [T,E]).
    Selection uses `scores + bias` (router.py:38-39); weights gather the UNBIASED scores
    (router.py:41) and, for norm == "sum", divide by (sum + 1e-20) with the sum taken in
    ascending expert order in float32 (router.py:45).  norm False leaves raw scores
    (router.py:46-47); norm == "softmax" is router.py:42-43.
    """
    logits = np.asarray(logits, dtype=np.float32)
    bias = np.asarray(bias, dtype=np.float32)
    T, E = logits.shape
    if not 1 <= k <= E:
        raise ValueError(f"k={k} must be in [1, E={E}]")
    scores = sigmoid32(logits)
    sel = (scores + bias[None, :]).astype(np.float32)
    # stable argsort of -sel: descending value, ties in ascending index order
    order = np.argsort(-sel, axis=1, kind="stable")[:, :k]
    idx = np.sort(order, axis=1).astype(np.int32)
    raw = np.take_along_axis(scores, idx.astype(np.int64), axis=1)
    if k > 1 and norm == "softmax":
        w = F.softmax(torch.from_numpy(raw), dim=-1).numpy()
    elif k > 1 and norm:
        s = np.zeros(T, dtype=np.float32)
        for j in range(k):                       # sequential float32 adds, ascending expert
            s = (s + raw[:, j]).astype(np.float32)
        w = (raw / (s + np.float32(SUM_NORM_EPS))[:, None]).astype(np.float32)
    else:
        w = raw
    return idx, w.astype(np.float32), scores


def boundary_gap(scores: np.ndarray, k: int) -> np.ndarray:
    """Per-token score_k - score_{k+1} on UNBIASED scores (router.py:33-36); caller takes the mean."""
    srt = -np.sort(-scores, axis=1)
    return (srt[:, k - 1] - srt[:, k]).astype(np.float32)


# --------------------------------------------------------------------------------------
# dispatch prologue: histogram, prefix sum, permutation (moe.py:56-68)
# --------------------------------------------------------------------------------------
def permute(idx: np.ndarray, E: int):
    """counts[E], offsets[E+1], perm_slot[S], perm_token[S] for idx [T,k] (moe.py:56-68).

    perm_slot is the stable sort of the flat slot ids 0..T*k-1 by expert; perm_token = slot // k.
    """
    idx = np.asarray(idx)
    T, k = idx.shape
    flat = idx.reshape(-1).astype(np.int64)
    if flat.size and (flat.min() < 0 or flat.max() >= E):
        raise ValueError("expert index out of range")
    counts = np.bincount(flat, minlength=E).astype(np.int32)                 # moe.py:65
    offsets = np.zeros(E + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(counts)                                          # moe.py:66-67
    perm_slot = np.argsort(flat, kind="stable").astype(np.int32)             # moe.py:61 (made stable)
    perm_token = (perm_slot // k).astype(np.int32)                           # moe.py:57-58,62
    return counts, offsets, perm_slot, perm_token


# --------------------------------------------------------------------------------------
# experts (moe.py:73-101)
# --------------------------------------------------------------------------------------
def radial_normsilu(gate: torch.Tensor, theta_e: torch.Tensor, act: str = "radial") -> torch.Tensor:
    """r^p * SiLU(g/r), r = sqrt(mean(g^2) + 1e-6) over the last dim, p = sigmoid(theta_e) (moe.py:87-89).
    Computed in gate's dtype (pass fp32 or fp64).

    `act` selects what the reference's training harness can switch its external kernel to
    (ablate/common/patches.py:53-69): "radial" = the module's own p = sigmoid(theta) (kernel act code 8),
    "tanh" = p = tanh(theta) in (-1,1) (code 10), "silu" = plain SiLU(g), no norm and no gain (code 0)."""
    if act == "silu":
        return F.silu(gate)
    r = torch.sqrt(gate.square().mean(-1, keepdim=True) + NORMSILU_EPS)
    t = theta_e.to(gate.dtype)
    p = torch.tanh(t) if act == "tanh" else torch.sigmoid(t)
    return F.silu(gate / r) * r.pow(p)


def expert_hidden(x_rows: torch.Tensor, w_gate_up_e: torch.Tensor, theta_e: torch.Tensor, act: str = "radial") -> torch.Tensor:
    """act(gate) * up for one expert (moe.py:84-92).  w_gate_up_e [2I,H]: rows 0..I-1 gate, I..2I-1 up."""
    gu = x_rows @ w_gate_up_e.t()
    gate, up = gu.chunk(2, dim=-1)                                            # moe.py:85
    return radial_normsilu(gate, theta_e, act) * up


def experts_forward(x, idx, w, w_gate_up, w_down, theta, dtype=torch.float32, return_hidden=False, n_pos=0, n_neg=0,
                    act="radial"):
    """Weighted sum over each token's experts, evaluated in `dtype` (moe.py:46-101).

    x [T,H]; idx [T,k] integer; w [T,k]; w_gate_up [Eg,2I,H]; w_down [Eg,H,I]; theta [Eg] hold the GLU experts;
    expert ids Eg .. Eg+n_pos-1 are +Identity (out += w*x, moe.py:95-96), the next n_neg -Identity (out -= w*x,
    moe.py:98-99).  Returns [T,H] in `dtype` (the caller rounds to the model dtype, moe.py:101).  With
    return_hidden=True also returns the [S,I] activations of the GLU rows in canonical sorted-row order.
    """
    x = x.to(dtype)
    idx_np = idx.cpu().numpy() if isinstance(idx, torch.Tensor) else np.asarray(idx)
    w_t = (w if isinstance(w, torch.Tensor) else torch.from_numpy(np.asarray(w))).to(dtype)
    T, H = x.shape
    Eg = w_gate_up.shape[0]
    E = Eg + n_pos + n_neg
    k = idx_np.shape[1]
    counts, offsets, perm_slot, perm_token = permute(idx_np, E)
    out = torch.zeros(T, H, dtype=dtype)
    hidden = torch.zeros(T * k, w_down.shape[2], dtype=dtype) if return_hidden else None
    w_flat = w_t.reshape(-1)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if lo == hi:                                                          # moe.py:78-79
            continue
        tok = torch.from_numpy(perm_token[lo:hi].astype(np.int64))
        slot = torch.from_numpy(perm_slot[lo:hi].astype(np.int64))
        if e >= Eg:                                                           # moe.py:95-99
            sign = 1.0 if e < Eg + n_pos else -1.0
            out.index_add_(0, tok, x[tok] * (sign * w_flat[slot]).unsqueeze(-1))
            continue
        h = expert_hidden(x[tok], w_gate_up[e].to(dtype), theta[e], act)
        if return_hidden:
            hidden[lo:hi] = h
        y = h @ w_down[e].to(dtype).t()                                       # moe.py:92
        out.index_add_(0, tok, y * w_flat[slot].unsqueeze(-1))                # moe.py:93
    return (out, hidden) if return_hidden else out


def moe_forward(x, w_router, bias, w_gate_up, w_down, theta, k, dtype=torch.float32, logits=None, n_pos=0, n_neg=0):
    """Whole layer (moe.py:157-183, eval mode, no shared expert).  If `logits` is given the
    routing is computed from them (the parity protocol: same fp32 logits on both sides)."""
    if logits is None:
        logits = router_logits(x, w_router)
    b = bias.detach().float().numpy() if isinstance(bias, torch.Tensor) else bias
    idx, w, _ = route_from_logits(logits, b, k)
    out = experts_forward(x, idx, w, w_gate_up, w_down, theta, dtype=dtype, n_pos=n_pos, n_neg=n_neg)
    return out, idx, w


# --------------------------------------------------------------------------------------
# backward pass: what torch.autograd computes for the reference's eager layer
# --------------------------------------------------------------------------------------
def route_weights(logits: torch.Tensor, idx, norm="sum") -> torch.Tensor:
    """Combine weights as a differentiable function of the logits for a FIXED selection `idx` [T,k]
    (router.py:31,41-47): the selection itself (router.py:38-39, with the bias) has no gradient."""
    idx_t = torch.as_tensor(np.asarray(idx), dtype=torch.int64)
    raw = torch.sigmoid(logits).gather(-1, idx_t)                             # router.py:31,41
    if idx_t.shape[1] > 1 and norm == "softmax":
        return F.softmax(raw, dim=-1)                                         # router.py:42-43
    if idx_t.shape[1] > 1 and norm:
        return raw / (raw.sum(-1, keepdim=True) + SUM_NORM_EPS)               # router.py:44-45
    return raw                                                                # router.py:46-47


def moe_backward(x, w_router, w_gate_up, w_down, theta, idx, d_out, norm="sum", act="radial", dtype=torch.float64,
                 n_pos=0, n_neg=0):
    """Gradients of sum(out * d_out) for out = BiBoMoELayer.forward(x) (moe.py:157-183, no shared expert) with the
    selection `idx` held fixed, as torch.autograd derives them from the restated forward evaluated in `dtype`:
    through the combine weights into the router weight (router.py:25-47), through each expert's down projection,
    Radial NormSiLU (theta included) and gate/up projection (moe.py:81-93).  The balancing bias gets none: it only
    enters the selection (router.py:38).  Returns a dict: x [T,H], w_router [E,H], w_gate_up, w_down, theta, and
    `w` [T,k], the gradient with respect to the combine weights."""
    leaf = lambda t: t.detach().to(dtype).clone().requires_grad_(True)
    xl, wr, gu, dn, th = leaf(x), leaf(w_router), leaf(w_gate_up), leaf(w_down), leaf(theta)
    logits = xl @ wr.t()                                                      # router.py:25-26
    w = route_weights(logits, idx, norm)
    w.retain_grad()
    out = experts_forward(xl, idx, w, gu, dn, th, dtype=dtype, n_pos=n_pos, n_neg=n_neg, act=act)
    (out * d_out.to(dtype)).sum().backward()
    return {"x": xl.grad, "w_router": wr.grad, "w_gate_up": gu.grad, "w_down": dn.grad, "theta": th.grad, "w": w.grad}


def shared_mlp(x, w_gate, w_up, w_down):
    """The shared expert, BiBoMLP.forward (src/modeling/ffn/mlp.py:34-35) with hidden_act = silu:
    down(silu(gate(x)) * up(x)); added to the routed output by the layer (moe.py:174-176).  fp32."""
    xf = x.float()
    return (F.silu(xf @ w_gate.float().t()) * (xf @ w_up.float().t())) @ w_down.float().t()


# --------------------------------------------------------------------------------------
# the caller of the block: RMSNorm in front, residual behind  (src/modeling/layers.py:57-67)
# --------------------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """BiBoRMSNorm.forward (src/modeling/norm.py:19-24): statistics in fp32, the normalised row rounded to
    the input dtype, then multiplied by the weight; returned in the input dtype."""
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)                                    # norm.py:22
    xn = (xf * torch.rsqrt(var + eps)).to(x.dtype)                            # norm.py:23-24
    return (weight.float() * xn.float()).to(x.dtype)


def ffn_forward(h, norm_weight, eps, w_router, bias, w_gate_up, w_down, theta, k, logits=None):
    """BiBoDecoderLayer._ffn_forward (layers.py:57-67): h + moe(post_attention_layernorm(h)), the block and the
    sum evaluated in fp32.  Returns (out fp32, xn in h's dtype, idx, w)."""
    xn = rmsnorm(h, norm_weight, eps)                                         # layers.py:60
    if logits is None:
        logits = router_logits(xn, w_router)
    y, idx, w = moe_forward(xn, w_router, bias, w_gate_up, w_down, theta, k, logits=logits)   # layers.py:61
    return h.float() + y.float(), xn, idx, w                                  # layers.py:64


# --------------------------------------------------------------------------------------
# the reference's eager CPU path, for timing (moe.py:46-101 + router.py:28-51 as written)
# --------------------------------------------------------------------------------------
@torch.no_grad()
def eager_loop_forward(x, w_router, bias, w_gate_up, w_down, theta, k):
    """The per-expert Python loop the reference runs, in the tensors' own dtype (bf16 rounding
    after each linear, fp32 activation, fp32 accumulation), using torch.topk / Tensor.sort as
    the reference does.  Used as the timed CPU baseline; not a parity oracle (tie order and
    rounding sequence are torch's)."""
    T, H = x.shape
    E = w_router.shape[0]
    scores = torch.sigmoid(F.linear(x, w_router).float())                    # router.py:26,31
    _, top_idx = torch.topk(scores + bias.float(), k, dim=-1, sorted=False)   # router.py:38-39
    top_w = scores.gather(-1, top_idx)                                        # router.py:41
    top_w = top_w / (top_w.sum(-1, keepdim=True) + SUM_NORM_EPS)              # router.py:45
    flat_e = top_idx.flatten()
    flat_t = torch.arange(T).unsqueeze(1).expand_as(top_idx).flatten()
    sorted_e, order = flat_e.sort()                                           # moe.py:61
    sorted_t = flat_t[order]
    sorted_w = top_w.flatten()[order]
    bounds = [0] + torch.cumsum(torch.bincount(sorted_e, minlength=E), 0).tolist()   # moe.py:65-68
    out = torch.zeros(T, H, dtype=torch.float32)
    for e in range(E):
        lo, hi = bounds[e], bounds[e + 1]
        if lo == hi:
            continue
        tok = sorted_t[lo:hi]
        gate, up = F.linear(x[tok], w_gate_up[e]).chunk(2, dim=-1)            # moe.py:84-85
        g = gate.float()
        r = torch.sqrt(g.square().mean(-1, keepdim=True) + NORMSILU_EPS)      # moe.py:88
        act = (F.silu(g / r) * r.pow(torch.sigmoid(theta[e].float()))).to(gate.dtype)   # moe.py:89-90
        y = F.linear(act * up, w_down[e])                                     # moe.py:92
        out.index_add_(0, tok, y * sorted_w[lo:hi].unsqueeze(-1))             # moe.py:93
    return out.to(x.dtype)                                                    # moe.py:101


# --------------------------------------------------------------------------------------
# synthetic workloads (seeded; values rounded to bf16 once so CPU and GPU see the same bits)
# --------------------------------------------------------------------------------------
CONFIGS = {
    # name: T, H, E, k, I, batch shape, bias kind, theta kind
    "c1": dict(T=512, H=512, E=64, k=6, I=256, B=1, bias="zero", theta="zero", seed=20261),
    "c2": dict(T=8192, H=768, E=64, k=6, I=384, B=8, bias="uniform", theta="normal", seed=20262),
    "c3": dict(T=64, H=1024, E=64, k=6, I=512, B=1, bias="zero", theta="zero", seed=20263),
    "c4": dict(T=16384, H=768, E=64, k=6, I=384, B=16, bias="hot4", theta="normal", seed=20264),
}


def make_inputs(T, H, E, k, I, bias="zero", theta="zero", seed=0, dtype=torch.bfloat16, **_):
    """Seeded synthetic tensors of a workload: hidden ~N(0,1), weights ~N(0,0.02), bias 0 /
    U(-0.01,0.01) / +2.0 on four hot experts, theta 0 / N(0,0.5).  Generated in fp32 on the CPU
    and rounded once to `dtype`; bias and theta stay fp32."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(dtype)
    w_router = (torch.randn(E, H, generator=g) * 0.02).to(dtype)
    w_gate_up = (torch.randn(E, 2 * I, H, generator=g) * 0.02).to(dtype)
    w_down = (torch.randn(E, H, I, generator=g) * 0.02).to(dtype)
    if bias == "zero":
        b = torch.zeros(E)
    else:
        b = (torch.rand(E, generator=g) * 0.02 - 0.01)
        if bias == "hot4":
            b[:4] = 2.0
    th = torch.zeros(E) if theta == "zero" else torch.randn(E, generator=g) * 0.5
    return dict(x=x, w_router=w_router, bias=b.float(), w_gate_up=w_gate_up, w_down=w_down,
                theta=th.float(), k=k)
