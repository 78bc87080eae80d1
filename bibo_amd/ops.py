"""Tensor-level wrappers over the C ABI: torch supplies device memory and the stream, nothing else."""
from __future__ import annotations

import ctypes

import torch

from . import _lib as L

_NORM = {"sum": L.NORM_SUM, True: L.NORM_SUM, "softmax": L.NORM_SOFTMAX, False: L.NORM_NONE, None: L.NORM_NONE}
_ALGO = {"auto": L.ALGO_AUTO, "generic": L.ALGO_GENERIC, "mfma": L.ALGO_MFMA, "stream": L.ALGO_STREAM,
         "fused": L.ALGO_FUSED}


_ACT = {"radial": L.ACT_RADIAL_SIGMOID, "radial_sigmoid": L.ACT_RADIAL_SIGMOID, "sigmoid": L.ACT_RADIAL_SIGMOID,
        "radial_tanh": L.ACT_RADIAL_TANH, "tanh": L.ACT_RADIAL_TANH, "silu": L.ACT_SILU}


def act_code(v) -> int:
    """Expert activation: 'radial' (= 'sigmoid', the reference module, kernel act code 8 of
    ablate/common/patches.py:53-69), 'tanh' (code 10: p = tanh(theta)) or 'silu' (code 0: plain SwiGLU)."""
    if isinstance(v, int) and not isinstance(v, bool):
        return v
    if v in _ACT:
        return _ACT[v]
    raise ValueError(f"act must be one of {sorted(_ACT)}, got {v!r}")


def norm_mode(v) -> int:
    if isinstance(v, str) or isinstance(v, bool) or v is None:
        if v in _NORM:
            return _NORM[v]
    raise ValueError(f"norm_topk_prob must be 'sum', 'softmax' or False, got {v!r}")


def algo_code(v) -> int:
    if isinstance(v, int):
        return v
    return _ALGO[v]


def select_algo(T, H, E, k, I, dtype_code=L.DTYPE_BF16, algo="auto", n_pos=0, n_neg=0) -> str:
    """Name of the kernel family the composite calls run for this shape (bibo_moe_select_algo)."""
    sh = L.Shape(T, H, E, k, I, dtype_code, n_pos, n_neg)
    out = ctypes.c_int(0)
    L.check(L.lib().bibo_moe_select_algo(ctypes.byref(sh), algo_code(algo), ctypes.byref(out)), "bibo_moe_select_algo")
    return {v: n for n, v in _ALGO.items()}[out.value]


def backward_supported(H, I, E, dtype, n_pos=0, n_neg=0) -> bool:
    """Whether bibo_moe_backward takes hidden size H and expert size I in `dtype` (torch.bfloat16 or torch.float32): the
    answer bibo_moe_backward_workspace_bytes gives for a single token."""
    sh = L.Shape(1, H, E, 1, I, L.DTYPE_BF16 if dtype == torch.bfloat16 else L.DTYPE_F32, n_pos, n_neg)
    n = ctypes.c_size_t(0)
    return L.lib().bibo_moe_backward_workspace_bytes(ctypes.byref(sh), ctypes.byref(n)) == 0


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return L.DTYPE_BF16
    if t.dtype == torch.float32:
        return L.DTYPE_F32
    raise TypeError(f"hidden states and weights must be bfloat16 or float32, got {t.dtype}")


def _chk(t: torch.Tensor, name: str, dtype=None, shape=None):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); bibo_amd has no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")   # a strided view would be silently misread
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(dev) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


_workspaces: dict = {}


def workspace(dev: torch.device, nbytes: int) -> torch.Tensor:
    """A grow-only byte buffer per (device, stream): calls on one stream are ordered, so they may share it."""
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
        _workspaces[key] = ws
    return ws


def workspace_bytes(T, H, E, k, I, dtype_code) -> int:
    sh = L.Shape(T, H, E, k, I, dtype_code)
    out = ctypes.c_size_t(0)
    L.check(L.lib().bibo_moe_workspace_bytes(ctypes.byref(sh), ctypes.byref(out)), "bibo_moe_workspace_bytes")
    return out.value


def router_fwd(x, w_router, bias, k, norm="sum", want_logits=False, want_gap=False):
    """x [T,H], w_router [E,H], bias fp32 [E] -> idx int32 [T,k], w fp32 [T,k], logits fp32 [T,E]|None, gap fp32 [T]|None."""
    T, H = x.shape
    E = w_router.shape[0]
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(w_router, "w_router", x.dtype, (E, H)); _chk(bias, "bias", torch.float32, (E,))
    dev = x.device
    idx = torch.empty(T, k, dtype=torch.int32, device=dev)
    w = torch.empty(T, k, dtype=torch.float32, device=dev)
    logits = torch.empty(T, E, dtype=torch.float32, device=dev) if want_logits else None
    gap = torch.empty(T, dtype=torch.float32, device=dev) if want_gap else None
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_router_fwd(_ptr(x), _ptr(w_router), _ptr(bias), T, H, E, k, dc, norm_mode(norm),
                                            _ptr(logits), _ptr(idx), _ptr(w), _ptr(gap), _stream(dev)),
                "bibo_moe_router_fwd")
    return idx, w, logits, gap


def permute(idx, E):
    """idx int32 [T,k] -> counts [E], offsets [E+1], perm_slot [T*k], perm_token [T*k] (all int32)."""
    T, k = idx.shape
    _chk(idx, "idx", torch.int32)
    dev = idx.device
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    perm_slot = torch.empty(T * k, dtype=torch.int32, device=dev)
    perm_token = torch.empty(T * k, dtype=torch.int32, device=dev)
    # one 64-entry histogram per 128 tokens and, for large batches, one sum per 256 histograms
    nb = (max(1, (T + 127) // 128) + (T + 32767) // 32768 + 1) * 64 * 4
    ws = workspace(dev, nb)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_permute(_ptr(idx), T, E, k, _ptr(counts), _ptr(offsets), _ptr(perm_slot),
                                         _ptr(perm_token), _ptr(ws), ws.numel(), _stream(dev)), "bibo_moe_permute")
    return counts, offsets, perm_slot, perm_token


def gateup_fwd(x, w_gate_up, theta, offsets, perm_token, k, algo="auto", act="radial"):
    """-> hidden [T*k, I] in x.dtype, rows in permuted order."""
    T, H = x.shape
    E, two_i, _ = w_gate_up.shape
    I = two_i // 2
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(w_gate_up, "w_gate_up", x.dtype, (E, 2 * I, H)); _chk(theta, "theta", torch.float32, (E,))
    _chk(offsets, "offsets", torch.int32, (E + 1,)); _chk(perm_token, "perm_token", torch.int32, (T * k,))
    hidden = torch.empty(T * k, I, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        L.check(L.lib().bibo_moe_gateup_fwd(_ptr(x), _ptr(w_gate_up), _ptr(theta), _ptr(offsets), _ptr(perm_token),
                                            T, H, E, k, I, dc, algo_code(algo), act_code(act), _ptr(hidden),
                                            _stream(x.device)),
                "bibo_moe_gateup_fwd")
    return hidden


def down_combine_fwd(hidden, w_down, w, offsets, perm_slot, T, algo="auto"):
    """-> out [T,H] in hidden.dtype."""
    E, H, I = w_down.shape
    k = w.shape[1]
    dc = _dtype_code(hidden)
    _chk(hidden, "hidden", None, (T * k, I)); _chk(w_down, "w_down", hidden.dtype); _chk(w, "w", torch.float32, (T, k))
    _chk(offsets, "offsets", torch.int32, (E + 1,)); _chk(perm_slot, "perm_slot", torch.int32, (T * k,))
    dev = hidden.device
    out = torch.empty(T, H, dtype=hidden.dtype, device=dev)
    ws = workspace(dev, T * k * H * 4)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_down_combine_fwd(_ptr(hidden), _ptr(w_down), _ptr(w), _ptr(offsets), _ptr(perm_slot),
                                                  T, H, E, k, I, dc, algo_code(algo), _ptr(out), _ptr(ws), ws.numel(),
                                                  _stream(dev)), "bibo_moe_down_combine_fwd")
    return out


def gateup_down_fwd(x, w_gate_up, w_down, theta, w, offsets, perm_slot, perm_token, act="radial"):
    """Both projections in one launch -> yw [T*k, H] bf16, routing-weighted rows in slot order."""
    T, H = x.shape
    E, two_i, _ = w_gate_up.shape
    I = two_i // 2
    k = w.shape[1]
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(w_gate_up, "w_gate_up", x.dtype, (E, 2 * I, H)); _chk(w_down, "w_down", x.dtype, (E, H, I))
    _chk(theta, "theta", torch.float32, (E,)); _chk(w, "w", torch.float32, (T, k))
    _chk(offsets, "offsets", torch.int32, (E + 1,)); _chk(perm_slot, "perm_slot", torch.int32, (T * k,))
    _chk(perm_token, "perm_token", torch.int32, (T * k,))
    yw = torch.zeros(T * k, H, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        L.check(L.lib().bibo_moe_gateup_down_fwd(_ptr(x), _ptr(w_gate_up), _ptr(w_down), _ptr(theta), _ptr(w),
                                                 _ptr(offsets), _ptr(perm_slot), _ptr(perm_token), T, H, E, k, I, dc,
                                                 act_code(act), _ptr(yw), _stream(x.device)), "bibo_moe_gateup_down_fwd")
    return yw


def combine_fwd(yw, T, k, dtype=None, idx=None, w=None, x=None, n_glu=0, n_pos=0, n_neg=0, residual=None):
    """out[t] = residual[t] + sum_j contribution(t, j) in fp32, rounded once -> [T,H] in `dtype` (default: yw.dtype).
    contribution = yw[t*k + j]; with idx (and w, x) given, +/- w[t,j] * x[t] for the +/-Identity specials and nothing
    for an index outside [0, n_glu + n_pos + n_neg)."""
    H = yw.shape[1]
    dtype = dtype or yw.dtype
    _chk(yw, "yw", None, (T * k, H))
    if yw.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError("yw must be bf16 or fp32")
    for t_, n_, d_, sh_ in ((idx, "idx", torch.int32, (T, k)), (w, "w", torch.float32, (T, k)), (x, "x", dtype, (T, H)),
                            (residual, "residual", dtype, (T, H))):
        if t_ is not None:
            _chk(t_, n_, d_, sh_)
    out = torch.empty(T, H, dtype=dtype, device=yw.device)
    dc = L.DTYPE_BF16 if dtype == torch.bfloat16 else L.DTYPE_F32
    with torch.cuda.device(yw.device):
        if idx is None and residual is None:
            L.check(L.lib().bibo_moe_combine_fwd(_ptr(yw), int(yw.dtype == torch.bfloat16), T, H, k, dc, _ptr(out),
                                                 _stream(yw.device)), "bibo_moe_combine_fwd")
        else:
            L.check(L.lib().bibo_moe_combine_ex_fwd(_ptr(yw), int(yw.dtype == torch.bfloat16), _ptr(idx), _ptr(w), _ptr(x),
                                                    n_glu, n_pos, n_neg, _ptr(residual), T, H, k, dc, _ptr(out),
                                                    _stream(yw.device)), "bibo_moe_combine_ex_fwd")
    return out


def experts_fwd(x, idx, w, w_gate_up, w_down, theta, algo="auto", want_counts=False, n_pos=0, n_neg=0, act="radial"):
    """Seam 2.  x [T,H]; idx int32 [T,k]; w fp32 [T,k] -> out [T,H] (x.dtype), counts int32 [E]|None.
    The weight tensors hold the GLU experts; expert ids Eg .. Eg+n_pos-1 are +Identity, the next n_neg -Identity
    specials (moe.py:39-44,95-99), and E = Eg + n_pos + n_neg."""
    T, H = x.shape
    Eg, two_i, _ = w_gate_up.shape
    E = Eg + n_pos + n_neg
    I = two_i // 2
    k = idx.shape[1]
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(idx, "idx", torch.int32, (T, k)); _chk(w, "w", torch.float32, (T, k))
    _chk(w_gate_up, "w_gate_up", x.dtype, (Eg, 2 * I, H)); _chk(w_down, "w_down", x.dtype, (Eg, H, I))
    _chk(theta, "theta", torch.float32, (Eg,))
    dev = x.device
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    counts = torch.empty(E, dtype=torch.int32, device=dev) if want_counts else None
    ws = workspace(dev, workspace_bytes(T, H, E, k, I, dc))
    sh = L.Shape(T, H, E, k, I, dc, n_pos, n_neg, act_code(act), 0)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_experts_fwd(_ptr(x), _ptr(idx), _ptr(w), _ptr(w_gate_up), _ptr(w_down), _ptr(theta),
                                             ctypes.byref(sh), algo_code(algo), _ptr(out), _ptr(counts), _ptr(ws),
                                             ws.numel(), _stream(dev)), "bibo_moe_experts_fwd")
    return out, counts


def moe_forward(x, w_router, bias, w_gate_up, w_down, theta, k, norm="sum", algo="auto", want_routing=False,
                want_counts=False, want_logits=False, n_pos=0, n_neg=0, act="radial"):
    """Seam 1.  -> out [T,H], idx int32 [T,k]|None, w fp32 [T,k]|None, counts int32 [E]|None, logits fp32 [T,E]|None.
    w_router / bias have E = Eg + n_pos + n_neg rows, the expert weights Eg (see experts_fwd)."""
    T, H = x.shape
    Eg, two_i, _ = w_gate_up.shape
    E = Eg + n_pos + n_neg
    I = two_i // 2
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(w_router, "w_router", x.dtype, (E, H)); _chk(bias, "bias", torch.float32, (E,))
    _chk(w_gate_up, "w_gate_up", x.dtype, (Eg, 2 * I, H)); _chk(w_down, "w_down", x.dtype, (Eg, H, I))
    _chk(theta, "theta", torch.float32, (Eg,))
    dev = x.device
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    idx = torch.empty(T, k, dtype=torch.int32, device=dev) if want_routing else None
    w = torch.empty(T, k, dtype=torch.float32, device=dev) if want_routing else None
    counts = torch.empty(E, dtype=torch.int32, device=dev) if want_counts else None
    logits = torch.empty(T, E, dtype=torch.float32, device=dev) if want_logits else None
    ws = workspace(dev, workspace_bytes(T, H, E, k, I, dc))
    sh = L.Shape(T, H, E, k, I, dc, n_pos, n_neg, act_code(act), 0)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_forward(_ptr(x), _ptr(w_router), _ptr(bias), _ptr(w_gate_up), _ptr(w_down),
                                         _ptr(theta), ctypes.byref(sh), norm_mode(norm), algo_code(algo), _ptr(out),
                                         _ptr(idx), _ptr(w), _ptr(counts), _ptr(logits), _ptr(ws), ws.numel(),
                                         _stream(dev)), "bibo_moe_forward")
    return out, idx, w, counts, logits


def moe_forward_static(x, w_router, bias, w_gate_up, w_down, theta, k, out, norm="sum", algo="auto", idx=None, w=None,
                       counts=None, logits=None, n_pos=0, n_neg=0, act="radial"):
    """bibo_moe_forward_static: the whole layer with the library's static per-GPU scratch array as workspace.  Nothing
    is allocated here either: `out` [T,H] and the optional `idx`, `w`, `counts`, `logits` are the caller's tensors."""
    T, H = x.shape
    Eg, two_i, _ = w_gate_up.shape
    E = Eg + n_pos + n_neg
    I = two_i // 2
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(w_router, "w_router", x.dtype, (E, H)); _chk(bias, "bias", torch.float32, (E,))
    _chk(w_gate_up, "w_gate_up", x.dtype, (Eg, 2 * I, H)); _chk(w_down, "w_down", x.dtype, (Eg, H, I))
    _chk(theta, "theta", torch.float32, (Eg,)); _chk(out, "out", x.dtype, (T, H))
    for t_, n_, d_, sh_ in ((idx, "idx", torch.int32, (T, k)), (w, "w", torch.float32, (T, k)),
                            (counts, "counts", torch.int32, (E,)), (logits, "logits", torch.float32, (T, E))):
        if t_ is not None:
            _chk(t_, n_, d_, sh_)
    sh = L.Shape(T, H, E, k, I, dc, n_pos, n_neg, act_code(act), 0)
    dev = x.device
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_forward_static(_ptr(x), _ptr(w_router), _ptr(bias), _ptr(w_gate_up), _ptr(w_down),
                                                _ptr(theta), ctypes.byref(sh), norm_mode(norm), algo_code(algo), _ptr(out),
                                                _ptr(idx), _ptr(w), _ptr(counts), _ptr(logits), _stream(dev)),
                "bibo_moe_forward_static")
    return out


def moe_backward(x, d_out, w_router, bias, w_gate_up, w_down, theta, k, norm="sum", act="radial", want_dw=False,
                 n_pos=0, n_neg=0):
    """Gradients of the layer (bibo_moe_backward) for the upstream gradient d_out [T,H] of its output: what autograd
    derives for BiBoMoELayer.forward (moe.py:157-183) with the selection held fixed.  w_router / bias have
    E = Eg + n_pos + n_neg rows, the expert weights Eg (see experts_fwd).
    -> d_x [T,H], d_w_router [E,H], d_w_gate_up [Eg,2I,H], d_w_down [Eg,H,I] (x.dtype), d_theta fp32 [Eg],
    d_w fp32 [T,k]|None."""
    T, H = x.shape
    Eg, two_i, _ = w_gate_up.shape
    E = Eg + n_pos + n_neg
    I = two_i // 2
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(d_out, "d_out", x.dtype, (T, H)); _chk(w_router, "w_router", x.dtype, (E, H))
    _chk(bias, "bias", torch.float32, (E,)); _chk(w_gate_up, "w_gate_up", x.dtype, (Eg, 2 * I, H))
    _chk(w_down, "w_down", x.dtype, (Eg, H, I)); _chk(theta, "theta", torch.float32, (Eg,))
    dev = x.device
    d_x = torch.empty_like(x)
    d_wr, d_gu, d_dn = torch.empty_like(w_router), torch.empty_like(w_gate_up), torch.empty_like(w_down)
    d_theta = torch.empty(Eg, dtype=torch.float32, device=dev)
    d_w = torch.empty(T, k, dtype=torch.float32, device=dev) if want_dw else None
    sh = L.Shape(T, H, E, k, I, dc, n_pos, n_neg, act_code(act), 0)
    nbytes = ctypes.c_size_t(0)
    L.check(L.lib().bibo_moe_backward_workspace_bytes(ctypes.byref(sh), ctypes.byref(nbytes)), "bibo_moe_backward_workspace_bytes")
    ws = workspace(dev, nbytes.value)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_backward(_ptr(x), _ptr(d_out), _ptr(w_router), _ptr(bias), _ptr(w_gate_up), _ptr(w_down),
                                          _ptr(theta), ctypes.byref(sh), norm_mode(norm), _ptr(d_x), _ptr(d_wr), _ptr(d_gu),
                                          _ptr(d_dn), _ptr(d_theta), _ptr(d_w), _ptr(ws), ws.numel(), _stream(dev)),
                "bibo_moe_backward")
    return d_x, d_wr, d_gu, d_dn, d_theta, d_w


def train_state_bytes(T, H, E, k, I, dtype, n_pos=0, n_neg=0, act="radial"):
    """Size of the buffer a training forward keeps for its backward pass (bibo_moe_train_state_bytes), or None where the
    shape has no such pair (anything but bf16 with H a multiple of 128 and I in {128, 256, 384})."""
    sh = L.Shape(T, H, E, k, I, L.DTYPE_BF16 if dtype == torch.bfloat16 else L.DTYPE_F32, n_pos, n_neg, act_code(act), 0)
    n = ctypes.c_size_t(0)
    rc = L.lib().bibo_moe_train_state_bytes(ctypes.byref(sh), ctypes.byref(n))
    return n.value if rc == 0 else None


def moe_forward_train(x, w_router, bias, w_gate_up, w_down, theta, k, norm="sum", want_counts=False, n_pos=0, n_neg=0,
                      act="radial"):
    """bibo_moe_forward_train: the layer's forward that keeps routing, permutation and gate/up pre-activations in a
    state tensor for moe_backward_saved.  -> out [T,H], counts int32 [E]|None, state (uint8)."""
    T, H = x.shape
    Eg, two_i, _ = w_gate_up.shape
    E = Eg + n_pos + n_neg
    I = two_i // 2
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(w_router, "w_router", x.dtype, (E, H)); _chk(bias, "bias", torch.float32, (E,))
    _chk(w_gate_up, "w_gate_up", x.dtype, (Eg, 2 * I, H)); _chk(w_down, "w_down", x.dtype, (Eg, H, I))
    _chk(theta, "theta", torch.float32, (Eg,))
    dev = x.device
    nbytes = train_state_bytes(T, H, E, k, I, x.dtype, n_pos, n_neg, act)
    if nbytes is None:
        raise NotImplementedError("no state-keeping training forward for this shape; use moe_forward and moe_backward")
    out = torch.empty(T, H, dtype=x.dtype, device=dev)
    counts = torch.empty(E, dtype=torch.int32, device=dev) if want_counts else None
    state = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    ws = workspace(dev, workspace_bytes(T, H, E, k, I, dc))
    sh = L.Shape(T, H, E, k, I, dc, n_pos, n_neg, act_code(act), 0)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_forward_train(_ptr(x), _ptr(w_router), _ptr(bias), _ptr(w_gate_up), _ptr(w_down), _ptr(theta),
                                               ctypes.byref(sh), norm_mode(norm), _ptr(out), _ptr(counts), _ptr(state),
                                               state.numel(), _ptr(ws), ws.numel(), _stream(dev)), "bibo_moe_forward_train")
    return out, counts, state


def moe_backward_saved(x, d_out, w_router, w_gate_up, w_down, theta, k, state, norm="sum", act="radial", want_dw=False,
                       n_pos=0, n_neg=0):
    """bibo_moe_backward_saved: moe_backward with the routing, the permutation and the pre-activations taken from the
    state tensor of moe_forward_train on the same x and weights (same results, bit for bit)."""
    T, H = x.shape
    Eg, two_i, _ = w_gate_up.shape
    E = Eg + n_pos + n_neg
    I = two_i // 2
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(d_out, "d_out", x.dtype, (T, H)); _chk(w_router, "w_router", x.dtype, (E, H))
    _chk(w_gate_up, "w_gate_up", x.dtype, (Eg, 2 * I, H)); _chk(w_down, "w_down", x.dtype, (Eg, H, I))
    _chk(theta, "theta", torch.float32, (Eg,)); _chk(state, "state", torch.uint8)
    dev = x.device
    d_x = torch.empty_like(x)
    d_wr, d_gu, d_dn = torch.empty_like(w_router), torch.empty_like(w_gate_up), torch.empty_like(w_down)
    d_theta = torch.empty(Eg, dtype=torch.float32, device=dev)
    d_w = torch.empty(T, k, dtype=torch.float32, device=dev) if want_dw else None
    sh = L.Shape(T, H, E, k, I, dc, n_pos, n_neg, act_code(act), 0)
    nbytes = ctypes.c_size_t(0)
    L.check(L.lib().bibo_moe_backward_workspace_bytes(ctypes.byref(sh), ctypes.byref(nbytes)), "bibo_moe_backward_workspace_bytes")
    ws = workspace(dev, nbytes.value)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_backward_saved(_ptr(x), _ptr(d_out), _ptr(w_router), _ptr(w_gate_up), _ptr(w_down),
                                                _ptr(theta), ctypes.byref(sh), norm_mode(norm), _ptr(state), state.numel(),
                                                _ptr(d_x), _ptr(d_wr), _ptr(d_gu), _ptr(d_dn), _ptr(d_theta), _ptr(d_w),
                                                _ptr(ws), ws.numel(), _stream(dev)), "bibo_moe_backward_saved")
    return d_x, d_wr, d_gu, d_dn, d_theta, d_w


def experts_backward(x, d_out, idx, w, w_gate_up, w_down, theta, act="radial", n_pos=0, n_neg=0):
    """bibo_moe_experts_backward: gradients of experts_fwd for a caller-owned routing (idx int32 [T,k], w fp32 [T,k];
    expert ids Eg .. Eg+n_pos-1 are +Identity, the next n_neg -Identity, as in experts_fwd).
    -> d_x [T,H], d_w fp32 [T,k], d_w_gate_up, d_w_down (x.dtype), d_theta fp32 [Eg]."""
    T, H = x.shape
    E, two_i, _ = w_gate_up.shape          # GLU experts
    I = two_i // 2
    k = idx.shape[1]
    dc = _dtype_code(x)
    _chk(x, "x"); _chk(d_out, "d_out", x.dtype, (T, H)); _chk(idx, "idx", torch.int32, (T, k)); _chk(w, "w", torch.float32, (T, k))
    _chk(w_gate_up, "w_gate_up", x.dtype, (E, 2 * I, H)); _chk(w_down, "w_down", x.dtype, (E, H, I))
    _chk(theta, "theta", torch.float32, (E,))
    dev = x.device
    d_x, d_gu, d_dn = torch.empty_like(x), torch.empty_like(w_gate_up), torch.empty_like(w_down)
    d_w = torch.empty(T, k, dtype=torch.float32, device=dev)
    d_theta = torch.empty(E, dtype=torch.float32, device=dev)
    sh = L.Shape(T, H, E + n_pos + n_neg, k, I, dc, n_pos, n_neg, act_code(act), 0)
    nbytes = ctypes.c_size_t(0)
    L.check(L.lib().bibo_moe_backward_workspace_bytes(ctypes.byref(sh), ctypes.byref(nbytes)), "bibo_moe_backward_workspace_bytes")
    ws = workspace(dev, nbytes.value)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_experts_backward(_ptr(x), _ptr(d_out), _ptr(idx), _ptr(w), _ptr(w_gate_up), _ptr(w_down),
                                                  _ptr(theta), ctypes.byref(sh), _ptr(d_x), _ptr(d_w), _ptr(d_gu), _ptr(d_dn),
                                                  _ptr(d_theta), _ptr(ws), ws.numel(), _stream(dev)),
                "bibo_moe_experts_backward")
    return d_x, d_w, d_gu, d_dn, d_theta


def attn_res_fwd(candidates, score_weight, eps):
    """bibo_moe_exp_attn_res_fwd: softmax-weighted average of the candidate rows, scores rsqrt(mean c^2 + eps) <c, score_weight>
    (apply_attention_residual, exp/modeling_bibo.py:119-232).  candidates: list of [T,H] bf16; score_weight fp32 [H]."""
    T, H = candidates[0].shape
    for c in candidates:
        _chk(c, "candidate", torch.bfloat16, (T, H))
    _chk(score_weight, "score_weight", torch.float32, (H,))
    out = torch.empty_like(candidates[0])
    arr = (ctypes.c_void_p * len(candidates))(*[c.data_ptr() for c in candidates])
    dev = out.device
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_exp_attn_res_fwd(ctypes.cast(arr, ctypes.c_void_p), len(candidates), _ptr(score_weight),
                                              ctypes.c_float(eps), T, H, _dtype_code(out), _ptr(out), _stream(dev)),
                "bibo_moe_exp_attn_res_fwd")
    return out


def rmsnorm_fwd(x, norm_weight, eps):
    """out = norm_weight * round(x * rsqrt(mean(x^2) + eps)) in x.dtype (the block's input norm, norm.py:19-24)."""
    T, H = x.shape
    _chk(x, "x"); _chk(norm_weight, "norm_weight", torch.float32, (H,))
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        L.check(L.lib().bibo_moe_rmsnorm_fwd(_ptr(x), _ptr(norm_weight), ctypes.c_float(eps), T, H, _dtype_code(x),
                                             _ptr(out), _stream(x.device)), "bibo_moe_rmsnorm_fwd")
    return out


def ffn_forward(h, norm_weight, eps, w_router, bias, w_gate_up, w_down, theta, k, norm="sum", algo="auto",
                want_routing=False, want_counts=False, n_pos=0, n_neg=0, act="radial", round_block_out=False,
                residual=None, out=None):
    """Seam 3 (the block's caller).  -> out = h + moe(rmsnorm(h)) [T,H], idx|None, w|None, counts|None.
    round_block_out: round the block's output to h.dtype before the residual add (bf16_moe_out, layers.py:62-63).
    residual: None adds h itself (layers.py:57-64); a [T,H] tensor is added instead of h; False adds nothing,
    out = moe(rmsnorm(h)) (the experimental layer's _attn_res_mlp_forward, exp/modeling_bibo.py:429-431).
    out: optional preallocated result (may be the residual tensor)."""
    T, H = h.shape
    Eg, two_i, _ = w_gate_up.shape
    E = Eg + n_pos + n_neg
    I = two_i // 2
    dc = _dtype_code(h)
    _chk(h, "h"); _chk(norm_weight, "norm_weight", torch.float32, (H,)); _chk(w_router, "w_router", h.dtype, (E, H))
    _chk(bias, "bias", torch.float32, (E,)); _chk(w_gate_up, "w_gate_up", h.dtype, (Eg, 2 * I, H))
    _chk(w_down, "w_down", h.dtype, (Eg, H, I)); _chk(theta, "theta", torch.float32, (Eg,))
    dev = h.device
    if out is None:
        out = torch.empty(T, H, dtype=h.dtype, device=dev)
    else:
        _chk(out, "out", h.dtype, (T, H))
    flags = L.FLAG_ROUND_BLOCK_OUT if round_block_out else 0
    if residual is False:
        flags |= L.FLAG_NO_RESIDUAL
        residual = None
    elif residual is not None:
        _chk(residual, "residual", h.dtype, (T, H))
    idx = torch.empty(T, k, dtype=torch.int32, device=dev) if want_routing else None
    w = torch.empty(T, k, dtype=torch.float32, device=dev) if want_routing else None
    counts = torch.empty(E, dtype=torch.int32, device=dev) if want_counts else None
    sh = L.Shape(T, H, E, k, I, dc, n_pos, n_neg, act_code(act), flags)
    nbytes = ctypes.c_size_t(0)
    L.check(L.lib().bibo_moe_ffn_workspace_bytes(ctypes.byref(sh), ctypes.byref(nbytes)), "bibo_moe_ffn_workspace_bytes")
    ws = workspace(dev, nbytes.value)
    with torch.cuda.device(dev):
        L.check(L.lib().bibo_moe_ffn_forward(_ptr(h), _ptr(norm_weight), ctypes.c_float(eps), _ptr(residual), _ptr(w_router), _ptr(bias),
                                             _ptr(w_gate_up), _ptr(w_down), _ptr(theta), ctypes.byref(sh),
                                             norm_mode(norm), algo_code(algo), _ptr(out), _ptr(idx), _ptr(w),
                                             _ptr(counts), _ptr(ws), ws.numel(), _stream(dev)), "bibo_moe_ffn_forward")
    return out, idx, w, counts
