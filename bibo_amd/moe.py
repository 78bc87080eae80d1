"""Drop-in modules for the reference's sparse-MoE block, running on the HIP kernels of libbibo_moe.so.

Class names, constructor argument, attribute names, parameter shapes and state_dict keys follow
src/modeling/ffn/router.py and src/modeling/ffn/moe.py of the reference, so a reference checkpoint
loads with strict=True and code that pokes at `layer.gate.bias` or `layer.experts.radial_theta`
keeps working.  The modules are differentiable: `BiBoMoELayer.forward` is one autograd node (backward =
bibo_moe_backward); with hooks present, or called on their own, `BiBoFusedExperts` is one node (backward =
bibo_moe_experts_backward) and `BiBoMoERouter` returns the kernel's selection with differentiable weights.  bf16
compute on sizes that are multiples of 128 trains on the MFMA kernels, fp32 compute and other sizes on generic ones."""
from __future__ import annotations

import torch
import torch.nn as nn

from . import _lib as L
from . import ops

__all__ = ["BiBoMoERouter", "BiBoFusedExperts", "BiBoMoELayer"]

try:
    _no_compile = torch.compiler.disable
except AttributeError:                                    # older torch
    _no_compile = torch._dynamo.disable


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class _MoELayerFn(torch.autograd.Function):
    """The whole layer as one autograd node.  Gradients are what autograd gives the reference's eager layer with the
    selection held fixed (moe.py:157-183); the balancing bias gets none (router.py:38).  The per-expert row counts come
    out as a second, non-differentiable result.  `cd` is the compute dtype: bf16 runs the MFMA backward where its tiles
    divide the sizes, anything else the generic kernels.  Two ways through the library: with `keep` and a shape that
    has the pair, forward = bibo_moe_forward_train, which leaves routing, permutation and pre-activations in a state
    tensor (about 4 I bytes per routed slot), and backward = bibo_moe_backward_saved; otherwise forward =
    bibo_moe_forward and backward = bibo_moe_backward, which computes all of that again from the saved input rows.
    The gradients are the same bits either way."""

    @staticmethod
    def forward(ctx, x, w_router, w_gate_up, w_down, theta, bias, k, norm, act, algo, want_counts, n_pos=0, n_neg=0,
                casts=None, cd=torch.bfloat16, keep=True):
        cast = lambda t, d: (t if t.dtype == d else t.to(d)).contiguous()
        xb = cast(x.detach(), cd)
        # `casts`: kernel-dtype copies of the three weight tensors the caller already holds (the layer's cast cache), so
        # fp32 master weights are rounded once per optimiser step, not once per forward
        wr, gu, dn = casts if casts is not None else (cast(w_router.detach(), cd), cast(w_gate_up.detach(), cd),
                                                      cast(w_down.detach(), cd))
        th = cast(theta.detach(), torch.float32)
        # A private copy of the E selection biases: the layer's balancing step writes gate.bias in place later in the
        # same forward (update_bias), and the backward pass has to route with the values the forward saw.
        b = bias.detach().to(torch.float32).clone()
        T, H = xb.shape
        state = None
        if keep and algo in ("auto", "fused") and ops.train_state_bytes(T, H, wr.shape[0], k, gu.shape[1] // 2, cd, n_pos,
                                                                        n_neg, act) is not None:
            out, counts, state = ops.moe_forward_train(xb, wr, b, gu, dn, th, k, norm=norm, want_counts=want_counts, act=act,
                                                       n_pos=n_pos, n_neg=n_neg)
        else:
            out, _, _, counts, _ = ops.moe_forward(xb, wr, b, gu, dn, th, k, norm=norm, algo=algo, want_counts=want_counts,
                                                   act=act, n_pos=n_pos, n_neg=n_neg)
        ctx.has_state = state is not None
        ctx.save_for_backward(xb, wr, gu, dn, th, b, *((state,) if state is not None else ()))
        ctx.conf = (k, norm, act, n_pos, n_neg)
        ctx.in_dtypes = (x.dtype, w_router.dtype, w_gate_up.dtype, w_down.dtype, theta.dtype)
        if counts is None:
            counts = torch.empty(0, dtype=torch.int32, device=x.device)
        ctx.mark_non_differentiable(counts)
        return out, counts

    @staticmethod
    def backward(ctx, d_out, _d_counts):
        saved = ctx.saved_tensors                        # read once: activation checkpointing unpacks on access
        xb, wr, gu, dn, th, b = saved[:6]
        k, norm, act, n_pos, n_neg = ctx.conf
        d = d_out.to(xb.dtype).contiguous()
        if ctx.has_state:
            grads = ops.moe_backward_saved(xb, d, wr, gu, dn, th, k, saved[6], norm=norm, act=act, n_pos=n_pos,
                                           n_neg=n_neg)[:5]
        else:
            grads = ops.moe_backward(xb, d, wr, b, gu, dn, th, k, norm=norm, act=act, n_pos=n_pos, n_neg=n_neg)[:5]
        return tuple(g.to(dt) for g, dt in zip(grads, ctx.in_dtypes)) + (None,) * 11


class _ExpertsFn(torch.autograd.Function):
    """BiBoFusedExperts.forward as one autograd node for a caller-owned routing: forward = bibo_moe_experts_fwd, backward
    = bibo_moe_experts_backward.  The gradient of the combine weights (moe.py:93) flows back to whoever made them."""

    @staticmethod
    def forward(ctx, x, top_w, w_gate_up, w_down, theta, idx, act, algo, want_counts, n_pos=0, n_neg=0, casts=None,
                cd=torch.bfloat16):
        cast = lambda t, d: (t if t.dtype == d else t.to(d)).contiguous()
        xb = cast(x.detach(), cd)
        gu, dn = casts if casts is not None else (cast(w_gate_up.detach(), cd), cast(w_down.detach(), cd))
        th, w = cast(theta.detach(), torch.float32), cast(top_w.detach(), torch.float32)
        out, counts = ops.experts_fwd(xb, idx, w, gu, dn, th, algo=algo, want_counts=want_counts, act=act, n_pos=n_pos,
                                      n_neg=n_neg)
        ctx.save_for_backward(xb, w, gu, dn, th, idx)
        ctx.act, ctx.specials = act, (n_pos, n_neg)
        ctx.in_dtypes = (x.dtype, top_w.dtype, w_gate_up.dtype, w_down.dtype, theta.dtype)
        if counts is None:
            counts = torch.empty(0, dtype=torch.int32, device=x.device)
        ctx.mark_non_differentiable(counts)
        return out, counts

    @staticmethod
    def backward(ctx, d_out, _d_counts):
        xb, w, gu, dn, th, idx = ctx.saved_tensors
        grads = ops.experts_backward(xb, d_out.to(xb.dtype).contiguous(), idx, w, gu, dn, th, act=ctx.act,
                                     n_pos=ctx.specials[0], n_neg=ctx.specials[1])
        return tuple(g.to(dt) for g, dt in zip(grads, ctx.in_dtypes)) + (None,) * 8


def _backward_covers(experts, cd) -> bool:
    """Whether bibo_moe_backward takes this size in compute dtype cd, as the library itself answers: the MFMA kernels
    for bf16 with hidden and expert sizes that are multiples of 128 (expert size up to 512), the generic kernels for
    everything else that keeps a row's 2H + 5I floats within 64 KB of LDS."""
    return ops.backward_supported(experts.hidden_size, experts.intermediate_size, experts.num_routed_experts, cd,
                                  experts.num_pos, experts.num_neg)


_NO_BACKWARD = ("no backward pass for this size: the MFMA kernels take bf16 with hidden and expert sizes that are multiples "
                "of 128 and expert sizes up to 512, the generic ones rows of 2 * hidden_size + 5 * moe_intermediate_size "
                "floats up to 64 KB")


class _CastCache:
    """Device copies of parameters in the dtype the kernels want, refreshed when the parameter changes.

    A change is seen through the parameter's storage address, version counter, device and dtype.  In-place writes
    through `p.data` (`p.data.copy_(...)`, `p.data.fill_(...)`) bump none of them; after such a write call
    `invalidate()` (the modules below expose it as `refresh_weights()`), as `load_state_dict` and `Module._apply`
    (`.to()`, `.cuda()`, `.bfloat16()`) do by themselves here."""

    def __init__(self):
        self._store = {}

    def invalidate(self):
        self._store.clear()

    def get(self, name: str, p: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        if p.dtype == dtype and p.is_contiguous():
            return p.detach()
        key = (name, dtype)
        tag = (p.data_ptr(), p._version, p.device, p.dtype)
        hit = self._store.get(key)
        if hit is None or hit[0] != tag:
            hit = (tag, p.detach().to(dtype).contiguous())
            self._store[key] = hit
        return hit[1]


def _compute_dtype(x: torch.Tensor) -> torch.dtype:
    """bf16 activations, or fp32 activations under bf16 autocast, run the bf16 kernels; plain fp32 runs the
    fp32 generic kernels (the regimes of ablate/common/train.py:589,677 and tests/test_moe.py:252-259)."""
    if x.dtype == torch.bfloat16:
        return torch.bfloat16
    if x.dtype == torch.float32:
        if torch.is_autocast_enabled() and torch.get_autocast_dtype("cuda") == torch.bfloat16:
            return torch.bfloat16
        return torch.float32
    raise TypeError(f"hidden states must be bfloat16 or float32, got {x.dtype}")


class BiBoMoERouter(nn.Module):
    """Sigmoid router with a non-grad selection bias (src/modeling/ffn/router.py:10-51)."""

    def __init__(self, config):
        super().__init__()
        self.num_routed_experts = config.num_routed_experts
        self.top_k = config.num_experts_per_tok
        self.norm_topk_prob = config.norm_topk_prob
        if self.num_routed_experts > L.MAX_EXPERTS or self.top_k > L.MAX_TOPK:
            raise NotImplementedError(f"the HIP router supports at most {L.MAX_EXPERTS} experts and top-{L.MAX_TOPK}")
        self.bias = nn.Parameter(torch.zeros(self.num_routed_experts), requires_grad=False)
        self._probe_gap = False
        self.boundary_gap = None
        self.gate_proj = nn.Linear(config.hidden_size, self.num_routed_experts, bias=False)
        nn.init.normal_(self.gate_proj.weight, mean=0.0, std=getattr(config, "initializer_range", 0.02))
        self._cache = _CastCache()
        self.register_load_state_dict_post_hook(lambda module, incompatible: module._cache.invalidate())

    def refresh_weights(self):
        """Drop the cached kernel-dtype copies of weight and bias (needed after a write through `.data`)."""
        self._cache.invalidate()

    def _apply(self, fn, *a, **kw):
        self._cache.invalidate()
        return super()._apply(fn, *a, **kw)

    def _operands(self, hidden_states):
        cd = _compute_dtype(hidden_states)
        x = hidden_states.detach().reshape(-1, hidden_states.shape[-1])
        x = x.to(cd) if x.dtype != cd else x
        return (x.contiguous(), self._cache.get("w", self.gate_proj.weight, cd),
                self._cache.get("b", self.bias, torch.float32))

    @_no_compile
    def router_logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """fp32 logits [B*S, E] (router.py:25-26); kept in fp32, never rounded to the model dtype."""
        x, w, b = self._operands(hidden_states)
        return ops.router_fwd(x, w, b, self.top_k, self.norm_topk_prob, want_logits=True)[2]

    @_no_compile
    def forward(self, hidden_states: torch.Tensor):
        bsz, seq, _ = hidden_states.shape
        x, w, b = self._operands(hidden_states)
        probe = self._probe_gap and self.top_k < self.num_routed_experts
        idx, wgt, _, gap = ops.router_fwd(x, w, b, self.top_k, self.norm_topk_prob, want_gap=probe)
        if probe:
            self.boundary_gap = gap.mean()                                   # router.py:33-36
        idx = idx.view(bsz, seq, -1).long()
        if _wants_grad(hidden_states, self.gate_proj.weight):
            # the kernel's selection, the weights again as differentiable tensor operations (router.py:25-26,31,41-47)
            scores = torch.sigmoid(self.gate_proj(hidden_states).float())
            raw = scores.gather(-1, idx)
            if self.top_k > 1 and self.norm_topk_prob == "softmax":
                return idx, torch.softmax(raw, dim=-1)
            if self.top_k > 1 and self.norm_topk_prob:
                return idx, raw / (raw.sum(dim=-1, keepdim=True) + 1e-20)
            return idx, raw
        return idx, wgt.view(bsz, seq, -1)


class BiBoFusedExperts(nn.Module):
    """Stacked GLU experts with the Radial NormSiLU activation (src/modeling/ffn/moe.py:19-101)."""

    def __init__(self, config):
        super().__init__()
        self.num_glu_experts = config.num_glu_experts
        self.special_expert_pairs = config.special_expert_pairs
        self.num_routed_experts = config.num_routed_experts
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.moe_intermediate_size
        num_pos = getattr(config, "num_pos_identity_experts", self.special_expert_pairs)
        num_neg = getattr(config, "num_neg_identity_experts", self.special_expert_pairs)
        self.pos_start = self.num_glu_experts
        self.pos_end = self.pos_start + num_pos
        self.neg_start = self.pos_end
        self.neg_end = self.neg_start + num_neg
        self.num_pos, self.num_neg = num_pos, num_neg
        if self.neg_end != self.num_routed_experts:
            raise ValueError(f"{self.num_glu_experts} GLU + {num_pos} +Identity + {num_neg} -Identity experts do not add "
                             f"up to num_routed_experts={self.num_routed_experts}")
        if self.num_routed_experts > L.MAX_EXPERTS:
            raise NotImplementedError(f"the HIP kernels support at most {L.MAX_EXPERTS} experts")
        std = getattr(config, "initializer_range", 0.02)
        self.gate_up_proj = nn.Parameter(torch.empty(self.num_glu_experts, 2 * self.intermediate_size, self.hidden_size))
        self.down_proj = nn.Parameter(torch.empty(self.num_glu_experts, self.hidden_size, self.intermediate_size))
        nn.init.normal_(self.gate_up_proj, mean=0.0, std=std)
        nn.init.normal_(self.down_proj, mean=0.0, std=std)
        self.radial_theta = nn.Parameter(torch.zeros(self.num_glu_experts))
        self.algo = "auto"
        # The reference module hardcodes p = sigmoid(theta) (moe.py:89); its harness switches the external kernel
        # to p = tanh(theta) or to plain SwiGLU through two globals (RADIAL_P / EXPERT_ACT,
        # ablate/common/patches.py:53-69).  Here they are attributes of the module.
        self.radial_p = getattr(config, "radial_p", "sigmoid")
        self.expert_act = getattr(config, "expert_act", "radial")
        self._cache = _CastCache()
        self.register_load_state_dict_post_hook(lambda module, incompatible: module._cache.invalidate())

    @property
    def act(self) -> str:
        if self.expert_act == "silu":
            return "silu"
        if self.expert_act != "radial" or self.radial_p not in ("sigmoid", "tanh"):
            raise ValueError(f"expert_act={self.expert_act!r} / radial_p={self.radial_p!r}: expected 'radial' or 'silu' "
                             "and 'sigmoid' or 'tanh'")
        return "radial_tanh" if self.radial_p == "tanh" else "radial"

    def refresh_weights(self):
        """Drop the cached kernel-dtype copies of the weights (needed after a write through `.data`)."""
        self._cache.invalidate()

    def _apply(self, fn, *a, **kw):
        self._cache.invalidate()
        return super()._apply(fn, *a, **kw)

    def _weights(self, cd):
        return (self._cache.get("gu", self.gate_up_proj, cd), self._cache.get("dn", self.down_proj, cd),
                self._cache.get("th", self.radial_theta, torch.float32))

    @_no_compile
    def forward(self, hidden_states: torch.Tensor, top_k_indices: torch.Tensor, top_k_weights: torch.Tensor,
                _want_counts: bool = False):
        if _wants_grad(hidden_states, top_k_weights, self.gate_up_proj, self.down_proj, self.radial_theta):
            cd = _compute_dtype(hidden_states)
            if not _backward_covers(self, cd):
                raise NotImplementedError(_NO_BACKWARD)
            out, counts = _ExpertsFn.apply(hidden_states, top_k_weights, self.gate_up_proj, self.down_proj, self.radial_theta,
                                           top_k_indices.detach().to(torch.int32).contiguous(), self.act, self.algo,
                                           _want_counts, self.num_pos, self.num_neg, self._weights(cd)[:2], cd)
            out = out if out.dtype == hidden_states.dtype else out.to(hidden_states.dtype)
            return (out, counts) if _want_counts else out
        cd = _compute_dtype(hidden_states)
        x = hidden_states.detach()
        x = (x.to(cd) if x.dtype != cd else x).contiguous()
        idx = top_k_indices.detach().to(torch.int32).contiguous()
        w = top_k_weights.detach().to(torch.float32).contiguous()
        gu, dn, th = self._weights(cd)
        out, counts = ops.experts_fwd(x, idx, w, gu, dn, th, algo=self.algo, want_counts=_want_counts,
                                      n_pos=self.num_pos, n_neg=self.num_neg, act=self.act)   # specials: moe.py:95-99
        out = out if out.dtype == hidden_states.dtype else out.to(hidden_states.dtype)   # moe.py:101
        return (out, counts) if _want_counts else out


class BiBoSharedMLP(nn.Module):
    """The shared expert: BiBoMLP (src/modeling/ffn/mlp.py:9-35) at width moe_intermediate_size * num_shared_experts;
    same parameter names, so `shared_experts_list.0.*` of a reference checkpoint loads."""

    def __init__(self, config, intermediate_size):
        super().__init__()
        act = getattr(config, "hidden_act", "silu")
        if act != "silu":
            raise NotImplementedError(f"shared expert with hidden_act={act!r}; only 'silu' is implemented")
        self.hidden_size = config.hidden_size
        self.intermediate_size = intermediate_size
        self.gate_proj = nn.Linear(self.hidden_size, intermediate_size, bias=False)
        self.up_proj = nn.Linear(self.hidden_size, intermediate_size, bias=False)
        self.down_proj = nn.Linear(intermediate_size, self.hidden_size, bias=False)

    def forward(self, x):
        return self.down_proj(nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))         # mlp.py:34-35


class BiBoCausalConv1D(nn.Module):
    """The convolutional shared expert (src/modeling/ffn/experts.py:11-34): the gate is a causal Conv1d over the
    sequence (left padding kernel_size - 1), up and down are linear; same parameter names, so
    `shared_experts_list.0.*` of a reference checkpoint loads.  Dense over every token: stock operations."""

    def __init__(self, config):
        super().__init__()
        act = getattr(config, "hidden_act", "silu")
        if act != "silu":
            raise NotImplementedError(f"shared expert with hidden_act={act!r}; only 'silu' is implemented")
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.moe_intermediate_size
        self.kernel_size_gate = int(getattr(config, "kernel_size", 3))
        self.causal_padding_gate = self.kernel_size_gate - 1
        self.gate_conv = nn.Conv1d(self.hidden_size, self.intermediate_size, self.kernel_size_gate, padding=0, bias=False)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=False)

    def forward(self, x):
        xp = nn.functional.pad(x.transpose(1, 2), (self.causal_padding_gate, 0))              # experts.py:26-27
        gate = self.gate_conv(xp).transpose(1, 2)                                              # [B,S,I]
        return self.down_proj(nn.functional.silu(gate) * self.up_proj(x))                      # experts.py:30


class BiBoMoELayer(nn.Module):
    """Router + experts + balancing state (src/modeling/ffn/moe.py:104-183)."""

    def __init__(self, config):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.num_routed_experts = config.num_routed_experts
        self.num_experts_per_tok = config.num_experts_per_tok
        self.bias_update_factor = config.bias_update_factor
        self.bias_update_threshold = config.bias_update_threshold
        self.register_buffer("accumulated_tpe", torch.zeros(config.num_routed_experts, dtype=torch.float))
        self._fwd_step = 0
        self._update_every = None
        # Training forwards keep routing, permutation and gate/up pre-activations for their backward pass (about
        # 4 * moe_intermediate_size bytes per routed slot until that backward has run), as autograd keeps the reference
        # layer's activations; False makes the backward pass compute them again from the input rows instead.
        self.keep_activations = True
        self.experts = BiBoFusedExperts(config)
        self.use_shared_expert = getattr(config, "use_shared_expert", False)
        self.shared_experts_list = nn.ModuleList()
        if self.use_shared_expert:
            # moe.py:118-127.  The shared expert is a dense SwiGLU over every token: stock GEMMs, not part of the
            # sparse path, so it runs as ordinary tensor operations next to the library call.
            if getattr(config, "shared_expert_type", "mlp") == "conv":
                self.shared_experts_list.append(BiBoCausalConv1D(config))
            else:
                n_sh = int(getattr(config, "num_shared_experts", 1))
                self.shared_experts_list.append(BiBoSharedMLP(config, config.moe_intermediate_size * n_sh))
        self.gate = BiBoMoERouter(config)

    # ---- balancing (host logic over device tensors, moe.py:131-155) ----
    @torch.no_grad()
    def update_bias(self, tokens_per_expert: torch.Tensor):
        u = self.bias_update_factor
        if u <= 0:
            return
        load = tokens_per_expert.detach().float()
        load = load / load.sum().clamp_min(1.0)
        self.gate.bias.add_(u * (load.mean() - load))        # proportional step; deviations sum to zero

    @_no_compile
    @torch.no_grad()
    def _balance_step(self, top_k_indices, num_tokens, counts=None):
        """Accumulate this forward's per-expert token counts; every `_update_every` forwards hand the
        accumulated vector back (all-reduced across ranks when a process group exists) and reset it.
        `counts` lets the caller pass the histogram the permutation kernel already produced."""
        if counts is None:
            counts = torch.bincount(top_k_indices.reshape(-1), minlength=self.num_routed_experts)
        self.accumulated_tpe += counts.to(self.accumulated_tpe.dtype)
        if self._update_every is None:
            self._update_every = max(1, round(self.bias_update_threshold / max(num_tokens, 1)))
        self._fwd_step += 1
        if self._fwd_step % self._update_every != 0:
            return None
        import torch.distributed as dist
        if dist.is_available() and dist.is_initialized():
            dist.all_reduce(self.accumulated_tpe, op=dist.ReduceOp.SUM)
        tpe = self.accumulated_tpe.clone()
        self.accumulated_tpe.zero_()
        return tpe

    def _hooks_present(self) -> bool:
        g, e = self.gate, self.experts
        return bool(g._forward_hooks or g._forward_pre_hooks or e._forward_hooks or e._forward_pre_hooks
                    or g._probe_gap or nn.modules.module._global_forward_hooks
                    or nn.modules.module._global_forward_pre_hooks)

    @_no_compile
    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        bsz, seq, hdim = hidden_states.shape
        num_tokens = bsz * seq
        balancing = self.training and self.bias_update_factor > 0
        if self._hooks_present():
            # module-by-module, so hooks on `gate` and `experts` observe exactly what the reference's
            # would (ablate/common/router_trace.py hooks both)
            top_idx, top_w = self.gate(hidden_states)
            res = self.experts(hidden_states.reshape(num_tokens, hdim), top_idx.view(num_tokens, -1),
                               top_w.view(num_tokens, -1), _want_counts=balancing)
            out, counts = res if balancing else (res, None)
        elif _wants_grad(hidden_states, self.gate.gate_proj.weight, self.experts.gate_up_proj, self.experts.down_proj,
                         self.experts.radial_theta):
            out, counts = self._differentiable_forward(hidden_states.reshape(num_tokens, hdim), balancing)
            out = out if out.dtype == hidden_states.dtype else out.to(hidden_states.dtype)
            top_idx = None
        else:
            cd = _compute_dtype(hidden_states)
            x = hidden_states.detach().reshape(num_tokens, hdim)
            x = (x.to(cd) if x.dtype != cd else x).contiguous()
            gu, dn, th = self.experts._weights(cd)
            wr = self.gate._cache.get("w", self.gate.gate_proj.weight, cd)
            b = self.gate._cache.get("b", self.gate.bias, torch.float32)
            out, _, _, counts, _ = ops.moe_forward(x, wr, b, gu, dn, th, self.num_experts_per_tok,
                                                   norm=self.gate.norm_topk_prob, algo=self.experts.algo,
                                                   want_counts=balancing, n_pos=self.experts.num_pos,
                                                   n_neg=self.experts.num_neg, act=self.experts.act)
            out = out if out.dtype == hidden_states.dtype else out.to(hidden_states.dtype)
            top_idx = None
        out = out.view(bsz, seq, hdim)
        if self.use_shared_expert:                             # moe.py:174-176
            out = out + self.shared_experts_list[0](hidden_states).to(out.dtype)
        if balancing:                                          # exactly once per training forward
            tpe = self._balance_step(top_idx, num_tokens, counts=counts)
            if tpe is not None:
                self.update_bias(tpe)
        return out

    def _differentiable_forward(self, x: torch.Tensor, want_counts: bool):
        """x [T,H] -> (out [T,H] in the compute dtype with an autograd graph, counts|None).  bf16 compute (bf16
        activations, or fp32 activations under bf16 autocast) with H and I multiples of 128 and I <= 512 runs the MFMA
        backward; fp32 compute and every other size run the generic kernels."""
        e = self.experts
        cd = _compute_dtype(x)
        if not _backward_covers(e, cd):
            raise NotImplementedError(_NO_BACKWARD)
        gu, dn, _ = e._weights(cd)
        casts = (self.gate._cache.get("w", self.gate.gate_proj.weight, cd), gu, dn)
        out, counts = _MoELayerFn.apply(x, self.gate.gate_proj.weight, e.gate_up_proj, e.down_proj, e.radial_theta,
                                        self.gate.bias, self.num_experts_per_tok, self.gate.norm_topk_prob, e.act, e.algo,
                                        want_counts, e.num_pos, e.num_neg, casts, cd, self.keep_activations)
        return out, (counts if want_counts else None)

    @_no_compile
    def ffn_forward(self, hidden_states: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                    bf16_stream: bool = False, bf16_moe_out: bool = False, residual=None) -> torch.Tensor:
        """The caller's seam, BiBoDecoderLayer._ffn_forward (src/modeling/layers.py:57-67):
        `hidden_states + self(rmsnorm(hidden_states))` with `norm_weight`/`eps` of post_attention_layernorm
        (src/modeling/norm.py:19-24), as ONE library call: the norm feeds the block from the workspace and the
        residual is added in the combine kernel.  With hooks or a gap probe present, or with an fp32 stream
        under bf16 autocast, the block runs as in forward and norm and residual are ordinary tensor operations
        around it.  `bf16_stream` and `bf16_moe_out` are the decoder layer's two switches (layers.py:28,37):
        the sum is cast to bf16, and the block's output is rounded to bf16 before it enters the sum.
        `residual`: None adds `hidden_states` itself; a tensor of the same shape is added instead; False adds
        nothing (norm + block only: `_attn_res_mlp_forward` of the experimental layer, exp/modeling_bibo.py:429-431)."""
        bsz, seq, hdim = hidden_states.shape
        num_tokens = bsz * seq
        if (self._hooks_present() or self.use_shared_expert or hidden_states.dtype != _compute_dtype(hidden_states)
                or (bf16_moe_out and hidden_states.dtype != torch.bfloat16)
                or _wants_grad(hidden_states, norm_weight, self.gate.gate_proj.weight, self.experts.gate_up_proj,
                               self.experts.down_proj, self.experts.radial_theta)):
            # (an fp32 residual stream under bf16 autocast keeps its fp32 norm and fp32 residual add; with autograd
            # on, norm and residual are ordinary differentiable operations around the differentiable block)
            xf = hidden_states.float()
            xn = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(hidden_states.dtype)    # norm.py:21-24
            blk = self.forward((norm_weight * xn).to(hidden_states.dtype))                             # layers.py:60-61
            blk = blk.to(torch.bfloat16) if bf16_moe_out else blk                                      # layers.py:62-63
            base = hidden_states if residual is None else residual
            out = blk.to(hidden_states.dtype) if residual is False else base + blk.to(hidden_states.dtype)   # layers.py:64
            return out.to(torch.bfloat16) if bf16_stream else out
        balancing = self.training and self.bias_update_factor > 0
        cd = _compute_dtype(hidden_states)
        h = hidden_states.detach().reshape(num_tokens, hdim)
        h = (h.to(cd) if h.dtype != cd else h).contiguous()
        gu, dn, th = self.experts._weights(cd)
        wr = self.gate._cache.get("w", self.gate.gate_proj.weight, cd)
        b = self.gate._cache.get("b", self.gate.bias, torch.float32)
        nw = norm_weight.detach().float().contiguous()
        out, _, _, counts = ops.ffn_forward(h, nw, float(eps), wr, b, gu, dn, th, self.num_experts_per_tok,
                                            norm=self.gate.norm_topk_prob, algo=self.experts.algo, want_counts=balancing,
                                            n_pos=self.experts.num_pos, n_neg=self.experts.num_neg, act=self.experts.act,
                                            round_block_out=bf16_moe_out and cd == torch.bfloat16,
                                            residual=(residual if residual is None or residual is False
                                                      else residual.detach().reshape(num_tokens, hdim).to(cd).contiguous()))
        if balancing:                                          # exactly once per training forward
            tpe = self._balance_step(None, num_tokens, counts=counts)
            if tpe is not None:
                self.update_bias(tpe)
        out = out.view(bsz, seq, hdim)
        out = out if out.dtype == hidden_states.dtype else out.to(hidden_states.dtype)
        return out.to(torch.bfloat16) if bf16_stream else out

