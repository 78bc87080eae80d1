"""CPU-side checks: the C-ABI library loads and exports what the header declares, argument errors are
reported before anything is launched, and the host mirror keeps the reference's module contract
(tests/test_moe.py:14-24,198-310 of the reference for layout and balancing closed forms)."""
import ctypes
import pathlib
import re

import pytest
import torch

import bibo_amd
from bibo_amd import _lib as L
from bibo_amd import ops

ROOT = pathlib.Path(__file__).resolve().parents[1]


def make_config(**kw):
    base = dict(hidden_size=64, intermediate_size=96, moe_intermediate_size=96, num_routed_experts=8,
                special_expert_pairs=0, num_experts_per_tok=2)
    base.update(kw)
    return bibo_amd.BiBoMoEConfig(**base)


# ------------------------------------------------------------------ C ABI
def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "bibo_moe.h").read_text()
    declared = set(re.findall(r"^(?:int|const char\*)\s+(bibo_moe_\w+)\s*\(", header, re.M))
    assert declared == set(L.SYMBOLS), "binding and header disagree"
    lib = L.lib()
    for name in declared:
        assert hasattr(lib, name)
    assert lib.bibo_moe_abi_version() == L.ABI_VERSION == 3
    m = re.search(r"#define BIBO_MOE_ABI_VERSION (\d+)", header)
    assert m and int(m.group(1)) == L.ABI_VERSION


def test_shape_struct_matches_the_header_and_the_documented_binding():
    """bibo_moe_shape is read by pointer: a binding with fewer fields makes the library read past the caller's
    struct.  The ctypes structure, the header and the example in the integration guide at the repository root must agree field for field."""
    header = (ROOT / "include" / "bibo_moe.h").read_text()
    body = re.search(r"typedef struct bibo_moe_shape \{(.*?)\} bibo_moe_shape;", header, re.S).group(1)
    fields = re.findall(r"int32_t\s+(\w+);", body)
    assert fields == [n for n, _ in L.Shape._fields_]
    assert ctypes.sizeof(L.Shape) == 4 * len(fields) == 40
    doc = (ROOT / "INTEGRATION.md").read_text()
    names = re.search(r"for n in \(([^)]*)\)\]", doc).group(1)
    assert [n.strip().strip('"') for n in names.split(",")] == fields
    assert "strerror.restype = ctypes.c_char_p" in doc


def test_argument_errors_are_reported_without_a_gpu():
    lib = L.lib()
    out = ctypes.c_size_t(0)
    ok = L.Shape(8192, 768, 64, 6, 384, L.DTYPE_BF16)
    assert lib.bibo_moe_workspace_bytes(ctypes.byref(ok), ctypes.byref(out)) == 0 and out.value > 0
    for bad in (L.Shape(8, 64, 65, 2, 32, 0), L.Shape(8, 64, 8, 9, 32, 0), L.Shape(8, 64, 4, 5, 32, 0),
                L.Shape(-1, 64, 8, 2, 32, 0), L.Shape(8, 0, 8, 2, 32, 0)):
        assert lib.bibo_moe_workspace_bytes(ctypes.byref(bad), ctypes.byref(out)) == -2
    assert lib.bibo_moe_workspace_bytes(ctypes.byref(L.Shape(8, 64, 8, 2, 32, 7)), ctypes.byref(out)) == -3
    assert lib.bibo_moe_workspace_bytes(None, ctypes.byref(out)) == -1
    # stage entry points validate before launching
    assert lib.bibo_moe_router_fwd(None, None, None, 4, 64, 8, 2, 0, 1, None, None, None, None, None) == -1
    assert lib.bibo_moe_router_fwd(None, None, None, 4, 64, 8, 9, 0, 1, None, None, None, None, None) == -2
    assert lib.bibo_moe_gateup_fwd(None, None, None, None, None, 4, 64, 8, 2, 96, 0, L.ALGO_MFMA, 0, None, None) == -6
    # the streaming kernels exist only behind the composite entry points
    assert lib.bibo_moe_gateup_fwd(None, None, None, None, None, 4, 1024, 64, 6, 512, 0, L.ALGO_STREAM, 0, None, None) == -6
    assert lib.bibo_moe_gateup_fwd(None, None, None, None, None, 4, 64, 8, 2, 96, 0, L.ALGO_GENERIC, 3, None, None) == -6   # no such activation
    assert lib.bibo_moe_permute(None, 4, 8, 2, None, None, None, None, None, 0, None) == -1
    # fused-kernel and caller-seam entry points
    assert lib.bibo_moe_gateup_down_fwd(None, None, None, None, None, None, None, None, 4, 768, 64, 6, 512, 0, 0, None, None) == -6
    assert lib.bibo_moe_gateup_down_fwd(None, None, None, None, None, None, None, None, 4, 768, 64, 6, 384, 0, 0, None, None) == -1
    assert lib.bibo_moe_combine_fwd(None, 1, 4, 64, 2, L.DTYPE_F32, None, None) == -3      # bf16 slot rows need a bf16 output
    assert lib.bibo_moe_rmsnorm_fwd(None, None, ctypes.c_float(1e-6), 4, 64, 0, None, None) == -1
    ffn = ctypes.c_size_t(0)
    assert lib.bibo_moe_ffn_workspace_bytes(ctypes.byref(ok), ctypes.byref(ffn)) == 0
    assert ffn.value >= out.value + 8192 * 768 * 2                 # the block's workspace plus the normalised activations
    assert lib.bibo_moe_ffn_forward(None, None, ctypes.c_float(1e-6), None, None, None, None, None, None, ctypes.byref(ok), 1, 0,
                                    None, None, None, None, None, 0, None) == -1
    assert b"workspace" in lib.bibo_moe_strerror(-4)
    with pytest.raises(RuntimeError, match="workspace"):
        L.check(-4, "x")


def test_training_pair_checks_its_arguments_without_a_gpu():
    """bibo_moe_train_state_bytes / bibo_moe_forward_train / bibo_moe_backward_saved: which shapes have the pair, and the
    errors found on the host before any launch."""
    lib = L.lib()
    n = ctypes.c_size_t(0)
    ok = L.Shape(8192, 768, 64, 6, 384, L.DTYPE_BF16)
    assert lib.bibo_moe_train_state_bytes(ctypes.byref(ok), ctypes.byref(n)) == 0
    assert n.value >= 8192 * 6 * (2 * 384 * 2 + 16) + 8192 * 64 * 4      # pre-activations, routing, permutation, logits
    assert lib.bibo_moe_train_state_bytes(ctypes.byref(ok), None) == -1
    assert lib.bibo_moe_train_state_bytes(None, ctypes.byref(n)) == -1
    for other in (L.Shape(64, 768, 64, 6, 384, L.DTYPE_F32), L.Shape(64, 1024, 64, 6, 512, L.DTYPE_BF16),
                  L.Shape(64, 200, 8, 2, 128, L.DTYPE_BF16)):
        assert lib.bibo_moe_train_state_bytes(ctypes.byref(other), ctypes.byref(n)) == -6
        assert lib.bibo_moe_forward_train(None, None, None, None, None, None, ctypes.byref(other), 1, None, None, None, 0, None, 0,
                                          None) == -6
    assert lib.bibo_moe_forward_train(None, None, None, None, None, None, ctypes.byref(ok), 1, None, None, None, 0, None, 0,
                                      None) == -1                                       # no state buffer
    assert lib.bibo_moe_forward_train(None, None, None, None, None, None, ctypes.byref(ok), 7, None, None, None, 0, None, 0,
                                      None) == -6                                       # no such normalisation mode
    fake = ctypes.c_void_p(4096)                                                        # aligned, never dereferenced here
    assert lib.bibo_moe_forward_train(None, None, None, None, None, None, ctypes.byref(ok), 1, None, None, fake, 256, None, 0,
                                      None) == -4                                       # state buffer too small
    assert lib.bibo_moe_backward_saved(None, None, None, None, None, None, ctypes.byref(ok), 1, None, 0, None, None, None, None,
                                       None, None, None, 0, None) == -1
    assert lib.bibo_moe_backward_saved(None, None, None, None, None, None, ctypes.byref(ok), 1, fake, 256, None, None, None, None,
                                       None, None, fake, 0, None) == -4
    assert lib.bibo_moe_backward_saved(None, None, None, None, None, None, ctypes.byref(ok), 1, ctypes.c_void_p(4100), 1 << 40,
                                       None, None, None, None, None, None, fake, 0, None) == -5   # misaligned state


def test_kernel_family_selection_is_exported():
    """bibo_moe_select_algo: what the composite calls run per workload, and which requests cannot be met."""
    from bibo_amd import ops
    assert ops.select_algo(8192, 768, 64, 6, 384) == "fused"            # prefill workload
    assert ops.select_algo(16384, 768, 64, 6, 384) == "fused"
    assert ops.select_algo(64, 1024, 64, 6, 512) == "stream"            # decode workload: 6 rows per expert
    assert ops.select_algo(512, 512, 64, 6, 256) == "fused"             # 48 rows per expert: past the streaming limit
    assert ops.select_algo(250, 512, 64, 6, 256) == "stream"            # 23.4 rows, register-resident weight rows
    assert ops.select_algo(300, 512, 64, 6, 256) == "fused"             # 28 rows: the fused kernel wins from about 24
    assert ops.select_algo(100, 768, 64, 6, 384) == "stream"            # 9.4 rows of 1.5 KB
    assert ops.select_algo(128, 768, 64, 6, 384) == "fused"             # 12 rows: wider rows are re-streamed per pass
    assert ops.select_algo(170, 1024, 64, 6, 512) == "stream"           # 16 rows; I = 512 is not fused, the tile path is slow
    assert ops.select_algo(341, 1024, 64, 6, 512) == "mfma"             # 32 rows of 2 KB: tiles win
    assert ops.select_algo(8192, 768, 64, 6, 384, L.DTYPE_F32) == "generic"
    assert ops.select_algo(8192, 768, 64, 6, 384, algo="mfma") == "mfma"
    with pytest.raises(RuntimeError, match="does not support"):
        ops.select_algo(8192, 768, 64, 6, 384, L.DTYPE_F32, algo="fused")
    with pytest.raises(RuntimeError, match="does not support"):
        ops.select_algo(64, 1000, 64, 6, 500, algo="stream")
    out = ctypes.c_int(0)
    assert L.lib().bibo_moe_select_algo(None, 0, ctypes.byref(out)) == -1


def test_bench_refuses_more_than_one_gpu():
    import subprocess, sys
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_cpu_tensors_are_refused_loudly():
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.router_fwd(x, torch.zeros(8, 64, dtype=torch.bfloat16), torch.zeros(8), 2)
    layer = bibo_amd.BiBoMoELayer(make_config())
    with torch.no_grad(), pytest.raises(RuntimeError, match="GPU"):
        layer(torch.zeros(1, 4, 64))


# ------------------------------------------------------------------ config + module contract
def test_config_derivations_follow_the_reference():
    c = bibo_amd.BiBoMoEConfig(intermediate_size=2304, num_experts_per_tok=6, num_routed_experts=64,
                               special_expert_pairs=0, norm_topk_prob=True)
    assert c.moe_intermediate_size == 384 and c.norm_topk_prob == "sum"
    assert c.bias_update_factor == 0.4 and c.bias_update_threshold == 8000 and c.num_glu_experts == 64
    c = bibo_amd.BiBoMoEConfig(num_routed_experts=8, special_expert_pairs=1, num_experts_per_tok=2)
    assert c.num_glu_experts == 6 and c.num_pos_identity_experts == 1
    with pytest.raises(ValueError):
        bibo_amd.BiBoMoEConfig(num_routed_experts=4, num_experts_per_tok=5, special_expert_pairs=0)
    with pytest.raises(ValueError):
        bibo_amd.BiBoMoEConfig(num_routed_experts=2, special_expert_pairs=1, num_experts_per_tok=1)
    with pytest.raises(ValueError):
        bibo_amd.BiBoMoEConfig(norm_topk_prob="max", special_expert_pairs=0)


def test_state_dict_layout_matches_the_reference_layer():
    c = make_config()
    layer = bibo_amd.BiBoMoELayer(c)
    sd = layer.state_dict()
    assert {k: tuple(v.shape) for k, v in sd.items()} == {
        "accumulated_tpe": (8,), "gate.bias": (8,), "gate.gate_proj.weight": (8, 64),
        "experts.gate_up_proj": (8, 192, 64), "experts.down_proj": (8, 64, 96), "experts.radial_theta": (8,)}
    assert layer.gate.bias.requires_grad is False and layer.experts.radial_theta.requires_grad
    assert float(layer.experts.radial_theta.detach().abs().max()) == 0.0
    e = layer.experts
    assert (e.pos_start, e.pos_end, e.neg_start, e.neg_end) == (8, 8, 8, 8)
    assert layer.gate.top_k == 2 and layer.gate.norm_topk_prob == "sum" and layer.gate._probe_gap is False
    assert not hasattr(layer.gate, "gate_conv")


def test_unsupported_configurations_raise():
    with pytest.raises(NotImplementedError, match="hidden_act"):
        bibo_amd.BiBoMoELayer(make_config(use_shared_expert=True, shared_expert_type="conv", hidden_act="gelu"))
    with pytest.raises(NotImplementedError, match="hidden_act"):
        bibo_amd.BiBoMoELayer(make_config(use_shared_expert=True, hidden_act="gelu"))
    with pytest.raises(ValueError, match="GLU"):
        make_config(num_routed_experts=4, num_pos_identity_experts=2, num_neg_identity_experts=2)


def test_conv_shared_expert_layout_and_causality():
    """src/modeling/ffn/experts.py:11-34: parameter names and shapes of the reference's conv expert; the gate is a
    causal convolution (output at position s sees inputs s-2..s only) and equals an explicit sum of shifted GEMMs."""
    layer = bibo_amd.BiBoMoELayer(make_config(use_shared_expert=True, shared_expert_type="conv", kernel_size=3))
    sd = layer.state_dict()
    assert sd["shared_experts_list.0.gate_conv.weight"].shape == (96, 64, 3)
    assert sd["shared_experts_list.0.up_proj.weight"].shape == (96, 64)
    assert sd["shared_experts_list.0.down_proj.weight"].shape == (64, 96)
    conv = layer.shared_experts_list[0].double()
    x = torch.randn(2, 7, 64, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    y = conv(x)
    w = conv.gate_conv.weight                                                    # [I, H, 3]; tap j looks back 2 - j
    xp = torch.nn.functional.pad(x, (0, 0, 2, 0))
    gate = sum(xp[:, j:j + 7] @ w[:, :, j].t() for j in range(3))
    ref = (torch.nn.functional.silu(gate) * (x @ conv.up_proj.weight.t())) @ conv.down_proj.weight.t()
    assert torch.allclose(y, ref, atol=1e-12)
    x2 = x.clone(); x2[:, 4:] += 1.0                                            # the future must not leak backwards
    assert torch.equal(conv(x2)[:, :4], y[:, :4]) and not torch.allclose(conv(x2)[:, 4:], y[:, 4:])


def test_expert_activation_switches():
    """The harness's RADIAL_P / EXPERT_ACT globals (ablate/common/patches.py:53-69) as module attributes."""
    e = bibo_amd.BiBoFusedExperts(make_config())
    assert e.act == "radial" and ops.act_code(e.act) == L.ACT_RADIAL_SIGMOID
    e.radial_p = "tanh"
    assert ops.act_code(e.act) == L.ACT_RADIAL_TANH
    e.expert_act = "silu"
    assert ops.act_code(e.act) == L.ACT_SILU
    e.expert_act = "gelu"
    with pytest.raises(ValueError, match="expert_act"):
        e.act
    with pytest.raises(ValueError, match="act must be"):
        ops.act_code("relu")
    assert ops.act_code(bibo_amd.BiBoFusedExperts(make_config(radial_p="tanh")).act) == L.ACT_RADIAL_TANH


def test_cast_cache_refreshes_on_load_and_on_request():
    """Kernel-dtype copies of the parameters follow load_state_dict, .to() and refresh_weights(); a write through
    `.data` alone is not seen (documented on _CastCache)."""
    from bibo_amd.moe import _CastCache
    c = _CastCache()
    p = torch.nn.Parameter(torch.ones(4))
    a = c.get("w", p, torch.bfloat16)
    assert a.dtype == torch.bfloat16 and c.get("w", p, torch.bfloat16) is a           # cached
    with torch.no_grad():
        p.mul_(2)                                                                      # in-place op: version bump
    assert float(c.get("w", p, torch.bfloat16)[0]) == 2.0
    p.data.fill_(5.0)                                                                  # invisible to the cache ...
    assert float(c.get("w", p, torch.bfloat16)[0]) == 2.0
    c.invalidate()                                                                     # ... until asked
    assert float(c.get("w", p, torch.bfloat16)[0]) == 5.0
    layer = bibo_amd.BiBoMoELayer(make_config())
    layer.experts._cache.get("gu", layer.experts.gate_up_proj, torch.bfloat16)
    layer.gate._cache.get("w", layer.gate.gate_proj.weight, torch.bfloat16)
    assert layer.experts._cache._store and layer.gate._cache._store
    layer.load_state_dict(layer.state_dict())
    assert not layer.experts._cache._store and not layer.gate._cache._store
    layer.experts._cache.get("gu", layer.experts.gate_up_proj, torch.bfloat16)
    layer.double()
    assert not layer.experts._cache._store
    layer.experts._cache.get("gu", layer.experts.gate_up_proj, torch.bfloat16)
    layer.experts.refresh_weights()
    assert not layer.experts._cache._store


def test_specials_and_shared_expert_follow_the_reference_layout():
    """moe.py:19-44,118-127: the weight tensors hold only the GLU experts, the router has a row per routed expert
    (specials included), the shared expert is a SwiGLU of width moe_intermediate_size * num_shared_experts."""
    layer = bibo_amd.BiBoMoELayer(make_config(num_routed_experts=8, special_expert_pairs=1, use_shared_expert=True,
                                              num_shared_experts=2))
    e = layer.experts
    assert (e.num_glu_experts, e.pos_start, e.pos_end, e.neg_start, e.neg_end) == (6, 6, 7, 7, 8)
    sd = layer.state_dict()
    assert sd["experts.gate_up_proj"].shape == (6, 192, 64) and sd["experts.down_proj"].shape == (6, 64, 96)
    assert sd["experts.radial_theta"].shape == (6,) and sd["gate.gate_proj.weight"].shape == (8, 64)
    assert sd["gate.bias"].shape == (8,) and sd["accumulated_tpe"].shape == (8,)
    assert sd["shared_experts_list.0.gate_proj.weight"].shape == (192, 64)
    assert sd["shared_experts_list.0.up_proj.weight"].shape == (192, 64)
    assert sd["shared_experts_list.0.down_proj.weight"].shape == (64, 192)
    asym = bibo_amd.BiBoMoELayer(make_config(num_routed_experts=8, num_pos_identity_experts=3, num_neg_identity_experts=0))
    assert (asym.experts.num_glu_experts, asym.experts.pos_end, asym.experts.neg_end) == (5, 8, 8)


def test_forward_under_autograd_has_no_cpu_path_either():
    """With gradients wanted the modules go to the library as without: host tensors are refused, not computed here."""
    layer = bibo_amd.BiBoMoELayer(make_config())
    with pytest.raises(RuntimeError, match="no CPU path"):
        layer(torch.zeros(1, 4, 64))
    with pytest.raises(RuntimeError, match="no CPU path"):
        layer.experts(torch.zeros(4, 64), torch.zeros(4, 2, dtype=torch.long), torch.ones(4, 2))


# ------------------------------------------------------------------ balancing closed forms
def test_bias_update_moves_toward_balance_and_keeps_the_mean():
    layer = bibo_amd.BiBoMoELayer(make_config(bias_update_factor=0.4))
    tpe = torch.full((8,), 10.0); tpe[0] = 100.0
    layer.update_bias(tpe)
    b = layer.gate.bias
    assert b[0] < 0 and (b[1:] > 0).all() and abs(float(b.mean())) < 1e-6
    share = tpe / tpe.sum()
    assert torch.allclose(b, 0.4 * (share.mean() - share), atol=1e-7)


def test_balanced_load_gives_no_update_and_zero_factor_disables():
    layer = bibo_amd.BiBoMoELayer(make_config(bias_update_factor=1.0))
    layer.update_bias(torch.full((8,), 100.0))
    assert float(layer.gate.bias.abs().max()) < 1e-6
    off = bibo_amd.BiBoMoELayer(make_config(bias_update_factor=0.0))
    off.update_bias(torch.tensor([1000.0] + [10.0] * 7))
    assert float(off.gate.bias.abs().max()) == 0.0
    empty = bibo_amd.BiBoMoELayer(make_config(bias_update_factor=0.4))
    empty.update_bias(torch.zeros(8))                       # nothing routed: clamp avoids 0/0
    assert torch.isfinite(empty.gate.bias).all()


def test_balance_step_fires_on_the_forward_step_interval():
    tokens = 16
    layer = bibo_amd.BiBoMoELayer(make_config(bias_update_threshold=tokens * 3)).train()
    idx = torch.zeros(2, 8, 2, dtype=torch.long)
    fired = [layer._balance_step(idx, tokens) is not None for _ in range(7)]
    assert layer._update_every == 3 and fired == [False, False, True, False, False, True, False]
    # counts accumulate between firings and reset after
    layer = bibo_amd.BiBoMoELayer(make_config(bias_update_threshold=tokens * 2)).train()
    assert layer._balance_step(idx, tokens) is None
    tpe = layer._balance_step(None, tokens, counts=torch.tensor([1, 2, 3, 4, 5, 6, 7, 4], dtype=torch.int32))
    assert tpe.tolist() == [33.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 4.0]
    assert float(layer.accumulated_tpe.abs().max()) == 0.0
