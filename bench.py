"""Benchmark of the BiBo sparse-MoE layer forward on one MI355X.

One step = one forward of the whole layer (router, permutation, gate/up + Radial NormSiLU, down +
combine) over one batch of the prefill workload (T=8192, H=768, E=64, k=6, I=384, bf16), inputs and
weights resident in HBM.  Prints one JSON line; see --help for the flags."""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import pathlib
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E

REPEATS = 5                   # timed repeats of --steps forwards; the median is reported


def measured_traffic(workload, kernel):
    """HBM-side bytes per launch of a kernel, as the rocprofv3 --pmc summaries under profiles/ record them
    (lines `traffic_bytes_per_launch <workload> <kernel> = <bytes>`); None when no profile covers it."""
    import re
    for f in sorted((ROOT / "profiles").glob("*.md")):
        m = re.search(rf"^traffic_bytes_per_launch {workload} {kernel} = (\d+)", f.read_text(), re.M)
        if m:
            return int(m.group(1))
    return None


def flops_layer(T, H, E, k, I):
    return 2 * T * H * E + 6 * T * k * H * I


def bytes_layer(T, H, E, k, I, e_active):
    return 2 * (3 * H * I * e_active + E * H + 2 * T * H) + 8 * E


class Layer:
    """Pre-allocated operands and a direct ctypes call per stage, so the timed loop does no allocation."""

    def __init__(self, name, dev, algo="auto"):
        import torch
        from bibo_amd import _lib as L
        from bibo_amd import ops
        from oracle import bibo_moe_oracle as O
        self.torch, self.L, self.ops = torch, L, ops
        self.cfg = cfg = O.CONFIGS[name]
        self.name = name
        p = O.make_inputs(**cfg)
        self.host = p
        self.dev = dev
        self.T, self.H, self.E, self.k, self.I = cfg["T"], cfg["H"], cfg["E"], cfg["k"], cfg["I"]
        self.S = self.T * self.k
        self.x = p["x"].to(dev)
        self.wr = p["w_router"].to(dev)
        self.bias = p["bias"].to(dev)
        self.wgu = p["w_gate_up"].to(dev)
        self.wd = p["w_down"].to(dev)
        self.theta = p["theta"].to(dev)
        T, H, E, k, I, S = self.T, self.H, self.E, self.k, self.I, self.S
        self.out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
        self.idx = torch.empty(T, k, dtype=torch.int32, device=dev)
        self.w = torch.empty(T, k, dtype=torch.float32, device=dev)
        self.counts = torch.empty(E, dtype=torch.int32, device=dev)
        self.offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
        self.perm_slot = torch.empty(S, dtype=torch.int32, device=dev)
        self.perm_token = torch.empty(S, dtype=torch.int32, device=dev)
        self.hidden = torch.empty(S, I, dtype=torch.bfloat16, device=dev)
        self.yw = torch.empty(S, H, dtype=torch.bfloat16, device=dev)
        self.ws = torch.empty(ops.workspace_bytes(T, H, E, k, I, L.DTYPE_BF16), dtype=torch.uint8, device=dev)
        self.shape = L.Shape(T, H, E, k, I, L.DTYPE_BF16)
        self.algo = ops.algo_code(algo)
        self.lib = L.lib()
        self.stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        self._fwd_args = (P(self.x), P(self.wr), P(self.bias), P(self.wgu), P(self.wd), P(self.theta),
                          ctypes.byref(self.shape), L.NORM_SUM, self.algo, P(self.out), P(self.idx), P(self.w),
                          None, None, P(self.ws), self.ws.numel(), self.stream)   # eval forward: no counts, no logits
        self._stages = {
            "router": (self.lib.bibo_moe_router_fwd,
                       (P(self.x), P(self.wr), P(self.bias), T, H, E, k, L.DTYPE_BF16, L.NORM_SUM, None, P(self.idx),
                        P(self.w), None, self.stream)),
            "permute": (self.lib.bibo_moe_permute,
                        (P(self.idx), T, E, k, P(self.counts), P(self.offsets), P(self.perm_slot), P(self.perm_token),
                         P(self.ws), self.ws.numel(), self.stream)),
        }
        # the expert stages the composite call runs for this shape: one fused launch + combine where the library
        # picks the fused kernel, else one kernel per projection (the streaming kernels have no stage entry points)
        self.family = ops.select_algo(T, H, E, k, I, L.DTYPE_BF16, algo)
        self.fused = self.family == "fused"
        if self.fused:
            self._stages.update({
                "gateup_down": (self.lib.bibo_moe_gateup_down_fwd,
                                (P(self.x), P(self.wgu), P(self.wd), P(self.theta), P(self.w), P(self.offsets),
                                 P(self.perm_slot), P(self.perm_token), T, H, E, k, I, L.DTYPE_BF16,
                                 L.ACT_RADIAL_SIGMOID, P(self.yw), self.stream)),
                "combine": (self.lib.bibo_moe_combine_fwd, (P(self.yw), 1, T, H, k, L.DTYPE_BF16, P(self.out), self.stream)),
            })
        else:
            stage_algo = self.algo if algo != "stream" else ops.algo_code("auto")
            self._stages.update({
                "gateup": (self.lib.bibo_moe_gateup_fwd,
                           (P(self.x), P(self.wgu), P(self.theta), P(self.offsets), P(self.perm_token), T, H, E, k, I,
                            L.DTYPE_BF16, stage_algo, L.ACT_RADIAL_SIGMOID, P(self.hidden), self.stream)),
                "down_combine": (self.lib.bibo_moe_down_combine_fwd,
                                 (P(self.hidden), P(self.wd), P(self.w), P(self.offsets), P(self.perm_slot), T, H, E, k, I,
                                  L.DTYPE_BF16, stage_algo, P(self.out), P(self.ws), self.ws.numel(), self.stream)),
            })

    def forward(self):
        rc = self.lib.bibo_moe_forward(*self._fwd_args)
        if rc != 0:
            self.L.check(rc, "bibo_moe_forward")

    def time_ffn_seam(self, steps, warmup):
        """One call of the block's caller seam, out = h + moe(rmsnorm(h)) (bibo_moe_ffn_forward), per step."""
        torch, L = self.torch, self.L
        nbytes = ctypes.c_size_t(0)
        L.check(self.lib.bibo_moe_ffn_workspace_bytes(ctypes.byref(self.shape), ctypes.byref(nbytes)), "ffn workspace")
        ws = torch.empty(nbytes.value, dtype=torch.uint8, device=self.dev)
        nw = torch.ones(self.H, dtype=torch.float32, device=self.dev)
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        args = (P(self.x), P(nw), ctypes.c_float(1e-6), None, P(self.wr), P(self.bias), P(self.wgu), P(self.wd), P(self.theta),
                ctypes.byref(self.shape), L.NORM_SUM, self.algo, P(self.out), None, None, None, P(ws), ws.numel(),
                self.stream)
        for _ in range(warmup):
            L.check(self.lib.bibo_moe_ffn_forward(*args), "bibo_moe_ffn_forward")
        torch.cuda.synchronize(self.dev)
        t0 = time.perf_counter()
        for _ in range(steps):
            self.lib.bibo_moe_ffn_forward(*args)
        torch.cuda.synchronize(self.dev)
        return (time.perf_counter() - t0) / steps

    def stage(self, name):
        fn, args = self._stages[name]
        rc = fn(*args)
        if rc != 0:
            self.L.check(rc, name)

    def time_forward(self, steps, warmup, repeats=REPEATS, weight_sets=1):
        """Seconds per step: `repeats` timed runs of `steps` forwards each (after `warmup` untimed ones), every run
        bracketed by a device synchronisation; returns (median, all runs).  weight_sets > 1 rotates the expert
        weights over that many separately allocated copies, so that no step finds its weights in the 256 MB
        Infinity Cache the step before left behind."""
        torch = self.torch
        calls = [self._fwd_args]
        if weight_sets > 1:
            P = lambda t: ctypes.c_void_p(t.data_ptr())
            self._rot = [(self.wgu.clone(), self.wd.clone()) for _ in range(weight_sets - 1)]
            for gu, dn in self._rot:
                a = list(self._fwd_args)
                a[3], a[4] = P(gu), P(dn)
                calls.append(tuple(a))
        fn = self.lib.bibo_moe_forward
        for i in range(warmup):
            self.L.check(fn(*calls[i % len(calls)]), "bibo_moe_forward")
        runs = []
        for _ in range(repeats):
            torch.cuda.synchronize(self.dev)
            t0 = time.perf_counter()
            for i in range(steps):
                fn(*calls[i % len(calls)])
            torch.cuda.synchronize(self.dev)
            runs.append((time.perf_counter() - t0) / steps)
        self._rot = None
        return sorted(runs)[len(runs) // 2], runs

    def time_stages(self, steps):
        """Average duration of each stage, HIP events on the launch stream around every call (an event pair also
        spans the gap to the next launch, so a stage reads 1-2 us longer than its kernel alone)."""
        torch = self.torch
        names = list(self._stages)
        for n in names:
            self.stage(n)
        torch.cuda.synchronize(self.dev)
        acc = {n: 0.0 for n in names}
        for _ in range(steps):
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(len(names) + 1)]
            evs[0].record()
            for i, n in enumerate(names):
                self.stage(n)
                evs[i + 1].record()
            torch.cuda.synchronize(self.dev)
            for i, n in enumerate(names):
                acc[n] += evs[i].elapsed_time(evs[i + 1]) * 1e-3
        return {n: v / steps for n, v in acc.items()}

    def check(self):
        """Parity of the benchmarked configuration against the oracle on a token sample."""
        import numpy as np
        from oracle import bibo_moe_oracle as O
        torch = self.torch
        self.forward()
        torch.cuda.synchronize(self.dev)
        idx = self.idx.cpu().numpy()
        w = self.w.cpu().numpy()
        rng = np.random.default_rng(0)
        sample = rng.choice(self.T, min(self.T, 128), replace=False)
        p = self.host
        ref = O.experts_forward(p["x"][sample], idx[sample], w[sample], p["w_gate_up"], p["w_down"], p["theta"])
        got = self.out.cpu()[sample].double()
        active = int(np.unique(idx).size)                      # experts that received at least one token
        return ((got - ref.double()).abs().max() / ref.double().abs().max()).item(), active


def cpu_baseline(name, budget_s=20.0, sample_tokens=8192):
    """The reference's eager CPU path (oracle restatement) timed on this box's host cores: bf16 weights and
    activations as the workload names them, and fp32 as a second line (CPU bf16 GEMMs are slow without a matrix
    unit); 3 warm-up forwards, then at least 5 timed ones within the time budget, median."""
    import statistics
    import torch
    from oracle import bibo_moe_oracle as O
    cfg = dict(O.CONFIGS[name])
    T = min(cfg["T"], sample_tokens)
    p = O.make_inputs(**{**cfg, "T": T})
    cores = torch.get_num_threads()
    lines = {}
    for label, cast in (("bf16", lambda t: t), ("fp32", lambda t: t.float())):
        q = {k_: (cast(v) if isinstance(v, torch.Tensor) and v.dtype == torch.bfloat16 else v) for k_, v in p.items()}
        for _ in range(3):
            O.eager_loop_forward(**q)
        times = []
        t_start = time.perf_counter()
        while len(times) < 5 or (time.perf_counter() - t_start) < budget_s / 2:
            t0 = time.perf_counter()
            O.eager_loop_forward(**q)
            times.append(time.perf_counter() - t0)
            if len(times) >= 400:
                break
        med = statistics.median(times)
        lines[label] = {"tokens_per_s": T / med, "median_s": med, "timed_forwards": len(times)}
    best = max(lines, key=lambda l: lines[l]["tokens_per_s"])
    return {"value": lines[best]["tokens_per_s"], "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"first {T} tokens of the {name} workload (same weights), eager per-expert loop; value = the faster "
                      f"dtype ({best}); 3 warm-up forwards, median of the timed ones",
            "bf16": lines["bf16"], "fp32": lines["fp32"]}


def side_workload(name, dev, algo, steps, warmup):
    """A parity-test workload timed next to the headline one: us/step, TFLOP/s, % of peak, load shape."""
    import numpy as np
    lay = Layer(name, dev, algo)
    rel, active = lay.check()
    sec, _ = lay.time_forward(steps, warmup)
    cnt = np.bincount(lay.idx.cpu().numpy().reshape(-1), minlength=lay.E)
    fl = flops_layer(lay.T, lay.H, lay.E, lay.k, lay.I)
    nbytes = bytes_layer(lay.T, lay.H, lay.E, lay.k, lay.I, active)
    hot = np.sort(cnt)[::-1]
    return {"workload": f"{name}: T={lay.T} H={lay.H} E={lay.E} k={lay.k} I={lay.I} bf16", "kernel_family": lay.family,
            "us_per_step": sec * 1e6, "tokens_per_s": lay.T / sec, "tflops": fl / sec / 1e12,
            "pct_bf16_mfma_peak": 100.0 * fl / sec / 1e12 / PEAK_BF16_TFLOPS,
            "algorithmic_gbs": nbytes / sec / 1e9, "pct_hbm_peak": 100.0 * nbytes / sec / 1e9 / PEAK_HBM_GBS,
            "experts_active": active, "rows_per_expert_max": int(hot[0]), "rows_per_expert_min": int(hot[-1]),
            "share_of_slots_on_4_busiest_experts": float(hot[:4].sum() / max(1, cnt.sum())),
            "parity_rel_err_sample": rel}


def backward_pass(lay, steps, warmup):
    """The layer's backward (bibo_moe_backward) on the headline workload, next to its forward: us/step and algorithmic
    TFLOP/s (twice the forward's contraction flops: one GEMM per operand gradient; what the call recomputes does not
    count)."""
    import torch
    from bibo_amd import ops
    g = torch.Generator(device=lay.dev).manual_seed(9)
    d_out = torch.randn(lay.T, lay.H, device=lay.dev, generator=g).to(torch.bfloat16)
    args = (lay.x, d_out, lay.wr, lay.bias, lay.wgu, lay.wd, lay.theta, lay.k)
    for _ in range(max(2, warmup // 4)):
        grads = ops.moe_backward(*args)
    runs = []
    n = max(5, steps // 10)
    for _ in range(3):
        torch.cuda.synchronize(lay.dev)
        t0 = time.perf_counter()
        for _ in range(n):
            grads = ops.moe_backward(*args)
        torch.cuda.synchronize(lay.dev)
        runs.append((time.perf_counter() - t0) / n)
    sec = sorted(runs)[1]
    fl = 2.0 * flops_layer(lay.T, lay.H, lay.E, lay.k, lay.I)
    res = {"entry": "bibo_moe_backward: d_x, d_w_router, d_w_gate_up, d_w_down, d_theta from d_out", "us_per_step": sec * 1e6,
           "steps_timed": n, "tflops": fl / sec / 1e12, "pct_bf16_mfma_peak": 100.0 * fl / sec / 1e12 / PEAK_BF16_TFLOPS,
           "gradients_finite": all(bool(torch.isfinite(t.float()).all()) for t in grads[:5])}
    # the pair that keeps routing, permutation and pre-activations from the forward pass for the backward pass
    if ops.train_state_bytes(lay.T, lay.H, lay.E, lay.k, lay.I, torch.bfloat16) is not None:
        fargs = (lay.x, lay.wr, lay.bias, lay.wgu, lay.wd, lay.theta, lay.k)

        def timed(fn):
            rr = []
            for _ in range(3):
                torch.cuda.synchronize(lay.dev)
                t0 = time.perf_counter()
                for _ in range(n):
                    fn()
                torch.cuda.synchronize(lay.dev)
                rr.append((time.perf_counter() - t0) / n)
            return sorted(rr)[1]
        # the forward call is short enough for the binding's per-call host work to show: call the library directly on
        # buffers allocated once, as Layer.forward does
        _, _, state = ops.moe_forward_train(*fargs)
        bargs = (lay.x, d_out, lay.wr, lay.wgu, lay.wd, lay.theta, lay.k, state)
        saved = ops.moe_backward_saved(*bargs)
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        c_args = (P(lay.x), P(lay.wr), P(lay.bias), P(lay.wgu), P(lay.wd), P(lay.theta), ctypes.byref(lay.shape), lay.L.NORM_SUM,
                  P(lay.out), None, P(state), state.numel(), P(lay.ws), lay.ws.numel(), lay.stream)

        def forward_train():
            rc = lay.lib.bibo_moe_forward_train(*c_args)
            if rc != 0:
                lay.L.check(rc, "bibo_moe_forward_train")
        fwd_train = timed(forward_train)
        fwd_plain = timed(lay.forward)
        bwd_saved = timed(lambda: ops.moe_backward_saved(*bargs))
        res["kept_activations"] = {
            "entry": "bibo_moe_forward_train + bibo_moe_backward_saved",
            "forward_train_us_per_step": fwd_train * 1e6, "forward_us_per_step_same_loop": fwd_plain * 1e6,
            "backward_saved_us_per_step": bwd_saved * 1e6,
            "backward_saved_tflops": fl / bwd_saved / 1e12,
            "backward_saved_pct_bf16_mfma_peak": 100.0 * fl / bwd_saved / 1e12 / PEAK_BF16_TFLOPS,
            "state_bytes": int(state.numel()),
            "same_gradients": all(bool(torch.equal(a, b)) for a, b in zip(saved[:5], grads[:5]))}
    return res


def full_model(dev, batch=8, seq=2048, steps=10, warmup=3):
    """Config 5: the 10-layer experimental forward (HIP MoE block in layers 1-8, dense SwiGLU in 0 and 9, hybrid
    global / window-128 attention, Block Attention Residuals, tied 32000-token head), bf16, random init, uniform
    random token ids; end-to-end forward tokens/s, logits included."""
    import torch
    from bibo_amd import exp_model as X
    cfg = X.BiBoExpConfig()
    torch.manual_seed(20265)
    model = X.BiBoExpForCausalLM(cfg).to(dev).to(torch.bfloat16).eval()
    ids = torch.randint(0, cfg.vocab_size, (batch, seq), device=dev, generator=torch.Generator(device=dev).manual_seed(5))
    for _ in range(warmup):
        out = model(ids)
    runs = []
    for _ in range(3):
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        for _ in range(steps):
            out = model(ids)
        torch.cuda.synchronize(dev)
        runs.append((time.perf_counter() - t0) / steps)
    sec = sorted(runs)[1]
    # the MoE layers alone, timed inside the same model: ffn seam calls on the layer inputs of the last forward
    finite = bool(torch.isfinite(out.float()).all())
    n_moe = sum(l.is_moe_layer for l in model.model.layers)
    return {"workload": f"c5: 10-layer experimental forward, batch {batch} x seq {seq}, H=768, 4q/2kv heads of 192, "
                        f"window 128 on [G,S,S], AttnRes block 3, E=64 k=6 I=384 in {n_moe} MoE layers, vocab 32000, bf16",
            "tokens_per_s": batch * seq / sec, "ms_per_forward": sec * 1e3, "ms_per_forward_runs": [r * 1e3 for r in runs],
            "logits_finite": finite, "params": sum(p.numel() for p in model.parameters()),
            "note": "HIP MoE block per layer through bibo_moe_ffn_forward (norm + block + residual in one call), HIP depth "
                    "mix (bibo_moe_exp_attn_res_fwd) and row norms (bibo_moe_rmsnorm_fwd); attention, dense layers and the "
                    "head are stock PyTorch-ROCm operations"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4"])
    ap.add_argument("--algo", default="auto", choices=["auto", "generic", "mfma", "stream", "fused"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-model", action="store_true", help="skip the 10-layer forward (c5)")
    ap.add_argument("--no-side", action="store_true", help="skip the c1 / c4 lines, the seam and the backward pass")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only copy 256 MiB device to device a few times: the known-size kernel the FETCH_SIZE / WRITE_SIZE "
                         "counters of a profile are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    from bibo_amd import _lib
    if not _lib.LIB_PATH.exists():
        import __graft_entry__
        __graft_entry__.build()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calibrate_copy:
        src = torch.full((256 << 20,), 3, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize(dev)
        print(json.dumps({"calibrate_copy_bytes": src.numel(), "copies": 5}))
        return

    layer = Layer(args.workload, dev, args.algo)
    rel, e_active = layer.check()
    sec, runs = layer.time_forward(args.steps, args.warmup)
    stages = layer.time_stages(max(10, min(args.steps, 100)))
    T, H, E, k, I, S = layer.T, layer.H, layer.E, layer.k, layer.I, layer.S
    fl = flops_layer(T, H, E, k, I)
    if layer.fused:
        dom, dom_name, dom_flops = "gateup_down", "experts_fused_kernel (gate/up GEMM + Radial NormSiLU + down GEMM)", 6 * S * H * I
    else:
        dom, dom_name, dom_flops = "gateup", "gateup_dma_kernel (grouped gate/up GEMM + Radial NormSiLU)", 4 * S * H * I
    out = {
        "metric": "moe_layer_tokens_per_s", "value": T / sec, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: MoE layer forward T={T} H={H} E={E} k={k} I={I} bf16, seeded synthetic",
                   "algo": args.algo},
        "timing": f"median of {REPEATS} timed runs of {args.steps} steps each", "ms_per_step_runs": [r * 1e3 for r in runs],
        "tflops": fl / sec / 1e12, "pct_bf16_mfma_peak": 100.0 * fl / sec / 1e12 / PEAK_BF16_TFLOPS,
        "parity_rel_err_sample": rel, "experts_active": e_active,
        "stage_us": {n: v * 1e6 for n, v in stages.items()},
        "stage_us_note": "HIP events around each stage entry point; includes the gap to the next launch",
        "roofline": {"kernel": dom_name, "bound": "mfma",
                     "achieved": dom_flops / stages[dom] / 1e12, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": dom_flops / stages[dom] / 1e12 / PEAK_BF16_TFLOPS,
                     "traffic": measured_traffic(args.workload, dom)},
    }
    if layer.family == "stream":
        # The streaming kernels only exist behind the composite call (the stage entry points time the tile kernels):
        # the roofline of this workload is the HBM one, algorithmic bytes of the layer over the whole step, with the
        # expert weights rotated over four copies so that every step streams them from HBM.
        nbytes = bytes_layer(T, H, E, k, I, e_active)
        rsec, _ = layer.time_forward(args.steps, args.warmup, weight_sets=4)
        out["roofline"] = {"kernel": "gateup_stream_kernel + down_stream_kernel (whole bibo_moe_forward step, 4 weight sets)",
                           "bound": "hbm", "achieved": nbytes / rsec / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                           "frac": nbytes / rsec / 1e9 / PEAK_HBM_GBS, "traffic": measured_traffic(args.workload, "stream")}
        out["stage_us"] = {n: v for n, v in out["stage_us"].items() if n in ("router", "permute")}
    if not args.no_side:
        ffn_sec = layer.time_ffn_seam(args.steps, args.warmup)
        out["ffn_seam"] = {"entry": "bibo_moe_ffn_forward: out = h + moe(rmsnorm(h))", "us_per_step": ffn_sec * 1e6,
                           "extra_us_over_layer": (ffn_sec - sec) * 1e6}
        if args.workload == "c2":
            out["backward"] = backward_pass(layer, args.steps, args.warmup)
    if not args.no_decode and args.workload == "c2":
        d = Layer("c3", dev, args.algo)
        drel, dact = d.check()
        warm, _ = d.time_forward(args.steps, args.warmup)
        sets = 4
        rot, rot_runs = d.time_forward(args.steps, args.warmup, weight_sets=sets)
        db = bytes_layer(d.T, d.H, d.E, d.k, d.I, dact)
        out["decode"] = {"workload": f"c3: T={d.T} H={d.H} E={d.E} k={d.k} I={d.I} bf16", "tokens_per_s": d.T / rot,
                         "us_per_step": rot * 1e6, "algorithmic_bytes": db, "hbm_gbs": db / rot / 1e9,
                         "pct_hbm_peak": 100.0 * db / rot / 1e9 / PEAK_HBM_GBS,
                         "weight_sets": sets, "weight_bytes_rotated": sets * 2 * 3 * d.H * d.I * d.E,
                         "cache_warm_us_per_step": warm * 1e6, "cache_warm_gbs": db / warm / 1e9,
                         "cache_warm_pct_hbm_peak": 100.0 * db / warm / 1e9 / PEAK_HBM_GBS,
                         "experts_active": dact, "parity_rel_err_sample": drel,
                         "note": "whole layer through bibo_moe_forward (weight-streaming kernels); hbm_gbs rotates the "
                                 "expert weights over 4 separately allocated sets (805 MB, more than the 256 MB Infinity "
                                 "Cache) so every step streams them from HBM; cache_warm re-reads one 201 MB set"}
        if not args.no_side:
            out["c1"] = side_workload("c1", dev, args.algo, args.steps, args.warmup)
            out["c4"] = side_workload("c4", dev, args.algo, max(10, args.steps // 2), args.warmup)
        if not args.no_model:
            out["c5"] = full_model(dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.workload)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
