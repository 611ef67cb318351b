#!/usr/bin/env python3
"""Benchmark of the MoE expert path on one MI355X.

A step is one forward+backward pass of the MoE layer (router linear, top-k routing,
dispatch, grouped expert FFN, combine, and the whole backward) over one batch of synthetic
input that is already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3] [--no-cpu]
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (config 3), each
# scaled by the same counter's reading for a plain 1 GiB copy; the runs and the scale factors
# are in profiles/grouped_gemm_cfg3_pmc.txt.  bench.py cannot run the profiler on itself, so
# the figures are carried here and refreshed whenever that profile is.
MEASURED_HBM_BYTES_PER_LAUNCH = {
    (3, "gemm_gateup_swiglu_fwd_blocked"): 3.980e9,
    (3, "gemm_gateup_swiglu_fwd"): 3.980e9,
    (3, "gemm_down_fwd"): 1.813e9,
    (3, "gemm_dgrad_down_swiglu_bwd_blocked"): 2.450e9,
    (3, "gemm_dgrad_down_swiglu_bwd"): 2.450e9,
    (3, "gemm_dgrad_gateup_packed"): 3.790e9,
    (3, "gemm_dgrad_gateup"): 3.790e9,
    (3, "gemm_wgrad_down"): 1.074e9,
    (3, "gemm_wgrad"): 1.074e9,
    (3, "gemm_wgrad_pair"): 2.18e9,                # from the average over both weight-gradient launches
    (3, "gemm_wgrad_gate_and_up_pair"): 2.18e9,
}


def _event_time_ms(torch, fn, iters, warmup):
    """Average duration of fn() measured with HIP events recorded on the stream the kernels
    are launched on (torch's current stream is the one handed to the library)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    s = torch.cuda.Event(enable_timing=True)
    e = torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters


def _timed_steps(torch, step, steps, warmup):
    """W untimed steps, then K steps bracketed by synchronisations: -> (wall-clock mean ms per step,
    HIP-event median, HIP-event minimum).  One event is recorded on the launch stream after every
    step (K+1 records in all), so that the spread over the steps is seen next to the mean."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    per = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    median = per[len(per) // 2] if len(per) % 2 else 0.5 * (per[len(per) // 2 - 1] + per[len(per) // 2])
    return wall, median, per[0]


# flops of one launch of each GEMM entry point, in units of R*H*I
_GEMM_RHI = {"moe_gemm_gateup_swiglu_fwd": 4, "moe_gemm_gateup_swiglu_fwd_blocked": 4,
             "moe_gemm_down_fwd": 2, "moe_gemm_dgrad_down_swiglu_bwd": 2,
             "moe_gemm_dgrad_down_swiglu_bwd_dgate": 2, "moe_gemm_dgrad_down_swiglu_bwd_packed": 2,
             "moe_gemm_dgrad_down_swiglu_bwd_blocked": 2,
             "moe_gemm_dgrad_gateup": 4, "moe_gemm_dgrad_gateup_packed": 4, "moe_gemm_wgrad_pair": 4,
             "moe_gemm_wgrad": 2}


def _launches_in_step(torch, P, step, steps, RHI, flops):
    """The same K steps once more with a pair of HIP events around every launch of the library
    (its `observer` hook): -> (records per launch in step order, roofline fields of the GEMM launch
    with the largest duration, ms per step of this instrumented region)."""
    watch = _LaunchEvents(torch)
    P.lib.load().observer = watch
    t0 = time.perf_counter()
    try:
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
    finally:
        P.lib.load().observer = None
    ms_events = (time.perf_counter() - t0) * 1e3 / steps
    in_step = watch.per_launch_ms(steps)
    recs = []
    # moe_gemm_wgrad also serves the router's small split-k product, and (with few experts) the
    # row segments of one stack: a launch counts as an expert weight gradient of 2*R*H*I when it
    # lasts at least a tenth of the longest one
    longest_wgrad = max([m for n, m in in_step if n == "moe_gemm_wgrad"], default=0.0)
    for name, kms in in_step:
        rec = {"entry": name, "ms": round(kms, 4)}
        f = _GEMM_RHI.get(name)
        if f and kms > 0 and not (name == "moe_gemm_wgrad" and kms < 0.1 * longest_wgrad):
            rec.update(achieved=round(f * RHI / kms / 1e9, 1), unit="TFLOP/s",
                       frac=round(f * RHI / kms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4))
        recs.append(rec)
    roof = None
    g_in = [r for r in recs if "frac" in r]
    if g_in:
        dom = max(g_in, key=lambda r: r["ms"])
        g_ms = sum(r["ms"] for r in g_in)
        roof = {"kernel": dom["entry"].replace("moe_", "", 1), "bound": "mfma", "achieved": dom["achieved"],
                "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac"], "traffic": None,
                "ms": dom["ms"],
                "measured": f"HIP events around this launch in each of {steps} steps that follow the timed "
                            f"ones ({round(ms_events, 4)} ms per step with the events)",
                "all_gemms_tflops": round(flops / g_ms / 1e9, 1),
                "all_gemms_frac": round(flops / g_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                "launches_ms_sum": round(sum(r["ms"] for r in recs), 4)}
    return recs, roof, ms_events


class _LaunchEvents:
    """Observer of the library's launches: a pair of HIP events around every entry point,
    recorded on torch's current stream (the stream the launch is handed), so that each kernel's
    duration can be read inside the timed steps themselves."""

    def __init__(self, torch):
        self.torch = torch
        self.pairs = []
        self._start = None

    def before(self, name):
        self._start = self.torch.cuda.Event(enable_timing=True)
        self._start.record()

    def after(self, name):
        end = self.torch.cuda.Event(enable_timing=True)
        end.record()
        self.pairs.append((name, self._start, end))

    def per_launch_ms(self, steps):
        """[(entry point, mean ms)] in the order of one step's launches (every step launches the
        same sequence), after a synchronisation."""
        n = len(self.pairs) // steps
        if n == 0 or n * steps != len(self.pairs):
            return []
        if any(self.pairs[i][0] != self.pairs[i % n][0] for i in range(len(self.pairs))):
            return []
        out = []
        for j in range(n):
            ms = [self.pairs[i][1].elapsed_time(self.pairs[i][2]) for i in range(j, len(self.pairs), n)]
            out.append((self.pairs[j][0], sum(ms) / len(ms)))
        return out


def _moe_dominant_kernel(torch, P, s, x_bf16, wr_bf16, ws_bf16):
    """HIP-event duration of the gate/up grouped GEMM (the kernel with the largest share of the
    layer) on the layer's own routing of `x_bf16`: the `roofline` object of a configuration."""
    ops = P.ops
    with torch.no_grad():
        logits = x_bf16 @ wr_bf16.t()
        ids, _ = ops.router_topk(logits, s.k, None)
        _, offs, p2r, r2p = ops.histogram_scan(ids, s.E)
        xp = ops.permute_fwd(x_bf16, p2r, s.k, r2p)
        ms = _event_time_ms(torch, lambda: ops.gemm_gateup_blocked(xp, ws_bf16[0], ws_bf16[1], offs), 10, 2)
    fl = 4 * s.R * s.H * s.I
    return {"kernel": "gemm_gateup_swiglu_fwd", "bound": "mfma", "achieved": round(fl / ms / 1e9, 1),
            "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(fl / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
            "traffic": None, "ms": round(ms, 4)}


def bench_block(args, torch, P, dev, steps=None, warmup=None, cpu=True):
    """Configuration 5: one GPT-MoE block (RMSNorm, GQA attention, MoE) forward+backward under
    bf16 autocast with fp32 parameters; reports tokens/s and the MoE's share of the time."""
    steps = steps or args.steps
    warmup = args.warmup if warmup is None else warmup
    s = P.configs.SHAPES[5]
    B, T = 2, 4096
    cfg = P.ModelConfig(hidden_size=s.H, num_attention_heads=32, num_key_value_heads=8, num_experts=s.E,
                        num_experts_per_tok=s.k, moe_intermediate_size=s.I, init_std=0.02, use_moe=True,
                        seed=P.configs.BASE_SEED, vocab_size=50304)
    blk = P.Block(cfg, s.k)
    wte = torch.nn.Embedding(cfg.vocab_size, s.H, device=dev)
    torch.nn.init.normal_(wte.weight, mean=0.0, std=0.02)
    g = torch.Generator().manual_seed(P.configs.BASE_SEED)
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=g).to(dev)
    dy = torch.randn(B, T, s.H, generator=g).to(dev)
    seen = {}
    hook = blk.mlp.register_forward_hook(lambda m, i, o: seen.update(moe_in=i[0].detach()))

    def step():
        blk.zero_grad(set_to_none=True)
        wte.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = blk(wte(ids))
        out.backward(dy)

    def timed():
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    # the caller as the reference writes it (gpt.py:32-33: norm, layer, residual add as three
    # calls), then with the norm and the residual add inside the layer's call
    ms_separate = timed()
    hook.remove()
    blk.fused_prenorm = True
    ms = timed()
    moe_in = seen["moe_in"].clone().requires_grad_(True)

    def moe_step():
        blk.mlp.zero_grad(set_to_none=True)
        moe_in.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            o = blk.mlp(moe_in)[0]
        o.backward(dy)

    moe_ms = _event_time_ms(torch, moe_step, max(steps // 2, 3), 2)
    flops = P.configs.gemm_flops(s)
    bf = torch.bfloat16
    m = blk.mlp
    wb = [w.detach().to(bf) for w in (m.experts_gate_weights, m.experts_up_weights, m.experts_down_weights)]
    x2 = moe_in.detach().reshape(B * T, s.H).to(bf)
    roofline = _moe_dominant_kernel(torch, P, s, x2, m.router.weight.detach().to(bf), wb)
    cpu_rec = None
    if cpu:
        # the oracle's per-expert loop on the rows the MoE received inside the block (1/4 of them)
        from oracle import moe_oracle as O
        ncores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(ncores)
        n = B * T // 4
        xc = x2[:n].cpu()
        wc = [w.cpu().float() for w in wb]
        wrc = m.router.weight.detach().to(bf).cpu().float()
        dyc = dy.reshape(B * T, s.H)[:n].cpu()
        t0 = time.perf_counter()
        f = O.moe_forward(xc, wrc, *wc, s.k, logits_dtype=bf)
        O.moe_backward(f, dyc, wrc, *wc)
        dt = time.perf_counter() - t0
        cpu_rec = {"value": round(n / dt, 1), "unit": "tokens/s", "cores": ncores, "kind": "port",
                   "sample": f"MoE part only (oracle per-expert loop, fp32 math on the bf16 rows the layer received in "
                             f"the block), {n} of {B * T} tokens, one timed pass of {dt:.2f} s; attention and norms "
                             f"are stock torch on both sides and are not in the sample",
                   "moe_tflops": round(18 * n * s.k * s.H * s.I / dt / 1e12, 4)}
    del blk, wte
    torch.cuda.empty_cache()
    return {
        "metric": "gpt_moe_block_fwd_bwd_tokens_per_s", "value": round(B * T / (ms * 1e-3), 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": s.name + " inside one GPT-MoE block (RMSNorm, GQA 32/8 heads x 64, seq 4096, batch 2), "
                               "fp32 parameters under bf16 autocast, ln_2 and the residual add inside the layer's call "
                               "(MoE.forward_prenorm)", "tokens": B * T},
        "ms_per_step_separate_norm_and_residual": round(ms_separate, 4),
        "moe_ms": round(moe_ms, 4), "moe_share_of_block_time": round(moe_ms / ms, 4),
        "moe_gemm_tflops": round(flops / moe_ms / 1e9, 1),
        "roofline": roofline, "cpu_baseline": cpu_rec,
    }


def time_layer_config(P, torch, dev, cfg_id, steps, warmup):
    """ms per step of one benchmark configuration (1, 2, 3 or 4) through the entry the module
    uses (`routed_moe`; `experts_rows` for the post-dispatch configuration 4)."""
    inp = P.configs.make_inputs(cfg_id)
    s = inp["shape"]
    if s.rows_entry:
        x = inp["x"].to(dev).requires_grad_(True)
        ids = inp["ids"].to(dev)
        ws = [inp[n].to(dev).requires_grad_(True) for n in ("w1", "w3", "w2")]
        dy = inp["dy"].to(dev)
        leaves = (x, *ws)

        def step():
            for t in leaves:
                t.grad = None
            P.experts_rows(x, ids, *ws).backward(dy)
    else:
        x = inp["x"].to(dev).requires_grad_(s.backward)
        wr = inp["wr"].to(dev).requires_grad_(s.backward)
        ws = [inp[n].to(dev).requires_grad_(s.backward) for n in ("w1", "w3", "w2")]
        dy = inp["dy"].to(dev) if s.backward else None
        bias = inp["bias"].to(dev) if "bias" in inp else None
        leaves = (x, wr, *ws)

        def step():
            for t in leaves:
                t.grad = None
            out, _ = P.routed_moe(x, wr, *ws, s.k, bias=bias)
            if s.backward:
                out.backward(dy)
    ms, ms_median, ms_min = _timed_steps(torch, step, steps, warmup)
    flops = P.configs.gemm_flops(s)
    recs, roof, _ = _launches_in_step(torch, P, step, steps, s.R * s.H * s.I, flops)
    return {"config": cfg_id, "workload": s.name, "entry": "experts_rows" if s.rows_entry else "routed_moe",
            "ms_per_step": round(ms, 4), "ms_per_step_median": round(ms_median, 4), "ms_per_step_min": round(ms_min, 4),
            "tflops": round(flops / ms / 1e9, 1),
            "mfma_peak_frac": round(flops / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
            "tokens_per_s": round(s.T / (ms * 1e-3), 1), "steps": steps, "roofline": roof,
            "kernels_in_step": recs}


def cpu_leg(P, torch, cfg_id, fraction=1.0):
    """The oracle's per-expert loop (forward, and backward where the configuration has one) on
    the host cores: the CPU baseline of a configuration.  The two small configurations are run
    once to warm up and then three times (the median is reported); the large ones, which take
    seconds, once."""
    from oracle import moe_oracle as O
    ncores = os.cpu_count() or 1
    ncores = min(ncores, int(os.environ.get("OMP_NUM_THREADS", ncores)))
    torch.set_num_threads(ncores)
    cin = P.configs.make_inputs(cfg_id, scale_tokens=fraction)
    s = cin["shape"]
    w32 = [cin[n].float() for n in ("w1", "w3", "w2")]

    def one_pass():
        t0 = time.perf_counter()
        if s.rows_entry:
            f = O.experts_rows_forward(cin["x"], cin["ids"].numpy(), *w32)
            O.experts_rows_backward(f, cin["dy"].float(), *w32)
        else:
            wr32 = cin["wr"].float()
            f = O.moe_forward(cin["x"], wr32, *w32, s.k, bias=cin.get("bias"), logits_dtype=torch.bfloat16)
            if s.backward:
                O.moe_backward(f, cin["dy"].float(), wr32, *w32)
        return time.perf_counter() - t0

    if s.rows_entry:
        rows = cin["x"].shape[0]
        toks = rows / s.k
    else:
        toks = cin["x"].shape[0]
        rows = toks * s.k
    small = cfg_id in (1, 2)
    if small:
        one_pass()
        times = sorted(one_pass() for _ in range(3))
        dt, how = times[1], f"one warm-up pass, then the median of three timed passes ({times[1]:.3f} s)"
    else:
        dt = one_pass()
        how = f"one timed pass of {dt:.2f} s"
    cflops = (18 if s.backward else 6) * rows * s.H * s.I
    return {"value": round(cflops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": ncores, "kind": "port",
            "sample": f"oracle per-expert loop, fp32 math on the same bf16 inputs, {int(toks)} of {s.T} tokens "
                      f"({rows} routed rows, all {s.E} experts), {how}",
            "tokens_per_s": round(toks / dt, 1)}


def module_config3(P, torch, dev, steps, warmup):
    """Configuration 3 through the module as the reference's trainer calls it (trainer.py:209-216,
    241-248): fp32 master weights and fp32 residual input under bf16 autocast, fp32 weight
    gradients; a fresh step (gradients created) and a gradient-accumulation micro-step with the
    weight-gradient kernel adding into `.grad`."""
    s = P.configs.SHAPES[3]
    inp = P.configs.make_inputs(3)
    cfg = P.ModelConfig(hidden_size=s.H, num_experts=s.E, num_experts_per_tok=s.k, moe_intermediate_size=s.I,
                        init_std=0.02, seed=P.configs.BASE_SEED)
    m = P.MoE(cfg, s.k)
    x = inp["x"].float().reshape(4, 4096, s.H).to(dev).requires_grad_(True)
    dy = inp["dy"].float().reshape(4, 4096, s.H).to(dev)
    flops = P.configs.gemm_flops(s)
    out = {}
    for name, accumulate, in_kernel in (("fresh_grads", False, False),
                                        ("accumulating_micro_step_autograd_adds", True, False),
                                        ("accumulating_micro_step_kernel_adds", True, True)):
        m.accumulate_wgrad_into_grad = in_kernel

        def step():
            if not accumulate:
                m.zero_grad(set_to_none=True)
            x.grad = None
            with torch.autocast("cuda", dtype=torch.bfloat16):
                o, _ = m(x)
            o.backward(dy)

        m.zero_grad(set_to_none=True)
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        out[name] = {"ms_per_step": round(ms, 4), "tflops": round(flops / ms / 1e9, 1),
                     "tokens_per_s": round(s.T / (ms * 1e-3), 1)}
    # the same fresh step with the module under `torch.compile` (the reference's --use_compile,
    # trainer.py:130-131, default backend): the layer body is the pair of registered operators,
    # which cast the fp32 expert weights in every forward as the reference does
    try:
        m.accumulate_wgrad_into_grad = False
        cm = torch.compile(m, fullgraph=True)

        def cstep():
            m.zero_grad(set_to_none=True)
            x.grad = None
            with torch.autocast("cuda", dtype=torch.bfloat16):
                o, _ = cm(x)
            o.backward(dy)

        for _ in range(max(warmup, 2)):
            cstep()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            cstep()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        out["fresh_grads_torch_compile"] = {"ms_per_step": round(ms, 4), "tflops": round(flops / ms / 1e9, 1),
                                            "tokens_per_s": round(s.T / (ms * 1e-3), 1)}
        del cm
    except Exception as e:  # a broken compiler stack on the box must not cost the benchmark line
        out["fresh_grads_torch_compile"] = {"error": repr(e)[:300]}
    torch._dynamo.reset()
    del m
    torch.cuda.empty_cache()
    return {"config": 3, "workload": s.name + ", MoE module with fp32 master weights and fp32 input under bf16 "
                                              "autocast (the reference trainer's calling convention), fp32 weight gradients",
            "entry": "MoE.forward", **out}


MFMA_F32_PEAK_TFLOPS = 157.3     # MI355X dense fp32 matrix


def fp32_config3(P, torch, dev, steps=3, warmup=1):
    """Configuration 3 in fp32 from end to end (`moe_ffn_f32`: what the reference computes when its
    layer is called without autocast on fp32 tensors), priced against the fp32 matrix peak."""
    s = P.configs.SHAPES[3]
    inp = P.configs.make_inputs(3)
    x = inp["x"].float().to(dev).requires_grad_(True)
    wr = inp["wr"].float().to(dev)
    ws = [inp[n].float().to(dev).requires_grad_(True) for n in ("w1", "w3", "w2")]
    dy = inp["dy"].float().to(dev)
    logits = torch.nn.functional.linear(x.detach(), wr).requires_grad_(True)
    leaves = (x, logits, *ws)

    def step():
        for t in leaves:
            t.grad = None
        P.moe_ffn_f32(x, logits, *ws, s.k).backward(dy)

    ms, ms_median, ms_min = _timed_steps(torch, step, steps, warmup)
    flops = P.configs.gemm_flops(s)
    watch = _LaunchEvents(torch)
    P.lib.load().observer = watch
    try:
        step()
        torch.cuda.synchronize()
    finally:
        P.lib.load().observer = None
    per = {"moe_f32_gemm_rows": 2, "moe_f32_gemm_wgrad": 2}  # flops per launch in units of R*H*I
    recs, g_ms = [], 0.0
    for name, kms in watch.per_launch_ms(1):
        rec = {"entry": name, "ms": round(kms, 4)}
        if name in per and kms > 0:
            tf = per[name] * s.R * s.H * s.I / kms / 1e9
            rec.update(achieved=round(tf, 1), unit="TFLOP/s", frac=round(tf / MFMA_F32_PEAK_TFLOPS, 4))
            g_ms += kms
        recs.append(rec)
    dom = max((r for r in recs if "frac" in r), key=lambda r: r["ms"])
    roof = {"kernel": dom["entry"].replace("moe_", "", 1), "bound": "mfma", "achieved": dom["achieved"],
            "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac"], "traffic": None, "ms": dom["ms"],
            "measured": "HIP events around this launch in one step that follows the timed ones",
            "all_gemms_tflops": round(flops / g_ms / 1e9, 1),
            "all_gemms_frac": round(flops / g_ms / 1e9 / MFMA_F32_PEAK_TFLOPS, 4)}
    del x, ws, dy, logits, leaves
    torch.cuda.empty_cache()
    return {"config": 3, "workload": s.name + ", every tensor and every product in fp32 (no autocast)",
            "entry": "moe_ffn_f32", "dtype": "f32", "ms_per_step": round(ms, 4),
            "ms_per_step_median": round(ms_median, 4), "ms_per_step_min": round(ms_min, 4),
            "tflops": round(flops / ms / 1e9, 1), "fp32_matrix_peak_frac": round(flops / ms / 1e9 / MFMA_F32_PEAK_TFLOPS, 4),
            "tokens_per_s": round(s.T / (ms * 1e-3), 1), "steps": steps, "roofline": roof, "kernels_in_step": recs}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=3, choices=(1, 2, 3, 4, 5))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--graph", action="store_true",
                    help="also time the step captured in one HIP graph (extra field ms_per_step_graph_replay)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (a kernel of known traffic, for scaling "
                         "profiler byte counters)")
    ap.add_argument("--cpu-fraction", type=float, default=1.0,
                    help="fraction of the tokens the CPU baseline sample processes")
    ap.add_argument("--no-kernel-events", dest="kernel_events", action="store_false",
                    help="record no HIP events around the launches inside the timed steps")
    ap.add_argument("--no-kernel-loops", action="store_true",
                    help="skip the separate back-to-back timing loops of the single kernels and the library's "
                         "dense reference (a profiler then sees the launches of the steps only)")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the short runs of the other benchmark configurations (field other_configs)")
    ap.add_argument("--fp32", action="store_true",
                    help="time only configuration 3 in fp32 from end to end (the other_configs entry "
                         "`moe_ffn_f32`) and print its record")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (one rank's share of the MoE layer, "
              "no collectives); --gpus must be 1", file=sys.stderr)
        return 2

    import torch
    import torch.nn.functional as F
    P = importlib.import_module("train-large-model-from-scratch_amd")
    if not os.path.exists(P.lib.LIB_PATH):
        importlib.import_module("__graft_entry__").build()
    P.lib.load()
    ops = P.ops
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.fp32:
        print(json.dumps(fp32_config3(P, torch, dev, steps=min(args.steps, 5), warmup=min(args.warmup, 2))),
              flush=True)
        return 0
    if args.config == 5:
        print(json.dumps(bench_block(args, torch, P, dev, cpu=not args.no_cpu)), flush=True)
        return 0

    inp = P.configs.make_inputs(args.config)
    s = inp["shape"]
    flops = P.configs.gemm_flops(s)
    RHI = s.R * s.H * s.I

    # ---------------- the timed step: inputs resident in HBM
    if s.rows_entry:
        x = inp["x"].to(dev).requires_grad_(True)
        ids = inp["ids"].to(dev)
        ws = [inp[n].to(dev).requires_grad_(True) for n in ("w1", "w3", "w2")]
        dy = inp["dy"].to(dev)

        def step():
            for t in (x, *ws):
                t.grad = None
            out = P.experts_rows(x, ids, *ws)
            out.backward(dy)
    else:
        x = inp["x"].to(dev).requires_grad_(s.backward)
        wr = inp["wr"].to(dev).requires_grad_(s.backward)
        ws = [inp[n].to(dev).requires_grad_(s.backward) for n in ("w1", "w3", "w2")]
        dy = inp["dy"].to(dev) if s.backward else None
        bias = inp["bias"].to(dev) if "bias" in inp else None

        def step():
            for t in (x, wr, *ws):
                t.grad = None
            out, _ = P.routed_moe(x, wr, *ws, s.k, bias=bias)
            if s.backward:
                out.backward(dy)

    ms, ms_median, ms_min = _timed_steps(torch, step, args.steps, args.warmup)
    tflops = flops / ms / 1e9
    # The same K steps once more, now with a pair of HIP events around every launch: each
    # kernel's duration inside the step.  A region of its own because the 2 x 15 event records
    # per step cost about 1 % of the step (5.33 against 5.28 ms on configuration 3), which the
    # headline figure should not carry.  (Where the step is bound by the host's launches, the two
    # small configurations, the events lengthen the step but not the kernels they bracket.)
    in_step_recs, roof_in_step, ms_events = [], None, None
    if args.kernel_events:
        in_step_recs, roof_in_step, ms_events = _launches_in_step(torch, P, step, args.steps, RHI, flops)
    tokens_per_s = s.T / (ms * 1e-3)

    # the same step captured once in a HIP graph and replayed: what a caller gets who removes
    # the host's launch cost (it only shows where a step is shorter than its ~30 launches)
    ms_graph = None
    if args.graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        for t in ((x, *ws) if s.rows_entry else (x, wr, *ws)):
            t.grad = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        ms_graph = (time.perf_counter() - t0) * 1e3 / args.steps
        del graph

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # ---------------- per-kernel durations (HIP events), for the roofline object
    per_kernel, lib_ref = [], {}
    if not args.no_kernel_loops:
        with torch.no_grad():
            xd = x.detach()
            w1, w3, w2 = (w.detach() for w in ws)
            if s.rows_entry:
                _, offs, p2r, r2p = ops.histogram_scan(ids.to(torch.int32), s.E)
                kk, gates = 1, None
            else:
                logits = F.linear(xd, wr.detach())
                rids, gates = ops.router_topk(logits, s.k, bias)
                _, offs, p2r, r2p = ops.histogram_scan(rids, s.E)
                kk = s.k
            xp = ops.permute_fwd(xd, p2r, kk, r2p)
            gu, act = ops.gemm_gateup_blocked(xp, w1, w3, offs)
            y = ops.gemm_down(act, w2, offs)
            dyy = dy if dy is not None else torch.randn_like(xd)
            dyp, _ = ops.combine_bwd(dyy, None, gates, p2r, kk, r2p)
            routed = gates is not None  # the gate gradients' block sums ride in the dgrad-down kernel
            # (dg and du side by side in one buffer, as the backward pass keeps them when I % 256 == 0:
            # their two weight gradients are then one launch)
            packed = s.I % 256 == 0
            if packed:
                dgu = ops.gemm_dgrad_down_blocked(dyp, w2, gu, offs, dgate_blocks=routed, packed=True)[0]
                dxp = ops.gemm_dgrad_gateup_packed(dgu, w1, w3, offs)
                dg = dgu[:, :s.I].contiguous()
            else:
                dg, du = ops.gemm_dgrad_down_blocked(dyp, w2, gu, offs, dgate_blocks=routed)[:2]
                dxp = ops.gemm_dgrad_gateup(dg, du, w1, w3, offs)
            bf = torch.bfloat16
            a = 2  # bytes per bf16 element
            T, R, H, I, E = xd.shape[0], s.R, s.H, s.I, s.E
            kernels = [
                # name, callable, algorithmic flops, algorithmic bytes, launches per step
                ("gemm_gateup_swiglu_fwd", lambda: ops.gemm_gateup_blocked(xp, w1, w3, offs), 4 * RHI, 0, 1),
                ("gemm_down_fwd", lambda: ops.gemm_down(act, w2, offs), 2 * RHI, 0, 1),
                ("gemm_dgrad_down_swiglu_bwd",
                 (lambda: ops.gemm_dgrad_down_blocked(dyp, w2, gu, offs, dgate_blocks=routed, packed=packed)),
                 2 * RHI, 0, 1),
                ("gemm_dgrad_gateup",
                 (lambda: ops.gemm_dgrad_gateup_packed(dgu, w1, w3, offs)) if packed else
                 (lambda: ops.gemm_dgrad_gateup(dg, du, w1, w3, offs)), 4 * RHI, 0, 1),
                ("gemm_wgrad_down", lambda: ops.gemm_wgrad(dyp, act, offs, E, bf), 2 * RHI, 0, 1),
                (("gemm_wgrad_gate_and_up_pair", lambda: ops.gemm_wgrad_pair(dgu, xp, offs, E, bf), 4 * RHI, 0, 1) if packed
                 else ("gemm_wgrad_gate_or_up", lambda: ops.gemm_wgrad(dg, xp, offs, E, bf), 2 * RHI, 0, 2)),
                ("permute_fwd", lambda: ops.permute_fwd(xd, p2r, kk, r2p), 0, T * H * a + R * H * a + R * 4, 1),
                ("combine_fwd", lambda: ops.combine_fwd(y, gates, r2p, T, kk, xd.dtype), 0,
                 R * H * a + R * 8 + T * H * a, 1),
                ("combine_bwd", lambda: ops.combine_bwd(dyy, None, gates, p2r, kk, r2p), 0,
                 T * H * a + R * H * a + R * 8, 1),
                ("permute_bwd", lambda: ops.permute_bwd(dxp, r2p, T, kk, xd.dtype), 0, R * H * a + T * H * a, 1),
            ]
            # fp32 master -> bf16 operand cast of one weight stack: not part of this step (the
            # configuration hands over bf16 weights); the module pays it once per optimizer step
            # and stack, the reference once per forward and stack
            w_master = torch.empty(w1.shape, dtype=torch.float32, device=dev).normal_()
            kernels.append(("cast_f32_bf16_one_weight_stack", lambda: ops.cast_bf16(w_master), 0,
                            w_master.numel() * 6, 0))
            # what the memory system of this part gives plain streaming kernels of the runtime, in the
            # same run: the yardstick for the row movers (a 1 GiB device copy, a 1 GiB fill)
            src_c = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
            dst_c = torch.empty_like(src_c)
            kernels.append(("reference_device_copy_1GiB", lambda: dst_c.copy_(src_c), 0, 2 * src_c.numel() * 4, 0))
            kernels.append(("reference_device_fill_1GiB", lambda: dst_c.zero_(), 0, src_c.numel() * 4, 0))
            per_kernel = []
            for name, fn, fl, by, launches in kernels:
                kms = _event_time_ms(torch, fn, 10, 2)
                rec = {"kernel": name, "ms": round(kms, 4), "launches_per_step": launches}
                if fl:
                    rec.update(bound="mfma", achieved=round(fl / kms / 1e9, 1), unit="TFLOP/s",
                               frac=round(fl / kms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4))
                else:
                    rec.update(bound="hbm", achieved=round(by / kms / 1e6, 1), unit="GB/s",
                               frac=round(by / kms / 1e6 / HBM_PEAK_GBS, 4))
                per_kernel.append(rec)
            del src_c, dst_c
            # what the vendor's dense GEMM library reaches on this part on problems of the same size
            # with none of the layer's structure (one weight for all rows, no ragged groups, no fused
            # epilogue, one output): the practical ceiling the grouped kernels are measured against
            lib_ref = {}
            if True:
                wd = torch.randn(2 * I, H, device=dev).to(bf) * 0.02
                wdn = torch.randn(H, I, device=dev).to(bf) * 0.02
                t_gu = _event_time_ms(torch, lambda: torch.mm(xp, wd.t()), 10, 3)
                t_dn = _event_time_ms(torch, lambda: torch.mm(act, wdn.t()), 10, 3)
                lib_ref = {"what": "torch.mm (hipBLASLt) on dense problems of the gate/up and down sizes: "
                                   "[R,H]x[H,2I] and [R,I]x[I,H], bf16, same random data scale",
                           "gateup_size_tflops": round(4 * RHI / t_gu / 1e9, 1), "down_size_tflops": round(2 * RHI / t_dn / 1e9, 1),
                           "gateup_size_frac_of_peak": round(4 * RHI / t_gu / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)}
                del wd, wdn
    gemms = [r for r in per_kernel if r["bound"] == "mfma"]
    if not s.backward:
        gemms = gemms[:2]
    roofline = {"kernel": None, "bound": "mfma", "achieved": None, "peak": MFMA_BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": None, "traffic": None}
    dominant = None
    if gemms:
        dominant = max(gemms, key=lambda r: r["ms"] * r["launches_per_step"])
        gemm_ms = sum(r["ms"] * r["launches_per_step"] for r in gemms)
        roofline.update(kernel=dominant["kernel"], achieved=dominant["achieved"], frac=dominant["frac"],
                        all_gemms_tflops=round(flops / gemm_ms / 1e9, 1),
                        all_gemms_frac=round(flops / gemm_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4))

    # the same kernels inside the timed steps (events around every launch): these are the
    # durations the roofline object reports where they exist; the figures from the separate
    # loops above stay beside them
    if roof_in_step:
        roofline.update(roof_in_step)
        roofline["achieved_back_to_back"] = dominant["achieved"] if dominant else None

    roofline["traffic"] = MEASURED_HBM_BYTES_PER_LAUNCH.get((args.config, roofline["kernel"]))
    roofline["traffic_source"] = ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this benchmark, "
                                  "profiles/grouped_gemm_cfg3_pmc.txt (not measured by this run)"
                                  if roofline["traffic"] is not None else None)

    # ---------------- CPU baseline: the oracle's per-expert loop on a bounded sample
    cpu = None if args.no_cpu else cpu_leg(P, torch, args.config, args.cpu_fraction)

    # ---------------- the other benchmark configurations, briefly (the default run only)
    others = None
    if args.config == 3 and not args.no_others:
        others = []
        for cid, fraction in ((1, 1.0), (2, 1.0), (4, 1.0)):
            # (the two small configurations take well under a millisecond per step: more steps, so
            # that one hiccup of the host does not show in their wall-clock mean)
            n_steps = max(args.steps * 2, 40) if cid in (1, 2) else max(args.steps // 2, 5)
            rec = time_layer_config(P, torch, dev, cid, n_steps, args.warmup)
            if not args.no_cpu:
                rec["cpu_baseline"] = cpu_leg(P, torch, cid, fraction)
            others.append(rec)
        others.append(module_config3(P, torch, dev, max(args.steps // 2, 5), args.warmup))
        others.append(fp32_config3(P, torch, dev))
        blk = bench_block(args, torch, P, dev, steps=max(args.steps // 2, 5), warmup=3, cpu=not args.no_cpu)
        others.append({"config": 5, "workload": blk["config"]["workload"], "entry": "Block.forward",
                       "ms_per_step": blk["ms_per_step"], "tokens_per_s": blk["value"],
                       "ms_per_step_separate_norm_and_residual": blk["ms_per_step_separate_norm_and_residual"],
                       "moe_ms": blk["moe_ms"], "moe_share_of_block_time": blk["moe_share_of_block_time"],
                       "moe_gemm_tflops": blk["moe_gemm_tflops"], "roofline": blk["roofline"],
                       "cpu_baseline": blk["cpu_baseline"], "steps": blk["steps"]})

    line = {
        "metric": "moe_layer_fwd_bwd_tflops" if s.backward else "moe_layer_fwd_tflops",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "ms_per_step_median": round(ms_median, 4), "ms_per_step_min": round(ms_min, 4),
        "ms_per_step_timing": "ms_per_step: wall clock around the K steps between two synchronisations, / K; "
                              "median and min: HIP events recorded on the launch stream after every step",
        "config": {"workload": s.name, "tokens": s.T, "hidden": s.H, "experts": s.E, "top_k": s.k,
                   "ffn": s.I, "routed_rows": s.R, "gemm_flops_per_step": flops},
        "tokens_per_s": round(tokens_per_s, 1),
        "ms_per_step_graph_replay": None if ms_graph is None else round(ms_graph, 4),
        "mfma_peak_frac_whole_step": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
        "roofline": roofline, "cpu_baseline": cpu, "kernels": per_kernel, "kernels_in_step": in_step_recs or None,
        "library_dense_reference": lib_ref,
        "other_configs": others,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
